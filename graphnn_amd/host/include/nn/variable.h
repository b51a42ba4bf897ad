// Variables of the computation graph (interface of graphnn's include/nn/variable.h):
// a named handle around a dense tensor (value + gradient), a CSR tensor, or the batch
// GraphStruct.  Placeholders are bound per batch with SetRef (a shallow copy).
#ifndef VARIABLE_H
#define VARIABLE_H

#include <string>
#include <vector>
#include "tensor/tensor_all.h"
#include "util/graph_struct.h"

namespace gnn
{

class FactorGraph;

class IDifferentiable
{
public:
    virtual ~IDifferentiable() {}
    virtual void ZeroGrad() = 0;
    virtual void OnesGrad() = 0;
    // Shapes the gradient like the value and reports its device buffer WITHOUT clearing it, so that the
    // caller can clear many gradients in one launch; false: the gradient has no such buffer, use ZeroGrad.
    virtual bool GradBuffer(void** device_ptr, size_t* bytes) { (void)device_ptr; (void)bytes; return false; }
};

namespace detail
{
template<typename mode, typename Dtype>
inline bool grad_buffer(DTensor<mode, Dtype>&, RowSpTensor<mode, Dtype>&, void**, size_t*) { return false; }
inline bool grad_buffer(DTensor<GPU, float>& value, RowSpTensor<GPU, float>& grad, void** device_ptr, size_t* bytes)
{
    if (!(grad.shape == value.shape)) grad.Reshape(value.shape.dims);
    grad.is_full = true;
    *device_ptr = grad.data->ptr;
    *bytes = sizeof(float) * grad.shape.Count();
    return true;
}
}  // namespace detail

class Variable
{
public:
    Variable(std::string _name) : name(_name) {}
    virtual ~Variable() {}
    virtual void SetRef(void* p) NOT_IMPLEMENTED
    virtual EleType GetEleType() = 0;
    virtual MatMode GetMode() = 0;
    std::string name;
};

class GraphVar : public Variable
{
public:
    GraphVar(std::string _name) : Variable(_name), graph(nullptr) {}
    virtual EleType GetEleType() override { return EleType::UNKNOWN; }
    virtual MatMode GetMode() override { return MatMode::cpu; }
    virtual void SetRef(void* p) override { graph = static_cast<GraphStruct*>(p); }
    GraphStruct* graph;
};

template<typename mode, typename matType, typename Dtype> class TensorVarTemplate;
template<typename mode, typename Dtype> using DTensorVar = TensorVarTemplate<mode, DENSE, Dtype>;
template<typename mode, typename Dtype> using SpTensorVar = TensorVarTemplate<mode, CSR_SPARSE, Dtype>;

template<typename mode, typename Dtype>
class TensorVar : public Variable
{
public:
    TensorVar(std::string _name) : Variable(_name) {}

    template<typename matType>
    TensorVarTemplate<mode, matType, Dtype>& Derived()
    {
        auto* p = dynamic_cast<TensorVarTemplate<mode, matType, Dtype>*>(this);
        ASSERT(p, "wrong derived type of TensorVar");
        return *p;
    }
    virtual EleType GetEleType() override { return Dtype2Enum<Dtype>(); }
    virtual MatMode GetMode() override { return mode::type; }
    virtual Dtype AsScalar() = 0;
    virtual MatType GetMatType() = 0;
};

template<typename mode, typename matType, typename Dtype>
class TensorVarTemplate : TensorVar<mode, Dtype> {};

template<typename mode, typename Dtype>
class TensorVarTemplate<mode, DENSE, Dtype> : public TensorVar<mode, Dtype>, public IDifferentiable
{
public:
    TensorVarTemplate(std::string _name) : TensorVar<mode, Dtype>(_name) {}
    TensorVarTemplate(std::string _name, std::vector<size_t> l) : TensorVar<mode, Dtype>(_name) { value.Reshape(l); }
    TensorVarTemplate(std::string _name, std::vector<int> l)
        : TensorVarTemplate(_name, std::vector<size_t>(l.begin(), l.end())) {}
    TensorVarTemplate(std::string _name, std::vector<uint> l)
        : TensorVarTemplate(_name, std::vector<size_t>(l.begin(), l.end())) {}

    virtual void SetRef(void* p) override { value.ShallowCopy(*static_cast< DTensor<mode, Dtype>* >(p)); }
    virtual Dtype AsScalar() override { return value.AsScalar(); }
    virtual MatType GetMatType() override { return MatType::dense; }
    virtual void ZeroGrad() override
    {
        if (!(grad.shape == value.shape)) grad.Reshape(value.shape.dims);
        grad.FullZeros();
    }
    virtual void OnesGrad() override
    {
        grad.Reshape(value.shape.dims);
        grad.Full().Fill(1);
    }
    virtual bool GradBuffer(void** device_ptr, size_t* bytes) override { return detail::grad_buffer(value, grad, device_ptr, bytes); }
    void Serialize(FILE* fid) { value.Serialize(fid); }
    void Deserialize(FILE* fid) { value.Deserialize(fid); }

    DTensor<mode, Dtype> value;
    RowSpTensor<mode, Dtype> grad;
};

template<typename mode, typename Dtype>
class TensorVarTemplate<mode, CSR_SPARSE, Dtype> : public TensorVar<mode, Dtype>
{
public:
    TensorVarTemplate(std::string _name) : TensorVar<mode, Dtype>(_name) {}
    virtual void SetRef(void* p) override { value.ShallowCopy(*static_cast< SpTensor<mode, Dtype>* >(p)); }
    virtual Dtype AsScalar() override { return 0; }
    virtual MatType GetMatType() override { return MatType::sparse; }
    SpTensor<mode, Dtype> value;
};

}  // namespace gnn
#endif
