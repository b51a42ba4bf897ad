// Parameter updates on the device (include/nn/optimizer.h, src/nn/optimizer.cpp:16-92):
// plain SGD, momentum SGD and Adam over the full (dense) gradients of a ParamSet.
#ifndef OPTIMIZER_H
#define OPTIMIZER_H

#include <cmath>
#include <map>
#include <memory>
#include <string>
#include <vector>
#include "nn/param_set.h"

namespace gnn
{

template<typename mode, typename Dtype>
class IOptimizer
{
public:
    IOptimizer(ParamSet<mode, Dtype>* _param_set, Dtype _init_lr, Dtype _l2_penalty = 0)
        : param_set(_param_set), init_lr(_init_lr), l2_penalty(_l2_penalty), cur_lr(_init_lr),
          clip_threshold(5), clipping_enabled(true), cur_iter(0) {}
    virtual ~IOptimizer() {}
    virtual void Update() = 0;

    // factor that brings the global gradient norm down to clip_threshold (1 when it already is)
    Dtype ClipGradients()
    {
        if (!clipping_enabled) return 1.0;
        Dtype sq = 0;
        for (auto& kv : param_set->params) {
            const Dtype n2 = kv.second->grad.Norm2();
            sq += n2 * n2;
        }
        const Dtype norm = std::sqrt(sq);
        return norm > clip_threshold ? clip_threshold / norm : (Dtype)1.0;
    }

    ParamSet<mode, Dtype>* param_set;
    Dtype init_lr;
    Dtype l2_penalty;
    Dtype cur_lr;
    Dtype clip_threshold;
    bool clipping_enabled;
    int cur_iter;
};

template<typename mode, typename Dtype>
class SGDOptimizer : public IOptimizer<mode, Dtype>
{
public:
    SGDOptimizer(ParamSet<mode, Dtype>* m, Dtype _init_lr, Dtype _l2_penalty = 0) : IOptimizer<mode, Dtype>(m, _init_lr, _l2_penalty) {}
    // w <- (1 - lr * l2) w - lr * g
    virtual void Update() override
    {
        for (auto& kv : this->param_set->params) {
            auto& p = kv.second;
            auto g = p->grad.Full();
            p->value.Axpby(-this->cur_lr, g, 1 - this->cur_lr * this->l2_penalty);
            p->grad.RowSpZeros();
        }
    }
};

namespace detail
{
// Every tensor of the parameter set updated by one launch (device, full gradients); false where that route
// does not apply and the caller updates tensor by tensor.
template<typename mode, typename Dtype>
struct BatchedMomentumUpdate
{
    static bool Run(ParamSet<mode, Dtype>*, std::map<std::string, std::shared_ptr< DTensor<mode, Dtype> > >&, Dtype, Dtype, Dtype) { return false; }
};
template<>
struct BatchedMomentumUpdate<GPU, float>
{
    static bool Run(ParamSet<GPU, float>* set, std::map<std::string, std::shared_ptr< DTensor<GPU, float> > >& velocity,
                    float lr, float momentum, float l2)
    {
        std::vector<float*> w, g, v;
        std::vector<size_t> count;
        for (auto& kv : set->params) {
            auto& p = kv.second;
            if (!p->grad.is_full || !(p->grad.shape == p->value.shape)) return false;
            if (momentum > 0) {
                auto& vel = velocity[kv.first];
                if (!vel) {
                    vel = std::make_shared< DTensor<GPU, float> >(p->grad.shape);
                    vel->Zeros();
                }
                v.push_back(vel->data->ptr);
            }
            w.push_back(p->value.data->ptr);
            g.push_back(p->grad.data->ptr);
            count.push_back(p->value.shape.Count());
        }
        GNN_HIP(gnnhip_momentum_sgd_batch_f32((int)w.size(), w.data(), g.data(), momentum > 0 ? v.data() : nullptr, count.data(),
                                              lr, momentum, l2, GpuHandle::Stream()));
        return true;
    }
};
}  // namespace detail

template<typename mode, typename Dtype>
class MomentumSGDOptimizer : public IOptimizer<mode, Dtype>
{
public:
    MomentumSGDOptimizer(ParamSet<mode, Dtype>* m, Dtype _init_lr, Dtype _momentum = 0.9, Dtype _l2_penalty = 0)
        : IOptimizer<mode, Dtype>(m, _init_lr, _l2_penalty), momentum(_momentum) {}

    // g <- g + l2 * w ;  v <- momentum * v + lr * g ;  w <- w - v     (plain SGD when momentum == 0)
    virtual void Update() override
    {
        if (detail::BatchedMomentumUpdate<mode, Dtype>::Run(this->param_set, acc_grad_dict, this->cur_lr, momentum, this->l2_penalty)) return;
        for (auto& kv : this->param_set->params) {
            auto& p = kv.second;
            auto g = p->grad.Full();
            if (momentum > 0) {
                auto& v = acc_grad_dict[kv.first];
                if (!v) {
                    v = std::make_shared< DTensor<mode, Dtype> >(p->grad.shape);
                    v->Zeros();
                }
                g.Axpy(this->l2_penalty, p->value);
                v->Axpby(this->cur_lr, g, momentum);
                p->value.Axpy(-1.0, *v);
            } else {
                p->value.Axpby(-this->cur_lr, g, 1 - this->cur_lr * this->l2_penalty);
            }
            p->grad.RowSpZeros();
        }
    }

    Dtype momentum;
    std::map<std::string, std::shared_ptr< DTensor<mode, Dtype> > > acc_grad_dict;
};

namespace detail
{
// AdamOptimizer::Update of every tensor by two launches (norm of all gradients, update); false where that route does
// not apply.
template<typename mode, typename Dtype>
struct BatchedAdamUpdate
{
    typedef std::map<std::string, std::shared_ptr< DTensor<mode, Dtype> > > Moments;
    static bool Run(ParamSet<mode, Dtype>*, Moments&, Moments&, Dtype, Dtype, Dtype, Dtype, Dtype, Dtype, int) { return false; }
};
template<>
struct BatchedAdamUpdate<GPU, float>
{
    typedef std::map<std::string, std::shared_ptr< DTensor<GPU, float> > > Moments;
    static bool Run(ParamSet<GPU, float>* set, Moments& first, Moments& second, float lr, float l2, float clip,
                    float beta_1, float beta_2, float eps, int iter)
    {
        std::vector<float*> w, g, m, v;
        std::vector<size_t> count;
        for (auto& kv : set->params) {
            auto& p = kv.second;
            if (!p->grad.is_full || !(p->grad.shape == p->value.shape)) return false;
        }
        for (auto& kv : set->params) {
            auto& p = kv.second;
            for (Moments* mom : {&first, &second}) {
                auto& t = (*mom)[kv.first];
                if (!t) {
                    t = std::make_shared< DTensor<GPU, float> >(p->grad.shape);
                    t->Zeros();
                }
            }
            w.push_back(p->value.data->ptr);
            g.push_back(p->grad.data->ptr);
            m.push_back(first[kv.first]->data->ptr);
            v.push_back(second[kv.first]->data->ptr);
            count.push_back(p->value.shape.Count());
        }
        // 1 / (1 - beta^t), as the reference forms them
        const float s1 = (float)(1.0 / (1 - std::pow(beta_1, iter)));
        const float s2 = (float)(1.0 / (1 - std::pow(beta_2, iter)));
        GNN_HIP(gnnhip_adam_batch_f32((int)w.size(), w.data(), g.data(), m.data(), v.data(), count.data(), lr, l2, clip,
                                      beta_1, beta_2, eps, s1, s2, GpuHandle::Stream()));
        return true;
    }
};
}  // namespace detail

// Adam with the reference's weight decay and gradient clipping (include/nn/optimizer.h:128-150,
// src/nn/optimizer.cpp:97-160): g <- l2 w + clip factor * g; m, v the two running moments; the step
// lr / (1 - beta_1^t) * m / (sqrt(v / (1 - beta_2^t)) + eps).  Device tensors with full gradients only.
template<typename mode, typename Dtype>
class AdamOptimizer : public IOptimizer<mode, Dtype>
{
public:
    AdamOptimizer(ParamSet<mode, Dtype>* m, Dtype _init_lr, Dtype _l2_penalty = 0, Dtype _beta_1 = 0.9, Dtype _beta_2 = 0.999,
                  Dtype _eps = 1e-8)
        : IOptimizer<mode, Dtype>(m, _init_lr, _l2_penalty), beta_1(_beta_1), beta_2(_beta_2), eps(_eps) {}

    virtual void Update() override
    {
        this->cur_iter++;
        const Dtype clip = this->clipping_enabled ? this->clip_threshold : (Dtype)0;
        const bool done = detail::BatchedAdamUpdate<mode, Dtype>::Run(this->param_set, first_moments, second_moments, this->cur_lr,
                                                                      this->l2_penalty, clip, beta_1, beta_2, eps, this->cur_iter);
        ASSERT(done, "AdamOptimizer: device tensors with full gradients only");
    }

    std::map<std::string, std::shared_ptr< DTensor<mode, Dtype> > > first_moments, second_moments;
    Dtype beta_1, beta_2, eps;
};

}  // namespace gnn
#endif
