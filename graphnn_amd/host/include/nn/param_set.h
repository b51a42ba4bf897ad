// Named collection of trainable tensors with graphnn's checkpoint format
// (include/nn/param_set.h, src/nn/param_set.cpp:29-54): parameters in name order, each as
// rank, dims, element count (size_t each) and the raw elements; no header or version.
#ifndef PARAM_SET_H
#define PARAM_SET_H

#include <map>
#include <string>
#include "nn/variable.h"

namespace gnn
{

template<typename mode, typename Dtype>
class ParamSet
{
public:
    typedef std::shared_ptr< DTensorVar<mode, Dtype> > ParamPtr;
    ParamSet() {}

    void AddParam(ParamPtr param)
    {
        ASSERT(params.count(param->name) == 0, "param " + param->name + " already created");
        params[param->name] = param;
    }
    void AddNondiff(ParamPtr param)
    {
        ASSERT(nondiff_params.count(param->name) == 0, "nondiff param " + param->name + " already created");
        nondiff_params[param->name] = param;
    }
    void Save(std::string filename)
    {
        FILE* fid = fopen(filename.c_str(), "wb");
        ASSERT(fid, "file " + filename + " cannot be opened for writing");
        for (auto& kv : params) kv.second->Serialize(fid);
        for (auto& kv : nondiff_params) kv.second->Serialize(fid);
        fclose(fid);
    }
    void Load(std::string filename)
    {
        FILE* fid = fopen(filename.c_str(), "rb");
        ASSERT(fid, "file " + filename + " is not found");
        for (auto& kv : params) kv.second->Deserialize(fid);
        for (auto& kv : nondiff_params) kv.second->Deserialize(fid);
        fclose(fid);
    }
    void DeepCopyFrom(ParamSet<mode, Dtype>& src)
    {
        for (auto& kv : src.params) {
            if (!params.count(kv.first)) params[kv.first] = std::make_shared< DTensorVar<mode, Dtype> >(kv.first);
            params[kv.first]->value.CopyFrom(kv.second->value);
        }
        for (auto& kv : src.nondiff_params) {
            if (!nondiff_params.count(kv.first)) nondiff_params[kv.first] = std::make_shared< DTensorVar<mode, Dtype> >(kv.first);
            nondiff_params[kv.first]->value.CopyFrom(kv.second->value);
        }
    }

    std::map<std::string, ParamPtr> params;
    std::map<std::string, ParamPtr> nondiff_params;
};

template<template <typename, typename> class ParamType, typename mode, typename Dtype, typename... Args>
std::shared_ptr< ParamType<mode, Dtype> > add_diff(ParamSet<mode, Dtype>& pset, std::string param_name, Args&&... args)
{
    auto p = std::make_shared< ParamType<mode, Dtype> >(param_name, std::forward<Args>(args)...);
    pset.AddParam(p);
    return p;
}

// shape given as a braced list: add_diff<DTensorVar>(model, "w", {rows, cols})
template<template <typename, typename> class ParamType, typename mode, typename Dtype, typename IdxType, typename... Args>
std::shared_ptr< ParamType<mode, Dtype> > add_diff(ParamSet<mode, Dtype>& pset, std::string param_name,
                                                  std::initializer_list<IdxType> l, Args&&... args)
{
    auto p = std::make_shared< ParamType<mode, Dtype> >(param_name, std::vector<IdxType>(l), std::forward<Args>(args)...);
    pset.AddParam(p);
    return p;
}

template<template <typename, typename> class ParamType, typename mode, typename Dtype, typename... Args>
std::shared_ptr< ParamType<mode, Dtype> > add_nondiff(ParamSet<mode, Dtype>& pset, std::string param_name, Args&&... args)
{
    auto p = std::make_shared< ParamType<mode, Dtype> >(param_name, std::forward<Args>(args)...);
    pset.AddNondiff(p);
    return p;
}

template<template <typename, typename> class ParamType, typename mode, typename Dtype, typename IdxType, typename... Args>
std::shared_ptr< ParamType<mode, Dtype> > add_nondiff(ParamSet<mode, Dtype>& pset, std::string param_name,
                                                     std::initializer_list<IdxType> l, Args&&... args)
{
    auto p = std::make_shared< ParamType<mode, Dtype> >(param_name, std::vector<IdxType>(l), std::forward<Args>(args)...);
    pset.AddNondiff(p);
    return p;
}

}  // namespace gnn
#endif
