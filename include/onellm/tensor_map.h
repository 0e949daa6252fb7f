// String-keyed bundle of Tensor views, the argument type of the oneLLM layer forward() methods
// (src/utils/tensor.h:160-296).  Same spelling of the members the layers and example drivers use:
// brace construction from {name, Tensor} pairs, operator[], at(), isExist(), insert(), getPtr<T>(key),
// getVal<T>(key), keys(), size().  Tensors without data or shape are dropped on construction, as in
// the reference (src/utils/tensor.h:165-175).
#pragma once
#include <initializer_list>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>
#include "onellm/tensor.h"

struct TensorMap {
    std::unordered_map<std::string, Tensor> tensor_map_;

    TensorMap() = default;
    TensorMap(std::initializer_list<std::pair<std::string, Tensor>> entries)
    {
        for (const auto& e : entries)
            if (isValid(e.second)) tensor_map_[e.first] = e.second;
    }
    explicit TensorMap(const std::unordered_map<std::string, Tensor>& entries)
    {
        for (const auto& e : entries)
            if (isValid(e.second)) tensor_map_[e.first] = e.second;
    }

    size_t size() const { return tensor_map_.size(); }
    bool isExist(const std::string& key) const { return tensor_map_.count(key) != 0; }
    bool isValid(const Tensor& t) const { return t.data != nullptr && t.size() > 0; }

    void insert(const std::string& key, const Tensor& value) { tensor_map_[key] = value; }
    void insert(std::pair<std::string, Tensor> p) { tensor_map_.insert(std::move(p)); }

    Tensor& at(const std::string& key)
    {
        auto it = tensor_map_.find(key);
        ONELLM_CHECK_WITH_INFO(it != tensor_map_.end(), "Cannot find a tensor of name " + key + " in the tensor map (keys: " + joined_keys() + ")");
        return it->second;
    }
    Tensor& operator[](const std::string& key) { return at(key); }

    template<typename T> T getVal(const std::string& key) const { return tensor_map_.at(key).getVal<T>(); }
    template<typename T> T getValByOffset(const std::string& key, int index) const { return tensor_map_.at(key).getVal<T>(index); }
    template<typename T> T* getPtr(const std::string& key) const { return tensor_map_.at(key).getPtr<T>(); }
    template<typename T> T* getPtrWithOffset(const std::string& key, int index) const { return tensor_map_.at(key).getPtrByOffset<T>(index); }

    std::vector<std::string> keys() const
    {
        std::vector<std::string> names;
        names.reserve(tensor_map_.size());
        for (const auto& e : tensor_map_) names.push_back(e.first);
        return names;
    }
    std::string toString()
    {
        std::string s = "{";
        bool first = true;
        for (const auto& e : tensor_map_) {
            s += (first ? "" : ", ") + e.first + ": " + e.second.toString();
            first = false;
        }
        return s + "}";
    }

private:
    std::string joined_keys() const
    {
        std::string s;
        for (const auto& e : tensor_map_) s += (s.empty() ? "" : ", ") + e.first;
        return s;
    }
};
