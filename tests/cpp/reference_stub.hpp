// The few declarations of danielmriley/vesper that the code blocks of the integration guide refer to, as a stand-in so that
// tests/test_integration_snippets.py can compile those blocks against include/vsp_attn.h without the reference tree.
// Shapes of the declarations follow include/vesper/core/{tensor,dtype,device,stream}.h and include/vesper/nn/transformer.h;
// nothing here is executed.
#pragma once
#include <cmath>
#include <cstdint>
#include <stdexcept>
#include <utility>
#include <vector>

#include "vsp_attn.h"

namespace vesper {
enum class DType { Float32, BFloat16, Int8 };
enum class Device { CPU, HIP };
class Tensor {
public:
    const std::vector<int64_t>& shape() const;
    const std::vector<int64_t>& strides() const;
    int64_t ndim() const;
    DType dtype() const;
    template <typename T>
    T* data_ptr() const;
};
Tensor empty(const std::vector<int64_t>& shape, DType dtype, Device device);
class Stream {
public:
    static Stream current(Device d);
    void* raw_handle() const;
};
namespace nn {
class KVCache {
public:
    std::pair<Tensor, Tensor> update(const Tensor& new_k, const Tensor& new_v, int start_pos);
    void reset();

private:
    std::pair<Tensor, Tensor> views();
    void* stream();
    vsp_kv_cache desc_;
    int current_len_ = 0;
};
}  // namespace nn
}  // namespace vesper
