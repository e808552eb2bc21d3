// dz = delta .* act'(y, pre) for VEC consecutive elements, and the matching store: shared by the streaming
// pullback kernels of bias_activation and by the passes that write dz in a second layout as well.
#pragma once

#include "common.h"

namespace luxhip {

template <typename T, int ACT, int VEC>
__device__ __forceinline__ void dx_vec(const T* delta, const T* out, const T* pre, size_t off, float (&dx)[VEC]) {
    float d[VEC], o[VEC], p[VEC];
    if constexpr (VEC == 1) {
        d[0] = ld(delta + off);
        if constexpr (ACT != LUXHIP_ACT_IDENTITY && !Act<ACT>::needs_pre) o[0] = ld(out + off);
        if constexpr (Act<ACT>::needs_pre) p[0] = ld(pre + off);
    } else {
        Vec<T>::load(delta + off, d);
        if constexpr (ACT != LUXHIP_ACT_IDENTITY && !Act<ACT>::needs_pre) Vec<T>::load(out + off, o);
        if constexpr (Act<ACT>::needs_pre) Vec<T>::load(pre + off, p);
    }
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
        if constexpr (ACT == LUXHIP_ACT_IDENTITY) dx[k] = d[k];
        else if constexpr (Act<ACT>::needs_pre) dx[k] = d[k] * Act<ACT>::d(Act<ACT>::f(p[k]), p[k]);
        else dx[k] = d[k] * Act<ACT>::d(o[k], 0.0f);
    }
}

template <typename T, int VEC>
__device__ __forceinline__ void store_vec(T* p, size_t off, const float (&v)[VEC]) {
    if constexpr (VEC == 1) st(p + off, v[0]);
    else Vec<T>::store(p + off, v);
}

}  // namespace luxhip
