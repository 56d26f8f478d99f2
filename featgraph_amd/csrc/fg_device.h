// Device-side helpers shared by the kernels (included by .hip files only).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace fg {

// Four consecutive words that are only known to be 4-byte aligned: read with one 128-bit load.
template <typename T> struct __attribute__((packed, aligned(4))) Words4 { T v[4]; };

// o[i] = p[min(4 * lane + i, n - 1) * stride], n >= 1: the lane's four consecutive elements of a
// stream of n, lanes past the end repeating the last element so that no load is conditional.
// With unit stride and n >= 4 (both uniform) that is one 128-bit load per lane from a window that
// is shifted back to end at the last element.
template <typename T>
__device__ __forceinline__ void load_four(const T *p, int n, int lane, int stride, T (&o)[4]) {
    if (stride == 1 && n >= 4) {
        const int s = min(4 * lane, n - 4), d = 4 * lane - s;
        const Words4<T> c = *reinterpret_cast<const Words4<T> *>(p + s);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = min(d + i, 3);
            o[i] = k == 0 ? c.v[0] : k == 1 ? c.v[1] : k == 2 ? c.v[2] : c.v[3];
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = p[(int64_t)min(4 * lane + i, n - 1) * stride];
    }
}

}  // namespace fg
