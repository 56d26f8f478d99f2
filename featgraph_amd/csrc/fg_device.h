// Device-side helpers shared by the kernels (included by .hip files only).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace fg {

// Four consecutive elements that are only known to be aligned like one of them (4 bytes for 32-bit words, 2 for
// 16-bit ones): read with one 128-bit or 64-bit load.
template <typename T> struct __attribute__((packed, aligned(sizeof(T) < 4 ? sizeof(T) : 4))) Words4 { T v[4]; };

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

// The lane's four column ids of a stream of n (as load_four): from the 16-bit copy `ids16` when there is one
// (uniform over the wavefront), else from `ids`.
__device__ __forceinline__ void load_four_ids(const int32_t *ids, const uint16_t *ids16, int64_t base, int n, int lane,
                                              int32_t (&c)[4]) {
    if (ids16) {
        uint16_t c16[4];
        load_four(ids16 + base, n, lane, 1, c16);
#pragma unroll
        for (int i = 0; i < 4; ++i) c[i] = c16[i];
    } else {
        load_four(ids + base, n, lane, 1, c);
    }
}

// Orders this wavefront's LDS writes before its later LDS reads (and the reverse); for staging buffers
// that are private to one wavefront, so no workgroup barrier is involved.
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// v from another lane of the same 16-lane row, chosen by a DPP control word (no LDS traffic).
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}

// Sum over the L (4, 8 or 16) consecutive lanes of a lane group; every lane of the group gets it.
template <int L>
__device__ __forceinline__ float group_sum(float v) {
    static_assert(L == 4 || L == 8 || L == 16, "lane groups inside one 16-lane row");
    v += dpp_move<0xB1>(v);                  // quad_perm [1,0,3,2]
    v += dpp_move<0x4E>(v);                  // quad_perm [2,3,0,1]
    if (L >= 8) v += dpp_move<0x141>(v);     // row_half_mirror
    if (L >= 16) v += dpp_move<0x140>(v);    // row_mirror
    return v;
}

}  // namespace fg
