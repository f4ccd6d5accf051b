// Device-side helpers shared by the SDDMM kernels (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sddmm {

constexpr int WAVE = 64;
constexpr int NUM_XCD = 8;  // MI355X: 8 accelerator complex dies, one L2 each

// ---- cross-lane -----------------------------------------------------------
// DPP control words (gfx9 encoding)
constexpr int DPP_QUAD_XOR1 = 0xB1;        // quad_perm:[1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;        // quad_perm:[2,3,0,1]
constexpr int DPP_ROW_HALF_MIRROR = 0x141; // lane i <-> 7-i inside each 8
constexpr int DPP_ROW_MIRROR = 0x140;      // lane i <-> 15-i inside each 16

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    // old = 0 with bound_ctrl lets the compiler fold the move into the consuming
    // VALU instruction (v_add_f32_dpp); every pattern used here reads a valid lane
    int i = __builtin_bit_cast(int, v);
    i = __builtin_amdgcn_update_dpp(0, i, CTRL, 0xF, 0xF, true);
    return __builtin_bit_cast(float, i);
}

// Sum over aligned groups of LPN lanes; every lane of the group ends with the
// total.  The addition tree is fixed (1,2,4,8,16,32), so the value does not
// depend on which kernel calls it.
template <int LPN>
__device__ __forceinline__ float group_sum(float v) {
    if constexpr (LPN >= 2) v += dpp_f32<DPP_QUAD_XOR1>(v);
    if constexpr (LPN >= 4) v += dpp_f32<DPP_QUAD_XOR2>(v);
    if constexpr (LPN >= 8) v += dpp_f32<DPP_ROW_HALF_MIRROR>(v);
    if constexpr (LPN >= 16) v += dpp_f32<DPP_ROW_MIRROR>(v);
    if constexpr (LPN >= 32) {
        // swap the two 16-lane halves of each 32: ds_swizzle bit mode, xor 0x10
        int i = __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F);
        v += __builtin_bit_cast(float, i);
    }
    if constexpr (LPN >= 64) v += __shfl_xor(v, 32, WAVE);
    return v;
}

__device__ __forceinline__ int lane_id() { return threadIdx.x & (WAVE - 1); }
// index of the wavefront inside its workgroup, as a scalar
__device__ __forceinline__ int wave_in_block() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }

// LDS that only one wavefront touches: its LDS operations execute in program order, so a
// write followed by a read of another lane's slot needs no workgroup barrier, only that the
// compiler keeps the order.
__device__ __forceinline__ void wave_lds_order() {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// Workgroups are handed to the 8 XCDs round-robin by id.  Give every XCD one
// contiguous eighth of the logical work so that neighbouring row panels (which
// touch neighbouring B rows) share an L2.  Returns the logical index, or -1 for
// the padding blocks of the rounded-up grid.
__device__ __forceinline__ int64_t xcd_remap(int64_t bid, int64_t nblocks) {
    int64_t per = (nblocks + NUM_XCD - 1) / NUM_XCD;
    int64_t logical = (bid % NUM_XCD) * per + bid / NUM_XCD;
    return logical < nblocks ? logical : -1;
}
inline int64_t xcd_grid(int64_t nblocks) {
    return ((nblocks + NUM_XCD - 1) / NUM_XCD) * NUM_XCD;
}

// Streamed operands (column indices, S values, row indices, P) are touched once
// per run.  Marking them non-temporal (SDDMM_NT=1) was measured SLOWER on MI355X
// (FEM-banded K=32: 119 us vs 86 us; power-law unchanged): repeated runs find the
// index arrays in the last-level cache, and the hint gives that up.  Off by default.
#ifndef SDDMM_NT
#define SDDMM_NT 0
#endif
template <class T>
__device__ __forceinline__ T ld_stream(const T *p) {
#if SDDMM_NT
    return __builtin_nontemporal_load(p);
#else
    return *p;
#endif
}
template <class T>
__device__ __forceinline__ void st_stream(T *p, T v) {
#if SDDMM_NT
    __builtin_nontemporal_store(v, p);
#else
    *p = v;
#endif
}

// One work item of the wave-per-segment kernel: entries [start,end) of one row.
struct RowItem {
    int32_t row;
    int32_t start;
    int32_t end;
    int32_t pad;
};

// ---- units of the K dimension ----------------------------------------------
// A "unit" is what one lane loads per step along K: 16 bytes where alignment
// allows (4 fp32, 8 bf16 or 8 fp16), one fp32 otherwise.  dot() extends an fp32
// accumulator with fused multiply-adds in element order.
// element types of A and B as template arguments of the kernels
constexpr int DT_F32 = 0, DT_BF16 = 1, DT_F16 = 2;

struct UnitF32x4 {
    static constexpr int DT = DT_F32;
    using T = float4;
    static constexpr int ELEMS = 4;
    static __device__ __forceinline__ T zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
    static __device__ __forceinline__ float dot(const T &a, const T &b, float acc) {
        acc = __builtin_fmaf(a.x, b.x, acc);
        acc = __builtin_fmaf(a.y, b.y, acc);
        acc = __builtin_fmaf(a.z, b.z, acc);
        acc = __builtin_fmaf(a.w, b.w, acc);
        return acc;
    }
    // acc[e] += p * (element e of b)
    static __device__ __forceinline__ void axpy(float p, const T &b, float (&acc)[ELEMS]) {
        acc[0] = __builtin_fmaf(p, b.x, acc[0]);
        acc[1] = __builtin_fmaf(p, b.y, acc[1]);
        acc[2] = __builtin_fmaf(p, b.z, acc[2]);
        acc[3] = __builtin_fmaf(p, b.w, acc[3]);
    }
};
struct UnitF32x1 {
    static constexpr int DT = DT_F32;
    using T = float;
    static constexpr int ELEMS = 1;
    static __device__ __forceinline__ T zero() { return 0.f; }
    static __device__ __forceinline__ float dot(const T &a, const T &b, float acc) {
        return __builtin_fmaf(a, b, acc);
    }
};
struct UnitBF16x8 {
    static constexpr int DT = DT_BF16;
    using T = uint4;  // 8 bfloat16, two per 32-bit word, low half first
    static constexpr int ELEMS = 8;
    static __device__ __forceinline__ T zero() { return make_uint4(0u, 0u, 0u, 0u); }
    static __device__ __forceinline__ float lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
    static __device__ __forceinline__ float hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xFFFF0000u); }
    static __device__ __forceinline__ float dot(const T &a, const T &b, float acc) {
        acc = __builtin_fmaf(lo(a.x), lo(b.x), acc);
        acc = __builtin_fmaf(hi(a.x), hi(b.x), acc);
        acc = __builtin_fmaf(lo(a.y), lo(b.y), acc);
        acc = __builtin_fmaf(hi(a.y), hi(b.y), acc);
        acc = __builtin_fmaf(lo(a.z), lo(b.z), acc);
        acc = __builtin_fmaf(hi(a.z), hi(b.z), acc);
        acc = __builtin_fmaf(lo(a.w), lo(b.w), acc);
        acc = __builtin_fmaf(hi(a.w), hi(b.w), acc);
        return acc;
    }
    static __device__ __forceinline__ void axpy(float p, const T &b, float (&acc)[ELEMS]) {
        acc[0] = __builtin_fmaf(p, lo(b.x), acc[0]); acc[1] = __builtin_fmaf(p, hi(b.x), acc[1]);
        acc[2] = __builtin_fmaf(p, lo(b.y), acc[2]); acc[3] = __builtin_fmaf(p, hi(b.y), acc[3]);
        acc[4] = __builtin_fmaf(p, lo(b.z), acc[4]); acc[5] = __builtin_fmaf(p, hi(b.z), acc[5]);
        acc[6] = __builtin_fmaf(p, lo(b.w), acc[6]); acc[7] = __builtin_fmaf(p, hi(b.w), acc[7]);
    }
};

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
struct UnitF16x8 {
    static constexpr int DT = DT_F16;
    using T = uint4;  // 8 IEEE half floats, two per 32-bit word, low half first
    static constexpr int ELEMS = 8;
    static __device__ __forceinline__ T zero() { return make_uint4(0u, 0u, 0u, 0u); }
    // v_dot2c_f32_f16: acc + a.lo*b.lo + a.hi*b.hi with fp32 accumulation (products of
    // halves are exact in fp32)
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, a), __builtin_bit_cast(half2_t, b), acc, false);
    }
    static __device__ __forceinline__ float dot(const T &a, const T &b, float acc) {
        acc = dot2(a.x, b.x, acc);
        acc = dot2(a.y, b.y, acc);
        acc = dot2(a.z, b.z, acc);
        acc = dot2(a.w, b.w, acc);
        return acc;
    }
    static __device__ __forceinline__ float lo(uint32_t w) {
        const half2_t h = __builtin_bit_cast(half2_t, w);
        const _Float16 e = h[0];
        return (float)e;
    }
    static __device__ __forceinline__ float hi(uint32_t w) {
        const half2_t h = __builtin_bit_cast(half2_t, w);
        const _Float16 e = h[1];
        return (float)e;
    }
    static __device__ __forceinline__ void axpy(float p, const T &b, float (&acc)[ELEMS]) {
        acc[0] = __builtin_fmaf(p, lo(b.x), acc[0]); acc[1] = __builtin_fmaf(p, hi(b.x), acc[1]);
        acc[2] = __builtin_fmaf(p, lo(b.y), acc[2]); acc[3] = __builtin_fmaf(p, hi(b.y), acc[3]);
        acc[4] = __builtin_fmaf(p, lo(b.z), acc[4]); acc[5] = __builtin_fmaf(p, hi(b.z), acc[5]);
        acc[6] = __builtin_fmaf(p, lo(b.w), acc[6]); acc[7] = __builtin_fmaf(p, hi(b.w), acc[7]);
    }
};

}  // namespace sddmm
