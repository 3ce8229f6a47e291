// Shared device/host helpers for the gfx950 kernels. Wave size is 64 everywhere.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define BM_WAVE 64
#define BM_BLOCK 256                 // 4 independent waves per workgroup
#define BM_WAVES_PER_BLOCK (BM_BLOCK / BM_WAVE)

#define BM_CHECK(expr)                                  \
    do {                                                \
        hipError_t _e = (expr);                         \
        if (_e != hipSuccess) return (int)_e;           \
    } while (0)

namespace bm {

// ---------------------------------------------------------------- vector access
template <int W> struct Vec;
template <> struct Vec<1> {
    float x;
    __device__ __forceinline__ static Vec<1> zero() { return {0.f}; }
    __device__ __forceinline__ static Vec<1> load(const float* p) { return {*p}; }
    __device__ __forceinline__ void store(float* p) const { *p = x; }
    __device__ __forceinline__ void fma(const Vec<1>& a, float v) { x = fmaf(a.x, v, x); }
    __device__ __forceinline__ void add(const Vec<1>& a) { x += a.x; }
    __device__ __forceinline__ float dot(const Vec<1>& b) const { return x * b.x; }
    __device__ __forceinline__ float dotacc(const Vec<1>& b, float s) const { return fmaf(x, b.x, s); }
};
template <> struct Vec<4> {
    float4 v;
    __device__ __forceinline__ static Vec<4> zero() { return {make_float4(0.f, 0.f, 0.f, 0.f)}; }
    __device__ __forceinline__ static Vec<4> load(const float* p) {
        return {*reinterpret_cast<const float4*>(p)};
    }
    __device__ __forceinline__ void store(float* p) const { *reinterpret_cast<float4*>(p) = v; }
    __device__ __forceinline__ void fma(const Vec<4>& a, float s) {
        v.x = fmaf(a.v.x, s, v.x); v.y = fmaf(a.v.y, s, v.y);
        v.z = fmaf(a.v.z, s, v.z); v.w = fmaf(a.v.w, s, v.w);
    }
    __device__ __forceinline__ void add(const Vec<4>& a) {
        v.x += a.v.x; v.y += a.v.y; v.z += a.v.z; v.w += a.v.w;
    }
    __device__ __forceinline__ float dotacc(const Vec<4>& b, float s) const {
        s = fmaf(v.x, b.v.x, s); s = fmaf(v.y, b.v.y, s);
        s = fmaf(v.z, b.v.z, s); s = fmaf(v.w, b.v.w, s);
        return s;
    }
};

// ---------------------------------------------------------------- cross-lane moves
// DPP moves inside a row of 16 lanes (no LDS traffic). ctrl must be a constant.
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float x) {
    int r = __builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, false);
    return __int_as_float(r);
}
constexpr int DPP_QUAD_XOR1 = 0xB1;       // quad_perm [1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;       // quad_perm [2,3,0,1]
constexpr int DPP_ROW_HALF_MIRROR = 0x141;
constexpr int DPP_ROW_MIRROR = 0x140;

// Sum over aligned groups of N consecutive lanes (N a power of two <= 64); every lane of a
// group ends up with the group's sum. Butterfly: DPP for the steps that stay inside a
// 16-lane row, ds_bpermute-based xor shuffles for the two cross-row steps.
template <int N>
__device__ __forceinline__ float group_allsum(float x) {
    if (N >= 2) x += dpp_mov<DPP_QUAD_XOR1>(x);
    if (N >= 4) x += dpp_mov<DPP_QUAD_XOR2>(x);
    if (N >= 8) x += dpp_mov<DPP_ROW_HALF_MIRROR>(x);
    if (N >= 16) x += dpp_mov<DPP_ROW_MIRROR>(x);
    if (N >= 32) x += __shfl_xor(x, 16, 64);
    if (N >= 64) x += __shfl_xor(x, 32, 64);
    return x;
}

// Sums U values per lane over aligned groups of N lanes at once (U in {2,4,8}, N >= 8, N >= U).
// The first log2(U) butterfly steps are "transposed": instead of every lane adding up all U
// values, partners split them, each keeping the half selected by one bit of its slot label, so
// the work halves per step; the remaining steps are a plain butterfly on the one value left.
// Afterwards lane l holds the complete group sum of slot slot_label(l). Every sum is formed by
// the same tree of additions as group_allsum<N>, so the bits are the same.
//
// The steps' partners are lane^1, lane^2, 7-lane (within 8), 15-lane (within 16), lane^16,
// lane^32. A label whose bit t flips exactly under step t and under no later step is
//   bit0 = l0 ^ l2, bit1 = l1 ^ l2, bit2 = l2 ^ l3          (l0..l3 = low bits of the lane).
__device__ __forceinline__ int slot_label(int l) {
    return ((l ^ (l >> 2)) & 1) | ((((l >> 1) ^ (l >> 2)) & 1) << 1) | ((((l >> 2) ^ (l >> 3)) & 1) << 2);
}
// Which of the U consecutive lanes it0 .. it0+U-1 (it0 a multiple of U) carries slot u.
template <int U>
__device__ __forceinline__ int slot_offset(int u, int it0) {
    if constexpr (U == 8) {
        const int b3 = (it0 >> 3) & 1;
        const int b2 = ((u >> 2) & 1) ^ b3, b0 = (u & 1) ^ b2, b1 = ((u >> 1) & 1) ^ b2;
        return b0 | (b1 << 1) | (b2 << 2);
    } else if constexpr (U == 4) {
        const int b2 = (it0 >> 2) & 1;
        return ((u & 1) ^ b2) | ((((u >> 1) & 1) ^ b2) << 1);
    } else if constexpr (U == 2) {
        return (u & 1) ^ ((it0 >> 2) & 1);
    } else {
        return 0;
    }
}
template <int N, int U>
__device__ __forceinline__ float group_multisum(const float (&s)[U], int label) {
    static_assert(U == 2 || U == 4 || U == 8, "U must be 2, 4 or 8");
    static_assert(N >= 8 && N >= U, "group too small");
    float a[U / 2];
    {
        const bool hi = label & 1;
#pragma unroll
        for (int i = 0; i < U / 2; ++i) {
            const float keep = hi ? s[2 * i + 1] : s[2 * i];
            const float send = hi ? s[2 * i] : s[2 * i + 1];
            a[i] = keep + dpp_mov<DPP_QUAD_XOR1>(send);
        }
    }
    float x;
    if constexpr (U >= 4) {
        float b[U / 4];
        const bool hi = label & 2;
#pragma unroll
        for (int i = 0; i < U / 4; ++i) {
            const float keep = hi ? a[2 * i + 1] : a[2 * i];
            const float send = hi ? a[2 * i] : a[2 * i + 1];
            b[i] = keep + dpp_mov<DPP_QUAD_XOR2>(send);
        }
        if constexpr (U == 8) {
            const bool hi2 = label & 4;
            const float keep = hi2 ? b[1] : b[0];
            const float send = hi2 ? b[0] : b[1];
            x = keep + dpp_mov<DPP_ROW_HALF_MIRROR>(send);
        } else {
            x = b[0];
            x += dpp_mov<DPP_ROW_HALF_MIRROR>(x);
        }
    } else {
        x = a[0];
        x += dpp_mov<DPP_QUAD_XOR2>(x);
        x += dpp_mov<DPP_ROW_HALF_MIRROR>(x);
    }
    if (N >= 16) x += dpp_mov<DPP_ROW_MIRROR>(x);
    if (N >= 32) x += __shfl_xor(x, 16, 64);
    if (N >= 64) x += __shfl_xor(x, 32, 64);
    return x;
}

// Read lane `src` (a wave-uniform or per-lane index) of x.
__device__ __forceinline__ int lane_read(int x, int src) { return __shfl(x, src, 64); }
__device__ __forceinline__ float lane_read(float x, int src) { return __shfl(x, src, 64); }

__device__ __forceinline__ int wave_uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }

// ---------------------------------------------------------------- shape dispatch
// A dense column of k floats is covered by groups of LPN lanes, each lane holding V vectors
// of W floats: element index of vector i on lane l is (i*LPN + l)*W.
struct Shape { int W, V, LPN; };

static inline int pow2ceil(int x) { int p = 1; while (p < x) p <<= 1; return p; }

// W = 4 needs k % 4 == 0 and 16-byte aligned base pointers; V is rounded up to 1,2,4,8,16.
static inline Shape pick_shape(int k, bool aligned16) {
    Shape s;
    s.W = (aligned16 && (k % 4 == 0)) ? 4 : 1;
    int nv = (k + s.W - 1) / s.W;          // vectors per column
    s.LPN = pow2ceil(nv) < 64 ? pow2ceil(nv) : 64;
    int v = (nv + s.LPN - 1) / s.LPN;
    s.V = pow2ceil(v);
    return s;
}

}  // namespace bm
