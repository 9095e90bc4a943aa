// Shared device helpers for the gfx950 kernels: wave64 shuffles, vector loads
// of fp32 / bf16 feature rows, launch and error plumbing for the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdio>
#include <cstring>

namespace yitu {

constexpr int kWave = 64;
constexpr int kBlock = 256;  // 4 waves per workgroup for every row kernel
constexpr int kWavesPerBlock = kBlock / kWave;

// ---- error plumbing -------------------------------------------------------
// Entry points return 0 on success, a negative value for rejected arguments
// and a positive hipError_t for runtime failures; the message is kept per
// thread and read back through yitu_last_error().
void set_error(const char *fmt, ...);

#define YITU_REQUIRE(cond, ...)            \
    do {                                   \
        if (!(cond)) {                     \
            ::yitu::set_error(__VA_ARGS__); \
            return -1;                     \
        }                                  \
    } while (0)

#define YITU_HIP(call)                                                              \
    do {                                                                            \
        hipError_t e_ = (call);                                                     \
        if (e_ != hipSuccess) {                                                     \
            ::yitu::set_error("%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), \
                              __FILE__, __LINE__);                                  \
            return (int)e_;                                                         \
        }                                                                           \
    } while (0)

#define YITU_LAUNCH_CHECK() YITU_HIP(hipGetLastError())

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// ---- bf16 -----------------------------------------------------------------
struct bf16_t {
    uint16_t bits;
};

__device__ __forceinline__ float bf16_lo(uint32_t packed) { return __uint_as_float(packed << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t packed) {
    return __uint_as_float(packed & 0xffff0000u);
}

// Lane exchanges of the gfx950 vector ALU (no trip through the LDS unit). For two
// registers a, b: pair_sum32 leaves a[l] + a[l + 32] in the lower half of the wave and
// b[l - 32] + b[l] in the upper half; pair_sum16 leaves, in the four quarters of the
// wave, a(q0) + a(q1), b(q0) + b(q1), a(q2) + a(q3), b(q2) + b(q3). One exchange and
// one add thus fold two values at once, each half (quarter pair) keeping one of them.
__device__ __forceinline__ float pair_sum32(float a, float b) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false,
                                                    false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float pair_sum16(float a, float b) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false,
                                                    false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// ---- vector loads: VEC consecutive elements of a feature row -> fp32 -------
template <int VEC, typename T>
struct RowLoad;

template <>
struct RowLoad<1, float> {
    static __device__ __forceinline__ void ld(const float *p, float (&v)[1]) { v[0] = *p; }
};
template <>
struct RowLoad<2, float> {
    static __device__ __forceinline__ void ld(const float *p, float (&v)[2]) {
        float2 t = *reinterpret_cast<const float2 *>(p);
        v[0] = t.x;
        v[1] = t.y;
    }
};
template <>
struct RowLoad<4, float> {
    static __device__ __forceinline__ void ld(const float *p, float (&v)[4]) {
        float4 t = *reinterpret_cast<const float4 *>(p);
        v[0] = t.x;
        v[1] = t.y;
        v[2] = t.z;
        v[3] = t.w;
    }
};
template <>
struct RowLoad<1, bf16_t> {
    static __device__ __forceinline__ void ld(const bf16_t *p, float (&v)[1]) {
        v[0] = __uint_as_float(static_cast<uint32_t>(p->bits) << 16);
    }
};
template <>
struct RowLoad<2, bf16_t> {
    static __device__ __forceinline__ void ld(const bf16_t *p, float (&v)[2]) {
        uint32_t t = *reinterpret_cast<const uint32_t *>(p);
        v[0] = bf16_lo(t);
        v[1] = bf16_hi(t);
    }
};
template <>
struct RowLoad<4, bf16_t> {
    static __device__ __forceinline__ void ld(const bf16_t *p, float (&v)[4]) {
        uint2 t = *reinterpret_cast<const uint2 *>(p);
        v[0] = bf16_lo(t.x);
        v[1] = bf16_hi(t.x);
        v[2] = bf16_lo(t.y);
        v[3] = bf16_hi(t.y);
    }
};
template <>
struct RowLoad<8, bf16_t> {
    static __device__ __forceinline__ void ld(const bf16_t *p, float (&v)[8]) {
        uint4 t = *reinterpret_cast<const uint4 *>(p);
        v[0] = bf16_lo(t.x);
        v[1] = bf16_hi(t.x);
        v[2] = bf16_lo(t.y);
        v[3] = bf16_hi(t.y);
        v[4] = bf16_lo(t.z);
        v[5] = bf16_hi(t.z);
        v[6] = bf16_lo(t.w);
        v[7] = bf16_hi(t.w);
    }
};

template <int VEC>
__device__ __forceinline__ void store_row(float *p, const float (&v)[VEC]) {
    if constexpr (VEC % 4 == 0) {
#pragma unroll
        for (int i = 0; i < VEC; i += 4)
            *reinterpret_cast<float4 *>(p + i) = make_float4(v[i], v[i + 1], v[i + 2], v[i + 3]);
    } else if constexpr (VEC == 2) {
        *reinterpret_cast<float2 *>(p) = make_float2(v[0], v[1]);
    } else {
        p[0] = v[0];
    }
}

// The same for rows that are written once and not read again by this kernel: the store
// does not claim a place in the caches.
template <int VEC>
__device__ __forceinline__ void store_row_streaming(float *p, const float (&v)[VEC]) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    if constexpr (VEC % 4 == 0) {
#pragma unroll
        for (int i = 0; i < VEC; i += 4) {
            f4 t = {v[i], v[i + 1], v[i + 2], v[i + 3]};
            __builtin_nontemporal_store(t, reinterpret_cast<f4 *>(p + i));
        }
    } else if constexpr (VEC == 2) {
        typedef float f2 __attribute__((ext_vector_type(2)));
        f2 t = {v[0], v[1]};
        __builtin_nontemporal_store(t, reinterpret_cast<f2 *>(p));
    } else {
#pragma unroll
        for (int i = 0; i < VEC; i++) __builtin_nontemporal_store(v[i], p + i);
    }
}

// ---- wave64 helpers ---------------------------------------------------------
__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }
// The wave's index in its workgroup as a scalar: what is derived from it (row ranges,
// loop bounds) then stays in scalar registers and scalar branches.
__device__ __forceinline__ int wave_id() {
    return __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
}

// Sum over the lanes whose ids differ only in bits >= log2(stride): the
// butterfly leaves every lane with the total of its residue class mod stride.
template <int STRIDE>
__device__ __forceinline__ float wave_sum_strided(float v) {
#pragma unroll
    for (int o = 32; o >= STRIDE; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}
template <int STRIDE>
__device__ __forceinline__ float wave_max_strided(float v) {
#pragma unroll
    for (int o = 32; o >= STRIDE; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}
// One lane permutation inside rows of 16 lanes on the vector ALU's data-parallel
// primitives: no LDS round trip, which is what __shfl_xor compiles to.
template <int CTRL>
__device__ __forceinline__ float dpp_permute(float v) {
    return __int_as_float(
        __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
// Sum over aligned groups of WIDTH consecutive lanes, left in every lane of the group.
// Up to 16 lanes: pairs, quads (quad permutes), halves of a row (mirror inside 8 lanes),
// rows (mirror inside 16 lanes); beyond that, shuffles across rows. The order of the
// additions is fixed.
template <int WIDTH>
__device__ __forceinline__ float group_sum(float v) {
    if constexpr (WIDTH >= 2) v += dpp_permute<0xb1>(v);   // quad_perm [1,0,3,2]
    if constexpr (WIDTH >= 4) v += dpp_permute<0x4e>(v);   // quad_perm [2,3,0,1]
    if constexpr (WIDTH >= 8) v += dpp_permute<0x141>(v);  // row_half_mirror
    if constexpr (WIDTH >= 16) v += dpp_permute<0x140>(v); // row_mirror
    if constexpr (WIDTH >= 32) v += __shfl_xor(v, 16, kWave);
    if constexpr (WIDTH >= 64) v += __shfl_xor(v, 32, kWave);
    return v;
}

}  // namespace yitu
