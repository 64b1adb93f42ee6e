// Device-side helpers shared by the MatchAttention kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace ma {

typedef _Float16 half_t;
typedef __bf16 bf16_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kMaxR = 3;  // window radius supported by every kernel
constexpr int kWave = 64;

// ---- storage-type traits -------------------------------------------------------------
template <typename T> struct Traits;
template <> struct Traits<float> {
    static constexpr int kEPV = 4;  // elements per 16-byte vector
    static __device__ __forceinline__ float to_f(float v) { return v; }
    static __device__ __forceinline__ float from_f(float v) { return v; }
    static __device__ __forceinline__ float round(float v) { return v; }
};
template <> struct Traits<half_t> {
    static constexpr int kEPV = 8;
    static __device__ __forceinline__ float to_f(half_t v) { return (float)v; }
    static __device__ __forceinline__ half_t from_f(float v) { return (half_t)v; }
    static __device__ __forceinline__ float round(float v) { return (float)(half_t)v; }
};
template <> struct Traits<bf16_t> {
    static constexpr int kEPV = 8;
    static __device__ __forceinline__ float to_f(bf16_t v) { return (float)v; }
    static __device__ __forceinline__ bf16_t from_f(float v) { return (bf16_t)v; }
    static __device__ __forceinline__ float round(float v) { return (float)(bf16_t)v; }
};

__device__ __forceinline__ float as_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t as_u32(float f) { return __builtin_bit_cast(uint32_t, f); }
__device__ __forceinline__ half2_t as_h2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }
__device__ __forceinline__ uint32_t h2_as_u32(half2_t h) { return __builtin_bit_cast(uint32_t, h); }

// Element e (0..kEPV-1) of a 16-byte vector, widened to fp32.
template <typename T> __device__ __forceinline__ float vec_elem(const u32x4 &v, int e);
template <> __device__ __forceinline__ float vec_elem<float>(const u32x4 &v, int e) { return as_f32(v[e]); }
template <> __device__ __forceinline__ float vec_elem<half_t>(const u32x4 &v, int e) {
    half2_t p = as_h2(v[e >> 1]);
    return (float)((e & 1) ? p.y : p.x);
}
template <> __device__ __forceinline__ float vec_elem<bf16_t>(const u32x4 &v, int e) {
    uint32_t w = v[e >> 1];
    return as_f32((e & 1) ? (w & 0xffff0000u) : (w << 16));
}

// Pack kEPV fp32 values into a 16-byte vector of T (round to nearest even).
template <typename T> __device__ __forceinline__ u32x4 vec_pack(const float *f);
template <> __device__ __forceinline__ u32x4 vec_pack<float>(const float *f) {
    return u32x4{as_u32(f[0]), as_u32(f[1]), as_u32(f[2]), as_u32(f[3])};
}
template <> __device__ __forceinline__ u32x4 vec_pack<half_t>(const float *f) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = h2_as_u32(half2_t{(half_t)f[2 * i], (half_t)f[2 * i + 1]});
    return r;
}
template <> __device__ __forceinline__ u32x4 vec_pack<bf16_t>(const float *f) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        uint32_t lo = (uint32_t)__builtin_bit_cast(uint16_t, (bf16_t)f[2 * i]);
        uint32_t hi = (uint32_t)__builtin_bit_cast(uint16_t, (bf16_t)f[2 * i + 1]);
        r[i] = lo | (hi << 16);
    }
    return r;
}

// Elementwise product of two 16-byte vectors of T, rounded to T once (the exact product of two 16-bit
// floats fits fp32).
template <typename T> __device__ __forceinline__ u32x4 vec_mul(const u32x4 &a, const u32x4 &b) {
    float f[Traits<T>::kEPV];
#pragma unroll
    for (int e = 0; e < Traits<T>::kEPV; ++e) f[e] = vec_elem<T>(a, e) * vec_elem<T>(b, e);
    return vec_pack<T>(f);
}

// sum_e |q_e - k_e| over one 16-byte vector, added to acc (fp32 accumulator).
// fp16 subtracts in packed half (the rounding point of the PyTorch definition in
// half precision), then accumulates |d| in fp32 with a dot-product against (1,1).
template <typename T> __device__ __forceinline__ float l1_accum(const u32x4 &q, const u32x4 &k, float acc);
template <> __device__ __forceinline__ float l1_accum<float>(const u32x4 &q, const u32x4 &k, float acc) {
#pragma unroll
    for (int e = 0; e < 4; ++e) acc += __builtin_fabsf(as_f32(q[e]) - as_f32(k[e]));
    return acc;
}
template <> __device__ __forceinline__ float l1_accum<half_t>(const u32x4 &q, const u32x4 &k, float acc) {
    const half2_t ones = {(half_t)1.0f, (half_t)1.0f};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        half2_t d = as_h2(q[e]) - as_h2(k[e]);
        half2_t a = as_h2(h2_as_u32(d) & 0x7fff7fffu);
        acc = __builtin_amdgcn_fdot2(a, ones, acc, false);
    }
    return acc;
}
// bf16: the difference is stored in bf16 by the definition.  Both differences of a 32-bit word are rounded by one
// packed conversion, the sign bits cleared together, and the pair added to the fp32 sum by a dot product with (1, 1).
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t bf16_abs_diff2(uint32_t qw, uint32_t kw) {
    const float d_lo = as_f32(qw << 16) - as_f32(kw << 16), d_hi = as_f32(qw & 0xffff0000u) - as_f32(kw & 0xffff0000u);
    const bf16x2_t d = {(__bf16)d_lo, (__bf16)d_hi};
    return __builtin_bit_cast(uint32_t, d) & 0x7fff7fffu;
}
template <> __device__ __forceinline__ float l1_accum<bf16_t>(const u32x4 &q, const u32x4 &k, float acc) {
    const bf16x2_t ones = {(__bf16)1.0f, (__bf16)1.0f};
#pragma unroll
    for (int e = 0; e < 4; ++e)
        acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, bf16_abs_diff2(q[e], k[e])), ones, acc, false);
    return acc;
}

// The same sum started from zero.  fp16: the first product-sum names its zero addend as an operand; the
// accumulating form the compiler selects for the builtin would clear its destination register first.
template <typename T> __device__ __forceinline__ float l1_sum(const u32x4 &q, const u32x4 &k) {
    return l1_accum<T>(q, k, 0.f);
}
template <> __device__ __forceinline__ float l1_sum<half_t>(const u32x4 &q, const u32x4 &k) {
    const half2_t ones = {(half_t)1.0f, (half_t)1.0f};
    const half2_t d0 = as_h2(q[0]) - as_h2(k[0]);
    float acc;
    asm("v_dot2_f32_f16 %0, %1, %2, 0" : "=v"(acc) : "v"(h2_as_u32(d0) & 0x7fff7fffu), "v"(h2_as_u32(ones)));
#pragma unroll
    for (int e = 1; e < 4; ++e) {
        const half2_t d = as_h2(q[e]) - as_h2(k[e]);
        acc = __builtin_amdgcn_fdot2(as_h2(h2_as_u32(d) & 0x7fff7fffu), ones, acc, false);
    }
    return acc;
}

template <> __device__ __forceinline__ float l1_sum<bf16_t>(const u32x4 &q, const u32x4 &k) {
    const bf16x2_t ones = {(__bf16)1.0f, (__bf16)1.0f};
    float acc;
    asm("v_dot2_f32_bf16 %0, %1, %2, 0" : "=v"(acc) : "v"(bf16_abs_diff2(q[0], k[0])), "v"(__builtin_bit_cast(uint32_t, ones)));
#pragma unroll
    for (int e = 1; e < 4; ++e)
        acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, bf16_abs_diff2(q[e], k[e])), ones, acc, false);
    return acc;
}

// ---- cross-lane sums over aligned groups of LPH lanes (DPP, no LDS) ------------------
template <int CTRL> __device__ __forceinline__ float dpp_mov(float x) {
    return as_f32((uint32_t)__builtin_amdgcn_update_dpp(0, (int)as_u32(x), CTRL, 0xf, 0xf, false));
}
template <int LPH> __device__ __forceinline__ float group_sum(float x) {
    static_assert(LPH == 1 || LPH == 2 || LPH == 4 || LPH == 8 || LPH == 16 || LPH == 32 || LPH == 64, "group size");
    if (LPH >= 2) x += dpp_mov<0xB1>(x);   // quad_perm [1,0,3,2]
    if (LPH >= 4) x += dpp_mov<0x4E>(x);   // quad_perm [2,3,0,1]
    if (LPH >= 8) x += dpp_mov<0x141>(x);  // row_half_mirror
    if (LPH >= 16) x += dpp_mov<0x140>(x); // row_mirror
    // (beyond a row of 16 lanes: through the LDS crossbar)
    if (LPH >= 32) x += as_f32((uint32_t)__builtin_amdgcn_ds_bpermute((int)(((threadIdx.x & 63u) ^ 16u) * 4u), (int)as_u32(x)));
    if (LPH >= 64) x += as_f32((uint32_t)__builtin_amdgcn_ds_bpermute((int)(((threadIdx.x & 63u) ^ 32u) * 4u), (int)as_u32(x)));
    return x;
}

// Compile-time loop: f(integral_constant<int, I>) for I in [I0, N).
template <int I, int N, typename F> __device__ __forceinline__ void static_for(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

__device__ __forceinline__ int clampi(int v, int lo, int hi) { return min(max(v, lo), hi); }

// Integer window centre from the floored sampling position.  The float is bounded first: +inf (or any value
// beyond int) converts to INT_MAX, and `centre + tap` then overflows -- which the compiler, entitled to assume
// it does not, uses to fold clamp(centre + t, 0, n) into min(max(centre, -t) + t, n): a negative index, and a
// memory fault where the address is not range-checked.  Beyond +-30000 every tap is a border pixel anyway
// (maps are smaller than that), so the result does not change.  NaN becomes -30000.
constexpr float kCentreLimit = 30000.f;
__device__ __forceinline__ int centre_index(float floored) { return (int)fminf(fmaxf(floored, -kCentreLimit), kCentreLimit); }

// Raw buffer descriptor over `bytes` bytes at p: 32-bit byte offsets, and loads
// beyond `bytes` return zero instead of faulting.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ u32x4 buf_load16(__amdgpu_buffer_rsrc_t r, uint32_t byte_off) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_off, 0, 0);
}
// Same with a wavefront-uniform byte offset added from a scalar register (the range check
// covers the per-lane offset only, so lane offset + uniform offset must be valid by construction).
__device__ __forceinline__ u32x4 buf_load16(__amdgpu_buffer_rsrc_t r, uint32_t lane_off, uint32_t uniform_off) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, (int)lane_off, (int)uniform_off, 0);
}

// Stores through a buffer descriptor: a lane whose offset lies beyond the buffer (kDeadOffset)
// writes nothing, which predicates a store without a branch.
constexpr uint32_t kDeadOffset = 0xFFFFFF00u;
__device__ __forceinline__ void buf_store16(__amdgpu_buffer_rsrc_t r, uint32_t byte_off, u32x4 v) {
    __builtin_amdgcn_raw_buffer_store_b128(v, r, (int)byte_off, 0, 0);
}
__device__ __forceinline__ void buf_store8(__amdgpu_buffer_rsrc_t r, uint32_t byte_off, u32x2 v) {
    __builtin_amdgcn_raw_buffer_store_b64(v, r, (int)byte_off, 0, 0);
}

}  // namespace ma
