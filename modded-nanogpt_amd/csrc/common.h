// Device-side helpers shared by every kernel of the FP8 contraction path (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ngpt {

typedef int   v2i  __attribute__((ext_vector_type(2)));
typedef int   v4i  __attribute__((ext_vector_type(4)));
typedef int   v8i  __attribute__((ext_vector_type(8)));
typedef float v4f  __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

enum : int { FMT_E4M3 = 0, FMT_E5M2 = 1, FMT_BF16 = 2 };   // FMT_BF16: both operands bf16, contraction counted in bytes
// Added to the A format of the GEMM kernel: the A operand is given as the panel of its TRANSPOSE (rows =
// contraction index) and is transposed on the way from LDS to the MFMA registers.
constexpr int FMT_TRANSPOSED = 4;
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

constexpr int kWave = 64;

// ---------------------------------------------------------------- bf16 <-> f32
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// round-to-nearest-even; NaN stays NaN
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    uint32_t r = u + 0x7fffu + ((u >> 16) & 1u);
    r = (f != f) ? (u | 0x00400000u) : r;
    return r >> 16;
}

__device__ __forceinline__ float round_to_bf16(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    return f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
}

// Two fp32 values -> bf16 bit patterns packed lo | hi << 16 with the hardware converter
// (v_cvt_pk_bf16_f32, round to nearest even).
typedef __bf16 hw_bf16x2 __attribute__((ext_vector_type(2)));
typedef float hw_f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t cvt_pk_bf16(float lo, float hi) {
    hw_f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, hw_bf16x2));
}

// ---------------------------------------------------------------- f32 -> fp8 (OCP)
// The hardware converter (v_cvt_pk_fp8_f32 / v_cvt_pk_bf8_f32) rounds to nearest even and keeps
// subnormals.  What it does above the largest finite value depends on a mode bit, so overflow
// and NaN are decided here and only in-range magnitudes reach the converter.

// torch.float8_e4m3fn cast: |v| > 464 (the tie at 464 rounds down to 448) -> NaN code, no saturation.
__device__ __forceinline__ uint32_t f32_to_e4m3_torch(float v) {
    float a = fabsf(v);
    uint32_t sign = (__float_as_uint(v) >> 24) & 0x80u;
    bool bad = !(a <= 464.0f);                       // overflow, inf or NaN
    float c = bad ? 0.0f : v;
    uint32_t code = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(c, c, 0, false) & 0xffu;
    return bad ? (sign | 0x7fu) : code;
}

// torch.float8_e5m2 cast: |v| >= 61440 -> +-inf (the tie rounds to the even code, which is inf).
__device__ __forceinline__ uint32_t f32_to_e5m2_torch(float v) {
    float a = fabsf(v);
    uint32_t sign = (__float_as_uint(v) >> 24) & 0x80u;
    bool isnan_ = (v != v);
    bool ovf = (a >= 61440.0f);
    float c = (isnan_ || ovf) ? 0.0f : v;
    uint32_t code = (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(c, c, 0, false) & 0xffu;
    code = ovf ? (sign | 0x7cu) : code;
    return isnan_ ? (sign | 0x7fu) : code;
}

// Saturating e5m2 of two values (the cross-entropy gradient store): finite values clamp to +-57344.
__device__ __forceinline__ uint32_t f32x2_to_e5m2_sat(float a, float b) {
    a = __builtin_fminf(__builtin_fmaxf(a, -57344.0f), 57344.0f);
    b = __builtin_fminf(__builtin_fmaxf(b, -57344.0f), 57344.0f);
    return (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(a, b, 0, false) & 0xffffu;
}

// SAT = false: the caller knows that |value| <= 57344 and saves the clamps.  The converter writes one half
// of its destination and keeps the other: the first of the two conversions gets its own first source (dead
// afterwards) as the "old" value -- all 32 bits are overwritten in the end -- instead of a fresh zero.
template <bool SAT = true>
__device__ __forceinline__ uint32_t f32x4_to_e5m2_sat(float a, float b, float c, float d) {
    if (SAT) {
        a = __builtin_fminf(__builtin_fmaxf(a, -57344.0f), 57344.0f);
        b = __builtin_fminf(__builtin_fmaxf(b, -57344.0f), 57344.0f);
        c = __builtin_fminf(__builtin_fmaxf(c, -57344.0f), 57344.0f);
        d = __builtin_fminf(__builtin_fmaxf(d, -57344.0f), 57344.0f);
    }
    int r = __builtin_amdgcn_cvt_pk_bf8_f32(a, b, __builtin_bit_cast(int, a), false);
    r = __builtin_amdgcn_cvt_pk_bf8_f32(c, d, r, true);
    return (uint32_t)r;
}

// Saturating e4m3 of one value, input already clamped to <= 448 by the caller or here.
__device__ __forceinline__ uint32_t f32_to_e4m3_sat(float v) {
    v = __builtin_fminf(__builtin_fmaxf(v, -448.0f), 448.0f);
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(v, v, 0, false) & 0xffu;
}

// fp8(bf16_rne(fp32(x) / s)): the division is IEEE fp32 and is rounded to bf16 before the cast.
template <int FMT>
__device__ __forceinline__ uint32_t quant_one(uint32_t bf16_bits, float s) {
    float q = round_to_bf16(__fdiv_rn(bf16_bits_to_f32(bf16_bits), s));
    return FMT == FMT_E4M3 ? f32_to_e4m3_torch(q) : f32_to_e5m2_torch(q);
}

// Eight values at once.  Common case, taken when no lane of the wave holds a special value: the division
// is x * r followed by two corrections q <- RN(q + RN(x - q s) r) with r = RN(1 / s).  x * r can be more than
// one unit in the last place off; after the first correction q is within 2^-46 of the quotient, so the second
// remainder is exact and its correction gives the correctly rounded quotient (Markstein's theorem: q
// faithful, r correctly rounded, significand of s not all ones, s and r normal numbers -- `fast_ok` checks
// the last three and s > 0).  The bf16 rounding and the fp8 casts are the hardware's packed conversions
// (round to nearest even, subnormals kept).  A quotient that overflows the fp8 format, an infinity or a
// NaN (the corrected quotient of an infinite x is a NaN, so those are caught too) sends the whole wave
// through the per-element path, which decides them explicitly.
template <int FMT>
__device__ __forceinline__ v2i quant8_slow(v4i in, float s) {
    uint32_t w[4] = {(uint32_t)in.x, (uint32_t)in.y, (uint32_t)in.z, (uint32_t)in.w};
    uint32_t c[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        c[2 * i] = quant_one<FMT>(w[i] & 0xffffu, s);
        c[2 * i + 1] = quant_one<FMT>(w[i] >> 16, s);
    }
    v2i o;
    o.x = (int)(c[0] | (c[1] << 8) | (c[2] << 16) | (c[3] << 24));
    o.y = (int)(c[4] | (c[5] << 8) | (c[6] << 16) | (c[7] << 24));
    return o;
}

struct QuantScale {
    float s, r;
    bool fast_ok;
    __device__ explicit QuantScale(float scale) : s(scale), r(__fdiv_rn(1.0f, scale)) {
        const uint32_t sb = __float_as_uint(scale), rb = __float_as_uint(r);
        const uint32_t se = (sb >> 23) & 0xffu, re = (rb >> 23) & 0xffu;
        fast_ok = (sb >> 31) == 0 && (sb & 0x7fffffu) != 0x7fffffu && se != 0 && se != 0xff && re != 0 && re != 0xff;
    }
};

template <int FMT>
__device__ __forceinline__ v2i quant8(v4i in, const QuantScale& qs) {
    const uint32_t w[4] = {(uint32_t)in.x, (uint32_t)in.y, (uint32_t)in.z, (uint32_t)in.w};
    uint32_t pk[4];      // bf16(x / s), two per word
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float x0 = __uint_as_float(w[i] << 16), x1 = __uint_as_float(w[i] & 0xffff0000u);
        float q0 = x0 * qs.r, q1 = x1 * qs.r;
#pragma unroll
        for (int step = 0; step < 2; ++step) {
            q0 = __builtin_fmaf(__builtin_fmaf(-q0, qs.s, x0), qs.r, q0);
            q1 = __builtin_fmaf(__builtin_fmaf(-q1, qs.s, x1), qs.r, q1);
        }
        // a zero quotient comes out of the correction as +0: give it the sign of x (s > 0 on this path)
        pk[i] = cvt_pk_bf16(q0, q1) | (w[i] & 0x80008000u);
    }
    // largest magnitude (as bf16 bits) of the eight: at or beyond the first value that does not cast to a finite code?
    typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
    u16x2 m = __builtin_bit_cast(u16x2, pk[0] & 0x7fff7fffu);
#pragma unroll
    for (int i = 1; i < 4; ++i) m = __builtin_elementwise_max(m, __builtin_bit_cast(u16x2, pk[i] & 0x7fff7fffu));
    // e4m3: above 464 (0x43e8) the torch cast gives NaN; e5m2: from 61440 (0x4770) on it gives infinity
    constexpr unsigned kFirstBad = FMT == FMT_E4M3 ? 0x43e9u : 0x4770u;
    const bool special = m[0] >= kFirstBad || m[1] >= kFirstBad;
    if (!qs.fast_ok || __any(special)) return quant8_slow<FMT>(in, qs.s);
    v2i o;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const float f0 = __uint_as_float(pk[2 * j] << 16), f1 = __uint_as_float(pk[2 * j] & 0xffff0000u);
        const float f2 = __uint_as_float(pk[2 * j + 1] << 16), f3 = __uint_as_float(pk[2 * j + 1] & 0xffff0000u);
        int r;
        if (FMT == FMT_E4M3) {
            r = __builtin_amdgcn_cvt_pk_fp8_f32(f0, f1, __builtin_bit_cast(int, f0), false);
            r = __builtin_amdgcn_cvt_pk_fp8_f32(f2, f3, r, true);
        } else {
            r = __builtin_amdgcn_cvt_pk_bf8_f32(f0, f1, __builtin_bit_cast(int, f0), false);
            r = __builtin_amdgcn_cvt_pk_bf8_f32(f2, f3, r, true);
        }
        o[j] = r;
    }
    return o;
}
template <int FMT>
__device__ __forceinline__ v2i quant8(v4i in, float s) {
    return quant8<FMT>(in, QuantScale(s));
}

// ---------------------------------------------------------------- wave helpers
__device__ __forceinline__ int lane_id() { return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// 16-byte global -> LDS copy that bypasses registers.  `lds_wave_base` must be the same for all
// lanes of the wave; lane l's 16 bytes land at lds_wave_base + 16*l.
__device__ __forceinline__ void global_to_lds16(const void* gptr, void* lds_wave_base) {
    __builtin_amdgcn_global_load_lds(
        (const __attribute__((address_space(1))) void*)gptr,
        (__attribute__((address_space(3))) void*)lds_wave_base, 16, 0, 0);
}

// Workgroup barrier WITHOUT the implicit "wait for all outstanding memory operations" that
// __syncthreads() carries: the caller states which waits it needs (wait_vmem_le) so
// that operand loads of later pipeline stages can stay in flight across the barrier.
__device__ __forceinline__ void wg_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

}  // namespace ngpt
