/*
 * TEST INFRASTRUCTURE ONLY -- a scalar CPU restatement of the byte-level
 * arithmetic of the FP8 contraction path.  Nothing in the shipped package
 * links, loads or calls this file; only tests, the smoke check and the
 * benchmark's cpu_baseline leg may use it, and only as the checker.
 *
 * What it restates:
 *   - the OCP float8_e4m3fn / float8_e5m2 encoders that PyTorch eager applies
 *     in `x.div(s).to(torch.float8_e4m3fn)` (reference train_gpt_medium.py:45-46,
 *     train_gpt.py:78-79, triton_kernels.py:1212-1213) and
 *     `grad.div(grad_s).to(torch.float8_e5m2)` (train_gpt_medium.py:75,
 *     train_gpt.py:114): round-to-nearest-even, subnormals kept, NOT
 *     saturating (e4m3fn overflow -> NaN code 0x7f, e5m2 overflow -> +-inf);
 *   - the saturating e5m2 store of the cross-entropy kernel
 *     (`cvt.rn.satfinite.e5m2x2.f32`, triton_kernels.py:923-933);
 *   - the eager quantiser for a bf16 tensor and a Python-float scale:
 *     fp8(bf16_rne(fp32(x) / fp32(s))) -- the division is IEEE fp32 and its
 *     result is rounded to bf16 before the fp8 cast.
 *
 *   - the two per-tensor quantisers of the FP8 MLP with every rounding of the eager
 *     expressions written out (train_gpt.py:1645-1647 and :1419-1422); they pin the
 *     torch formulations in nanogpt_fp8_oracle.py (tests/test_oracle_math.py).
 *
 * Pinned by tests/test_oracle_fp8.py: closed-form decode of all 256 codes of
 * each format, encode(decode(c)) == c, monotonicity, tie-to-even at every
 * midpoint between adjacent codes, the overflow thresholds, and agreement
 * with the PyTorch CPU casts on all 65536 bf16 bit patterns (committed
 * tables under tests/golden/).
 */
#include <stdint.h>
#include <string.h>
#include <math.h>

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* fp32 -> bf16, round to nearest even; NaN stays NaN (quiet). */
uint16_t ngpt_oracle_f32_to_bf16(float f) {
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

float ngpt_oracle_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/*
 * Generic fp32 -> small-float encoder.  EBITS/MBITS describe the target,
 * BIAS its exponent bias.  Works on the exact binary value: the magnitude is
 * written as q * 2^e_min_sub with q rounded to nearest even, so normals,
 * subnormals and the carry from the top subnormal into the first normal are
 * one code path.  Returns the magnitude code without the sign; a result
 * above `max_code` is reported as max_code + 1 so the caller can apply the
 * format's overflow rule.
 */
static uint32_t encode_mag(float a /* >= 0, finite */, int ebits, int mbits, int bias) {
    (void)ebits;
    if (a == 0.0f) return 0;
    int e;
    (void)frexpf(a, &e);              /* a = m * 2^e, m in [0.5,1) -> floor(log2 a) = e-1 */
    int E = e - 1;
    int emin = 1 - bias;              /* exponent of the smallest normal */
    if (E < emin) E = emin;           /* subnormal range shares emin's quantum */
    /* quantum = 2^(E - mbits); q = a / quantum, exact in double */
    double q = ldexp((double)a, mbits - E);
    double fl = floor(q);
    double rem = q - fl;
    uint64_t qi = (uint64_t)fl;
    if (rem > 0.5 || (rem == 0.5 && (qi & 1u))) qi += 1;
    /* qi in [0, 2^(mbits+1)]: qi < 2^mbits only in the subnormal range */
    uint32_t code;
    if (E == emin && qi < (1u << mbits)) {
        code = (uint32_t)qi;                                  /* subnormal (or zero) */
    } else {
        if (qi == (2u << mbits)) { qi >>= 1; E += 1; }        /* mantissa carry */
        code = ((uint32_t)(E + bias) << mbits) | ((uint32_t)qi & ((1u << mbits) - 1u));
    }
    return code;
}

/* torch.float8_e4m3fn: 1-4-3, bias 7, no inf, only S.1111.111 is NaN, max 448. */
uint8_t ngpt_oracle_f32_to_e4m3fn(float f) {
    uint32_t u = f32_bits(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    if ((u & 0x7fffffffu) >= 0x7f800000u) return (uint8_t)(sign | 0x7fu);   /* inf, NaN -> NaN */
    uint32_t code = encode_mag(fabsf(f), 4, 3, 7);
    if (code > 0x7eu) code = 0x7fu;                                          /* overflow -> NaN */
    return (uint8_t)(sign | code);
}

/* torch.float8_e5m2: 1-5-2, bias 15, IEEE-like inf/NaN, max 57344. */
uint8_t ngpt_oracle_f32_to_e5m2(float f) {
    uint32_t u = f32_bits(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    uint32_t mag = u & 0x7fffffffu;
    if (mag > 0x7f800000u) return (uint8_t)(sign | 0x7fu);                   /* NaN */
    if (mag == 0x7f800000u) return (uint8_t)(sign | 0x7cu);                  /* inf */
    uint32_t code = encode_mag(fabsf(f), 5, 2, 15);
    if (code > 0x7bu) code = 0x7cu;                                          /* overflow -> inf */
    return (uint8_t)(sign | code);
}

/* e5m2 with saturation to +-57344 (the CE kernel's satfinite store). */
uint8_t ngpt_oracle_f32_to_e5m2_sat(float f) {
    uint32_t u = f32_bits(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    uint32_t mag = u & 0x7fffffffu;
    if (mag > 0x7f800000u) return (uint8_t)(sign | 0x7fu);
    if (mag == 0x7f800000u) return (uint8_t)(sign | 0x7bu);
    uint32_t code = encode_mag(fabsf(f), 5, 2, 15);
    if (code > 0x7bu) code = 0x7bu;
    return (uint8_t)(sign | code);
}

float ngpt_oracle_e4m3fn_to_f32(uint8_t c) {
    int s = c >> 7, e = (c >> 3) & 0xf, m = c & 7;
    float v;
    if (e == 0xf && m == 7) v = NAN;
    else if (e == 0) v = ldexpf((float)m, -9);               /* m/8 * 2^-6 */
    else v = ldexpf((float)(8 + m), e - 7 - 3);
    return s ? -v : v;
}

float ngpt_oracle_e5m2_to_f32(uint8_t c) {
    int s = c >> 7, e = (c >> 2) & 0x1f, m = c & 3;
    float v;
    if (e == 0x1f) v = m ? NAN : INFINITY;
    else if (e == 0) v = ldexpf((float)m, -16);              /* m/4 * 2^-14 */
    else v = ldexpf((float)(4 + m), e - 15 - 2);
    return s ? -v : v;
}

/* Eager quantiser: out[i] = fp8(bf16(fp32(in[i]) / s)); fmt 0 = e4m3fn, 1 = e5m2, 2 = e5m2 saturating. */
void ngpt_oracle_quant_bf16(const uint16_t* in, uint8_t* out, int64_t n, float s, int fmt) {
    for (int64_t i = 0; i < n; ++i) {
        float x = ngpt_oracle_bf16_to_f32(in[i]);
        float q = ngpt_oracle_bf16_to_f32(ngpt_oracle_f32_to_bf16(x / s));
        out[i] = fmt == 0 ? ngpt_oracle_f32_to_e4m3fn(q)
               : fmt == 1 ? ngpt_oracle_f32_to_e5m2(q)
                          : ngpt_oracle_f32_to_e5m2_sat(q);
    }
}

/* Encode an fp32 array directly (no bf16 step); same fmt codes. */
void ngpt_oracle_encode_f32(const float* in, uint8_t* out, int64_t n, int fmt) {
    for (int64_t i = 0; i < n; ++i)
        out[i] = fmt == 0 ? ngpt_oracle_f32_to_e4m3fn(in[i])
               : fmt == 1 ? ngpt_oracle_f32_to_e5m2(in[i])
                          : ngpt_oracle_f32_to_e5m2_sat(in[i]);
}

/*
 * Brute-force fp8 GEMM on codes: C[m,n] = scale * sum_k dec(A[m,k]) * dec(B[n,k]),
 * accumulated in double.  fmt_a / fmt_b: 0 = e4m3fn, 1 = e5m2.  Small shapes only.
 */
void ngpt_oracle_gemm_tn_codes(const uint8_t* A, const uint8_t* B, double* C,
                               int M, int N, int K, int fmt_a, int fmt_b, double scale) {
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            double acc = 0.0;
            for (int k = 0; k < K; ++k) {
                float a = fmt_a ? ngpt_oracle_e5m2_to_f32(A[(int64_t)m * K + k])
                                : ngpt_oracle_e4m3fn_to_f32(A[(int64_t)m * K + k]);
                float b = fmt_b ? ngpt_oracle_e5m2_to_f32(B[(int64_t)n * K + k])
                                : ngpt_oracle_e4m3fn_to_f32(B[(int64_t)n * K + k]);
                acc += (double)a * (double)b;
            }
            C[(int64_t)m * N + n] = acc * scale;
        }
}

static float bf16_round(float f) { return ngpt_oracle_bf16_to_f32(ngpt_oracle_f32_to_bf16(f)); }

/* max |v| over n bf16 values, clamped below by bf16(1e-12): `t.abs().max().clamp(min=1e-12)` on a bf16 tensor. */
static float bf16_amax_clamped(const uint16_t* v, int64_t n) {
    float m = 0.0f;
    for (int64_t i = 0; i < n; ++i) {
        float a = fabsf(ngpt_oracle_bf16_to_f32(v[i]));
        if (a > m) m = a;
    }
    float lo = bf16_round(1.0e-12f);
    return m < lo ? lo : m;
}

/*
 * MLP input quantiser, train_gpt.py:1645-1647, every bf16 operation of the eager expressions rounding:
 *   amax    = normed.abs().max().clamp(min=1e-12)                    bf16
 *   q       = 448.0 / amax = bf16(bf16(1 / amax) * 448)             (float / Tensor is reciprocal() * float)
 *   x_f8    = e4m3fn(bf16(normed * q))
 *   dequant = (up_scale * amax) / 448                                fp32, in-place mul_ then div_
 */
void ngpt_oracle_mlp_input_quant(const uint16_t* normed, int64_t n, float up_scale, uint8_t* x_f8, float* dequant) {
    float amax = bf16_amax_clamped(normed, n);
    float q = bf16_round(bf16_round(1.0f / amax) * 448.0f);
    for (int64_t i = 0; i < n; ++i)
        x_f8[i] = ngpt_oracle_f32_to_e4m3fn(bf16_round(ngpt_oracle_bf16_to_f32(normed[i]) * q));
    float d = up_scale * amax;
    *dequant = d / 448.0f;
}

/*
 * Up-projection weight quantiser, train_gpt.py:1419-1422, per layer l of w [layers, per_layer] bf16:
 *   scale[l] = bf16(amax_l / 448)  with amax_l = max |w_l| clamped below by bf16(1e-12)   (bf16 tensor / float)
 *   w_f8[l]  = e4m3fn(bf16(w_l / scale[l]))                                                 (bf16 tensor / bf16 tensor)
 * scales are returned as fp32 (`up_scales.float()`).
 */
void ngpt_oracle_quant_up_weights(const uint16_t* w, int layers, int64_t per_layer, uint8_t* w_f8, float* scales) {
    for (int l = 0; l < layers; ++l) {
        const uint16_t* wl = w + (int64_t)l * per_layer;
        float scale = bf16_round(bf16_amax_clamped(wl, per_layer) / 448.0f);
        scales[l] = scale;
        for (int64_t i = 0; i < per_layer; ++i)
            w_f8[(int64_t)l * per_layer + i] = ngpt_oracle_f32_to_e4m3fn(bf16_round(ngpt_oracle_bf16_to_f32(wl[i]) / scale));
    }
}
