// Softcapped cross-entropy: the standalone op on materialised logits and the lm_head-fused
// forward/backward that never stores the [M, V] logits.
//
// Reference semantics (ce_fwd_bwd_kernel): a logit l is a bf16 number; sigma = bf16(sigmoid(l/C + B/C));
// z = A*sigma; loss = sum_k w_k (lse - z[target_k]); dlogit = coef * (S_w * p - term2) * sigma * (1 - sigma),
// p = exp(z - lse), coef = grad_scale * (A/C) / grad_s, stored as saturating e5m2.
//
// Because l is a bf16 number, everything that depends only on l is a function of 16 bits.  Two
// tables indexed by the logit's bit pattern replace all transcendental work in the hot loops:
//   tabE[i] = exp(z - A)                     (forward: sum of exponentials, shifted by the cap A)
//   tabD[i] = exp(z - A) * sigma * (1-sigma) (backward: dlogit = rowf[m] * tabD[i])
// with rowf[m] = coef * S_w[m] * exp(A - lse[m]).  The tables cover |l| in [2^-12, 2^8) exactly
// (128 mantissa steps per binade, both signs); smaller magnitudes share the entry of l = 0 and
// larger ones the last entry, where sigma has saturated in bf16.
#include "epilogues.h"
#include "host_util.h"
#include "launch.h"
#include "panel.h"
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstring>
#include <numeric>

namespace ngpt {

constexpr int kCodeGroupBytes = 256 * 16;   // code panel block: [8 groups of 16 codes][256 tokens][16 bytes]
constexpr int TAB_LO = 0x3980;            // bf16 bits of 2^-12
constexpr int TAB_N = 0x4380 - 0x3980;    // 2560 entries per sign, up to 2^8
constexpr int TAB_NEG = 4096;             // negative logits start here, so the sign is one index bit
constexpr int TAB_ENTRIES = TAB_NEG + TAB_N;
constexpr int TAB_BYTES = TAB_ENTRIES * 4;
constexpr int MAX_CAND = NGPT_MAX_PREDICT + 1;   // shifted targets + the prefix target

// Sigma codes.  The gradient factor D(l) depends on the logit only through sigma = bf16(sigmoid(..)), and the bf16
// values in [SIGC_LOW, 1.0] are 255 consecutive bit patterns: code = bits - SIGC_LOW + 1 in 1..255 names one of them
// exactly, code 0 says "sigma below the window" (logits under about -13 with the reference's constants).  A forward
// that stores one code byte per logit (1 byte, like the reference's saved e5m2 gradient, instead of the 2-byte logit)
// lets the backward rebuild dl = e5m2(rowf * D) bit for bit without running the logits GEMM again.
constexpr int SIGC_LOW = 0x3f80 - 254;           // bf16 bits of 0.25390625
__device__ __forceinline__ uint32_t sigma_code(float sigma_bf16) {
    const int c = (int)(__float_as_uint(sigma_bf16) >> 16) - SIGC_LOW + 1;
    return (c >= 1 && c <= 255) ? (uint32_t)c : 0u;
}

struct Softcap {
    float A, inv_C, B_div_C;
};

__device__ __forceinline__ int tab_index(uint32_t bf16_bits) {
    int t = (int)(bf16_bits & 0x7fffu) - TAB_LO;
    t = max(0, min(t, TAB_N - 1));
    return t + (int)(bf16_bits >> 15) * TAB_NEG;
}

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));

// Two fp32 logits -> their bf16 bit patterns (round to nearest even) packed lo | hi << 16.
__device__ __forceinline__ uint32_t pack_logits(float a, float b) {
    f32x2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
// Byte offsets (4 * tab_index) of both packed logits, again packed lo | hi << 16; all 16-bit lane math.
__device__ __forceinline__ uint32_t tab_offsets2(uint32_t pk) {
    u16x2_t u = __builtin_bit_cast(u16x2_t, pk);
    u16x2_t t = __builtin_elementwise_sub_sat(u & (u16x2_t){0x7fff, 0x7fff}, (u16x2_t){TAB_LO, TAB_LO});
    t = __builtin_elementwise_min(t, (u16x2_t){TAB_N - 1, TAB_N - 1});
    // sign bits (bit 15 of each half) to the table's sign bit and merged in one instruction: written as
    // assembly because the compiler otherwise separates the merge from the extraction of the two halves
    // at the price of an extra instruction.  (A 32-bit shift moves bit 16 into bit 15, which the mask
    // drops: same as shifting the halves.)
    uint32_t off;
    asm("v_and_or_b32 %0, %1, %2, %3"
        : "=v"(off)
        : "v"(pk >> 1), "s"((uint32_t)(4 * TAB_NEG) * 0x10001u), "v"(__builtin_bit_cast(uint32_t, t << (u16x2_t){2, 2})));
    return off;
}
__device__ __forceinline__ float tab_at(const float* tab, uint32_t byte_off) {
    return *(const float*)((const uint8_t*)tab + byte_off);
}

// bf16(sigmoid(l * inv_C + B_div_C)) as an fp32 value; mul and add rounded separately.
__device__ __forceinline__ float softcap_sigma(float l, const Softcap& sc) {
    float u = __fadd_rn(__fmul_rn(l, sc.inv_C), sc.B_div_C);
    float s = __fdiv_rn(1.0f, 1.0f + expf(-u));
    return round_to_bf16(s);
}
__device__ __forceinline__ float softcap_E(float sigma, const Softcap& sc) { return expf(sc.A * sigma - sc.A); }

// embed_codes: every tabE entry carries the sigma code of its logit in the low 8 bits of its fp32 pattern, and the
// upper 24 bits are chosen so that the pattern read as a float is as close to exp(z - A) as those 8 bits allow
// (relative error at most 2^-16, either sign): one table read then serves the sum of exponentials and the code.
// tabE may be null (the backward from codes keeps its code table in that place).
__device__ __forceinline__ void ce_table_entry(int i, float* tabE, float* tabD, const Softcap& sc, bool embed_codes) {
    if (i >= TAB_ENTRIES) return;
    int t = i % TAB_NEG, neg = i / TAB_NEG;
    if (t >= TAB_N) {   // unused gap
        if (tabE) tabE[i] = 0.0f;
        tabD[i] = 0.0f;
        return;
    }
    uint32_t bits = t == 0 ? 0u : (uint32_t)(TAB_LO + t);
    float l = bf16_bits_to_f32(bits | (neg ? 0x8000u : 0u));
    float s = softcap_sigma(l, sc);
    float e = softcap_E(s, sc);
    tabD[i] = e * s * (1.0f - s);
    if (!tabE) return;
    if (embed_codes) {
        const uint32_t code = sigma_code(s), hi = __float_as_uint(e) & ~0xffu;
        float best = __uint_as_float(hi | code);
#pragma unroll
        for (int d = -1; d <= 1; d += 2) {
            const float cand = __uint_as_float((hi + (uint32_t)(d * 0x100)) | code);
            if (fabsf(cand - e) < fabsf(best - e)) best = cand;
        }
        e = best;
    }
    tabE[i] = e;
}
constexpr int TAB_BLOCKS = (TAB_ENTRIES + 255) / 256;
__global__ void ce_table_kernel(float* tabE, float* tabD, Softcap sc, bool embed_codes) {
    ce_table_entry(blockIdx.x * blockDim.x + threadIdx.x, tabE, tabD, sc, embed_codes);
}

// dcode[c] = D of the sigma with code c (the expression of ce_table_kernel's tabD), dcode[0] = 0; dcode[256] = D of
// the largest sigma below the window, which bounds D of every sigma there if D grows with sigma up to it, and
// infinity if it does not (D = exp(A sigma - A) sigma (1 - sigma) grows on (0, 1/2) whatever A > 0 is).
__device__ __forceinline__ float ce_d_below_window(const Softcap& sc) {
    const float s = bf16_bits_to_f32((uint32_t)(SIGC_LOW - 1));
    return s < 0.5f ? softcap_E(s, sc) * s * (1.0f - s) : __builtin_inff();
}
__device__ __forceinline__ void ce_dcode_entry(int c, float* dcode, const Softcap& sc) {   // c = 0 .. 255
    float d = 0.0f;
    if (c >= 1) {
        const float s = bf16_bits_to_f32((uint32_t)(SIGC_LOW + c - 1));
        d = softcap_E(s, sc) * s * (1.0f - s);
    }
    dcode[c] = d;
    if (c == 0) dcode[256] = ce_d_below_window(sc);
}

__global__ void fill_f32_kernel(float* p, int64_t n, float v) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// The lookup table of the GEMM-fused kernels lives in static LDS, so its address is a link-time
// constant that folds into the offset field of every ds_read.
__device__ __forceinline__ float* lds_table() {
    __shared__ float table[TAB_ENTRIES];
    return table;
}

__device__ __forceinline__ void load_table(float* lds_tab, const float* gtab) {
    for (int i = threadIdx.x; i < TAB_ENTRIES; i += blockDim.x) lds_tab[i] = gtab[i];
}

struct CandArgs {
    const int64_t* targets;          // [M]
    const int64_t* prefix_targets;   // [M], nullable
    const float* mtp_weights;        // [n_predict]
    const float* prefix_weight;      // [1], nullable
    int n_predict;
    int M, V;
};

// Candidate c of row m: c < n_predict -> targets[m + c] (if m + c < M), c == n_predict -> prefix target.
__device__ __forceinline__ int64_t cand_target(const CandArgs& ca, int m, int c) {
    if (c < ca.n_predict) return (m + c < ca.M) ? ca.targets[m + c] : -1;
    return ca.prefix_targets ? ca.prefix_targets[m] : -1;
}
__device__ __forceinline__ float cand_weight(const CandArgs& ca, int c) {
    if (c < ca.n_predict) return ca.mtp_weights[c];
    return ca.prefix_weight ? ca.prefix_weight[0] : 0.0f;
}
// Normaliser weight of a row: all n_predict weights (no bounds check on the shifted index, as in the
// reference) plus the prefix weight when the prefix target is valid.
__device__ __forceinline__ float row_weight_sum(const CandArgs& ca, int m) {
    float s = 0.0f;
    for (int k = 0; k < ca.n_predict; ++k) s += ca.mtp_weights[k];
    int64_t pt = ca.prefix_targets ? ca.prefix_targets[m] : -1;
    if (pt >= 0 && pt < ca.V) s += cand_weight(ca, ca.n_predict);
    return s;
}

// =====================================================================================================
// Standalone op on materialised logits: one workgroup walks rows; two sweeps over a row (the second
// one re-reads it from L2) instead of caching 100 KB per row in LDS.
constexpr int ROW_THREADS = 512;

__device__ __forceinline__ float block_sum(float v, float* red /* >= 16 floats */) {
    v = wave_sum(v);
    int wave = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float t = 0.0f;
    for (int w = 0; w < (int)(blockDim.x >> 6); ++w) t += red[w];
    return t;
}

__global__ __launch_bounds__(ROW_THREADS) void ce_rows_kernel(
    const uint16_t* __restrict__ logits, CandArgs ca, float* __restrict__ losses, uint8_t* __restrict__ grad,
    const float* __restrict__ gtabE, const float* __restrict__ gtabD, Softcap sc, float coef) {
    __shared__ float tabE[TAB_ENTRIES];
    __shared__ float tabD[TAB_ENTRIES];
    __shared__ float red[16];
    load_table(tabE, gtabE);
    load_table(tabD, gtabD);
    __syncthreads();
    const int V = ca.V, n8 = V / 8;
    for (int row = blockIdx.x; row < ca.M; row += gridDim.x) {
        const uint16_t* lrow = logits + (int64_t)row * V;
        float sum = 0.0f;
        for (int i = threadIdx.x; i < n8; i += ROW_THREADS) {
            v4i w = *(const v4i*)(lrow + i * 8);
            uint32_t u[4] = {(uint32_t)w.x, (uint32_t)w.y, (uint32_t)w.z, (uint32_t)w.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) sum += tabE[tab_index(u[j] & 0xffffu)] + tabE[tab_index(u[j] >> 16)];
        }
        float S = block_sum(sum, red);
        float lse = sc.A + logf(S);
        float s_w = row_weight_sum(ca, row);
        float p_scale = expf(sc.A - lse);
        float rowf = coef * (s_w * p_scale);
        if (threadIdx.x == 0) {
            float total = 0.0f;
            for (int c = 0; c <= ca.n_predict; ++c) {
                int64_t t = cand_target(ca, row, c);
                if (t >= 0 && t < V) {
                    float sg = softcap_sigma(bf16_bits_to_f32(lrow[t]), sc);
                    total += cand_weight(ca, c) * (lse - sc.A * sg);
                }
            }
            losses[row] = total;
        }
        uint8_t* grow = grad + (int64_t)row * V;
        for (int i = threadIdx.x; i < n8; i += ROW_THREADS) {
            v4i w = *(const v4i*)(lrow + i * 8);
            uint32_t u[4] = {(uint32_t)w.x, (uint32_t)w.y, (uint32_t)w.z, (uint32_t)w.w};
            float g[8];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                g[2 * j] = rowf * tabD[tab_index(u[j] & 0xffffu)];
                g[2 * j + 1] = rowf * tabD[tab_index(u[j] >> 16)];
            }
            v2i o;
            o.x = (int)f32x4_to_e5m2_sat(g[0], g[1], g[2], g[3]);
            o.y = (int)f32x4_to_e5m2_sat(g[4], g[5], g[6], g[7]);
            *(v2i*)(grow + i * 8) = o;
        }
        __syncthreads();   // dense stores of this row are complete before the target columns are rewritten
        if ((int)threadIdx.x <= ca.n_predict) {
            int c = threadIdx.x;
            int64_t t = cand_target(ca, row, c);
            if (t >= 0 && t < V) {
                float sg = softcap_sigma(bf16_bits_to_f32(lrow[t]), sc);
                float p = softcap_E(sg, sc) * p_scale;
                float term2 = 0.0f;
                for (int k = 0; k <= ca.n_predict; ++k) {
                    int64_t tk = cand_target(ca, row, k);
                    if (tk == t) term2 += cand_weight(ca, k);     // every prediction that lands on this column
                }
                float gz = s_w * p - term2;
                float gx = coef * gz * sg * (1.0f - sg);
                grow[t] = (uint8_t)(f32x2_to_e5m2_sat(gx, gx) & 0xffu);
            }
        }
        __syncthreads();
    }
}

// Rows of up to MAXC * 8 * ROWREG_THREADS columns: a thread keeps its 16-byte pieces of the row in
// registers -- as table offsets, which both sweeps use -- so the logits are read from memory once.  Two
// workgroups share a compute unit (at most 128 registers per thread): while one reduces, decides the
// target columns and meets at its barriers, the other streams.  The thread that owns a target column hands
// the raw logit to the candidate's thread through LDS and patches the exact gradient code into its own 8
// output bytes before storing them, so every byte of the gradient is written once.
constexpr int ROWREG_THREADS = 512;

template <int MAXC>
__global__ __launch_bounds__(ROWREG_THREADS, 4) void ce_rows_reg_kernel(
    const uint16_t* __restrict__ logits, CandArgs ca, float* __restrict__ losses, uint8_t* __restrict__ grad,
    const float* __restrict__ gtabE, const float* __restrict__ gtabD, Softcap sc, float coef) {
    __shared__ float tabE[TAB_ENTRIES];
    __shared__ float tabD[TAB_ENTRIES];
    __shared__ float red[16];
    __shared__ uint32_t tl[MAX_CAND];      // raw bf16 bits of the logit at each candidate's target column
    __shared__ uint32_t fix[MAX_CAND];     // exact e5m2 code for that column
    __shared__ float loss_term[MAX_CAND];
    load_table(tabE, gtabE);
    load_table(tabD, gtabD);
    const int V = ca.V, n8 = V / 8, tid = threadIdx.x, ncand = ca.n_predict + 1;
    auto load_row = [&](int row, v4i (&w)[MAXC]) {
        const uint16_t* lrow = logits + (int64_t)row * V;
#pragma unroll
        for (int s_ = 0; s_ < MAXC; ++s_) {
            const int i = tid + s_ * ROWREG_THREADS;
            w[s_] = (i < n8) ? *(const v4i*)(lrow + i * 8) : (v4i){0, 0, 0, 0};
        }
    };
    v4i cur[MAXC];
    int row = blockIdx.x;
    if (row < ca.M) load_row(row, cur);
    __syncthreads();
    for (; row < ca.M; row += gridDim.x) {
        const int next_row = row + gridDim.x;
        // candidate target columns: the owner publishes the raw logit
        int my_cand_slot[MAX_CAND], my_cand_pos[MAX_CAND];
#pragma unroll
        for (int c = 0; c < MAX_CAND; ++c) {
            my_cand_slot[c] = -1;
            my_cand_pos[c] = 0;
            if (c < ncand) {
                const int64_t t = cand_target(ca, row, c);
                if (t >= 0 && t < V) {
                    const int i8 = (int)(t >> 3);
                    if ((i8 % ROWREG_THREADS) == tid) {
                        my_cand_slot[c] = i8 / ROWREG_THREADS;
                        my_cand_pos[c] = (int)(t & 7);
                        uint32_t word = 0;
#pragma unroll
                        for (int s_ = 0; s_ < MAXC; ++s_)
#pragma unroll
                            for (int k = 0; k < 4; ++k)
                                if (s_ == my_cand_slot[c] && k == (my_cand_pos[c] >> 1)) word = (uint32_t)cur[s_][k];
                        tl[c] = (my_cand_pos[c] & 1) ? (word >> 16) : (word & 0xffffu);
                    }
                }
            }
        }
        // sweep 1: table offsets (kept) and the sum of exponentials
        float sum = 0.0f;
#pragma unroll
        for (int s_ = 0; s_ < MAXC; ++s_) {
            const bool live = tid + s_ * ROWREG_THREADS < n8;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t off = tab_offsets2((uint32_t)cur[s_][k]);
                cur[s_][k] = (int)off;
                if (live) sum += tab_at(tabE, off & 0xffffu) + tab_at(tabE, off >> 16);
            }
        }
        const float S = block_sum(sum, red);      // (its barriers also publish tl[])
        const float lse = sc.A + logf(S);
        const float s_w = row_weight_sum(ca, row);
        const float p_scale = expf(sc.A - lse);
        const float rowf = coef * (s_w * p_scale);
        if (tid < ncand) {
            const int c = tid;
            const int64_t t = cand_target(ca, row, c);
            float term = 0.0f;
            uint32_t code = 0;
            if (t >= 0 && t < V) {
                const float sg = softcap_sigma(bf16_bits_to_f32(tl[c]), sc);
                term = cand_weight(ca, c) * (lse - sc.A * sg);
                const float p = softcap_E(sg, sc) * p_scale;
                float term2 = 0.0f;
                for (int k = 0; k < ncand; ++k)
                    if (cand_target(ca, row, k) == t) term2 += cand_weight(ca, k);   // every prediction that lands on this column
                const float gx = coef * (s_w * p - term2) * sg * (1.0f - sg);
                code = f32x2_to_e5m2_sat(gx, gx) & 0xffu;
            }
            loss_term[c] = term;
            fix[c] = code;
        }
        __syncthreads();
        if (tid == 0) {
            float total = 0.0f;
            for (int c = 0; c < ncand; ++c) total += loss_term[c];
            losses[row] = total;
        }
        // sweep 2: gradient codes, the exact ones patched in by their owners
        const bool big = !(fabsf(rowf) <= 4.0f * 57344.0f);
        uint8_t* grow = grad + (int64_t)row * V;
#pragma unroll
        for (int s_ = 0; s_ < MAXC; ++s_) {
            const int i = tid + s_ * ROWREG_THREADS;
            if (i < n8) {
                float g[8];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t off = (uint32_t)cur[s_][k];
                    g[2 * k] = rowf * tab_at(tabD, off & 0xffffu);
                    g[2 * k + 1] = rowf * tab_at(tabD, off >> 16);
                }
                uint32_t o[2];
                if (big) {
                    o[0] = f32x4_to_e5m2_sat<true>(g[0], g[1], g[2], g[3]);
                    o[1] = f32x4_to_e5m2_sat<true>(g[4], g[5], g[6], g[7]);
                } else {
                    o[0] = f32x4_to_e5m2_sat<false>(g[0], g[1], g[2], g[3]);
                    o[1] = f32x4_to_e5m2_sat<false>(g[4], g[5], g[6], g[7]);
                }
#pragma unroll
                for (int c = 0; c < MAX_CAND; ++c)
                    if (my_cand_slot[c] == s_) {
                        const int sh = 8 * (my_cand_pos[c] & 3);
                        uint32_t& word = o[my_cand_pos[c] >> 2];
                        word = (word & ~(0xffu << sh)) | (fix[c] << sh);
                    }
                *(v2i*)(grow + i * 8) = (v2i){(int)o[0], (int)o[1]};
            }
        }
        if (next_row < ca.M) load_row(next_row, cur);
        __syncthreads();     // tl / fix / loss_term / red are reused by the next row
    }
}

// =====================================================================================================
// Fused forward.  GEMM orientation: rows = vocabulary (A = w_f8 [V, K]), columns = tokens
// (B = x_f8 [M, K]), so one lane owns one token per MFMA tile column and sums exponentials in
// registers.  A job = (token tile, vocabulary split); the workgroup walks the split's vocabulary
// tiles with the token tile fixed and flushes its row sums at the end of the job.
//
// L2-aware placement (workgroup b runs on XCD b % 8, each XCD has its own 4 MB L2): XCD x owns a
// contiguous block of token tiles.  Its workgroups form an MG x CE_SPLITS grid: MG token tiles are
// processed at the same time, each by CE_SPLITS workgroups that take one vocabulary split each.
// The MG token tiles (MG * 196 KB at K = 768) stay L2-resident for the whole round, and every
// weight tile streamed from memory is used by the MG workgroups of its split at about the same time.
constexpr int CE_SPLITS = 4;
constexpr int CE_XCDS = 8;

struct CEJobIter {
    int tiles_v, tile_m_end, tile_m, mg, split, tr_, tr_begin, tr_end;
    __device__ CEJobIter(const GemmOperands& g, int BM, int BN, int bid, int G) {
        tiles_v = (g.R + BM - 1) / BM;
        const int tiles_m = (g.C + BN - 1) / BN;
        const int xcd = bid % CE_XCDS, slot = bid / CE_XCDS;
        mg = G / (CE_XCDS * CE_SPLITS);                       // token tiles in flight per XCD
        const int per_xcd = (tiles_m + CE_XCDS - 1) / CE_XCDS;
        split = slot / mg;
        tile_m = xcd * per_xcd + slot % mg;
        tile_m_end = min(tiles_m, (xcd + 1) * per_xcd);
        tr_begin = tiles_v * split / CE_SPLITS;
        tr_end = tiles_v * (split + 1) / CE_SPLITS;
        tr_ = tr_begin;
        if (tr_begin >= tr_end) tile_m = tile_m_end;          // empty vocabulary range: nothing to do
    }
    __device__ bool valid() const { return tile_m < tile_m_end; }
    __device__ int tr() const { return tr_; }
    __device__ int tc() const { return tile_m; }
    __device__ int kt_begin(int) const { return 0; }
    __device__ int kt_end(int nk) const { return nk; }
    __device__ bool partial() const { return false; }
    __device__ int part_slot() const { return 0; }
    __device__ bool job_begin() const { return tr_ == tr_begin; }
    __device__ bool job_end() const { return tr_ + 1 == tr_end; }
    __device__ int job_id() const { return split; }
    __device__ void advance() {
        if (++tr_ == tr_end) {
            tr_ = tr_begin;
            tile_m += mg;
        }
    }
};

constexpr int CE_MAX_BN = 256;                                  // widest token tile of any config
constexpr int CAND_LDS_BYTES = MAX_CAND * CE_MAX_BN * 4;
constexpr int CE_FWD_EXTRA_LDS = (CAND_LDS_BYTES + 1023) / 1024 * 1024;

// Four code bytes (the low bytes of four table words) as one word, lowest register first.
__device__ __forceinline__ uint32_t pack_codes4(float w0, float w1, float w2, float w3) {
    const uint32_t t01 = __builtin_amdgcn_perm(__float_as_uint(w1), __float_as_uint(w0), 0x0c0c0400);
    const uint32_t t23 = __builtin_amdgcn_perm(__float_as_uint(w3), __float_as_uint(w2), 0x0c0c0400);
    return __builtin_amdgcn_perm(t23, t01, 0x05040100);
}

// CODES: the table entries carry sigma codes (ce_table_kernel with embed_codes) and every tile also writes its
// 256 x 256 codes into the code panel: blocks [token tile][vocabulary / 128] of 256 tokens x 128 codes, a lane's 16
// accumulator registers (16 vocabulary rows of one token, in register order, i.e. dw_pos order inside every
// 32-group) as one 16-byte store.  Inside a block the 16-byte pieces are ordered [8 groups of 16 codes][256 tokens]:
// the 32 lanes of a store instruction that hold consecutive tokens then write 512 contiguous bytes instead of 16
// bytes in each of 32 lines, which is what the vector memory unit is fast at.
template <bool CODES>
struct EpiCEFwdT {
    static constexpr int EXTRA_LDS = CE_FWD_EXTRA_LDS;
    static constexpr bool NEEDS_SCRATCH = false;
    static constexpr bool JOB_END_NEEDS_SCRATCH = true;    // job_end reduces through the stage
    static constexpr int TILE_STORES = CODES ? 8 : 0;      // 16-byte panel stores per wave and tile (the rare sigma stores come on top)
    uint8_t* codes;       // CODES: the code panel
    int nkp;              // CODES: 128-byte k-steps per token tile of the panel = vocabulary rounded up to 256, / 128
    const float* gtabE;
    float* part;          // [CE_SPLITS][M] partial sums of exp(z - A)
    float* saved_sigma;   // [MAX_CAND][M] bf16-rounded sigma at each candidate target column
    CandArgs ca;
    Softcap sc;
    float scale;
    int ncand;            // n_predict (+1 with prefix targets)
    int* cand;            // LDS: [MAX_CAND][CE_MAX_BN] valid target column of the job's tokens, else -1
    float sum[8];

    __device__ void partial(bool, int) {}
    __device__ void begin(int, int, uint8_t* extra) {
        cand = (int*)extra;
        load_table(lds_table(), gtabE);
#pragma unroll
        for (int i = 0; i < 8; ++i) sum[i] = 0.0f;
    }
    __device__ void end(uint8_t*, int, int) {}

    // A new (token tile, split) job: stage the candidate target columns of its tokens in LDS.
    template <class Cfg>
    __device__ void job_begin(int c0) {
        static_assert(Cfg::BN <= CE_MAX_BN, "token tile too wide");
        for (int i = threadIdx.x; i < ncand * Cfg::BN; i += Cfg::THREADS) {
            int c = i / Cfg::BN, j = i % Cfg::BN;
            int m = c0 + j;
            int64_t t = (m < ca.M) ? cand_target(ca, m, c) : -1;
            cand[c * CE_MAX_BN + j] = (t >= 0 && t < ca.V) ? (int)t : -1;
        }
    }

    template <class Cfg>
    __device__ void tile(v16f (&acc)[Cfg::TM][Cfg::TN], int r0 /* vocab */, int c0 /* token */,
                         const AccCoords<Cfg>& co, uint8_t*, int lane) {
        static_assert(Cfg::TN <= 8, "per-lane token columns");
        static_assert(!CODES || (Cfg::BM == kPanelRows && Cfg::BN == kPanelRows && Cfg::WTM == 64 && Cfg::WTN == 128),
                      "the code stores assume a 256 x 256 tile of 64 x 128 wave tiles");
        const int V = ca.V, M = ca.M;
        const float* tab = lds_table();
        // code panel: row = this lane's token, 16 bytes = the 16 vocabulary rows of one (tm, lane half) group;
        // address = wave-uniform pointer + ONE 32-bit per-lane offset + a constant per store
        uint8_t* cd_base = nullptr;
        uint32_t cd_lane = 0;
        if constexpr (CODES) {
            const int wr = co.wave_row0 >> 6, wc = co.wave_col0 >> 7;
            cd_base = codes + ((int64_t)(c0 >> 8) * nkp + (r0 >> 7) + (wr >> 1)) * kPanelBytes;
            cd_lane = (uint32_t)((4 * (wr & 1) + (lane >> 5)) * kCodeGroupBytes + (128 * wc + (lane & 31)) * 16);
        }
        auto code_store = [&](int tm, int tn, uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3) {
            *(v4i*)(cd_base + (cd_lane + tn * 512 + tm * 2 * kCodeGroupBytes)) = (v4i){(int)w0, (int)w1, (int)w2, (int)w3};
        };
        if (r0 + Cfg::BM <= V) {
            // Batches of 8 accumulator registers, software-pipelined by hand: while the 8 table reads of batch b are in
            // flight the index arithmetic of batch b + 1 runs; then batch b is consumed (the compiler waits for every
            // outstanding LDS read at that point, so nothing may be issued between a batch's reads and that arithmetic
            // that it would have to wait for as well) and the reads of batch b + 1 go out.
            constexpr int NB = Cfg::TN * Cfg::TM * 2;
            auto offsets_of = [&](int b, uint32_t (&off)[4]) {
                const v16f& a = acc[(b >> 1) % Cfg::TM][b / (2 * Cfg::TM)];
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    off[k] = tab_offsets2(pack_logits(a[8 * (b & 1) + 2 * k] * scale, a[8 * (b & 1) + 2 * k + 1] * scale));
            };
            auto gather = [&](const uint32_t (&off)[4], float (&v)[8]) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    v[2 * k] = tab_at(tab, off[k] & 0xffffu);
                    v[2 * k + 1] = tab_at(tab, off[k] >> 16);
                }
            };
            float cur[8];
            uint32_t off[4], cw[4];
            offsets_of(0, off);
            gather(off, cur);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                if (b + 1 < NB) offsets_of(b + 1, off);
                __builtin_amdgcn_sched_barrier(0);
                sum[b / (2 * Cfg::TM)] += ((cur[0] + cur[1]) + (cur[2] + cur[3])) + ((cur[4] + cur[5]) + (cur[6] + cur[7]));
                if constexpr (CODES) {
                    cw[2 * (b & 1)] = pack_codes4(cur[0], cur[1], cur[2], cur[3]);
                    cw[2 * (b & 1) + 1] = pack_codes4(cur[4], cur[5], cur[6], cur[7]);
                    if (b & 1) code_store((b >> 1) % Cfg::TM, b / (2 * Cfg::TM), cw[0], cw[1], cw[2], cw[3]);
                }
                __builtin_amdgcn_sched_barrier(0);
                if (b + 1 < NB) gather(off, cur);
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {   // last vocabulary tile: rows past V are clamped duplicates and must not count
#pragma unroll
            for (int tn = 0; tn < Cfg::TN; ++tn)
#pragma unroll
                for (int tm = 0; tm < Cfg::TM; ++tm) {
                    float s0 = 0.0f;
                    uint32_t cwe[4];
#pragma unroll
                    for (int v = 0; v < 16; v += 4) {
                        uint32_t o01 = tab_offsets2(pack_logits(acc[tm][tn][v] * scale, acc[tm][tn][v + 1] * scale));
                        uint32_t o23 = tab_offsets2(pack_logits(acc[tm][tn][v + 2] * scale, acc[tm][tn][v + 3] * scale));
                        const float e0 = tab_at(tab, o01 & 0xffffu), e1 = tab_at(tab, o01 >> 16);
                        const float e2 = tab_at(tab, o23 & 0xffffu), e3 = tab_at(tab, o23 >> 16);
                        s0 += (r0 + co.row(tm, v) < V) ? e0 : 0.0f;
                        s0 += (r0 + co.row(tm, v + 1) < V) ? e1 : 0.0f;
                        s0 += (r0 + co.row(tm, v + 2) < V) ? e2 : 0.0f;
                        s0 += (r0 + co.row(tm, v + 3) < V) ? e3 : 0.0f;
                        if constexpr (CODES) cwe[v >> 2] = pack_codes4(e0, e1, e2, e3);
                    }
                    sum[tn] += s0;
                    if constexpr (CODES)   // rows past V: codes of the clamped duplicates, which no reader of the panel looks at
                        code_store(tm, tn, cwe[0], cwe[1], cwe[2], cwe[3]);
                    __builtin_amdgcn_sched_barrier(0);
                }
        }
        // sigma at candidate target columns that fall inside this wave's vocabulary rows
        const int v_lo = r0 + co.wave_row0;
        for (int c = 0; c < ncand; ++c) {
            int rl[Cfg::TN];
            bool any_hit = false;
#pragma unroll
            for (int tn = 0; tn < Cfg::TN; ++tn) {
                int d = cand[c * CE_MAX_BN + co.col(tn)] - v_lo;
                rl[tn] = ((unsigned)d < (unsigned)Cfg::WTM) ? d : -1;
                any_hit |= rl[tn] >= 0;
            }
            if (!__any(any_hit)) continue;
#pragma unroll
            for (int tn = 0; tn < Cfg::TN; ++tn) {
                if (!__any(rl[tn] >= 0)) continue;
                float got = 0.0f;
                bool mine = false;
#pragma unroll
                for (int tm = 0; tm < Cfg::TM; ++tm)
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        if (co.row(tm, v) - co.wave_row0 == rl[tn]) { got = acc[tm][tn][v]; mine = true; }
                int m = c0 + co.col(tn);
                if (mine && m < M) {
                    float l = bf16_bits_to_f32(pack_logits(got * scale, 0.0f) & 0xffffu);
                    saved_sigma[(int64_t)c * M + m] = softcap_sigma(l, sc);
                }
            }
        }
    }

    // Fold the lane sums of one finished (token tile, split) job into part[split][m].
    template <class Cfg>
    __device__ void job_end(int c0, int split, const AccCoords<Cfg>& co, uint8_t* scratch) {
        float* red = (float*)scratch;                    // [WAVES_M][BN]
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        const int wr = wave / Cfg::WAVES_N;
#pragma unroll
        for (int tn = 0; tn < Cfg::TN; ++tn) {
            float s = sum[tn] + __shfl_xor(sum[tn], 32, 64);
            if (lane < 32) red[wr * Cfg::BN + co.col(tn)] = s;
            sum[tn] = 0.0f;
        }
        wg_barrier();
        for (int j = threadIdx.x; j < Cfg::BN; j += Cfg::THREADS) {
            float s = 0.0f;
#pragma unroll
            for (int w = 0; w < Cfg::WAVES_M; ++w) s += red[w * Cfg::BN + j];
            int m = c0 + j;
            if (m < ca.M) part[(int64_t)split * ca.M + m] = s;
        }
    }
};
using EpiCEFwd = EpiCEFwdT<false>;

__global__ void ce_finalize_kernel(const float* __restrict__ part, const float* __restrict__ saved_sigma,
                                   CandArgs ca, Softcap sc, float* __restrict__ losses, float* __restrict__ lse_out) {
    int m = blockIdx.x * blockDim.x + threadIdx.x;
    if (m >= ca.M) return;
    float S = 0.0f;
    for (int s = 0; s < CE_SPLITS; ++s) S += part[(int64_t)s * ca.M + m];
    float lse = sc.A + logf(S);
    float total = 0.0f;
    for (int c = 0; c <= ca.n_predict; ++c) {
        int64_t t = cand_target(ca, m, c);
        if (t >= 0 && t < ca.V) total += cand_weight(ca, c) * (lse - sc.A * saved_sigma[(int64_t)c * ca.M + m]);
    }
    losses[m] = total;
    lse_out[m] = lse;
}

}  // namespace ngpt
#include "token_stationary.h"
namespace ngpt {

// =====================================================================================================
// Backward, recomputing the logits.  rowf[m] = coef * S_w[m] * exp(A - lse[m]).
// One 256-thread block per 256 rows (one token tile of the recompute kernel).  rowf is written for the
// whole block, zero past M (zero codes in the panel's padding without any masking in the epilogue);
// big[block] says whether any |rowf| of the block is large enough for rowf * D to leave the e5m2 range:
// D = E * sigma * (1 - sigma) <= 1/4, so |rowf| <= 4 * 57344 needs no clamp.
__device__ __forceinline__ float ce_row_factor(const float* __restrict__ lse, const CandArgs& ca, const Softcap& sc, float coef, int m) {
    return m < ca.M ? coef * (row_weight_sum(ca, m) * expf(sc.A - lse[m])) : 0.0f;
}
__device__ __forceinline__ void ce_rowf_block(int block, const float* __restrict__ lse, const CandArgs& ca, const Softcap& sc, float coef,
                                              float* __restrict__ rowf, int* __restrict__ big) {
    const int m = block * 256 + threadIdx.x;
    const float f = ce_row_factor(lse, ca, sc, coef, m);
    rowf[m] = f;
    int b = __syncthreads_or(!(fabsf(f) <= 4.0f * 57344.0f));   // NaN counts as big
    if (threadIdx.x == 0) big[block] = b;
}

// ------------------------------------------------------------------------------------------------
// dlogits panel.  The e5m2 gradient is consumed twice: as an operand of dW = dl^T . x (rows =
// vocabulary, contraction = tokens) and as the A operand of dx = dl . W (rows = tokens, contraction =
// vocabulary).  It is written ONCE, vocabulary-major and panel-blocked (see GemmOperands): blocks
// [V / 256][tokens / 128], 128-byte rows = 128 tokens of one vocabulary column.  Inside such a row the
// tokens of every 32-group sit in the order in which the recompute kernel's accumulator registers hold
// them (dw_pos), so the panel leaves the registers as full 16-byte stores without a trip through
// LDS; x^T, the other operand of dW, is produced with the same token order by panel_transpose_kernel
// (a GEMM does not care about the order of its contraction as long as both operands agree).
// The dx GEMM reads the same panel as the transpose of its A operand and transposes it on the way from
// LDS to the MFMA registers (FMT_TRANSPOSED); its output rows come out in dw_pos order, which its
// epilogue undoes (AccCoords::perm).
//
// Epilogue of the backward's logits recompute (A = x chunk, rows = tokens; B = W, rows = vocabulary):
// dl = e5m2_sat(rowf[token] * D(logit)) written to the panel.  Rows past the last one have rowf = 0, i.e. zero
// codes, so the token padding of the panel contracts to nothing.
struct EpiDlStore {
    static constexpr int TILE_STORES = 8;    // 16-byte panel stores per wave and tile, always
    static constexpr bool HAS_TILE_BEGIN = true;
    static constexpr int EXTRA_LDS = 2048;   // row factors of the current and the next tile (2 x 256 floats)
    static constexpr bool NEEDS_SCRATCH = false;
    static constexpr bool JOB_END_NEEDS_SCRATCH = false;
    template <class Cfg>
    __device__ void job_begin(int) {}
    const float* gtabD;
    const float* rowf;     // already offset to the chunk's first row; zero past the last row up to a multiple of 256
    const int* big;        // per 256 rows of the chunk: some row factor may push a gradient out of the e5m2 range
    uint8_t* dw_panel;     // [Vp / 256][Mt / 128] blocks, Vp / Mt = V / Mc rounded up to 256
    int Mc, V, nkt;        // nkt = k-steps per panel row = Mt / 128
    float scale;
    float* rowf_lds;       // LDS [2][256]
    int rslot;
    int tile_big;

    __device__ void partial(bool, int) {}
    __device__ void begin(int, int, uint8_t* extra) {
        rowf_lds = (float*)extra;
        rslot = 0;
        load_table(lds_table(), gtabD);
    }
    __device__ void end(uint8_t*, int, int) {}
    template <class Cfg>
    __device__ void job_end(int, int, const AccCoords<Cfg>&, uint8_t*) {}

    // The tile's 256 row factors go straight to LDS with one wave-level load, issued before the k-loop, so
    // that tile() contains no global load: a load there would make the wave wait for its own earlier
    // panel stores (the memory counter retires in order).  Two slots: the other one may still be read
    // by waves that are finishing the previous tile.
    template <class Cfg>
    __device__ void tile_begin(int r0, int) {
        rslot ^= 1;
        // wave-uniform and written by an earlier kernel: read through the constant address space so that it is a
        // scalar load, which stays out of the vector memory counter the k-loop's waits are built on
        tile_big = ((const __attribute__((address_space(4))) int*)(uintptr_t)big)[r0 >> 8];
        if ((threadIdx.x >> 6) == 0) global_to_lds16(rowf + r0 + 4 * (int)(threadIdx.x & 63), rowf_lds + rslot * 256);
    }

    template <class Cfg>
    __device__ void tile(v16f (&acc)[Cfg::TM][Cfg::TN], int r0, int c0, const AccCoords<Cfg>& co,
                         uint8_t*, int lane) {
        if (tile_big) tile_impl<Cfg, true>(acc, r0, c0, co, lane);
        else tile_impl<Cfg, false>(acc, r0, c0, co, lane);
    }
    template <class Cfg, bool SAT>
    __device__ __forceinline__ void tile_impl(v16f (&acc)[Cfg::TM][Cfg::TN], int r0, int c0, const AccCoords<Cfg>& co, int lane) {
        static_assert(Cfg::BM == kPanelRows && Cfg::BN == kPanelRows && Cfg::WTM == 64 && Cfg::WTN == 128,
                      "the panel stores assume a 256 x 256 tile of 64 x 128 wave tiles");
        const int h = lane >> 5, j = lane & 31;
        const float* tab = lds_table();
        const int wr = co.wave_row0 >> 6, wc = co.wave_col0 >> 7;
        // row = vocabulary column of this lane, 16 bytes = 16 tokens of one (tm, h) group
        uint8_t* dw_base = dw_panel + ((int64_t)(c0 >> 8) * nkt + (r0 >> 7) + (wr >> 1)) * kPanelBytes;
        const uint32_t dw_lane = (uint32_t)((128 * wc + j) * 128 + 64 * (wr & 1) + 16 * h);
        // Batches of 8 accumulator registers (registers 4g ..+3 of two MFMA tiles of one row block), software-
        // pipelined by hand: index arithmetic of batch b, its 8 table reads (and the 4 row factors of a new
        // register group), then products and e5m2 packing of batch b - 1, whose reads have had the arithmetic
        // of b to return; the four 16-byte stores of a row block follow its last batch.
        static_assert(Cfg::TN == 4 && Cfg::TM == 2, "batches of two column blocks");
        constexpr int NB = Cfg::TM * 4 * 2;
        uint32_t pk[Cfg::TN][4];
        float pv[8], nv[8];
        v4f prf, nrf;
#pragma unroll
        for (int b = 0; b <= NB; ++b) {
            if (b < NB) {
                const int tm = b >> 3, g = (b >> 1) & 3, tn0 = 2 * (b & 1);
                uint32_t off[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const v16f& a = acc[tm][tn0 + (k >> 1)];
                    off[k] = tab_offsets2(pack_logits(a[4 * g + 2 * (k & 1)] * scale, a[4 * g + 2 * (k & 1) + 1] * scale));
                }
                __builtin_amdgcn_sched_barrier(0);
                if ((b & 1) == 0) nrf = *(const v4f*)(rowf_lds + rslot * 256 + co.wave_row0 + tm * 32 + 8 * g + 4 * h);
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    nv[2 * k] = tab_at(tab, off[k] & 0xffffu);
                    nv[2 * k + 1] = tab_at(tab, off[k] >> 16);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (b > 0) {
                const int q = b - 1, tm = q >> 3, g = (q >> 1) & 3, tn0 = 2 * (q & 1);
                pk[tn0][g] = f32x4_to_e5m2_sat<SAT>(prf[0] * pv[0], prf[1] * pv[1], prf[2] * pv[2], prf[3] * pv[3]);
                pk[tn0 + 1][g] = f32x4_to_e5m2_sat<SAT>(prf[0] * pv[4], prf[1] * pv[5], prf[2] * pv[6], prf[3] * pv[7]);
                if ((q & 7) == 7) {
#pragma unroll
                    for (int tn = 0; tn < Cfg::TN; ++tn)
                        *(v4i*)(dw_base + (dw_lane + tn * 4096 + tm * 32)) =
                            (v4i){(int)pk[tn][0], (int)pk[tn][1], (int)pk[tn][2], (int)pk[tn][3]};
                }
            }
#pragma unroll
            for (int k = 0; k < 8; ++k) pv[k] = nv[k];
            if ((b & 1) == 0) prf = nrf;
        }
    }
};

// Rewrites the (at most MAX_CAND) target columns of every row of the chunk with the exact gradient.
__global__ void ce_dl_fix_kernel(const float* __restrict__ lse, const float* __restrict__ saved_sigma,
                                 CandArgs ca, Softcap sc, float coef, int m_begin, int Mc, int nkt,
                                 uint8_t* __restrict__ dw_panel) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= Mc) return;
    int m = m_begin + i;
    float s_w = row_weight_sum(ca, m);
    float p_scale = expf(sc.A - lse[m]);
    for (int c = 0; c <= ca.n_predict; ++c) {
        int64_t t64 = cand_target(ca, m, c);
        if (t64 < 0 || t64 >= ca.V) continue;
        int t = (int)t64;
        float term2 = 0.0f;
        for (int k = 0; k <= ca.n_predict; ++k)
            if (cand_target(ca, m, k) == t64) term2 += cand_weight(ca, k);
        float sg = saved_sigma[(int64_t)c * ca.M + m];
        float gz = s_w * (softcap_E(sg, sc) * p_scale) - term2;
        float gx = coef * gz * sg * (1.0f - sg);
        uint8_t code = (uint8_t)(f32x2_to_e5m2_sat(gx, gx) & 0xffu);
        dw_panel[panel_offset(t, i, nkt) + dw_pos(i & 127)] = code;
    }
}

// Backward from the forward's sigma codes: the code panel (see EpiCEFwdT) of one pass becomes that
// pass's dlogits panel (vocabulary-major, tokens of a k-step in dw_pos order), dl = e5m2_sat(rowf[token] * dcode[code]):
// the same product and conversion as EpiDlStore, so the two agree bit for bit.  One workgroup moves 128 tokens x 128
// vocabulary entries: 16 KiB of one code block in, converted on the way into LDS, transposed as in
// panel_transpose_kernel, 16 KiB of one panel block out.  A code of 0 (sigma below the window) stands for a gradient of
// zero, which is exact whenever |rowf| * D(largest sigma below the window) is under half the smallest e5m2 subnormal
// (2^-17): every such product then rounds to zero in the recompute epilogue too.  Only a code of 0 inside the matrix in
// a row whose factor is larger than that puts the 256 x 256 tile it lies in on the list of tiles (each tile once:
// flags) that EpiDlStore then recomputes from the logits.  Such entries cluster in vocabulary columns (tokens
// that never occur as targets keep being pushed down), so the list stays a small part of the matrix.
// Some code of the word is 0 (a sigma below the window) in a row whose factor is too large for that to mean an exact zero.
__device__ __forceinline__ bool code_needs_logit(uint32_t w, float rf, float d_below) {
    return (((w - 0x01010101u) & ~w & 0x80808080u) != 0u) & !(fabsf(rf) * d_below < 0x1p-17f);
}

// Everything the backward needs before its first large kernel, in one launch of 256-thread workgroups; block ranges, in
// this order (a range may be empty): the table of the gradient factor; the code table; the row factors of all rows;
// zeros for the pass's tile list state; W^T as a panel; the pass's x^T as a panel; the weights in the token-stationary
// kernel's fragment order; the probe of the pass's codes.
//
// The probe looks at every `stride`-th 256 x 256 tile of the pass's codes and counts those that the conversion would
// put on the list.  If more than a given share of the sample is, the conversion is skipped and the whole panel
// recomputed from the logits (TileListIter walks the whole grid then): conversion plus the recompute of that many tiles
// would cost more than the recompute alone, so a step with codes never costs much more than one without.  Workgroup j
// of the probe takes the sampled tiles j, j + kProbeBlocks, .. and writes its own count to hits[j]: nothing to zero
// beforehand, and the readers add the kProbeBlocks counts up (probe_total).  It computes the row factors itself, with
// the expression of ce_rowf_block, since those are written by the same launch.
struct BwdPrepArgs {
    float *tabD, *dcode;
    Softcap sc;
    const float* lse;
    CandArgs ca;
    float coef;
    float* rowf;
    int* big;
    int* zero;
    int nzero;
    const uint8_t *w_f8, *x_f8;
    int K, V, nkv, m0, Mc, nkt;
    uint8_t *w_t, *x_t;
    const uint8_t* codes;
    int nkp, nbx, nvt, stride, nsample;
    int* hits;
    uint8_t* w_frag;
    int b_tab, b_dcode, b_rowf, b_zero, b_wt, b_xt, b_frag;      // workgroups of each range; the probe takes the rest
};

__device__ __forceinline__ void ce_codes_probe_block(const BwdPrepArgs& p, int b) {
    const int tid = threadIdx.x;
    const float d_below = ce_d_below_window(p.sc);
    int found = 0;
    for (int sample = b; sample < p.nsample; sample += kProbeBlocks) {
        const int idx = sample * p.stride, vt = idx % p.nvt, tt = idx / p.nvt;
        const int tok0 = p.m0 + tt * 256;
        // all loads first (branch-free), then the tests: a sample is one round trip to memory long
        const float rf = ce_row_factor(p.lse, p.ca, p.sc, p.coef, tok0 + tid);     // piece tid + 256 j of a block: group j of token tid
        v4i c[2][8];
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const int kv = min(2 * vt + q, p.nbx - 1);     // the last tile of an odd count holds one block: read it twice
            const uint8_t* src = p.codes + ((int64_t)(tok0 >> 8) * p.nkp + kv) * kPanelBytes;    // [8 groups][256 tokens] x 16 codes
#pragma unroll
            for (int j = 0; j < 8; ++j) c[q][j] = *(const v4i*)(src + (tid + 256 * j) * 16);
        }
        bool below = false;
        const bool inside = tok0 + tid < p.ca.M;
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
            for (int q = 0; q < 2; ++q)
#pragma unroll
                for (int k = 0; k < 4; ++k) below |= inside & code_needs_logit((uint32_t)c[q][j][k], rf, d_below);
        found += __syncthreads_or(below) ? 1 : 0;
    }
    if (tid == 0) p.hits[b] = found;
}

__global__ __launch_bounds__(256) void ce_bwd_prep_kernel(BwdPrepArgs p) {
    int b = blockIdx.x;
    const int tid = threadIdx.x;
    if (b < p.b_tab) { ce_table_entry(b * 256 + tid, nullptr, p.tabD, p.sc, false); return; }
    b -= p.b_tab;
    if (b < p.b_dcode) { ce_dcode_entry(tid, p.dcode, p.sc); return; }
    b -= p.b_dcode;
    if (b < p.b_rowf) { ce_rowf_block(b, p.lse, p.ca, p.sc, p.coef, p.rowf, p.big); return; }
    b -= p.b_rowf;
    if (b < p.b_zero) {
        if (b * 256 + tid < p.nzero) p.zero[b * 256 + tid] = 0;
        return;
    }
    b -= p.b_zero;
    const int ncg = (p.K + 127) / 128;      // column groups of both transposes: their columns are the K features
    if (b < p.b_wt) { panel_transpose_block<0, kPanelRaw>(p.w_f8, p.K, 0, p.V, p.K, p.nkv, 1.0f, p.w_t, b % ncg, b / ncg); return; }
    b -= p.b_wt;
    if (b < p.b_xt) { panel_transpose_block<2, kPanelRaw>(p.x_f8, p.K, p.m0, p.Mc, p.K, p.nkt, 1.0f, p.x_t, b % ncg, b / ncg); return; }
    b -= p.b_xt;
    if (b < p.b_frag) { xs_frag_from_f8(p.w_f8, p.V, p.K, p.w_frag, b, p.b_frag); return; }
    b -= p.b_frag;
    ce_codes_probe_block(p, b);
}

__global__ __launch_bounds__(256) void ce_codes_to_dl_kernel(const uint8_t* __restrict__ codes, int nkp, int m0, int M,
                                                             const float* __restrict__ rowf, const int* __restrict__ big,
                                                             const float* __restrict__ dcode,
                                                             int nkt, uint8_t* __restrict__ dl_panel, int nvt, int* __restrict__ flags,
                                                             int* __restrict__ list, int* __restrict__ count,
                                                             const int* __restrict__ probe_hits, int probe_limit) {
    constexpr int kStride = 33;
    __shared__ uint32_t tile[128 * kStride];
    __shared__ float dtab[256];
    const int kv = blockIdx.x, a = blockIdx.y, tid = threadIdx.x;
    const int tok0 = m0 + a * 128;
    const uint8_t* src = codes + ((int64_t)(tok0 >> 8) * nkp + kv) * kPanelBytes + (tok0 & 128) * 16;
    // The workgroup's codes and row factors are requested before anything else: the probe counts, the code table and
    // its barrier would otherwise put a round trip to memory in front of them (a workgroup lives only a few of those).
    v4i c[4];
    float rf[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int i = tid + 256 * j, r = i & 127, ch = i >> 7;   // 16 codes (group ch) of token tok0 + r
        c[j] = *(const v4i*)(src + ch * kCodeGroupBytes + r * 16);
        rf[j] = rowf[tok0 + r];                                   // zero past the last token
    }
    const float dcode_mine = dcode[tid], d_below = dcode[256];
    if (probe_total(probe_hits) > probe_limit) return;      // the whole panel is recomputed instead (see ce_bwd_prep_kernel)
    dtab[tid] = dcode_mine;
    __syncthreads();
    auto word_at = [&](int r, int w) -> uint32_t& { return tile[r * kStride + (w ^ (((r >> 4) & 7) << 2))]; };
    bool below = false;
    // the two 128-token halves of a 256-token block ask the same flag: no product of the block leaves the e5m2 range
    // unless it is set (see ce_rowf_block), and the conversion then needs no clamps
    const int may_saturate = ((const __attribute__((address_space(4))) int*)(uintptr_t)big)[tok0 >> 8];
    auto convert = [&](auto sat) {
        constexpr bool SAT = decltype(sat)::value;
        // per 16 codes: sixteen table reads in flight, then products, conversions, LDS writes
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = tid + 256 * j, r = i & 127, ch = i >> 7;
            float d[16];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t w = (uint32_t)c[j][k];
                d[4 * k] = dtab[w & 0xffu];
                d[4 * k + 1] = dtab[(w >> 8) & 0xffu];
                d[4 * k + 2] = dtab[(w >> 16) & 0xffu];
                d[4 * k + 3] = dtab[w >> 24];
            }
            __builtin_amdgcn_sched_barrier(0);
            const bool inside = tok0 + r < M;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                below |= inside & code_needs_logit((uint32_t)c[j][k], rf[j], d_below);
                word_at(r, ch * 4 + k) = f32x4_to_e5m2_sat<SAT>(rf[j] * d[4 * k], rf[j] * d[4 * k + 1], rf[j] * d[4 * k + 2], rf[j] * d[4 * k + 3]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    if (may_saturate) convert(std::true_type{});
    else convert(std::false_type{});
    if (__syncthreads_or(below) && tid == 0) {
        const int tt = (tok0 - m0) >> 8, vt = kv >> 1;
        if (atomicExch(&flags[tt * nvt + vt], 1) == 0) list[atomicAdd(count, 1)] = (tt << 16) | vt;
    }
    // as panel_transpose_kernel with PERM = 2: piece `sub` of a vocabulary entry's 128-byte row holds the tokens
    // 32 (sub / 2) + 8 g + 4 (sub % 2) + i at byte 4 g + i; the four code columns 4 cgp ..+3 of a thread are the
    // vocabulary entries vloc ..+3 (dw_pos order of the code panel's bytes undone)
    const int sub = tid & 7, cgp = tid >> 3;
    const int rbase = 32 * (sub >> 1) + 4 * (sub & 1);
    uint32_t w[4][4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
#pragma unroll
        for (int i = 0; i < 4; ++i) w[g][i] = word_at(rbase + 8 * g + i, cgp);
        transpose4x4_bytes(w[g]);
    }
    const int vloc = 32 * (cgp >> 3) + 8 * (cgp & 3) + 4 * ((cgp >> 2) & 1);
    uint8_t* dst = dl_panel + ((int64_t)(kv >> 1) * nkt + a) * kPanelBytes + ((kv & 1) * 128 + vloc) * 128 + sub * 16;
#pragma unroll
    for (int c = 0; c < 4; ++c) *(v4i*)(dst + c * 128) = (v4i){(int)w[0][c], (int)w[1][c], (int)w[2][c], (int)w[3][c]};
}

int gemm_store(const void* A, int fa, int64_t lda, const void* B, int fb, int64_t ldb, int R, int C, int K,
               float scale, void* out, int64_t ldc, int out_kind, hipStream_t st, int splits);
int gemm_balanced_bf16(const void* A, int fa, int64_t lda, const void* B, int fb, int64_t ldb, int layout, int R, int C, int K,
                       float scale, void* out_bf16, int64_t ldc, float* part32, int a_rows_pad, hipStream_t st,
                       const float* dscale_a = nullptr, const float* dscale_b = nullptr);
int gemm_balanced_f32(const void* A, int fa, int64_t lda, const void* B, int fb, int64_t ldb, int layout, int R, int C, int K,
                      float scale, float* out, int64_t ldc, bool accumulate, float* part32, hipStream_t st);
int64_t balanced_part_bytes(int R, int C, int K);


static Softcap make_softcap(float A, float B, float C) {
    Softcap sc;
    sc.A = A;
    sc.inv_C = 1.0f / C;
    sc.B_div_C = B * sc.inv_C;
    return sc;
}
// The tables hold the softcap exactly for |l| in [2^-12, 2^8); outside, a logit takes the entry of the nearest
// covered value, and the sum of exponentials is taken relative to the cap A without a running maximum.  Both are
// exact for constants like the reference's (A = 23, B = 5, C = 7.5) and silently wrong for others (a large C
// leaves sigma unsaturated at |l| = 256, a large A underflows exp(-A)), so every entry point checks its
// (A, B, C) here, on the host, with the kernel's own fp32 expressions:
//   * |l| < 2^-12 rounds to the same bf16 sigma as l = 0 (checked at the largest uncovered magnitude, both signs;
//     sigma is monotone in l);
//   * l >= 2^8 : bf16 sigma has reached 1 at the last covered value, l = 255;
//   * l <= -2^8: at l = -255 sigma is below 2^-36 and exp(A sigma - A) equals exp(-A) in fp32, so the summand is
//     that of sigma = 0, and the gradient there, at most coef * S_w * sigma, lies more than the whole e5m2
//     range (57344 / 2^-17 < 2^33) below any gradient entry that is itself representable: both the exact value
//     and the table's round to zero;
//   * exp(-A) is a normal fp32 number with room to spare, so neither a row's sum nor its products underflow.
static float host_bf16_round(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    u &= 0xffff0000u;
    memcpy(&f, &u, 4);
    return f;
}
static float host_bf16_value(uint32_t bits) {
    bits <<= 16;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}
static float host_sigma(float l, const Softcap& sc) {
    const float u = l * sc.inv_C + sc.B_div_C;
    return host_bf16_round(1.0f / (1.0f + expf(-u)));
}
static int check_softcap(const char* who, float A, float B, float C) {
    if (!(A > 0.0f) || !(C > 0.0f) || !std::isfinite(A) || !std::isfinite(B) || !std::isfinite(C))
        return fail(NGPT_ERANGE, "%s: softcap constants A=%g B=%g C=%g must be finite with A > 0 and C > 0", who, A, B, C);
    const Softcap sc = make_softcap(A, B, C);
    const float tiny = host_bf16_value(TAB_LO - 1), last = host_bf16_value(TAB_LO + TAB_N - 1);
    const float s0 = host_sigma(0.0f, sc);
    const char* why = nullptr;
    if (host_sigma(tiny, sc) != s0 || host_sigma(-tiny, sc) != s0) why = "logits below 2^-12 in magnitude do not round to sigma(0)";
    else if (host_sigma(last, sc) != 1.0f) why = "sigma has not reached 1 in bf16 at logit 255";
    else if (!(host_sigma(-last, sc) < 0x1p-36f) || expf(A * host_sigma(-last, sc) - A) != expf(-A))
        why = "sigma has not vanished at logit -255";
    else if (!(expf(-A) >= 0x1p-100f)) why = "exp(-A) is too small for sums of exponentials relative to the cap";
    if (why)
        return fail(NGPT_ERANGE, "%s: softcap A=%g B=%g C=%g is outside what the lookup tables cover (%s)", who, A, B, C, why);
    return NGPT_OK;
}

// grad_scale * (1/C * A) * (1/grad_s), in the reference's fp32 order
static float make_coef(float A, float C, float grad_s, float grad_scale) {
    return grad_scale * (1.0f / C * A) * (1.0f / grad_s);
}

static int check_cand(const char* who, const int64_t* targets, const float* mtp_weights, int n_predict) {
    if (!targets || !mtp_weights) return fail(NGPT_EINVAL, "%s: targets / mtp_weights are required", who);
    if (n_predict < 1 || n_predict > NGPT_MAX_PREDICT)
        return fail(NGPT_ERANGE, "%s: n_predict=%d outside [1, %d]", who, n_predict, NGPT_MAX_PREDICT);
    return NGPT_OK;
}

// One launch of the fused forward kernel for tile configuration Cfg.
template <class Cfg, bool CODES>
static int launch_ce_fwd(const GemmOperands& g, const EpiCEFwdT<CODES>& epi, hipStream_t st) {
    auto kernel = gemm_tn_kernel<Cfg, FMT_E4M3, FMT_E4M3, EpiCEFwdT<CODES>, CEJobIter>;
    constexpr int LDS = Cfg::SMEM_BYTES + EpiCEFwdT<CODES>::EXTRA_LDS;   // dynamic part; the table is static LDS
    static PerDeviceOnce configured;
    if (int e = configured.run([&] { return allow_lds(kernel, LDS); })) return e;
    int cus = num_cus();
    if (cus <= 0) return fail(NGPT_EINVAL, "lm_head CE forward: no HIP device");
    if (cus < CE_XCDS * CE_SPLITS)
        return fail(NGPT_EINVAL, "lm_head CE forward: the job walk needs at least %d compute units, the device has %d", CE_XCDS * CE_SPLITS, cus);
    int tiles_m = (g.C + Cfg::BN - 1) / Cfg::BN;
    int per_xcd = (tiles_m + CE_XCDS - 1) / CE_XCDS;
    int mg = cus * Cfg::WGS_PER_CU / (CE_XCDS * CE_SPLITS);      // token tiles in flight per XCD
    if (mg > per_xcd) mg = per_xcd;
    if (mg < 1) mg = 1;
    {
        ProfileScope prof(PROF_CE_FWD, st);
        kernel<<<CE_XCDS * CE_SPLITS * mg, Cfg::THREADS, LDS, st>>>(g, epi);
    }
    return check_launch("lm_head CE forward");
}

// The token-stationary forward (token_stationary.h) covers V % 64 == 0, K % 256 == 0, K <= XS_MAX_K; other shapes take the tile kernel.
static bool xs_eligible(int M, int K, int V) { return M > 0 && V % XS_UNIT == 0 && (K == 256 || K == 512 || K == 768 || K == 1024); }

template <int MODE, int NS>
static int launch_token_stationary(XsArgs a, hipStream_t st, int slot = -1) {
    auto kernel = token_stationary_kernel<MODE, NS>;
    // dynamic LDS: candidate targets / row factors + slab (the table is static LDS), or slab + the waves' line staging
    constexpr int HEAD = MODE >= XS_LINES ? XS_WAVES * XS_LINE_STAGE : XS_CAND_LDS + (MODE == XS_DL && NS <= 12 ? XS_WAVES * XS_LINE_STAGE : 0);
    const int LDS = HEAD + a.K * XS_TOK;
    static PerDeviceOnce configured;
    if (int e = configured.run([&] { return allow_lds(kernel, HEAD + NS * 64 * XS_TOK); })) return e;
    const int cus = num_cus();
    if (cus <= 0) return fail(NGPT_EINVAL, "token-stationary kernel: no HIP device");
    if (cus < CE_XCDS) return fail(NGPT_EINVAL, "token-stationary kernel: the job walk needs at least %d compute units, the device has %d", CE_XCDS, cus);
    // workgroups per XCD = token tiles in flight (mg) x vocabulary shares (splits); the split count that needs the
    // fewest unit-steps per workgroup wins, the smaller one on a tie (longer jobs, fewer slab loads)
    if (a.tiles_m <= 0) a.tiles_m = (a.M + XS_TOK - 1) / XS_TOK;
    const int per_xcd_slots = cus / CE_XCDS, tiles_m = a.tiles_m, per_xcd = (tiles_m + CE_XCDS - 1) / CE_XCDS;
    const int units = a.V / XS_UNIT;
    int best_splits = 1, best_mg = 1;
    int64_t best_cost = -1;
    for (int s = 1; s <= XS_MAX_SPLITS; s *= 2) {
        if (s > per_xcd_slots || s > units) break;
        int mg = per_xcd_slots / s;
        if (mg > per_xcd) mg = per_xcd;
        const int64_t cost = (int64_t)((per_xcd + mg - 1) / mg) * ((units + s - 1) / s);
        if (best_cost < 0 || cost < best_cost) { best_cost = cost; best_splits = s; best_mg = mg; }
    }
    a.splits = best_splits;
    {
        ProfileScope prof(slot >= 0 ? slot : MODE == XS_DL ? PROF_CE_DLOGITS : PROF_CE_FWD, st, slot != -2);     // -2: the caller's scope covers it
        if (MODE == XS_RELU2_EMIT && a.partial_amax && a.n_partials < CE_XCDS * best_splits * best_mg)
            return fail(NGPT_EINVAL, "fc + relu^2: %d partial maxima for %d workgroups", a.n_partials, CE_XCDS * best_splits * best_mg);
        kernel<<<CE_XCDS * best_splits * best_mg, XS_THREADS, LDS, st>>>(a);
    }
    return check_launch(MODE >= XS_LINES ? "fp8 GEMM (token-stationary)" : MODE == XS_DL ? "lm_head CE backward (dlogits, token-stationary)" : "lm_head CE forward (token-stationary)");
}

template <class Cfg, class Iter, class Epi>
static int launch_grid_kernel(const GemmOperands& g, const Epi& epi, hipStream_t st, int slot, const char* what) {
    auto kernel = gemm_tn_kernel<Cfg, FMT_E4M3, FMT_E4M3, Epi, Iter>;
    constexpr int LDS = Cfg::SMEM_BYTES + Epi::EXTRA_LDS;
    static PerDeviceOnce configured;
    if (int e = configured.run([&] { return allow_lds(kernel, LDS); })) return e;
    const int cus = num_cus();
    if (cus <= 0) return fail(NGPT_EINVAL, "no HIP device");
    int tiles = ((g.R + Cfg::BM - 1) / Cfg::BM) * ((g.C + Cfg::BN - 1) / Cfg::BN);
    int per_cu = Cfg::WGS_PER_CU > 1 ? Cfg::WGS_PER_CU : 1;
    int grid = tiles < cus * per_cu ? tiles : cus * per_cu;
    {
        ProfileScope prof(slot >= 0 ? slot : 0, st, slot >= 0);
        kernel<<<grid, Cfg::THREADS, LDS, st>>>(g, epi);
    }
    return check_launch(what);
}

// Tokens per pass of the backward: the dlogits panels of one pass take 2 * rows * V bytes of workspace.
constexpr int BWD_CHUNK_ROWS = 65536;
static int bwd_chunk_rows(int M) { return M < BWD_CHUNK_ROWS ? M : BWD_CHUNK_ROWS; }
static int64_t round256(int64_t n) { return (n + 255) / 256 * 256; }

}  // namespace ngpt

using namespace ngpt;

// ------------------------------------------------------------------------------------------------
extern "C" int ngpt_softcap_supported(float A, float B, float C) { return check_softcap("ngpt_softcap_supported", A, B, C); }

extern "C" int ngpt_ce_fwd_bwd(const void* logits_bf16, const int64_t* targets, const float* mtp_weights,
                               const int64_t* prefix_targets, const float* prefix_weight,
                               float* losses, void* grad_e5m2, int n_rows, int n_cols, int n_predict,
                               float A, float B, float C, float grad_s, float grad_scale,
                               void* workspace, int64_t workspace_bytes, void* stream) {
    if (!logits_bf16 || !losses || !grad_e5m2) return fail(NGPT_EINVAL, "ngpt_ce_fwd_bwd: null pointer");
    if (int e = check_cand("ngpt_ce_fwd_bwd", targets, mtp_weights, n_predict)) return e;
    if (int e = check_softcap("ngpt_ce_fwd_bwd", A, B, C)) return e;
    if (n_rows <= 0 || n_cols <= 0) return fail(NGPT_EINVAL, "ngpt_ce_fwd_bwd: empty logits %d x %d", n_rows, n_cols);
    if (n_cols % 8) return fail(NGPT_EALIGN, "ngpt_ce_fwd_bwd: n_cols=%d must be a multiple of 8", n_cols);
    if (!workspace || workspace_bytes < 2 * TAB_BYTES)
        return fail(NGPT_EWORKSPACE, "ngpt_ce_fwd_bwd: workspace %lld < %d bytes", (long long)workspace_bytes, 2 * TAB_BYTES);
    hipStream_t st = (hipStream_t)stream;
    Softcap sc = make_softcap(A, B, C);
    float* tabE = (float*)workspace;
    float* tabD = tabE + TAB_ENTRIES;
    ce_table_kernel<<<(TAB_ENTRIES + 255) / 256, 256, 0, st>>>(tabE, tabD, sc, false);
    CandArgs ca{targets, prefix_targets, mtp_weights, prefix_weight, n_predict, n_rows, n_cols};
    int grid = num_cus();
    if (grid <= 0) return fail(NGPT_EINVAL, "no HIP device");
    if (n_cols <= 16 * 8 * ROWREG_THREADS) {    // a row fits the registers of one workgroup
        const float coef = make_coef(A, C, grad_s, grad_scale);
        grid *= 2;
        if (grid > n_rows) grid = n_rows;
        auto launch = [&](auto kernel) {
            kernel<<<grid, ROWREG_THREADS, 0, st>>>((const uint16_t*)logits_bf16, ca, losses, (uint8_t*)grad_e5m2, tabE, tabD, sc, coef);
        };
        if (n_cols <= 4 * 8 * ROWREG_THREADS) launch(ce_rows_reg_kernel<4>);
        else if (n_cols <= 8 * 8 * ROWREG_THREADS) launch(ce_rows_reg_kernel<8>);
        else launch(ce_rows_reg_kernel<16>);
        return check_launch("ce_rows_reg_kernel");
    }
    grid *= 2;
    if (grid > n_rows) grid = n_rows;
    ce_rows_kernel<<<grid, ROW_THREADS, 0, st>>>((const uint16_t*)logits_bf16, ca, losses, (uint8_t*)grad_e5m2,
                                                 tabE, tabD, sc, make_coef(A, C, grad_s, grad_scale));
    return check_launch("ce_rows_kernel");
}

extern "C" int64_t ngpt_ce_fwd_bwd_workspace_bytes(void) { return 2 * TAB_BYTES; }

// ------------------------------------------------------------------------------------------------
// forward workspace: tabE | tabD | part [CE_SPLITS][M] | (IN_OUT only) nothing extra: the transposed
// quantiser writes w_f8_vk directly.
static int64_t fwd_base_workspace_bytes(int M) { return align_up(2 * TAB_BYTES, 256) + align_up((int64_t)CE_SPLITS * M * 4, 256); }
extern "C" int64_t ngpt_lmhead_ce_fwd_min_workspace_bytes(int M, int K, int V, int w_layout) {
    (void)K; (void)V; (void)w_layout;
    return fwd_base_workspace_bytes(M);
}
// ... | fragment-major copy of the weights (token-stationary kernel only)
extern "C" int64_t ngpt_lmhead_ce_fwd_workspace_bytes(int M, int K, int V, int w_layout) {
    (void)w_layout;
    return fwd_base_workspace_bytes(M) + (xs_eligible(M, K, V) ? align_up(xs_frag_bytes(V, K), 256) : 0);
}

namespace ngpt {
// Everything the forward's GEMM kernel starts from, in one launch.  Block ranges: [0, bx) the e4m3 copy of the
// activations; then bw blocks for the e4m3 copy of (out, in) weights, which also goes to the token-stationary kernel's
// fragment order if w_frag is given (each 8-byte piece of a row is 8 bytes of one 16-byte fragment entry, see
// xs_frag_from_f8_kernel); then b_tab blocks for the lookup tables; then the zeros of the partial sums (an empty vocabulary split must
// read as zero) and of the saved sigmas (entries of candidates without a target are never written by the kernel).
struct FwdPrepArgs {
    const v4i* x; v2i* x_f8; int64_t nx8; float x_s;
    const v4i* w; v2i* w_f8; int64_t nw8; float w_s; uint8_t* w_frag; int K8;
    int bx, bw, b_tab;
    float *tabE, *tabD; Softcap sc; bool embed_codes;
    float* zero0; int64_t n0; float* zero1; int64_t n1;
};
__global__ __launch_bounds__(256) void ce_fwd_prep_kernel(FwdPrepArgs p) {
    int b = blockIdx.x;
    const int tid = threadIdx.x;
    if (b < p.bx) {
        const QuantScale qs(p.x_s);
        for (int64_t i = (int64_t)b * 256 + tid; i < p.nx8; i += (int64_t)p.bx * 256) p.x_f8[i] = quant8<FMT_E4M3>(p.x[i], qs);
        return;
    }
    b -= p.bx;
    if (b < p.bw) {
        const QuantScale qs(p.w_s);
        for (int64_t i = (int64_t)b * 256 + tid; i < p.nw8; i += (int64_t)p.bw * 256) {
            const v2i q = quant8<FMT_E4M3>(p.w[i], qs);
            p.w_f8[i] = q;
            if (p.w_frag) {
                const int row = (int)(i / p.K8), c8 = (int)(i - (int64_t)row * p.K8);     // 8-byte piece c8 of the row
                const int u = row >> 6, tm = (row >> 5) & 1, ri = row & 31, ks = c8 >> 3, hh = (c8 >> 2) & 1, part = (c8 >> 1) & 1;
                *(v2i*)(p.w_frag + (((int64_t)u * (p.K8 >> 3) + ks) * 4 + tm * 2 + part) * 1024 + (hh * 32 + ri) * 16 + (c8 & 1) * 8) = q;
            }
        }
        return;
    }
    b -= p.bw;
    if (b < p.b_tab) {
        ce_table_entry(b * 256 + tid, p.tabE, p.tabD, p.sc, p.embed_codes);
        return;
    }
    const int64_t i = (int64_t)(b - p.b_tab) * 256 + tid;
    if (i < p.n0) p.zero0[i] = 0.0f;
    else if (i - p.n0 < p.n1) p.zero1[i - p.n0] = 0.0f;
}

bool xs_gemm_eligible(int M, int N, int K) { return xs_eligible(M, K, N); }
int64_t xs_gemm_frag_bytes(int N, int K) { return align_up(xs_frag_bytes(N, K), 256); }
int xs_gemm_make_frag(const void* w_f8, int N, int K, void* w_frag, hipStream_t st) {
    xs_frag_from_f8_kernel<<<std::min((N / XS_UNIT) * (K / 128), 8 * num_cus()), 256, 0, st>>>((const uint8_t*)w_f8, N, K, (uint8_t*)w_frag);
    return check_launch("xs_frag_from_f8_kernel");
}
static void prep_quant_blocks(FwdPrepArgs& a) {   // quantiser blocks in proportion to the sizes
    const int64_t cap = (int64_t)num_cus() * 16;
    int64_t bx = (a.nx8 + 255) / 256, bw = (a.nw8 + 255) / 256;
    if (bx + bw > cap) {
        bx = std::max<int64_t>(1, bx * cap / (bx + bw));
        bw = a.nw8 ? std::max<int64_t>(1, cap - bx) : 0;
    }
    a.bx = (int)bx;
    a.bw = (int)bw;
}
int xs_gemm_quant_pair_frag(const void* x_bf16, void* x_f8, int64_t nx, float x_s, const void* w_bf16, void* w_f8, int N, int K, float w_s,
                            void* w_frag, hipStream_t st) {
    FwdPrepArgs a{};
    a.x = (const v4i*)x_bf16; a.x_f8 = (v2i*)x_f8; a.nx8 = nx / 8; a.x_s = x_s;
    a.w = (const v4i*)w_bf16; a.w_f8 = (v2i*)w_f8; a.nw8 = (int64_t)N * K / 8; a.w_s = w_s;
    a.w_frag = (uint8_t*)w_frag;
    a.K8 = K / 8;
    prep_quant_blocks(a);
    ce_fwd_prep_kernel<<<a.bx + a.bw, 256, 0, st>>>(a);
    return check_launch("ce_fwd_prep_kernel");
}
int xs_gemm_lines(int mode, const void* x_f8, const void* w_frag, int M, int N, int K, float scale, const float* dscale,
                  void* out_bf16, int64_t ld_out, void* out_f8, int64_t ld_f8, const float* act_scale, float* partial_amax, int n_partials,
                  int slot, hipStream_t st) {
    XsArgs a{};
    a.w_frag = (const uint8_t*)w_frag;
    a.x_f8 = (const uint8_t*)x_f8;
    a.M = M; a.V = N; a.K = K;
    a.scale = scale;
    a.dscale = dscale;
    a.out = (uint16_t*)out_bf16; a.ld_out = ld_out;
    a.out_f8 = (uint8_t*)out_f8; a.ld_f8 = ld_f8;
    a.act_scale = act_scale; a.partial_amax = partial_amax; a.n_partials = n_partials;
    auto go = [&](auto ns) -> int {
        constexpr int NS = decltype(ns)::value;
        switch (mode) {
            case XS_LINES: return launch_token_stationary<XS_LINES, NS>(a, st, slot);
            case XS_RELU2: return launch_token_stationary<XS_RELU2, NS>(a, st, slot);
            case XS_RELU2_EMIT: return launch_token_stationary<XS_RELU2_EMIT, NS>(a, st, slot);
        }
        return fail(NGPT_EINVAL, "xs_gemm_lines: mode %d", mode);
    };
    switch (K / 64) {
        case 4: return go(std::integral_constant<int, 4>{});
        case 8: return go(std::integral_constant<int, 8>{});
        case 12: return go(std::integral_constant<int, 12>{});
        case 16: return go(std::integral_constant<int, 16>{});
    }
    return fail(NGPT_EINVAL, "xs_gemm_lines: K=%d", K);
}

// Forward of the fused lm_head + CE on a workspace that the caller (ngpt_lmhead_ce_fwd) or the library itself
// (ngpt_lmhead_ce_fwd_static) provides; `who` names the entry point in error messages.
static int lmhead_ce_fwd_impl(const char* who, const void* x_bf16, const void* w_bf16, const int64_t* targets,
                              const float* mtp_weights, int n_predict, const int64_t* prefix_targets, const float* prefix_weight,
                              int M, int K, int V, float x_s, float w_s, float A, float B, float C,
                              float* losses, float* lse, float* saved_sigma, void* x_f8, void* w_f8_vk,
                              int w_layout, void* workspace, int64_t workspace_bytes, void* stream, void* sigma_codes = nullptr) {
    if (!x_bf16 || !w_bf16 || !losses || !lse || !saved_sigma || !x_f8 || !w_f8_vk || !workspace)
        return fail(NGPT_EINVAL, "%s: null pointer", who);
    if (int e = check_cand(who, targets, mtp_weights, n_predict)) return e;
    if (int e = check_softcap(who, A, B, C)) return e;
    if (M <= 0 || K <= 0 || V <= 0) return fail(NGPT_EINVAL, "%s: empty problem M=%d K=%d V=%d", who, M, K, V);
    if (K % 128 || M % 16 || V % 16)
        return fail(NGPT_EALIGN, "%s: need K %% 128 == 0, M %% 16 == 0, V %% 16 == 0 (M=%d K=%d V=%d)", who, M, K, V);
    if (w_layout != NGPT_W_OUT_IN && w_layout != NGPT_W_IN_OUT) return fail(NGPT_EINVAL, "%s: w_layout=%d", who, w_layout);
    int64_t need = fwd_base_workspace_bytes(M);
    if (workspace_bytes < need)
        return fail(NGPT_EWORKSPACE, "%s: workspace %lld < %lld bytes", who, (long long)workspace_bytes, (long long)need);
    // the token-stationary kernel needs room for its copy of the weights; a workspace of the minimum size selects the tile kernel
    const bool use_xs = xs_eligible(M, K, V) && workspace_bytes >= ngpt_lmhead_ce_fwd_workspace_bytes(M, K, V, w_layout);
    hipStream_t st = (hipStream_t)stream;
    uint8_t* ws = (uint8_t*)workspace;
    float* tabE = (float*)ws;
    float* tabD = tabE + TAB_ENTRIES;
    float* part = (float*)(ws + align_up(2 * TAB_BYTES, 256));
    uint8_t* w_frag = ws + fwd_base_workspace_bytes(M);

    Softcap sc = make_softcap(A, B, C);
    {
        FwdPrepArgs a{};
        a.x = (const v4i*)x_bf16; a.x_f8 = (v2i*)x_f8; a.nx8 = (int64_t)M * K / 8; a.x_s = x_s;
        const bool w_here = w_layout == NGPT_W_OUT_IN;     // (in, out) weights go through the transposing quantiser below
        a.w = (const v4i*)w_bf16; a.w_f8 = (v2i*)w_f8_vk; a.nw8 = w_here ? (int64_t)V * K / 8 : 0; a.w_s = w_s;
        a.w_frag = (w_here && use_xs) ? w_frag : nullptr;
        a.K8 = K / 8;
        prep_quant_blocks(a);
        a.b_tab = TAB_BLOCKS;
        a.tabE = tabE; a.tabD = tabD; a.sc = sc; a.embed_codes = sigma_codes != nullptr;
        a.zero0 = part; a.n0 = (int64_t)CE_SPLITS * M;
        a.zero1 = saved_sigma; a.n1 = (int64_t)MAX_CAND * M;
        const int64_t fill_blocks = (a.n0 + a.n1 + 255) / 256;
        ce_fwd_prep_kernel<<<(int)(a.bx + a.bw + TAB_BLOCKS + fill_blocks), 256, 0, st>>>(a);
        if (int e = check_launch("ce_fwd_prep_kernel")) return e;
        if (!w_here)
            if (int e = ngpt_quant_fp8_2d(w_bf16, K, V, w_s, NGPT_FMT_E4M3, nullptr, w_f8_vk, stream)) return e;
    }

    GemmOperands g{(const uint8_t*)w_f8_vk, (const uint8_t*)x_f8, K, K, V, M, K, 1};
    const CandArgs ca{targets, prefix_targets, mtp_weights, prefix_weight, n_predict, M, V};
    auto fill = [&](auto& epi) {
        epi.gtabE = tabE;
        epi.part = part;
        epi.saved_sigma = saved_sigma;
        epi.ca = ca;
        epi.sc = sc;
        epi.scale = x_s * w_s;
        epi.ncand = prefix_targets ? n_predict + 1 : n_predict;
    };
    if (use_xs) {
        if (w_layout != NGPT_W_OUT_IN) {
            xs_frag_from_f8_kernel<<<std::min((V / XS_UNIT) * (K / 128), 8 * num_cus()), 256, 0, st>>>((const uint8_t*)w_f8_vk, V, K, w_frag);
            if (int e = check_launch("xs_frag_from_f8_kernel")) return e;
        }
        XsArgs a{};
        a.w_frag = w_frag;
        a.x_f8 = (const uint8_t*)x_f8;
        a.M = M; a.V = V; a.K = K;
        a.codes = (uint8_t*)sigma_codes;
        a.nkp = (int)(round256(V) / 128);
        a.gtabE = tabE;
        a.part = part;
        a.saved_sigma = saved_sigma;
        a.ca = ca;
        a.sc = sc;
        a.scale = x_s * w_s;
        a.ncand = prefix_targets ? n_predict + 1 : n_predict;
        int e = NGPT_EINVAL;
        switch (K / 64) {   // the contraction loop is unrolled completely: one instantiation per supported K
            case 4: e = sigma_codes ? launch_token_stationary<XS_FWD_CODES, 4>(a, st) : launch_token_stationary<XS_FWD, 4>(a, st); break;
            case 8: e = sigma_codes ? launch_token_stationary<XS_FWD_CODES, 8>(a, st) : launch_token_stationary<XS_FWD, 8>(a, st); break;
            case 12: e = sigma_codes ? launch_token_stationary<XS_FWD_CODES, 12>(a, st) : launch_token_stationary<XS_FWD, 12>(a, st); break;
            case 16: e = sigma_codes ? launch_token_stationary<XS_FWD_CODES, 16>(a, st) : launch_token_stationary<XS_FWD, 16>(a, st); break;
        }
        if (e) return e;
    } else if (sigma_codes) {
        EpiCEFwdT<true> epi{};
        fill(epi);
        epi.codes = (uint8_t*)sigma_codes;
        epi.nkp = (int)(round256(V) / 128);
        if (int e = launch_ce_fwd<MainCfg, true>(g, epi, st)) return e;
    } else {
        EpiCEFwd epi{};
        fill(epi);
        if (int e = launch_ce_fwd<MainCfg, false>(g, epi, st)) return e;
    }
    ce_finalize_kernel<<<(M + 255) / 256, 256, 0, st>>>(part, saved_sigma, ca, sc, losses, lse);
    return check_launch("ce_finalize_kernel");
}
}  // namespace ngpt

// ---- allocation-free forward -------------------------------------------------------------------
// The workspace of the forward (two lookup tables and the per-split partial sums of exponentials) for up to
// kStaticMaxRows tokens, as a file-scope device array: every GPU the library runs on holds its own copy at its own
// address until the process ends.  In host code the array's name is only a handle: its device address on the
// current GPU comes from hipGetSymbolAddress, once per device, and that pointer is what kernels are given.
constexpr int kStaticMaxRows = 65536;
constexpr int64_t kStaticBytes = (2 * TAB_BYTES + 255) / 256 * 256 + (int64_t)CE_SPLITS * kStaticMaxRows * 4;
static __device__ __align__(256) uint8_t scratch[kStaticBytes];

static std::atomic<void*> g_static_ptr[kMaxDevices];
static int static_scratch(void** out) {
    const int dev = current_device();
    if (dev < 0 || dev >= kMaxDevices) return fail(NGPT_EINVAL, "ngpt_lmhead_ce_fwd_static: no current HIP device (or its index is above %d)", kMaxDevices - 1);
    void* p = g_static_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return fail(e != hipSuccess ? (int)e : NGPT_EINVAL, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
        g_static_ptr[dev].store(p, std::memory_order_release);      // racing first calls store the same address
    }
    *out = p;
    return NGPT_OK;
}

extern "C" int ngpt_lmhead_ce_fwd(const void* x_bf16, const void* w_bf16, const int64_t* targets,
                                  const float* mtp_weights, int n_predict,
                                  const int64_t* prefix_targets, const float* prefix_weight,
                                  int M, int K, int V, float x_s, float w_s, float A, float B, float C,
                                  float* losses, float* lse, float* saved_sigma, void* x_f8, void* w_f8_vk,
                                  int w_layout, void* workspace, int64_t workspace_bytes, void* stream) {
    return lmhead_ce_fwd_impl("ngpt_lmhead_ce_fwd", x_bf16, w_bf16, targets, mtp_weights, n_predict, prefix_targets, prefix_weight,
                              M, K, V, x_s, w_s, A, B, C, losses, lse, saved_sigma, x_f8, w_f8_vk, w_layout,
                              workspace, workspace_bytes, stream);
}

extern "C" int ngpt_lmhead_ce_fwd_static_max_rows(void) { return kStaticMaxRows; }

extern "C" int ngpt_lmhead_ce_fwd_static(const void* x_bf16, const void* w_bf16, const int64_t* targets,
                                         const float* mtp_weights, int n_predict,
                                         const int64_t* prefix_targets, const float* prefix_weight,
                                         int M, int K, int V, float x_s, float w_s, float A, float B, float C,
                                         float* losses, float* lse, float* saved_sigma, void* x_f8, void* w_f8_vk,
                                         int w_layout, void* stream) {
    if (M > kStaticMaxRows)
        return fail(NGPT_ERANGE, "ngpt_lmhead_ce_fwd_static: M=%d exceeds the %d rows its built-in workspace holds; "
                    "use ngpt_lmhead_ce_fwd with a caller-provided workspace", M, kStaticMaxRows);
    void* ws = nullptr;
    if (int e = static_scratch(&ws)) return e;
    return lmhead_ce_fwd_impl("ngpt_lmhead_ce_fwd_static", x_bf16, w_bf16, targets, mtp_weights, n_predict, prefix_targets,
                              prefix_weight, M, K, V, x_s, w_s, A, B, C, losses, lse, saved_sigma, x_f8, w_f8_vk, w_layout,
                              ws, fwd_base_workspace_bytes(M), stream);      // the minimum size: always the tile kernel
}

// ------------------------------------------------------------------------------------------------
// backward workspace: tabE | tabD | rowf [M rounded up to 256] | big [same, one int per 256 rows used] | x^T panel [Kp, Mt] | W^T panel [Kp, V] | dlogits panel [Vp, Mt] |
// fp32 parts of the split tiles of dx, then of dW   (Mc = tokens per pass, Mt / Kp / Vp = Mc / K / V rounded up to 256)
static int64_t bwd_part_bytes(int64_t Mc, int64_t Mt, int K, int V) {
    return std::max(balanced_part_bytes((int)Mc, K, V), std::max(balanced_part_bytes(V, K, (int)Mt), balanced_part_bytes(K, V, (int)Mt)));
}
// codes backward: probe counts [kProbeBlocks] | count | flags [tiles] | list [tiles] of the 256 x 256 tiles of one pass's logits
static int64_t flag_bytes(int64_t Mt, int64_t Vp) { return align_up((kProbeBlocks + 1 + 2 * (Mt / 256) * (Vp / 256)) * 4, 256); }
extern "C" int64_t ngpt_lmhead_ce_bwd_workspace_bytes(int M, int K, int V, int w_layout) {
    (void)w_layout;
    int64_t Mc = bwd_chunk_rows(M), Mt = round256(Mc), Kp = round256(K), Vp = round256(V);
    return align_up(2 * TAB_BYTES, 256) + 2 * round256(M) * 4 + Kp * Mt + Kp * (int64_t)V + Vp * Mt + bwd_part_bytes(Mc, Mt, K, V) + flag_bytes(Mt, Vp) +
           (xs_eligible(M, K, V) ? align_up(xs_frag_bytes(V, K), 256) : 0);
}

extern "C" int64_t ngpt_lmhead_ce_codes_bytes(int M, int V) { return round256(M) * round256(V); }

namespace ngpt {
static int lmhead_ce_bwd_impl(const char* who, const void* x_f8, const void* w_f8_vk, const int64_t* targets,
                              const float* mtp_weights, int n_predict,
                              const int64_t* prefix_targets, const float* prefix_weight,
                              const float* lse, const float* saved_sigma, const void* sigma_codes, int M, int K, int V,
                              float x_s, float w_s, float grad_s, float grad_scale,
                              float A, float B, float C, void* dx_bf16, void* dw_f32, int w_layout,
                              void* workspace, int64_t workspace_bytes, void* stream) {
    if (!x_f8 || !w_f8_vk || !lse || !saved_sigma || !dx_bf16 || !dw_f32 || !workspace)
        return fail(NGPT_EINVAL, "%s: null pointer", who);
    if (int e = check_cand(who, targets, mtp_weights, n_predict)) return e;
    if (int e = check_softcap(who, A, B, C)) return e;
    if (M <= 0 || K <= 0 || V <= 0) return fail(NGPT_EINVAL, "%s: empty problem M=%d K=%d V=%d", who, M, K, V);
    if (K % 128 || M % 128 || V % 128)
        return fail(NGPT_EALIGN, "%s: need M, K, V multiples of 128 (M=%d K=%d V=%d)", who, M, K, V);
    if (w_layout != NGPT_W_OUT_IN && w_layout != NGPT_W_IN_OUT) return fail(NGPT_EINVAL, "%s: w_layout=%d", who, w_layout);
    int64_t need = ngpt_lmhead_ce_bwd_workspace_bytes(M, K, V, w_layout);
    if (workspace_bytes < need)
        return fail(NGPT_EWORKSPACE, "%s: workspace %lld < %lld bytes", who, (long long)workspace_bytes, (long long)need);
    hipStream_t st = (hipStream_t)stream;
    const int Mc_max = bwd_chunk_rows(M);
    const int64_t Mt_max = round256(Mc_max), Kp = round256(K), Vp = round256(V);
    uint8_t* ws = (uint8_t*)workspace;
    float* tabE = (float*)ws;
    float* tabD = tabE + TAB_ENTRIES;
    ws += align_up(2 * TAB_BYTES, 256);
    float* rowf = (float*)ws;
    ws += round256(M) * 4;
    int* big = (int*)ws;
    ws += round256(M) * 4;
    uint8_t* x_t = ws;       // x^T panel of the pass: rows = K features, contraction = tokens (dw_pos order)
    ws += Kp * Mt_max;
    uint8_t* w_t = ws;       // W^T panel: rows = K features, contraction = vocabulary
    ws += Kp * (int64_t)V;
    uint8_t* dw_panel = ws;
    ws += Vp * Mt_max;
    float* parts = (float*)ws;
    ws += bwd_part_bytes(Mc_max, Mt_max, K, V);
    int* hits = (int*)ws;                    // sampled tiles that would be listed, one count per workgroup of the probe
    int* count = hits + kProbeBlocks;        // number of listed tiles
    int* flags = count + 1;                  // per 256 x 256 tile of the pass's logits: a sigma of it lies below the code window and matters
    int* list = flags + (Mt_max / 256) * (Vp / 256);
    ws += flag_bytes(Mt_max, Vp);
    // the recompute of the logits runs on the token-stationary kernel where that covers the shape; it reads the weights
    // in fragment order
    const bool dl_xs = !sigma_codes && xs_eligible(M, K, V);
    uint8_t* w_frag = ws;
    static_assert(BWD_CHUNK_ROWS / 256 < 65536, "a list entry holds the token tile in its upper 16 bits");
    if (Vp / 256 >= 65536) return fail(NGPT_ERANGE, "%s: V=%d", who, V);

    Softcap sc = make_softcap(A, B, C);
    const float coef = make_coef(A, C, grad_s, grad_scale);
    CandArgs ca{targets, prefix_targets, mtp_weights, prefix_weight, n_predict, M, V};
    float* dcode = tabE;                     // the backward does not read tabE: its first 257 entries serve as the code table
    const int nkv = V / 128;
    const bool several = M > Mc_max;       // dw then accumulates over the passes
    if (several) fill_f32_kernel<<<(int)(((int64_t)V * K + 255) / 256), 256, 0, st>>>((float*)dw_f32, (int64_t)V * K, 0.0f);

    for (int m0 = 0; m0 < M; m0 += Mc_max) {
        const int Mc = (M - m0 < Mc_max) ? (M - m0) : Mc_max;
        const int Mt = (int)round256(Mc), nkt = Mt / 128;
        const int nvt = (int)(Vp / 256), nbx = V / 128, ntiles = (Mt / 256) * nvt;
        // a sample of a few hundred tiles decides between conversion and recompute, its stride coprime to the tiles per row
        // so that the sample walks through all vocabulary columns; the recompute of 45 % of the tiles costs what the conversion does
        int stride = std::max(1, ntiles / 300);
        while (stride > 1 && std::gcd(stride, nvt) != 1) ++stride;
        const int nsample = (ntiles + stride - 1) / stride;
        const int limit = nsample * 45 / 100;
        {   // tables, row factors and W^T with the first pass; x^T, the tile list's zeros and the probe with every pass
            BwdPrepArgs a{};
            a.tabD = tabD; a.dcode = dcode; a.sc = sc; a.lse = lse; a.ca = ca; a.coef = coef; a.rowf = rowf; a.big = big;
            a.zero = count; a.nzero = 1 + ntiles;
            a.w_f8 = (const uint8_t*)w_f8_vk; a.x_f8 = (const uint8_t*)x_f8;
            a.K = K; a.V = V; a.nkv = nkv; a.m0 = m0; a.Mc = Mc; a.nkt = nkt; a.w_t = w_t; a.x_t = x_t;
            a.codes = (const uint8_t*)sigma_codes; a.nkp = (int)(Vp / 128); a.nbx = nbx; a.nvt = nvt; a.stride = stride; a.nsample = nsample;
            a.hits = hits;
            const int ncg = (K + 127) / 128;
            const bool first = m0 == 0;
            a.b_tab = first ? TAB_BLOCKS : 0;
            a.b_dcode = (first && sigma_codes) ? 1 : 0;
            a.b_rowf = first ? (M + 255) / 256 : 0;
            a.b_zero = sigma_codes ? (a.nzero + 255) / 256 : 0;
            a.b_wt = first ? ncg * nkv : 0;
            a.b_xt = ncg * nkt;
            a.w_frag = w_frag;
            a.b_frag = (first && dl_xs) ? std::min((V / XS_UNIT) * (K / 128), 4 * num_cus()) : 0;
            const int b_probe = sigma_codes ? kProbeBlocks : 0;
            ce_bwd_prep_kernel<<<a.b_tab + a.b_dcode + a.b_rowf + a.b_zero + a.b_wt + a.b_xt + a.b_frag + b_probe, 256, 0, st>>>(a);
            if (int e = check_launch("ce_bwd_prep_kernel")) return e;
        }
        // 1. recompute the pass's logits and turn them into the e5m2 dlogits panel
        GemmOperands g{(const uint8_t*)x_f8 + (int64_t)m0 * K, (const uint8_t*)w_f8_vk, K, K, Mc, V, K, 1};
        EpiDlStore epi{};
        epi.gtabD = tabD;
        epi.rowf = rowf + m0;
        epi.big = big + (m0 >> 8);
        epi.dw_panel = dw_panel;
        epi.Mc = Mc;
        epi.V = V;
        epi.nkt = nkt;
        epi.scale = x_s * w_s;
        if (sigma_codes) {
            // 1'. the pass's dlogits panel from the forward's sigma codes; tiles with a sigma below the code window
            //     that matters (none, normally) are then redone from the logits
            ProfileScope prof(PROF_CE_DLOGITS, st);
            ce_codes_to_dl_kernel<<<dim3(nbx, nkt), 256, 0, st>>>((const uint8_t*)sigma_codes, (int)(Vp / 128), m0, M, rowf, big, dcode,
                                                                  nkt, dw_panel, nvt, flags, list, count, hits, limit);
            if (int e = check_launch("ce_codes_to_dl_kernel")) return e;
            g.tile_list = list;
            g.tile_count = count;
            g.probe_hits = hits;
            g.probe_limit = limit;
            if (int e = launch_grid_kernel<MainCfg, TileListIter>(g, epi, st, -1, "lm_head CE backward (dlogits of the listed tiles)")) return e;
        } else if (dl_xs) {
            XsArgs a{};
            a.w_frag = w_frag;
            a.x_f8 = (const uint8_t*)x_f8 + (int64_t)m0 * K;
            a.M = Mc; a.V = V; a.K = K;
            a.tiles_m = nkt;                   // every 128-token k-step of the panel, the padding's zeros included
            a.gtabE = tabD;
            a.sc = sc;
            a.scale = x_s * w_s;
            a.rowf = rowf + m0;
            a.big = big + (m0 >> 8);
            a.dl_panel = dw_panel;
            a.nkt = nkt;
            int e = NGPT_EINVAL;
            switch (K / 64) {
                case 4: e = launch_token_stationary<XS_DL, 4>(a, st); break;
                case 8: e = launch_token_stationary<XS_DL, 8>(a, st); break;
                case 12: e = launch_token_stationary<XS_DL, 12>(a, st); break;
                case 16: e = launch_token_stationary<XS_DL, 16>(a, st); break;
            }
            if (e) return e;
        } else if (int e = launch_grid_kernel<MainCfg, GridIter>(g, epi, st, PROF_CE_DLOGITS, "lm_head CE backward (dlogits)")) return e;
        // 2. exact gradient at the target columns
        ce_dl_fix_kernel<<<(Mc + 255) / 256, 256, 0, st>>>(lse, saved_sigma, ca, sc, coef, m0, Mc, nkt, dw_panel);
        if (int e = check_launch("ce_dl_fix_kernel")) return e;
        // 3. dx[pass] = dl [Mc, V] . (W^T [K, V])^T, dl read transposed from the panel
        {
            GemmSlot slot(PROF_CE_DX);
            if (int e = gemm_balanced_bf16(dw_panel, FMT_E5M2 | FMT_TRANSPOSED, 0, w_t, FMT_E4M3, 0, kBlockedB | kRowsPermuted, Mc, K, V, grad_s * w_s,
                                           (uint16_t*)dx_bf16 + (int64_t)m0 * K, K, parts, Mt, st)) return e;
        }
        // 4. dw (+)= dl^T . x over the tokens of the pass (zero padded to Mt)
        GemmSlot slot(PROF_CE_DW);
        if (w_layout == NGPT_W_OUT_IN) {   // dw [V, K] = dl^T [V, Mt] . (x^T [K, Mt])^T
            if (int e = gemm_balanced_f32(dw_panel, FMT_E5M2, 0, x_t, FMT_E4M3, 0, kBlockedA | kBlockedB, V, K, Mt, x_s * grad_s,
                                          (float*)dw_f32, K, several, parts, st)) return e;
        } else {                           // dw [K, V] = x^T [K, Mt] . (dl^T [V, Mt])^T
            if (int e = gemm_balanced_f32(x_t, FMT_E4M3, 0, dw_panel, FMT_E5M2, 0, kBlockedA | kBlockedB, K, V, Mt, x_s * grad_s,
                                          (float*)dw_f32, V, several, parts, st)) return e;
        }
    }
    return NGPT_OK;
}
}  // namespace ngpt

extern "C" int ngpt_lmhead_ce_bwd(const void* x_f8, const void* w_f8_vk, const int64_t* targets,
                                  const float* mtp_weights, int n_predict,
                                  const int64_t* prefix_targets, const float* prefix_weight,
                                  const float* lse, const float* saved_sigma, int M, int K, int V,
                                  float x_s, float w_s, float grad_s, float grad_scale,
                                  float A, float B, float C, void* dx_bf16, void* dw_f32, int w_layout,
                                  void* workspace, int64_t workspace_bytes, void* stream) {
    return lmhead_ce_bwd_impl("ngpt_lmhead_ce_bwd", x_f8, w_f8_vk, targets, mtp_weights, n_predict, prefix_targets, prefix_weight,
                              lse, saved_sigma, nullptr, M, K, V, x_s, w_s, grad_s, grad_scale, A, B, C, dx_bf16, dw_f32,
                              w_layout, workspace, workspace_bytes, stream);
}


extern "C" int ngpt_lmhead_ce_fwd_codes(const void* x_bf16, const void* w_bf16, const int64_t* targets,
                                        const float* mtp_weights, int n_predict,
                                        const int64_t* prefix_targets, const float* prefix_weight,
                                        int M, int K, int V, float x_s, float w_s, float A, float B, float C,
                                        float* losses, float* lse, float* saved_sigma, void* x_f8, void* w_f8_vk,
                                        void* sigma_codes, int w_layout, void* workspace, int64_t workspace_bytes, void* stream) {
    if (!sigma_codes) return fail(NGPT_EINVAL, "ngpt_lmhead_ce_fwd_codes: null pointer");
    return lmhead_ce_fwd_impl("ngpt_lmhead_ce_fwd_codes", x_bf16, w_bf16, targets, mtp_weights, n_predict, prefix_targets, prefix_weight,
                              M, K, V, x_s, w_s, A, B, C, losses, lse, saved_sigma, x_f8, w_f8_vk, w_layout,
                              workspace, workspace_bytes, stream, sigma_codes);
}

extern "C" int ngpt_lmhead_ce_bwd_codes(const void* x_f8, const void* w_f8_vk, const int64_t* targets,
                                        const float* mtp_weights, int n_predict,
                                        const int64_t* prefix_targets, const float* prefix_weight,
                                        const float* lse, const float* saved_sigma, const void* sigma_codes, int M, int K, int V,
                                        float x_s, float w_s, float grad_s, float grad_scale,
                                        float A, float B, float C, void* dx_bf16, void* dw_f32, int w_layout,
                                        void* workspace, int64_t workspace_bytes, void* stream) {
    if (!sigma_codes) return fail(NGPT_EINVAL, "ngpt_lmhead_ce_bwd_codes: null pointer");
    return lmhead_ce_bwd_impl("ngpt_lmhead_ce_bwd_codes", x_f8, w_f8_vk, targets, mtp_weights, n_predict, prefix_targets, prefix_weight,
                              lse, saved_sigma, sigma_codes, M, K, V, x_s, w_s, grad_s, grad_scale, A, B, C, dx_bf16, dw_f32,
                              w_layout, workspace, workspace_bytes, stream);
}
