// Epilogues for gemm_tn_kernel: what happens to a finished BM x BN fp32 accumulator tile.
#pragma once
#include "gemm_tn.h"

namespace ngpt {

// acc * scale into an fp32 matrix: plain stores, or fire-and-forget L2 atomics (no read-modify-write
// through registers) when `atomic`.  Shared by the fp32 output and by partial tiles of a split contraction.
template <class Cfg>
__device__ __forceinline__ void store_tile_f32(v16f (&acc)[Cfg::TM][Cfg::TN], float* out, int64_t ld, float scale, int R, int C,
                                               int r0, int c0, const AccCoords<Cfg>& co, bool atomic) {
    float* origin = out + ((int64_t)r0 * ld + c0);
    const uint32_t lane_off = (uint32_t)co.row_base * (uint32_t)ld + (uint32_t)co.col_base;
    const int rlim = R - r0 - co.row_base, clim = C - c0 - co.col_base;
    const bool full = (r0 + Cfg::BM <= R) && (c0 + Cfg::BN <= C);
#pragma unroll
    for (int tm = 0; tm < Cfg::TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < Cfg::TN; ++tn) {
#pragma unroll
            for (int v = 0; v < 16; v += 2) {
                const int dr = co.dr(tm, v), dc = tn * 32;
                float* pu = origin + ((int64_t)dr * ld + dc);
                float v0 = acc[tm][tn][v] * scale, v1 = acc[tm][tn][v + 1] * scale;
                if (full || (dr < rlim && dc < clim)) {
                    if (atomic) (void)__hip_atomic_fetch_add(&pu[lane_off], v0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    else pu[lane_off] = v0;
                }
                if (full || (dr + 1 < rlim && dc < clim)) {
                    if (atomic) (void)__hip_atomic_fetch_add(&pu[lane_off + (uint32_t)ld], v1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    else pu[lane_off + (uint32_t)ld] = v1;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
}

// ---------------------------------------------------------------------------------------------
// Partial results of split tiles.  A job that holds only part of its tile's contraction stores acc * scale as a whole
// BM x BN fp32 tile at part32 + slot * BM * BN (plain stores; rows / columns past the matrix edge hold whatever the
// clamped operands gave); a later pass adds a tile's parts up and writes the result (rem_tiles_kernel).  Adding
// them with device-scope atomics instead costs more than the contraction of a short split: the XCDs' L2 caches are
// not coherent with each other, so such atomics execute at the memory side.
template <class Cfg>
__device__ __forceinline__ void store_part_tile(v16f (&acc)[Cfg::TM][Cfg::TN], float* part32, int slot, float scale,
                                                const AccCoords<Cfg>& co) {
    store_tile_f32<Cfg>(acc, part32 + (int64_t)slot * (Cfg::BM * Cfg::BN), Cfg::BN, scale, Cfg::BM, Cfg::BN, 0, 0, co, false);
}

// out[r, c] = bf16(acc * scale)
struct EpiStoreBf16 {
    uint16_t* out;
    int64_t ld;
    float scale;
    int R, C;
    float* part32;       // required when the walk splits tiles: one BM x BN fp32 tile per partial job
    bool is_partial;
    int part_slot;
    // optional per-tensor scales that live in device memory (1-element fp32 buffers, both or neither): the result is
    // scaled by scale * (*dscale_a * *dscale_b), the product taken on the device, no host synchronisation
    const float* dscale_a;
    const float* dscale_b;
    static constexpr int EXTRA_LDS = 0;
    static constexpr bool NEEDS_SCRATCH = false;
    static constexpr bool JOB_END_NEEDS_SCRATCH = false;
    __device__ void partial(bool p, int slot) { is_partial = p; part_slot = slot; }
    __device__ void begin(int, int, uint8_t*) {
        if (dscale_a) {   // wave-uniform, written by an earlier kernel: scalar loads through the constant address space
            const float a = ((const __attribute__((address_space(4))) float*)(uintptr_t)dscale_a)[0];
            const float b = ((const __attribute__((address_space(4))) float*)(uintptr_t)dscale_b)[0];
            scale *= a * b;
        }
    }
    __device__ void end(uint8_t*, int, int) {}
    template <class Cfg>
    __device__ void job_begin(int) {}
    template <class Cfg>
    __device__ void job_end(int, int, const AccCoords<Cfg>&, uint8_t*) {}
    template <class Cfg>
    __device__ void tile(v16f (&acc)[Cfg::TM][Cfg::TN], int r0, int c0, const AccCoords<Cfg>& co,
                         uint8_t*, int) {
        if (is_partial) {
            store_part_tile<Cfg>(acc, part32, part_slot, scale, co);
            return;
        }
        // address = wave-uniform pointer (tile origin + the element's fixed position inside the wave
        // tile, all scalar) + ONE per-lane 32-bit offset, so no per-element address registers exist
        uint16_t* origin = out + ((int64_t)r0 * ld + c0);
        const uint32_t lane_off = (uint32_t)co.row_base * (uint32_t)ld + (uint32_t)co.col_base;
        const int rlim = R - r0 - co.row_base, clim = C - c0 - co.col_base;   // lane's element (dr, dc) exists iff dr < rlim && dc < clim
        const bool full = (r0 + Cfg::BM <= R) && (c0 + Cfg::BN <= C);
#pragma unroll
        for (int tm = 0; tm < Cfg::TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < Cfg::TN; ++tn) {
#pragma unroll
                for (int v = 0; v < 16; v += 2) {
                    const int dr = co.dr(tm, v), dc = tn * 32;
                    uint16_t* pu = origin + ((int64_t)dr * ld + dc);
                    uint32_t pk = cvt_pk_bf16(acc[tm][tn][v] * scale, acc[tm][tn][v + 1] * scale);
                    if (full || (dr < rlim && dc < clim)) pu[lane_off] = (uint16_t)pk;
                    if (full || (dr + 1 < rlim && dc < clim)) pu[lane_off + (uint32_t)ld] = (uint16_t)(pk >> 16);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
    }
};

// dpre = bf16(2 * bf16(acc) * sqrt(post)): the backward of relu(pre)^2 through the down projection, with
// relu(pre) recovered as sqrt(post) (linear_relu_square_kernel, FORWARD = False).
// The GEMM runs TRANSPOSED: tile rows = hidden units (A = W2), tile columns = tokens (B = dY), while post
// and dpre are [tokens, hidden] row-major.  A lane then owns one token and, per accumulator register
// group, four consecutive hidden units, i.e. 8 contiguous bytes of post / dpre: 32 wide loads and stores
// per wave tile instead of 128 two-byte ones.  All loads are issued before the first store (the memory
// counter retires in issue order: a load behind a store would wait for it to reach memory).
struct EpiDpre {
    uint16_t* out;          // dpre [C = tokens, R = hidden], row stride ld
    const uint16_t* post;   // same shape
    int64_t ld;
    int R, C;               // R % 8 == 0
    static constexpr int EXTRA_LDS = 32768;    // 4 KiB per wave
    static constexpr bool NEEDS_SCRATCH = false;
    static constexpr bool JOB_END_NEEDS_SCRATCH = false;
    static constexpr int TILE_STORES = 16;
    static constexpr bool DROPS_FRAGMENTS = true;   // 16 lines of post in flight next to the accumulators
    uint8_t* stage;
    bool stored_all;
    __device__ bool all_stores_issued() const { return stored_all; }
    __device__ void partial(bool, int) {}
    __device__ void begin(int, int, uint8_t* extra) {
        stage = extra + (threadIdx.x >> 6) * 4096;
        stored_all = false;
    }
    __device__ void end(uint8_t*, int, int) {}
    template <class Cfg>
    __device__ void job_begin(int) {}
    template <class Cfg>
    __device__ void job_end(int, int, const AccCoords<Cfg>&, uint8_t*) {}
    // A lane owns one token and four consecutive hidden units per register group, i.e. 8-byte pieces scattered
    // over 32 rows of post / dpre per memory instruction: issued like that, the address unit spends one cycle
    // per cache line and the epilogue takes longer than the GEMM.  Instead every 32-token x 64-hidden block
    // (4 KiB) goes through the wave's LDS region: read from post as whole 128-byte lines (16 bytes per lane),
    // picked up and replaced piece by piece, and written to dpre as whole lines again.  16-byte chunks are
    // XOR-swizzled by the row.  (LDS operations of one wave execute in order, so no waits are needed between
    // the steps; the square root is the hardware's v_sqrt_f32, 1 ulp: its result is multiplied and rounded to
    // bf16, and the reference's kernel uses an approximate square root too, triton_kernels.py:475.)
    template <class Cfg>
    __device__ void tile(v16f (&acc)[Cfg::TM][Cfg::TN], int r0, int c0, const AccCoords<Cfg>& co,
                         uint8_t*, int lane) {
        static_assert(Cfg::TM == 2 && Cfg::TN == 4 && Cfg::NWAVES * 4096 <= EXTRA_LDS, "64 x 128 wave tiles, 4 KiB of staging each");
        const int h = lane >> 5, j = lane & 31;
        const bool full = (r0 + Cfg::BM <= R) && (c0 + Cfg::BN <= C);
        stored_all = full;
        const int rd_row = lane >> 3, rd_chunk = lane & 7;
        const int n = r0 + co.wave_row0 + rd_chunk * 8;          // this lane's 8 hidden units in the line-wise steps
        v4i line[Cfg::TN][4];
        auto load_block = [&](int tn) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int m = c0 + co.wave_col0 + tn * 32 + 8 * k + rd_row;
                line[tn][k] = (full || (m < C && n < R)) ? *(const v4i*)(post + (int64_t)m * ld + n) : (v4i){0, 0, 0, 0};
            }
        };
        load_block(0);
        load_block(1);
#pragma unroll
        for (int tn = 0; tn < Cfg::TN; ++tn) {
            if (tn + 2 < Cfg::TN) load_block(tn + 2);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int row = 8 * k + rd_row;
                *(v4i*)(stage + row * 128 + ((rd_chunk ^ (row & 7)) << 4)) = line[tn][k];
            }
#pragma unroll
            for (int tm = 0; tm < Cfg::TM; ++tm)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    uint8_t* at = stage + j * 128 + (((tm * 4 + g) ^ (j & 7)) << 4) + 8 * h;
                    const v2i p = *(const v2i*)at;
                    const uint32_t p01 = (uint32_t)p.x, p23 = (uint32_t)p.y;
                    const v16f& c = acc[tm][tn];
                    const uint32_t c01 = cvt_pk_bf16(c[4 * g], c[4 * g + 1]), c23 = cvt_pk_bf16(c[4 * g + 2], c[4 * g + 3]);   // bf16(acc)
                    const float d0 = 2.0f * bf16_bits_to_f32(c01 & 0xffffu) * __builtin_amdgcn_sqrtf(bf16_bits_to_f32(p01 & 0xffffu));
                    const float d1 = 2.0f * bf16_bits_to_f32(c01 >> 16) * __builtin_amdgcn_sqrtf(bf16_bits_to_f32(p01 >> 16));
                    const float d2 = 2.0f * bf16_bits_to_f32(c23 & 0xffffu) * __builtin_amdgcn_sqrtf(bf16_bits_to_f32(p23 & 0xffffu));
                    const float d3 = 2.0f * bf16_bits_to_f32(c23 >> 16) * __builtin_amdgcn_sqrtf(bf16_bits_to_f32(p23 >> 16));
                    *(v2i*)at = (v2i){(int)cvt_pk_bf16(d0, d1), (int)cvt_pk_bf16(d2, d3)};
                }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int row = 8 * k + rd_row;
                const v4i v = *(const v4i*)(stage + row * 128 + ((rd_chunk ^ (row & 7)) << 4));
                const int m = c0 + co.wave_col0 + tn * 32 + row;
                if (full || (m < C && n < R)) *(v4i*)(out + (int64_t)m * ld + n) = v;
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
};

#ifdef NGPT_BENCH_BUILD
// Contraction-loop-only timing aid (measurement build of the library only): keeps the accumulators alive but writes
// (practically) nothing.
struct EpiDiscard {
    float* out;   // >= 4 floats; workgroup 0 leaves its shader-clock and 100 MHz wall-clock tick counts in out[2], out[3]
    static constexpr int EXTRA_LDS = 0;
    static constexpr bool NEEDS_SCRATCH = false;
    static constexpr bool JOB_END_NEEDS_SCRATCH = false;
    long long t_clk, t_wall;
    __device__ void partial(bool, int) {}
    __device__ void begin(int, int, uint8_t*) {
        t_clk = clock64();
        t_wall = wall_clock64();
    }
    __device__ void end(uint8_t*, int bid, int) {
        if (bid == 0 && threadIdx.x == 0) {
            out[2] = (float)(clock64() - t_clk);
            out[3] = (float)(wall_clock64() - t_wall);
        }
    }
    template <class Cfg>
    __device__ void job_begin(int) {}
    template <class Cfg>
    __device__ void job_end(int, int, const AccCoords<Cfg>&, uint8_t*) {}
    template <class Cfg>
    __device__ void tile(v16f (&acc)[Cfg::TM][Cfg::TN], int, int, const AccCoords<Cfg>&, uint8_t*, int) {
        float s = 0.0f;
#pragma unroll
        for (int tm = 0; tm < Cfg::TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < Cfg::TN; ++tn)
#pragma unroll
                for (int v = 0; v < 16; ++v) s += acc[tm][tn][v];
        if (s == 1.2345678e30f) out[0] = s;
    }
};
#endif  // NGPT_BENCH_BUILD

// out[r, c] (+)= acc * scale in fp32.  The += form (ACCUMULATE) uses floating-point atomics on an output the caller
// has initialised; so does a job that holds only part of its tile's contraction unless `part32` is given, in
// which case its tile goes there (store_part_tile) for a later pass to add up.
template <bool ACCUMULATE>
struct EpiStoreF32 {
    float* out;
    int64_t ld;
    float scale;
    int R, C;
    float* part32;       // nullable
    bool is_partial;
    int part_slot;
    static constexpr int EXTRA_LDS = 0;
    static constexpr bool NEEDS_SCRATCH = false;
    static constexpr bool JOB_END_NEEDS_SCRATCH = false;
    __device__ void partial(bool p, int slot) { is_partial = p; part_slot = slot; }
    __device__ void begin(int, int, uint8_t*) {}
    __device__ void end(uint8_t*, int, int) {}
    template <class Cfg>
    __device__ void job_begin(int) {}
    template <class Cfg>
    __device__ void job_end(int, int, const AccCoords<Cfg>&, uint8_t*) {}
    template <class Cfg>
    __device__ void tile(v16f (&acc)[Cfg::TM][Cfg::TN], int r0, int c0, const AccCoords<Cfg>& co,
                         uint8_t*, int) {
        if (is_partial && part32) store_part_tile<Cfg>(acc, part32, part_slot, scale, co);
        else if (ACCUMULATE || is_partial) store_tile_f32<Cfg>(acc, out, ld, scale, R, C, r0, c0, co, true);
        else store_tile_f32<Cfg>(acc, out, ld, scale, R, C, r0, c0, co, false);
    }
};

// post = bf16(max(bf16(acc * dequant), 0)^2) for a GEMM that runs TRANSPOSED (tile rows = hidden units, tile
// columns = tokens, post [tokens, hidden] row-major): a lane's four consecutive accumulator registers are
// four consecutive hidden units of one token.  Every 32-token x 64-hidden block (4 KiB) is collected in the
// wave's LDS region and written as whole 128-byte lines, 16 bytes per lane (see EpiDpre).  R % 8 == 0.
// EMIT (R % 16 == 0): also post_f8 = e4m3(min(post / act_scale, 448)), row-major like post, and the largest post of
// every workgroup in partial_amax[workgroup] (zeros in the slots past the grid).  The e4m3 block of 32 tokens x 64
// bytes takes the same LDS region after the bf16 lines have been read out of it (80-byte rows: the four-byte
// writes of 32 lanes then meet at most two per bank) and leaves as 16-byte pieces, 64 bytes per token.  Rows and
// columns past the matrix edge are copies of the last valid ones (the operand loads clamp), so the maximum needs no mask.
template <bool EMIT>
struct EpiRelu2LinesT {
    uint16_t* post;
    int64_t ld;
    const float* dequant;        // 1-element device tensor, or null for a scale of one (bf16 operands)
    int R, C;                    // R = hidden units (tile rows), C = tokens (tile columns)
    uint8_t* post_f8;            // EMIT
    int64_t ld_f8;
    const float* act_scale;      // EMIT: 1-element device tensor
    float* partial_amax;         // EMIT: n_partials entries, nullable
    int n_partials;
    static constexpr int EXTRA_LDS = 32768;
    static constexpr bool NEEDS_SCRATCH = false;
    static constexpr bool JOB_END_NEEDS_SCRATCH = false;
    static constexpr int TILE_STORES = EMIT ? 24 : 16;
    static constexpr int F8_STRIDE = 80;
    float scale, inv_act;
    uint32_t amax2;              // EMIT: running maximum of the bf16 patterns of post (all >= 0), two lanes of 16 bits
    uint8_t* stage;
    bool stored_all;
    __device__ bool all_stores_issued() const { return stored_all; }
    __device__ void partial(bool, int) {}
    __device__ void begin(int, int, uint8_t* extra) {
        scale = dequant ? *dequant : 1.0f;
        inv_act = EMIT ? 1.0f / *act_scale : 0.0f;
        amax2 = 0u;
        stage = extra + (threadIdx.x >> 6) * 4096;
        stored_all = false;
    }
    __device__ void end(uint8_t* smem, int bid, int G) {
        if (!EMIT || !partial_amax) return;
        const uint32_t top = amax2 > (amax2 << 16) ? (amax2 & 0xffff0000u) : (amax2 << 16);
        float m = wave_max(__uint_as_float(top));
        float* red = (float*)smem;
        int wave = threadIdx.x >> 6;
        if ((threadIdx.x & 63) == 0) red[wave] = m;
        wg_barrier();
        if (threadIdx.x == 0) {
            float t = 0.0f;
            for (int w = 0; w < (int)(blockDim.x >> 6); ++w) t = fmaxf(t, red[w]);
            partial_amax[bid] = t;
            for (int i = bid + G; i < n_partials; i += G) partial_amax[i] = 0.0f;
        }
    }
    template <class Cfg>
    __device__ void job_begin(int) {}
    template <class Cfg>
    __device__ void job_end(int, int, const AccCoords<Cfg>&, uint8_t*) {}
    template <class Cfg>
    __device__ void tile(v16f (&acc)[Cfg::TM][Cfg::TN], int r0, int c0, const AccCoords<Cfg>& co, uint8_t*, int lane) {
        static_assert(Cfg::TM == 2 && Cfg::TN == 4 && Cfg::NWAVES * 4096 <= EXTRA_LDS, "64 x 128 wave tiles, 4 KiB of staging each");
        typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
        const int h = lane >> 5, j = lane & 31;
        const bool full = (r0 + Cfg::BM <= R) && (c0 + Cfg::BN <= C);
        stored_all = full;
        const int rd_row = lane >> 3, rd_chunk = lane & 7;
        const int n = r0 + co.wave_row0 + rd_chunk * 8;
        // address = wave-uniform pointer (tile origin + the block's and line group's fixed position) + ONE per-lane offset
        uint16_t* origin = post + ((int64_t)c0 * ld + r0);
        const uint32_t lane_off = (uint32_t)(co.wave_col0 + rd_row) * (uint32_t)ld + (uint32_t)(co.wave_row0 + rd_chunk * 8);
        // the e4m3 block: lane -> row lane / 4 (+ 16), 16-byte piece lane % 4 of its 64 bytes
        const int f8_row = lane >> 2, f8_chunk = lane & 3;
        uint8_t* origin8 = EMIT ? post_f8 + ((int64_t)c0 * ld_f8 + r0) : nullptr;
        const uint32_t lane_off8 = EMIT ? (uint32_t)(co.wave_col0 + f8_row) * (uint32_t)ld_f8 + (uint32_t)(co.wave_row0 + f8_chunk * 16) : 0u;
        const int n8 = r0 + co.wave_row0 + f8_chunk * 16;
        // relu(bf16(x)) == bf16(relu(x)) (rounding keeps the sign, a NaN becomes 0 either way): the maximum is taken on
        // the product, which spares the canonicalising pass that a maximum on re-expanded bf16 bits needs
        auto relu2 = [&](float a0, float a1) {
            const uint32_t pre = cvt_pk_bf16(fmaxf(a0 * scale, 0.0f), fmaxf(a1 * scale, 0.0f));
            const float c0f = __uint_as_float(pre << 16), c1f = __uint_as_float(pre & 0xffff0000u);
            return cvt_pk_bf16(c0f * c0f, c1f * c1f);
        };
#pragma unroll
        for (int tn = 0; tn < Cfg::TN; ++tn) {
            uint32_t f8[EMIT ? 8 : 1];
#pragma unroll
            for (int tm = 0; tm < Cfg::TM; ++tm)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const v16f& a = acc[tm][tn];
                    const uint32_t p01 = relu2(a[4 * g], a[4 * g + 1]), p23 = relu2(a[4 * g + 2], a[4 * g + 3]);
                    *(v2i*)(stage + j * 128 + (((tm * 4 + g) ^ (j & 7)) << 4) + 8 * h) = (v2i){(int)p01, (int)p23};
                    if constexpr (EMIT) {
                        amax2 = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2, amax2), __builtin_bit_cast(u16x2, p01)));
                        amax2 = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2, amax2), __builtin_bit_cast(u16x2, p23)));
                        const float q0 = fminf(__uint_as_float(p01 << 16) * inv_act, 448.0f), q1 = fminf(__uint_as_float(p01 & 0xffff0000u) * inv_act, 448.0f);
                        const float q2 = fminf(__uint_as_float(p23 << 16) * inv_act, 448.0f), q3 = fminf(__uint_as_float(p23 & 0xffff0000u) * inv_act, 448.0f);
                        int r = __builtin_amdgcn_cvt_pk_fp8_f32(q0, q1, __builtin_bit_cast(int, q0), false);
                        f8[tm * 4 + g] = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(q2, q3, r, true);
                    }
                    if (g & 1) __builtin_amdgcn_sched_barrier(0);   // keep the arithmetic next to its LDS write (registers)
                }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int row = 8 * k + rd_row;
                const v4i v = *(const v4i*)(stage + row * 128 + ((rd_chunk ^ (row & 7)) << 4));
                const int m = c0 + co.wave_col0 + tn * 32 + row;
                if (full || (m < C && n < R)) *(v4i*)(origin + (int64_t)(tn * 32 + 8 * k) * ld + lane_off) = v;
            }
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (EMIT) {
                // hidden units 32 tm + 8 g + 4 h ..+3 of token j: dword 8 tm + 2 g + h of the token's 64 bytes
#pragma unroll
                for (int d = 0; d < 8; ++d) *(uint32_t*)(stage + j * F8_STRIDE + (2 * d + h) * 4) = f8[d];
#pragma unroll
                for (int k = 0; k < 2; ++k) {
                    const int row = 16 * k + f8_row;
                    const v4i v = *(const v4i*)(stage + row * F8_STRIDE + f8_chunk * 16);
                    const int m = c0 + co.wave_col0 + tn * 32 + row;
                    if (full || (m < C && n8 < R)) *(v4i*)(origin8 + (int64_t)(tn * 32 + 16 * k) * ld_f8 + lane_off8) = v;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
};
using EpiRelu2Lines = EpiRelu2LinesT<false>;

}  // namespace ngpt
