// Epilogues for gemm_tn_kernel: what happens to a finished BM x BN fp32 accumulator tile.
#pragma once
#include "gemm_tn.h"

namespace ngpt {

// ---------------------------------------------------------------------------------------------
// Staged byte stores.  An fp8 result tile cannot be written straight from the MFMA register
// layout (a lane owns one column and scattered rows: 1-byte or 4-byte pieces per row), so the
// wave parks a strip in its private LDS scratch and writes it back out in 16-byte pieces.

// Strip = 32 rows x WTN columns of bytes in the wave's LDS scratch, rows padded where the scratch allows it
// (fewer bank conflicts on the 16-byte reads).
template <class Cfg>
struct StripU8 {
    static constexpr int STRIDE = (32 * (Cfg::WTN + 16) <= Cfg::WAVE_SCRATCH) ? Cfg::WTN + 16 : Cfg::WTN;
    static_assert(32 * STRIDE <= Cfg::WAVE_SCRATCH, "strip does not fit the wave's LDS scratch");
    // byte of accumulator element (tn, v) of the strip's tm
    static __device__ __forceinline__ void put(uint8_t* scratch, int lane, int tn, int v, uint32_t code) {
        const int rl = 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        scratch[rl * STRIDE + tn * 32 + (lane & 31)] = (uint8_t)code;
    }
};
// The strip, complete in LDS, to global memory: row-major with leading dimension ld, 16 bytes per lane.
template <class Cfg>
__device__ __forceinline__ void strip_flush_rowmajor_u8(uint8_t* scratch, int lane, uint8_t* out, int64_t ld,
                                                        int grow0 /* global row of strip row 0 */, int gcol0, int R, int C) {
    constexpr int STRIDE = StripU8<Cfg>::STRIDE;
    __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): the wave's own LDS writes have landed
    constexpr int CH_PER_ROW = Cfg::WTN / 16;
#pragma unroll
    for (int p = 0; p < Cfg::WTN / 32; ++p) {
        int id = p * 64 + lane;
        int rl = id / CH_PER_ROW, ch = id % CH_PER_ROW;
        v4i val = *(const v4i*)(scratch + rl * STRIDE + ch * 16);
        int gr = grow0 + rl, gc = gcol0 + ch * 16;
        if (gr < R && gc + 16 <= C) *(v4i*)(out + (int64_t)gr * ld + gc) = val;
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
}

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
struct EpiRelu2Lines {
    uint16_t* post;
    int64_t ld;
    const float* dequant;        // 1-element device tensor, or null for a scale of one (bf16 operands)
    int R, C;                    // R = hidden units (tile rows), C = tokens (tile columns)
    static constexpr int EXTRA_LDS = 32768;
    static constexpr bool NEEDS_SCRATCH = false;
    static constexpr bool JOB_END_NEEDS_SCRATCH = false;
    static constexpr int TILE_STORES = 16;
    float scale;
    uint8_t* stage;
    bool stored_all;
    __device__ bool all_stores_issued() const { return stored_all; }
    __device__ void partial(bool, int) {}
    __device__ void begin(int, int, uint8_t* extra) {
        scale = dequant ? *dequant : 1.0f;
        stage = extra + (threadIdx.x >> 6) * 4096;
        stored_all = false;
    }
    __device__ void end(uint8_t*, int, int) {}
    template <class Cfg>
    __device__ void job_begin(int) {}
    template <class Cfg>
    __device__ void job_end(int, int, const AccCoords<Cfg>&, uint8_t*) {}
    template <class Cfg>
    __device__ void tile(v16f (&acc)[Cfg::TM][Cfg::TN], int r0, int c0, const AccCoords<Cfg>& co, uint8_t*, int lane) {
        static_assert(Cfg::TM == 2 && Cfg::TN == 4 && Cfg::NWAVES * 4096 <= EXTRA_LDS, "64 x 128 wave tiles, 4 KiB of staging each");
        const int h = lane >> 5, j = lane & 31;
        const bool full = (r0 + Cfg::BM <= R) && (c0 + Cfg::BN <= C);
        stored_all = full;
        const int rd_row = lane >> 3, rd_chunk = lane & 7;
        const int n = r0 + co.wave_row0 + rd_chunk * 8;
        // address = wave-uniform pointer (tile origin + the block's and line group's fixed position) + ONE per-lane offset
        uint16_t* origin = post + ((int64_t)c0 * ld + r0);
        const uint32_t lane_off = (uint32_t)(co.wave_col0 + rd_row) * (uint32_t)ld + (uint32_t)(co.wave_row0 + rd_chunk * 8);
        // relu(bf16(x)) == bf16(relu(x)) (rounding keeps the sign, a NaN becomes 0 either way): the maximum is taken on
        // the product, which spares the canonicalising pass that a maximum on re-expanded bf16 bits needs
        auto relu2 = [&](float a0, float a1) {
            const uint32_t pre = cvt_pk_bf16(fmaxf(a0 * scale, 0.0f), fmaxf(a1 * scale, 0.0f));
            const float c0f = __uint_as_float(pre << 16), c1f = __uint_as_float(pre & 0xffff0000u);
            return (int)cvt_pk_bf16(c0f * c0f, c1f * c1f);
        };
#pragma unroll
        for (int tn = 0; tn < Cfg::TN; ++tn) {
#pragma unroll
            for (int tm = 0; tm < Cfg::TM; ++tm)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const v16f& a = acc[tm][tn];
                    *(v2i*)(stage + j * 128 + (((tm * 4 + g) ^ (j & 7)) << 4) + 8 * h) =
                        (v2i){relu2(a[4 * g], a[4 * g + 1]), relu2(a[4 * g + 2], a[4 * g + 3])};
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
        }
    }
};

// post = bf16(max(bf16(acc * *dequant), 0)^2); optionally post_f8 = e4m3(min(post / act_scale, 448))
// and a per-workgroup running max of post written to partial_amax[bid].
template <bool EMIT>      // EMIT: also the e4m3 copy of post and the per-workgroup maxima
struct EpiRelu2T {
    uint16_t* post;
    int64_t ld;
    const float* dequant;        // 1-element device tensor
    uint8_t* post_f8;            // EMIT only
    int64_t ld_f8;
    const float* act_scale;      // 1-element device tensor, EMIT only
    float* partial_amax;         // EMIT only; n_partials entries
    int n_partials;
    int R, C;
    float scale, inv_act, amax;
    static constexpr int EXTRA_LDS = 0;
    static constexpr bool NEEDS_SCRATCH = EMIT;     // the e4m3 strip is staged through the free operand slot
    static constexpr bool JOB_END_NEEDS_SCRATCH = false;
    template <class Cfg>
    __device__ void job_begin(int) {}
    template <class Cfg>
    __device__ void job_end(int, int, const AccCoords<Cfg>&, uint8_t*) {}
    __device__ void partial(bool, int) {}
    __device__ void begin(int, int, uint8_t*) {
        scale = *dequant;
        inv_act = EMIT ? 1.0f / *act_scale : 0.0f;
        amax = 0.0f;
    }
    template <class Cfg>
    __device__ void tile(v16f (&acc)[Cfg::TM][Cfg::TN], int r0, int c0, const AccCoords<Cfg>& co,
                         uint8_t* scratch, int lane) {
        // address = wave-uniform pointer + ONE per-lane 32-bit offset, as in EpiStoreBf16
        uint16_t* origin = post + ((int64_t)r0 * ld + c0);
        const uint32_t lane_off = (uint32_t)co.row_base * (uint32_t)ld + (uint32_t)co.col_base;
        const int rlim = R - r0 - co.row_base, clim = C - c0 - co.col_base;
        const bool full = (r0 + Cfg::BM <= R) && (c0 + Cfg::BN <= C);
#pragma unroll
        for (int tm = 0; tm < Cfg::TM; ++tm) {
#pragma unroll
            for (int tn = 0; tn < Cfg::TN; ++tn) {
#pragma unroll
                for (int v = 0; v < 16; v += 2) {
                    const int dr = co.dr(tm, v), dc = tn * 32;
                    // c = bf16(acc * dequant); post = bf16(max(c, 0)^2): both roundings by the packed converter
                    // (the maximum on the product: relu(bf16(x)) == bf16(relu(x)), see EpiRelu2Lines)
                    const uint32_t pre = cvt_pk_bf16(fmaxf(acc[tm][tn][v] * scale, 0.0f), fmaxf(acc[tm][tn][v + 1] * scale, 0.0f));
                    const float c0f = __uint_as_float(pre << 16), c1f = __uint_as_float(pre & 0xffff0000u);
                    const uint32_t pk = cvt_pk_bf16(c0f * c0f, c1f * c1f);
                    uint16_t* pu = origin + ((int64_t)dr * ld + dc);
                    const bool ok0 = full || (dr < rlim && dc < clim), ok1 = full || (dr + 1 < rlim && dc < clim);
                    if (ok0) pu[lane_off] = (uint16_t)pk;
                    if (ok1) pu[lane_off + (uint32_t)ld] = (uint16_t)(pk >> 16);
                    if (EMIT) {
                        const float p0 = __uint_as_float(pk << 16), p1 = __uint_as_float(pk & 0xffff0000u);
                        StripU8<Cfg>::put(scratch, lane, tn, v, f32_to_e4m3_sat(fminf(p0 * inv_act, 448.0f)));
                        StripU8<Cfg>::put(scratch, lane, tn, v + 1, f32_to_e4m3_sat(fminf(p1 * inv_act, 448.0f)));
                        amax = ok0 ? fmaxf(amax, p0) : amax;
                        amax = ok1 ? fmaxf(amax, p1) : amax;
                    }
                }
                if (!EMIT) __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (EMIT)
                strip_flush_rowmajor_u8<Cfg>(scratch, lane, post_f8, ld_f8, r0 + co.wave_row0 + tm * 32, c0 + co.wave_col0, R, C);
        }
    }
    __device__ void end(uint8_t* smem, int bid, int G) {
        if (!EMIT || !partial_amax) return;
        float m = wave_max(amax);
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
};


}  // namespace ngpt
