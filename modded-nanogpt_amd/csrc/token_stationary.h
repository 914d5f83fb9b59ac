// Fused lm_head + softcapped CE, token-stationary kernel (included by ce.hip): the forward (XS_FWD, XS_FWD_CODES) and the
// backward's logits recompute that writes the e5m2 gradient panel (XS_DL).  The same contraction loop also serves plain
// fp8 GEMMs with a row-major bf16 output [tokens, N] whose rows are written as whole 128-byte lines: XS_LINES
// (bf16(acc * scale): nanogpt::mm forward), XS_RELU2 and XS_RELU2_EMIT (the FP8 c_fc with its ReLU^2 epilogue, see
// EpiRelu2LinesT); there "vocabulary" reads "output features".
//
// Same arithmetic as EpiCEFwdT / EpiDlStore on gemm_tn_kernel (rows = vocabulary, columns = tokens, 32x32x64 fp8 MFMAs over the
// contraction in ascending order, softcap through the bf16-indexed table), different data movement:
//   * a job = 128 tokens x one share of the vocabulary.  The tokens' fp8 activations (128 x K bytes) are loaded into
//     LDS ONCE per job and stay there; only the weights stream.
//   * the eight waves of the workgroup are independent inside a job.  A wave takes 64 vocabulary rows x 128 tokens at
//     a time (a "unit": 2 x 4 MFMA tiles, 128 accumulator registers) and reads the weights of ITS rows straight from
//     global memory into MFMA operand registers, a few steps ahead of their use -- no other wave needs them, so they
//     never pass through LDS and the contraction loop has no workgroup barrier at all.
//   * nothing keeps the two waves that share a SIMD in step, and the one in its contraction loop has the higher
//     priority: while one of them runs the table epilogue of its unit on the vector pipe and the LDS gather path, the
//     other one feeds the matrix pipe, which an eight-wave lockstep tile leaves idle for the whole epilogue.
//
// Weights are read in "fragment-major" order, written by the quantiser next to the row-major fp8 copy:
//   [V / 64 units][K / 64 steps][2 row blocks][2 parts][64 lanes][16 bytes]
// lane 32 h + i of (unit u, step s, row block t, part p) holds W[64 u + 32 t + i][64 s + 32 h + 16 p ..+15], so each
// wave-level 16-byte load reads 1 KiB of consecutive addresses and leaves every lane with exactly the bytes the MFMA
// wants from it (row i of the tile, contraction bytes 64 s + 32 h ..+31).
//
// Requirements (checked by the host): V % 64 == 0, K % 256 == 0, the token slab + tables fit LDS (K <= 1024).
#pragma once

namespace ngpt {

constexpr int XS_TOK = 128;                 // tokens per job
constexpr int XS_UNIT = 64;                 // vocabulary rows per unit
constexpr int XS_WAVES = 8;
constexpr int XS_THREADS = XS_WAVES * 64;
constexpr int XS_BDEPTH = 1;                // token fragments are read from LDS this many MFMA pairs ahead
constexpr int XS_CAND_LDS = (MAX_CAND * XS_TOK * 4 + 1023) / 1024 * 1024;
constexpr int XS_MAX_K = 1024;
constexpr int XS_MAX_SPLITS = CE_SPLITS;    // part[] has CE_SPLITS slots per token

__host__ __device__ inline int64_t xs_frag_bytes(int V, int K) { return (int64_t)V * K; }

enum { XS_FWD = 0, XS_FWD_CODES = 1, XS_DL = 2, XS_LINES = 3, XS_RELU2 = 4, XS_RELU2_EMIT = 5 };
constexpr int XS_LINE_STAGE = 4096;         // XS_LINES..: LDS bytes per wave for turning accumulator registers into whole lines

struct XsArgs {
    const uint8_t* w_frag;   // fragment-major weights
    const uint8_t* x_f8;     // [M, K] row-major
    int M, V, K;
    int tiles_m;             // 128-token tiles to walk: M / 128 rounded up (XS_DL: up to the panel's token padding)
    int splits;              // vocabulary shares per token tile (<= XS_MAX_SPLITS)
    uint8_t* codes;          // CODES: code panel (see EpiCEFwdT)
    int nkp;
    const float* gtabE;
    float* part;             // [CE_SPLITS][M]
    float* saved_sigma;      // [MAX_CAND][M]
    CandArgs ca;
    Softcap sc;
    float scale;
    int ncand;
    // XS_DL (gtabE then is the table of the gradient factor): see EpiDlStore
    const float* rowf;       // row factors, zero past the last token up to the panel's padding
    const int* big;          // per 256 tokens: a product may leave the e5m2 range
    uint8_t* dl_panel;       // [V / 256 rounded up][nkt] blocks of 256 vocabulary rows x 128 tokens
    int nkt;
    // XS_LINES, XS_RELU2, XS_RELU2_EMIT
    uint16_t* out;           // bf16 [M, ld_out]
    int64_t ld_out;
    const float* dscale;     // nullable: one more factor of the scale, read from device memory
    uint8_t* out_f8;         // XS_RELU2_EMIT: e4m3(min(out / *act_scale, 448)), [M, ld_f8]
    int64_t ld_f8;
    const float* act_scale;
    float* partial_amax;     // XS_RELU2_EMIT: largest output of every workgroup, zeros up to n_partials; nullable
    int n_partials;
};

template <int MODE, int NS /* K / 64 */>
__global__ __launch_bounds__(XS_THREADS, 1) void token_stationary_kernel(XsArgs p) {
    constexpr bool CODES = MODE == XS_FWD_CODES, DL = MODE == XS_DL, LINES = MODE >= XS_LINES, EMIT = MODE == XS_RELU2_EMIT;
    // XS_DL: the gradient bytes pass through the waves' line staging where LDS has room for it beside slab and table
    constexpr bool DL_STAGED = DL && NS <= 12;
    // weight fragment sets in registers (loads run XS_RING - 1 steps ahead); must divide the number of steps
    constexpr int XS_RING = 4;
    static_assert(NS % XS_RING == 0, "ring slots of a unit's first steps");
    extern __shared__ __attribute__((aligned(1024))) uint8_t xs_smem[];
    int* const cand = (int*)xs_smem;                  // [MAX_CAND][XS_TOK] valid target column of the job's tokens, else -1
    uint8_t* const xslab = xs_smem + (LINES ? 0 : XS_CAND_LDS);     // [K / 128][128 tokens][128 bytes], chunks swizzled as in gemm_tn.h
    const float* tab = nullptr;
    if constexpr (!LINES) {
        tab = lds_table();
        load_table(lds_table(), p.gtabE);
    }

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int M = p.M, K = p.K;
    // XS_LINES.., XS_DL (staged): the wave's staging block behind the slab; scale and running maximum of the ReLU^2 modes
    uint8_t* const line_stage = xslab + K * XS_TOK + wave * XS_LINE_STAGE;
    float line_scale = p.scale, inv_act = 0.0f;
    uint32_t amax2 = 0u;
    if constexpr (LINES) {
        if (p.dscale) line_scale *= ((const __attribute__((address_space(4))) float*)(uintptr_t)p.dscale)[0];
        if constexpr (EMIT) inv_act = 1.0f / ((const __attribute__((address_space(4))) float*)(uintptr_t)p.act_scale)[0];
    }
    const int64_t unit_bytes = (int64_t)K * XS_UNIT;

    // job walk: XCD x owns a contiguous block of token tiles, mg of them in flight, each shared by `splits` workgroups
    const int bid = blockIdx.x, G = gridDim.x;
    const int tiles_m = p.tiles_m, units = p.V / XS_UNIT;
    const int xcd = bid % CE_XCDS, slot = bid / CE_XCDS;
    const int mg = max(G / (CE_XCDS * p.splits), 1);
    const int per_xcd = (tiles_m + CE_XCDS - 1) / CE_XCDS;
    const int split = slot / mg;
    int tile_m = xcd * per_xcd + slot % mg;
    const int tile_m_end = min(tiles_m, (xcd + 1) * per_xcd);
    const int u_begin = units * split / p.splits, u_end = units * (split + 1) / p.splits;
    if (split >= p.splits || u_begin >= u_end) tile_m = tile_m_end;


    const uint32_t xs_addr = (uint32_t)(size_t)((const __attribute__((address_space(3))) uint8_t*)xslab);

    for (; tile_m < tile_m_end; tile_m += mg) {
        const int c0 = tile_m * XS_TOK;
        wg_barrier();                                  // every wave is done with the previous job's slab and scratch
        {   // the job's activations: K / 128 sub-slabs of 128 rows x 128 bytes; a wave-level 16-byte access covers 8 rows,
            // and the chunk a lane writes at position lane % 8 of its row is global chunk (lane % 8) ^ swizzle(row).
            // (Through registers, not direct-to-LDS loads: behind those the compiler makes every later LDS read of the
            // kernel wait for all vector memory operations in flight.)
            typedef __attribute__((address_space(3))) v4i* lds_w4;
#pragma unroll
            for (int li = 0; li < 2; ++li) {
                const int ld = 2 * wave + li, row = ld * 8 + (lane >> 3);
                const int q = (lane & 7) ^ ((row >> 1) & 7);
                const uint8_t* src = p.x_f8 + (int64_t)min(c0 + row, M - 1) * K + q * 16;
                const uint32_t dst = xs_addr + (uint32_t)(ld * 1024 + lane * 16);
#pragma unroll
                for (int kc = 0; kc < NS / 2; ++kc) *(lds_w4)(uintptr_t)(dst + kc * 16384) = *(const v4i*)(src + kc * 128);
            }
            if constexpr (DL) {
                if (tid < XS_TOK) ((float*)cand)[tid] = p.rowf[c0 + tid];
            } else if constexpr (!LINES) {
                for (int i = tid; i < p.ncand * XS_TOK; i += XS_THREADS) {
                    const int c = i / XS_TOK, jj = i % XS_TOK, m = c0 + jj;
                    const int64_t t = (m < M) ? cand_target(p.ca, m, c) : -1;
                    cand[c * XS_TOK + jj] = (t >= 0 && t < p.ca.V) ? (int)t : -1;
                }
            }
            wg_barrier();
        }
        int job_big = 0;
        if constexpr (DL) job_big = ((const __attribute__((address_space(4))) int*)(uintptr_t)p.big)[c0 >> 8];

        float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        v16f acc[2][4];
        v8i a[XS_RING][2];

        // Per-lane constants (lane offsets, LDS fragment addresses) are rebuilt from the lane id at the start of every unit
        // instead of being kept in registers across the epilogue, where every register counts: a value the compiler parks
        // in scratch memory comes back through a load that waits for all the weight loads in flight.
        auto fresh_lane = [] {
            int l = lane_id();
            asm volatile("" : "+v"(l));
            return l;
        };
        auto load_step = [&](const uint8_t* step_base, uint32_t w_lane, int ring) {
#pragma unroll
            for (int tm = 0; tm < 2; ++tm) {
                const v4i lo = *(const v4i*)(step_base + (tm * 2) * 1024 + w_lane);
                const v4i hi = *(const v4i*)(step_base + (tm * 2 + 1) * 1024 + w_lane);
                a[ring][tm] = (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            }
        };
        // token fragment of column block tn, step s of the quad whose four chunk addresses are bq[]: everything but
        // bq is a compile-time constant and lands in the offset field of the LDS read
        typedef const __attribute__((address_space(3))) v4i* lds_v4i;
        auto bfrag = [&](const uint32_t (&bq)[4], int tn, int s) -> v8i {
            const uint32_t c = (uint32_t)((s >> 1) * 16384 + tn * 4096);      // step s of the unit: sub-slab s / 2
            const v4i lo = *(lds_v4i)(uintptr_t)(bq[2 * (s & 1)] + c);
            const v4i hi = *(lds_v4i)(uintptr_t)(bq[2 * (s & 1) + 1] + c);
            return (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        };

        int u = u_begin + wave;
        if (u < u_end) {
            const uint8_t* w0 = p.w_frag + (int64_t)u * unit_bytes;
#pragma unroll
            for (int s = 0; s < XS_RING - 1; ++s) load_step(w0 + s * 4096, (uint32_t)lane * 16u, s);
        }
        for (; u < u_end; u += XS_WAVES) {
            const uint8_t* wcur = p.w_frag + (int64_t)u * unit_bytes;
            // steps past the unit's end belong to this wave's next unit (none left: the current one again, unused)
            const uint8_t* wnext = (u + XS_WAVES < u_end) ? wcur + XS_WAVES * unit_bytes : wcur;
            __builtin_amdgcn_s_setprio(2);     // the wave that feeds the matrix pipe goes first (measured: 3 % of the kernel)
            // The unit's K / 64 steps as straight-line code, ring slots and LDS offsets as compile-time constants.  Step
            // ks first sends off the loads of step ks + 3 (the unit's last steps: of the next unit's first steps) into
            // the slot that step ks - 1 has just finished with.
            const int kl = fresh_lane();
            const uint32_t w_lane = (uint32_t)kl * 16u;
            // token fragment of MFMA column block tn: 16-byte chunks 2h, 2h + 1 of the 64-byte half (step & 1) of the
            // 128-byte row 32 tn + j; the swizzle term of that row does not depend on tn
            const int fb0 = (kl & 31) * 128 + (((2 * (kl >> 5)) ^ (((kl & 31) >> 1) & 7)) << 4);
            uint32_t bq[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                bq[v] = xs_addr + (uint32_t)(fb0 ^ ((v >> 1) * 64) ^ ((v & 1) * 16));
                asm volatile("" : "+v"(bq[v]));     // keeps the compiler from folding the reads' constants into scalar bases instead of offset fields
            }
            // Token fragments run XS_BDEPTH MFMA pairs ahead of their use through a ring of XS_BDEPTH + 1 register sets: the
            // LDS is shared with the table gathers of the waves that are in their epilogue, and a read that is issued
            // only one pair ahead comes back too late.  Pair p = 4 ks + tn.
            constexpr int NP = 4 * NS;
            v8i b[XS_BDEPTH + 1];
#pragma unroll
            for (int pp = 0; pp < XS_BDEPTH; ++pp) b[pp] = bfrag(bq, pp & 3, pp >> 2);
#pragma unroll
            for (int pr = 0; pr < NP; ++pr) {
                const int ks = pr >> 2, tn = pr & 3;
                if (tn == 0) {
                    constexpr int AHEAD = XS_RING - 1;
                    if (ks + AHEAD >= NS) load_step(wnext + (ks + AHEAD - NS) * 4096, w_lane, (ks + AHEAD) % XS_RING);
                    else load_step(wcur + (ks + AHEAD) * 4096, w_lane, (ks + AHEAD) % XS_RING);
                }
                if (pr + XS_BDEPTH < NP) b[(pr + XS_BDEPTH) % (XS_BDEPTH + 1)] = bfrag(bq, (pr + XS_BDEPTH) & 3, (pr + XS_BDEPTH) >> 2);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int tm = 0; tm < 2; ++tm) {
                    const v16f zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                    // XS_DL: operands swapped, so that a lane owns a vocabulary row and its registers hold tokens
                    if constexpr (DL)
                        acc[tm][tn] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                            b[pr % (XS_BDEPTH + 1)], a[ks % XS_RING][tm], ks == 0 ? zero : acc[tm][tn], 0, 0, 0, 0, 0, 0);
                    else
                        acc[tm][tn] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                            a[ks % XS_RING][tm], b[pr % (XS_BDEPTH + 1)], ks == 0 ? zero : acc[tm][tn], 0, 0, 0, 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            __builtin_amdgcn_s_setprio(0);

            const int el = fresh_lane();
            const int j = el & 31, h = el >> 5;
            if constexpr (DL) {
                // ---- epilogue of the unit: dl = e5m2_sat(rowf[token] * D(logit)) into the panel (as EpiDlStore::tile).  A lane
                // owns vocabulary row 32 tm + j of the unit; registers 4 g ..+3 of acc[tm][tn] are the tokens
                // 32 tn + 8 g + 4 h ..+3, i.e. the four bytes at position 16 h + 4 g of token group tn of that row.
                uint8_t* dl_base = p.dl_panel + ((int64_t)(u >> 2) * p.nkt + (c0 >> 7)) * kPanelBytes + (u & 3) * (XS_UNIT * 128);
                const uint32_t dl_lane = (uint32_t)(j * 128 + 16 * h);
                const uint32_t rf_addr = (uint32_t)(size_t)((const __attribute__((address_space(3))) uint8_t*)cand) + 16 * h;
                auto run = [&](auto sat) {
                    constexpr bool SAT = decltype(sat)::value;
                    constexpr int NB = 16;
                    if constexpr (DL_STAGED) {
                        // batch b: vocabulary block b / 8, token block b / 2 % 4, registers 8 (b % 2) ..+7 (two groups of four
                        // tokens).  The block's 32 rows x 128 bytes are collected in the wave's LDS block (16-byte pieces
                        // swizzled by the row) and leave as whole 128-byte rows: a 64-lane store then touches 8 lines
                        // instead of 64, which is what the address unit charges for.
                        uint8_t* const stage = line_stage;
                        const int rd_row = el >> 3, rd_chunk = el & 7;
                        float pv[8], nv[8];
                        v4f prf[2], nrf[2];
#pragma unroll
                        for (int b = 0; b <= NB; ++b) {
                            if (b < NB) {
                                const int tm = b >> 3, tn = (b >> 1) & 3, gp = b & 1;
                                const v16f& r = acc[tm][tn];
                                uint32_t off[4];
#pragma unroll
                                for (int k = 0; k < 4; ++k) off[k] = tab_offsets2(pack_logits(r[8 * gp + 2 * k] * p.scale, r[8 * gp + 2 * k + 1] * p.scale));
                                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                                for (int q = 0; q < 2; ++q)
                                    nrf[q] = *(const __attribute__((address_space(3))) v4f*)(uintptr_t)(rf_addr + (32 * tn + 8 * (2 * gp + q)) * 4);
#pragma unroll
                                for (int k = 0; k < 4; ++k) {
                                    nv[2 * k] = tab_at(tab, off[k] & 0xffffu);
                                    nv[2 * k + 1] = tab_at(tab, off[k] >> 16);
                                }
                                __builtin_amdgcn_sched_barrier(0);
                            }
                            if (b > 0) {
                                const int q = b - 1, tm = q >> 3, tn = (q >> 1) & 3, gp = q & 1;
                                const uint32_t w0 = f32x4_to_e5m2_sat<SAT>(prf[0][0] * pv[0], prf[0][1] * pv[1], prf[0][2] * pv[2], prf[0][3] * pv[3]);
                                const uint32_t w1 = f32x4_to_e5m2_sat<SAT>(prf[1][0] * pv[4], prf[1][1] * pv[5], prf[1][2] * pv[6], prf[1][3] * pv[7]);
                                *(v2i*)(stage + j * 128 + (((2 * tn + h) ^ (j & 7)) << 4) + 8 * gp) = (v2i){(int)w0, (int)w1};
                                if ((q & 7) == 7) {     // the vocabulary block is complete
#pragma unroll
                                    for (int k = 0; k < 4; ++k) {
                                        const int row = 8 * k + rd_row;
                                        const v4i v = *(const v4i*)(stage + row * 128 + ((rd_chunk ^ (row & 7)) << 4));
                                        *(v4i*)(dl_base + ((tm * 32 + row) * 128 + rd_chunk * 16)) = v;
                                    }
                                }
                            }
#pragma unroll
                            for (int k = 0; k < 8; ++k) pv[k] = nv[k];
                            prf[0] = nrf[0];
                            prf[1] = nrf[1];
                        }
                        return;
                    }
                    // batch b: token block b / 4, register group b % 4, both vocabulary blocks; 16-byte stores from the registers
                    uint32_t pk[2][4];
                    float pv[8], nv[8];
                    v4f prf, nrf;
#pragma unroll
                    for (int b = 0; b <= NB; ++b) {
                        if (b < NB) {
                            const int tn = b >> 2, g = b & 3;
                            uint32_t off[4];
#pragma unroll
                            for (int k = 0; k < 4; ++k) {
                                const v16f& r = acc[k >> 1][tn];
                                off[k] = tab_offsets2(pack_logits(r[4 * g + 2 * (k & 1)] * p.scale, r[4 * g + 2 * (k & 1) + 1] * p.scale));
                            }
                            __builtin_amdgcn_sched_barrier(0);
                            nrf = *(const __attribute__((address_space(3))) v4f*)(uintptr_t)(rf_addr + (32 * tn + 8 * g) * 4);
#pragma unroll
                            for (int k = 0; k < 4; ++k) {
                                nv[2 * k] = tab_at(tab, off[k] & 0xffffu);
                                nv[2 * k + 1] = tab_at(tab, off[k] >> 16);
                            }
                            __builtin_amdgcn_sched_barrier(0);
                        }
                        if (b > 0) {
                            const int q = b - 1, tn = q >> 2, g = q & 3;
                            pk[0][g] = f32x4_to_e5m2_sat<SAT>(prf[0] * pv[0], prf[1] * pv[1], prf[2] * pv[2], prf[3] * pv[3]);
                            pk[1][g] = f32x4_to_e5m2_sat<SAT>(prf[0] * pv[4], prf[1] * pv[5], prf[2] * pv[6], prf[3] * pv[7]);
                            if (g == 3) {
#pragma unroll
                                for (int tm = 0; tm < 2; ++tm)
                                    *(v4i*)(dl_base + (dl_lane + tm * 4096 + tn * 32)) =
                                        (v4i){(int)pk[tm][0], (int)pk[tm][1], (int)pk[tm][2], (int)pk[tm][3]};
                            }
                        }
#pragma unroll
                        for (int k = 0; k < 8; ++k) pv[k] = nv[k];
                        prf = nrf;
                    }
                };
                if (job_big) run(std::true_type{});
                else run(std::false_type{});
                continue;
            }
            if constexpr (LINES) {
                // ---- epilogue of the unit: bf16 results as whole lines (as EpiRelu2LinesT::tile).  Registers 4 g ..+3 of
                // acc[tm][tn] are the output features 32 tm + 8 g + 4 h ..+3 of token 32 tn + j: every 32-token x 64-feature
                // block (4 KiB) is collected in the wave's LDS block and leaves as 128-byte lines, 16 bytes per lane.
                typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
                uint8_t* const stage = line_stage;
                const int rd_row = el >> 3, rd_chunk = el & 7;
                uint16_t* const obase = p.out + ((int64_t)c0 * p.ld_out + u * XS_UNIT);
                const uint32_t lane_off = (uint32_t)rd_row * (uint32_t)p.ld_out + (uint32_t)(rd_chunk * 8);
                const int f8_row = el >> 2, f8_chunk = el & 3;
                uint8_t* const obase8 = EMIT ? p.out_f8 + ((int64_t)c0 * p.ld_f8 + u * XS_UNIT) : nullptr;
                const uint32_t lane_off8 = EMIT ? (uint32_t)f8_row * (uint32_t)p.ld_f8 + (uint32_t)(f8_chunk * 16) : 0u;
                auto pair_of = [&](float a0, float a1) -> uint32_t {
                    if constexpr (MODE == XS_LINES) return cvt_pk_bf16(a0 * line_scale, a1 * line_scale);
                    // c = bf16(acc * scale); bf16(max(c, 0)^2): the maximum on the product (relu(bf16(x)) == bf16(relu(x)))
                    const uint32_t pre = cvt_pk_bf16(fmaxf(a0 * line_scale, 0.0f), fmaxf(a1 * line_scale, 0.0f));
                    const float c0f = __uint_as_float(pre << 16), c1f = __uint_as_float(pre & 0xffff0000u);
                    return cvt_pk_bf16(c0f * c0f, c1f * c1f);
                };
#pragma unroll
                for (int tn = 0; tn < 4; ++tn) {
                    uint32_t f8[EMIT ? 8 : 1];
#pragma unroll
                    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            const v16f& r = acc[tm][tn];
                            const uint32_t p01 = pair_of(r[4 * g], r[4 * g + 1]), p23 = pair_of(r[4 * g + 2], r[4 * g + 3]);
                            *(v2i*)(stage + j * 128 + (((tm * 4 + g) ^ (j & 7)) << 4) + 8 * h) = (v2i){(int)p01, (int)p23};
                            if constexpr (EMIT) {
                                amax2 = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2, amax2), __builtin_bit_cast(u16x2, p01)));
                                amax2 = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2, amax2), __builtin_bit_cast(u16x2, p23)));
                                const float q0 = fminf(__uint_as_float(p01 << 16) * inv_act, 448.0f), q1 = fminf(__uint_as_float(p01 & 0xffff0000u) * inv_act, 448.0f);
                                const float q2 = fminf(__uint_as_float(p23 << 16) * inv_act, 448.0f), q3 = fminf(__uint_as_float(p23 & 0xffff0000u) * inv_act, 448.0f);
                                int rr = __builtin_amdgcn_cvt_pk_fp8_f32(q0, q1, __builtin_bit_cast(int, q0), false);
                                f8[tm * 4 + g] = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(q2, q3, rr, true);
                            }
                            if (g & 1) __builtin_amdgcn_sched_barrier(0);
                        }
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const int row = 8 * k + rd_row;
                        const v4i v = *(const v4i*)(stage + row * 128 + ((rd_chunk ^ (row & 7)) << 4));
                        if (c0 + tn * 32 + row < M) *(v4i*)(obase + (int64_t)(tn * 32 + 8 * k) * p.ld_out + lane_off) = v;
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (EMIT) {
                        constexpr int F8_STRIDE = 80;
#pragma unroll
                        for (int d = 0; d < 8; ++d) *(uint32_t*)(stage + j * F8_STRIDE + (2 * d + h) * 4) = f8[d];
#pragma unroll
                        for (int k = 0; k < 2; ++k) {
                            const int row = 16 * k + f8_row;
                            const v4i v = *(const v4i*)(stage + row * F8_STRIDE + f8_chunk * 16);
                            if (c0 + tn * 32 + row < M) *(v4i*)(obase8 + (int64_t)(tn * 32 + 16 * k) * p.ld_f8 + lane_off8) = v;
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                continue;
            }
            // ---- epilogue of the unit: softcap table, sum of exponentials, sigma codes (as EpiCEFwdT::tile)
            // code panel (layout: EpiCEFwdT): row = this lane's token, 16 bytes = the 16 vocabulary rows of one (tm, lane half) group
            uint8_t* cd_base = nullptr;
            uint32_t cd_lane = 0;
            if constexpr (CODES) {
                cd_base = p.codes + ((int64_t)(c0 >> 8) * p.nkp + (u >> 1)) * kPanelBytes + 4 * (u & 1) * kCodeGroupBytes;
                cd_lane = (uint32_t)(h * kCodeGroupBytes + ((c0 & 255) + j) * 16);
            }
            {
                constexpr int NB = 16;
                auto offsets_of = [&](int b, uint32_t (&off)[4]) {
                    const v16f& r = acc[(b >> 1) & 1][b >> 2];
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        off[k] = tab_offsets2(pack_logits(r[8 * (b & 1) + 2 * k] * p.scale, r[8 * (b & 1) + 2 * k + 1] * p.scale));
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
                    sum[b >> 2] += ((cur[0] + cur[1]) + (cur[2] + cur[3])) + ((cur[4] + cur[5]) + (cur[6] + cur[7]));
                    // nothing reads the sums before the job ends: without this the compiler moves all the additions
                    // behind the epilogue and keeps every table value alive until then
                    asm volatile("" : "+v"(sum[b >> 2]));
                    if constexpr (CODES) {
                        cw[2 * (b & 1)] = pack_codes4(cur[0], cur[1], cur[2], cur[3]);
                        cw[2 * (b & 1) + 1] = pack_codes4(cur[4], cur[5], cur[6], cur[7]);
                        if (b & 1)      // (tn, tm) = (b / 4, b / 2 % 2)
                            // non-temporal: the codes are next read by the conversion pass, long after they have left every
                            // cache, and should not push the weights out of L2 on their way (measured: 0.05 ms of the step)
                            __builtin_nontemporal_store((v4i){(int)cw[0], (int)cw[1], (int)cw[2], (int)cw[3]},
                                                        (v4i*)(cd_base + (cd_lane + (b >> 2) * 512 + ((b >> 1) & 1) * 2 * kCodeGroupBytes)));
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    if (b + 1 < NB) gather(off, cur);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            // sigma at candidate target columns that fall inside this unit's vocabulary rows
            const int v_lo = u * XS_UNIT;
            for (int c = 0; c < p.ncand; ++c) {
                int rl[4];
                bool any_hit = false;
#pragma unroll
                for (int tn = 0; tn < 4; ++tn) {
                    const int d = cand[c * XS_TOK + tn * 32 + j] - v_lo;
                    rl[tn] = ((unsigned)d < (unsigned)XS_UNIT) ? d : -1;
                    any_hit |= rl[tn] >= 0;
                }
                if (!__any(any_hit)) continue;
#pragma unroll
                for (int tn = 0; tn < 4; ++tn) {
                    if (!__any(rl[tn] >= 0)) continue;
                    float got = 0.0f;
                    bool mine = false;
#pragma unroll
                    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            if (tm * 32 + 8 * (v >> 2) + 4 * h + (v & 3) == rl[tn]) { got = acc[tm][tn][v]; mine = true; }
                    const int m = c0 + tn * 32 + j;
                    if (mine && m < M) {
                        const float l = bf16_bits_to_f32(pack_logits(got * p.scale, 0.0f) & 0xffffu);
                        p.saved_sigma[(int64_t)c * M + m] = softcap_sigma(l, p.sc);
                    }
                }
            }
        }

        if constexpr (DL || LINES) continue;
        // ---- job end: the lanes' sums -> part[split][token]
        wg_barrier();                                  // every wave is done reading the slab: it becomes scratch
        float* red = (float*)xslab;                    // [XS_WAVES][XS_TOK]
#pragma unroll
        for (int tn = 0; tn < 4; ++tn) {
            const float s = sum[tn] + __shfl_xor(sum[tn], 32, 64);
            if (lane < 32) red[wave * XS_TOK + tn * 32 + lane] = s;
        }
        wg_barrier();
        if (tid < XS_TOK) {
            float s = 0.0f;
#pragma unroll
            for (int w = 0; w < XS_WAVES; ++w) s += red[w * XS_TOK + tid];
            const int m = c0 + tid;
            if (m < M) p.part[(int64_t)split * M + m] = s;
        }
    }
    if constexpr (EMIT) {
        if (p.partial_amax) {      // the outputs are >= 0: the larger bf16 pattern is the larger value
            const uint32_t top = amax2 > (amax2 << 16) ? (amax2 & 0xffff0000u) : (amax2 << 16);
            const float m = wave_max(__uint_as_float(top));
            wg_barrier();          // the last job's slab is done with
            float* red = (float*)xslab;
            if (lane == 0) red[wave] = m;
            wg_barrier();
            if (tid == 0) {
                float t = 0.0f;
                for (int w = 0; w < XS_WAVES; ++w) t = fmaxf(t, red[w]);
                p.partial_amax[bid] = t;
                for (int i = bid + G; i < p.n_partials; i += G) p.partial_amax[i] = 0.0f;
            }
        }
    }
}

// Fragment-major copy of the weights (layout at the top of this file) from the row-major fp8 matrix [V, K]:
// one workgroup iteration moves 64 rows x 128 contraction bytes = 8 KiB, consecutive in both layouts' units.
__device__ __forceinline__ void xs_frag_from_f8(const uint8_t* __restrict__ w_f8, int V, int K, uint8_t* __restrict__ w_frag, int block, int nblocks) {
    const int nkc = K / 128, items = (V / XS_UNIT) * nkc;
    for (int it = block; it < items; it += nblocks) {
        const int u = it / nkc, kc = it % nkc;
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int t = threadIdx.x + 256 * r, row = t >> 3, cc = t & 7;     // 16-byte chunk cc of the 128-byte piece of row `row`
            const v4i v = *(const v4i*)(w_f8 + (int64_t)(u * XS_UNIT + row) * K + kc * 128 + cc * 16);
            const int ks = 2 * kc + (cc >> 2), hh = (cc >> 1) & 1, part = cc & 1, tm = row >> 5, i = row & 31;
            *(v4i*)(w_frag + (((int64_t)u * (K / 64) + ks) * 4 + tm * 2 + part) * 1024 + (hh * 32 + i) * 16) = v;
        }
    }
}
__global__ __launch_bounds__(256) void xs_frag_from_f8_kernel(const uint8_t* __restrict__ w_f8, int V, int K, uint8_t* __restrict__ w_frag) {
    xs_frag_from_f8(w_f8, V, K, w_frag, blockIdx.x, gridDim.x);
}

}  // namespace ngpt
