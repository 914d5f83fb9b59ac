// Persistent FP8 "TN" GEMM core for gfx950:  C[r, c] = sum_k A[r, k] * B[c, k]
//
// Both operands are fp8 bytes (or bf16 pairs, FMT_BF16) with the contraction index contiguous.  One
// workgroup owns a BM x BN tile at a time and walks a list of jobs (tiles, or contraction ranges of
// tiles); the k-loop of consecutive jobs is one continuous software pipeline: operand loads run two
// k-steps ahead of the MFMAs, across job boundaries and epilogues.
//
// Data path per k-step (BK = 128 bytes of contraction):
//   HBM/L2 --global_load_lds_dwordx4--> LDS (two 64 KiB slots, no register staging)
//   LDS --ds_read_b128--> MFMA operand registers --v_mfma_f32_32x32x64_f8f6f4--> fp32 accumulators
// (A operand given as the panel of its transpose, FMT_TRANSPOSED: LDS --ds_read_b64_tr_b8--> registers.)
//
// LDS layout of an operand slab: rows of 128 bytes; the eight 16-byte chunks of row r are stored
// at chunk position q ^ ((r >> 1) & 7).  A direct-to-LDS load writes 1 KiB (8 rows) per wave
// instruction with lane l at byte 16*l, so the swizzle is applied on the global-address side.
// With it, the 16 lanes that a ds_read_b128 serves together (16 consecutive rows, same chunk) hit
// 16 distinct 16-byte bank groups.
//
// MFMA 32x32x64 f8f6f4 register layouts used here (lane l, h = l / 32):
//   A operand: row  i = l % 32, 32 contraction bytes  [64*ks + 32*h, +32)
//   B operand: col  j = l % 32, the same 32 contraction bytes
//   D (16 fp32): col j = l % 32, row i = 8*(v/4) + 4*h + (v%4) for register v
// Any permutation of the contraction bytes is harmless as long as A and B use the same one.
#pragma once
#include "common.h"
#include <type_traits>

namespace ngpt {

// Operand layouts.  Row-major: row r, contraction byte c at r * ld + c.  Panel-blocked (256-row tiles,
// 128-byte k-steps only): the 256 x 128 slab that one k-step of one tile consumes is one contiguous
// 32 KiB block, blocks ordered [row tile][k-step]:  ((r / 256) * (K / 128) + c / 128) * 32768 +
// (r % 256) * 128 + c % 128.  A blocked operand is allocated for whole tiles (rows padded to 256).
// One k-step then reads 2 x 32 KiB of consecutive addresses instead of 512 rows that lie a full
// matrix row apart, which for long rows costs a TLB entry and a DRAM page per 128 bytes.
// Transposed A (kernel instantiations with FMT_TRANSPOSED): `A` points at the panel-blocked TRANSPOSE of
// the A matrix -- rows = the contraction index of this GEMM, 128-byte k-step rows = 128 rows of this
// GEMM's output, blocks [contraction / 256][R / 128] -- and `a_rows_pad` is R rounded up to 256.  One
// k-step of a tile then reads two contiguous 16 KiB pieces (128 contraction rows x 128 output rows each).
// kRowsPermuted: the 128-byte rows of a transposed A panel hold the output rows of every 32-group in dw_pos
// order (panel.h); the epilogue's row arithmetic undoes it (AccCoords::perm).
// Transposed bf16 operand (FMT_BF16 | FMT_TRANSPOSED, either operand): the pointer is a row-major matrix with the
// CONTRACTION index as its rows (row stride lda / ldb BYTES) and this operand's output rows / columns contiguous,
// i.e. C = A^T . B style products without a transposed copy.  One k-step = 64 contraction rows x 256 bf16 = 32 KiB;
// the contraction length must be a multiple of 64 rows, R / C multiples of 8.
constexpr int kBlockedA = 1, kBlockedB = 2, kRowsPermuted = 4;
constexpr int kPanelRows = 256, kPanelBytes = kPanelRows * 128;

struct GemmOperands {
    const uint8_t* A;   // [R, K] fp8, row stride lda bytes
    const uint8_t* B;   // [C, K] fp8, row stride ldb bytes
    int64_t lda, ldb;   // ignored for a blocked operand
    int R, C, K;        // K % 128 == 0
    int splits;         // split-K: the contraction of a split tile is cut into this many jobs (>= 1); needs an accumulating epilogue if > 1
    int layout;         // kBlockedA | kBlockedB | kRowsPermuted
    int full_tiles;     // the first full_tiles tiles (in walk order) are never split; 0 = `splits` applies to every tile
    int a_rows_pad;     // transposed A only: R rounded up to 256
    // TileListIter only: the kernel works on the tiles tile_list[0 .. *tile_count) instead of on all of them, unless the
    // counts probe_hits[0 .. kProbeBlocks) that an earlier kernel wrote add up to more than probe_limit: then on all of them
    const int* tile_list;
    const int* tile_count;
    const int* probe_hits;
    int probe_limit;
};

// Sum of the per-workgroup counts of a probe (written by an earlier kernel, hence read as scalar loads).
constexpr int kProbeBlocks = 64;
__device__ __forceinline__ int probe_total(const int* hits) {
    const __attribute__((address_space(4))) int* h = (const __attribute__((address_space(4))) int*)(uintptr_t)hits;
    int s = 0;
#pragma unroll
    for (int i = 0; i < kProbeBlocks; ++i) s += h[i];
    return s;
}

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int BK_ = 128, int NSTAGES_ = 2, int WGS_PER_CU_ = 1>
struct TileCfg {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, NSTAGES = NSTAGES_;
    static constexpr int WGS_PER_CU = WGS_PER_CU_;                 // co-resident workgroups the register budget allows
    static constexpr int WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
    static constexpr int NWAVES = WAVES_M * WAVES_N;
    static constexpr int THREADS = NWAVES * 64;
    static constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;   // wave tile
    static constexpr int TM = WTM / 32, TN = WTN / 32;             // MFMA tiles per wave
    static constexpr int KSUB = BK / 64;                           // 64-byte MFMA contraction steps per k-step
    static constexpr int CPR = BK / 16;                            // 16-byte chunks per LDS row
    static constexpr int RPB = 256 / BK;                           // LDS rows per 256-byte bank row
    static constexpr int ROWS_PER_LOAD = 1024 / BK;                // rows one wave-level 1 KiB load covers
    static constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK;
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int SMEM_BYTES = NSTAGES * STAGE_BYTES;
    static constexpr int A_LOADS = BM / ROWS_PER_LOAD / NWAVES;    // wave-level loads per k-step and wave
    static constexpr int B_LOADS = BN / ROWS_PER_LOAD / NWAVES;
    static constexpr int LOADS = A_LOADS + B_LOADS;
    static constexpr int WAVE_SCRATCH = STAGE_BYTES / NWAVES;      // epilogue staging per wave
    static_assert(BK == 64 || BK == 128, "BK is 64 or 128 bytes");
    static_assert(NSTAGES >= 2 && NSTAGES <= 4, "2..4 LDS stages");
    static_assert(BM % (ROWS_PER_LOAD * NWAVES) == 0 && BN % (ROWS_PER_LOAD * NWAVES) == 0, "tile rows must split over waves");
    static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be made of 32x32 MFMA tiles");
    // LDS swizzle: chunk q of row r is stored at chunk position q ^ swz(r)
    static __device__ __forceinline__ int swz(int r) { return (r / RPB) % CPR; }
};

// Tile order: groups of 4 tile-rows, column-major inside a group, so 32 consecutive sequence
// numbers form a 4 x 8 block of tiles that shares 4 A panels and 8 B panels.  Workgroups are
// dealt to the 8 XCDs round-robin by the dispatcher (workgroup b runs on XCD b % 8); giving
// XCD x the sequence numbers [32x, 32x+32) of every batch of 256 keeps such a block inside one
// XCD's L2.  An output with few tile columns (the skinny backward GEMMs: 3) is walked row-major
// instead: the tiles of one row, which share the long A panel, are consecutive, so only the rows that
// straddle a multiple of 32 are fetched by two XCDs.
struct TileOrder {
    int tiles_r, tiles_c, total;
    __device__ TileOrder(int R, int C, int BM, int BN)
        : tiles_r((R + BM - 1) / BM), tiles_c((C + BN - 1) / BN), total(tiles_r * tiles_c) {}
    __device__ void coords(int seq, int& tr, int& tc) const {
        constexpr int GROUP = 4;
        if (tiles_c <= 8 && tiles_r > GROUP) {
            tr = seq / tiles_c;
            tc = seq - tr * tiles_c;
            return;
        }
        int per_group = GROUP * tiles_c;
        int grp = seq / per_group;
        int first = grp * GROUP;
        int gsz = min(tiles_r - first, GROUP);
        int rem = seq - grp * per_group;
        tr = first + rem % gsz;
        tc = rem / gsz;
    }
    // sequence number handled by workgroup `bid` of `G` in its `it`-th turn
    static __device__ int seq_of(int it, int bid, int G) {
        if ((G & 7) == 0) return it * G + (bid & 7) * (G >> 3) + (bid >> 3);
        return it * G + bid;
    }
};

template <int N>
__device__ __forceinline__ void wait_vmem_le() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    if constexpr (N == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Operand addresses are a wave-uniform 64-bit base (SGPRs) plus a 32-bit per-lane offset, which keeps
// the k-loop free of 64-bit VGPR pointer arithmetic; a tile's operand slab must span < 4 GiB.
template <class Cfg>
struct LaneOffsets {
    uint32_t a_off[Cfg::A_LOADS], b_off[Cfg::B_LOADS];   // byte offset of this lane's chunk from the tile's first row
    // Transposed bf16 slab: LDS row = contraction row (64 per k-step) of 512 bytes = 32 chunks; one wave-level load
    // covers two rows.  The chunk stored at position p of row m is global chunk p ^ (4 * (m & 3)): with it the 32
    // lanes that a transposing read serves together hit 32 distinct 8-byte bank pairs (see frag offsets below).
    // `lim` = columns of this operand left from the tile's origin (a multiple of 8): chunks past it are clamped.
    static __device__ uint32_t tr16_off(int load, int wave, int lane, int64_t ld, int lim) {
        const int m = 2 * (wave + load * Cfg::NWAVES) + (lane >> 5);
        int chunk = (lane & 31) ^ (4 * (m & 3));
        chunk = min(chunk, lim / 8 - 1);
        return (uint32_t)((int64_t)m * ld + chunk * 16);
    }
    // A tile's offsets depend on its position only where rows (or, for a transposed bf16 slab, columns) past the end of
    // the operand are clamped, i.e. in the last tile row / column of a matrix that is not a multiple of the tile:
    // init_a / init_b are called again only when the new or the previous tile is such an edge tile.
    __device__ void init_a(const GemmOperands& g, int wave, int lane, int r0, bool a_transposed, bool a_tr16) {
        int lrow = lane / Cfg::CPR, lchunk = lane % Cfg::CPR;
#pragma unroll
        for (int i = 0; i < Cfg::A_LOADS; ++i) {
            if (a_tr16) { a_off[i] = tr16_off(i, wave, lane, g.lda, g.R - r0); continue; }
            if (a_transposed) {
                // 1 KiB piece `c32` of the k-step's 32: half (token block) c32 / 16, contraction rows 8 * (c32 % 16) ..+7;
                // the 16-byte chunk q of contraction row r lands at chunk position q ^ (r & 7)
                const int c32 = wave + i * Cfg::NWAVES;
                const int r = 8 * (c32 & 15) + lrow;
                a_off[i] = (uint32_t)((c32 >> 4) * kPanelBytes + r * 128 + ((lchunk ^ (r & 7)) << 4));
                continue;
            }
            int R = (wave + i * Cfg::NWAVES) * Cfg::ROWS_PER_LOAD + lrow;
            int q = lchunk ^ Cfg::swz(R);
            if (g.layout & kBlockedA) { a_off[i] = (uint32_t)(R * 128 + q * 16); continue; }   // padded: no clamp
            int rr = min(R, g.R - 1 - r0);                       // clamp rows past the end
            a_off[i] = (uint32_t)((int64_t)rr * g.lda + q * 16);
        }
    }
    __device__ void init_b(const GemmOperands& g, int wave, int lane, int c0, bool b_tr16) {
        int lrow = lane / Cfg::CPR, lchunk = lane % Cfg::CPR;
#pragma unroll
        for (int i = 0; i < Cfg::B_LOADS; ++i) {
            if (b_tr16) { b_off[i] = tr16_off(i, wave, lane, g.ldb, g.C - c0); continue; }
            int R = (wave + i * Cfg::NWAVES) * Cfg::ROWS_PER_LOAD + lrow;
            int q = lchunk ^ Cfg::swz(R);
            if (g.layout & kBlockedB) { b_off[i] = (uint32_t)(R * 128 + q * 16); continue; }
            int rr = min(R, g.C - 1 - c0);
            b_off[i] = (uint32_t)((int64_t)rr * g.ldb + q * 16);
        }
    }
};

template <class Cfg, int AFMT, int BFMT>
struct TileMainloop {
    LaneOffsets<Cfg> lo;
    const uint8_t* a_next;   // wave-uniform: slab of the next k-step to load (first row of the tile)
    const uint8_t* b_next;
    int frag_a[Cfg::TM];     // LDS byte offset of this lane's first 16-byte chunk, stage 0, ksub 0
    int frag_b[Cfg::TN];
    int a_step, b_step;      // bytes from one k-step's slab to the next
    const uint8_t* b_pending;   // B slab whose loads issue_loads_b() still has to issue, or null
    int pending_stage;
    int lo_state;            // bit 0 / 1: a_off / b_off hold the offsets of a tile that needs no clamping (they fit every such tile)
    int a_kt;                // transposed A: index of the next k-step to load; a_next then is the tile's base
    int64_t a_pair_stride;   // transposed A: bytes between the panel rows of two consecutive 256-blocks of the contraction
    int wave, lane, wr, wc;
    static constexpr bool BF16 = (AFMT & 3) == FMT_BF16;
    static constexpr bool ATR = (AFMT & FMT_TRANSPOSED) != 0 && !BF16;      // fp8 A given as the panel of its transpose
    static constexpr bool ATR16 = (AFMT & FMT_TRANSPOSED) != 0 && BF16;     // bf16 operands with the contraction as rows
    static constexpr bool BTR16 = (BFMT & FMT_TRANSPOSED) != 0 && BF16;
    static_assert(!(BFMT & FMT_TRANSPOSED) || BF16, "a transposed B operand exists for bf16 only");
    // bf16 fragments are read by hand-placed assembly and handed over between k-steps (the 256 x 256 configuration)
    static constexpr bool kAsmFrags16 = BF16 && Cfg::TM == 2 && Cfg::TN == 4 && Cfg::BK == 128;
    v4i h16a[2][Cfg::TM], h16b[2][Cfg::TN];   // kAsmFrags16: two alternating fragment sets
    static_assert(!(ATR16 || BTR16) || (Cfg::BM == 256 && Cfg::BN == 256 && Cfg::BK == 128), "transposed bf16 slabs are 64 x 256");

    __device__ void init() {
        int tid = threadIdx.x;
        lane = tid & 63;
        b_pending = nullptr;
        pending_stage = 0;
        lo_state = 0;
        wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        wr = wave / Cfg::WAVES_N;
        wc = wave % Cfg::WAVES_N;
        // first 16-byte chunk of this lane's operand fragment: fp8 MFMAs (32x32x64) take 32 bytes per
        // lane (chunks 2h, 2h+1), the bf16 MFMA (32x32x16) takes 16 bytes (chunk h)
        int q0 = BF16 ? (lane >> 5) : (lane >> 5) * 2;
#pragma unroll
        for (int t = 0; t < Cfg::TM; ++t) {
            int row = wr * Cfg::WTM + t * 32 + (lane & 31);
            frag_a[t] = row * Cfg::BK + ((q0 ^ Cfg::swz(row)) << 4);
            if (ATR16) frag_a[t] = tr16_frag(wr * Cfg::WTM + t * 32);
            if (ATR) {
                // Source address of this lane for the transposing read (ds_read_b64_tr_b8: inside each block
                // of 16 lanes, lane i receives byte i % 8 of the 8-byte rows of lanes 2j + i / 8, j = 0..7).
                // Lane s' of a block supplies contraction row s' / 2 and output rows 8 * (s' % 2) ..+7, so lane i
                // ends up with 8 consecutive contraction bytes of output row i.  Blocks 0, 1 serve MFMA rows
                // 0..15, 16..31 of the first 32 contraction bytes, blocks 2, 3 the same rows of the second 32.
                static_assert(!ATR || (Cfg::BM == 256 && Cfg::BK == 128 && Cfg::WTM == 64), "transposed A geometry");
                const int sl = lane & 15, blk = lane >> 4;
                const int krow = 32 * (blk >> 1) + (sl >> 1);
                const int pos = (wr & 1) * 64 + 32 * t + 16 * (blk & 1) + 8 * (sl & 1);   // byte inside the 128-byte row
                frag_a[t] = (wr >> 1) * (kPanelBytes / 2) + krow * 128 + ((((pos >> 4) ^ (sl >> 1)) << 4) | (pos & 15));
            }
        }
#pragma unroll
        for (int t = 0; t < Cfg::TN; ++t) {
            int row = wc * Cfg::WTN + t * 32 + (lane & 31);
            frag_b[t] = Cfg::A_BYTES + row * Cfg::BK + ((q0 ^ Cfg::swz(row)) << 4);
            if (BTR16) frag_b[t] = Cfg::A_BYTES + tr16_frag(wc * Cfg::WTN + t * 32);
        }
    }
    // Source address of this lane for the transposing 16-bit read (ds_read_b64_tr_b16: inside each block of 16
    // lanes, lane i receives element i % 4 of the 4-element rows of lanes 4j + i / 4, j = 0..3).  Lane s of a
    // block supplies contraction row s / 4 and output rows 4 * (s % 4) ..+3, so lane i ends up with 4 consecutive
    // contraction elements of output row i.  Blocks 0, 1 serve rows 0..15, 16..31 of the MFMA tile for the first 8
    // of a sub-step's 16 contraction rows (two reads, 4 rows = 2 KiB apart), blocks 2, 3 the same for the second 8:
    // a lane half holds its 8 contraction elements in natural order, as a row-major operand's 16-byte chunk does.
    // `row0`: first output row of the MFMA tile inside the workgroup tile.
    __device__ int tr16_frag(int row0) const {
        const int s = lane & 15, blk = lane >> 4;
        const int m = 8 * (blk >> 1) + (s >> 2);                      // contraction row inside the sub-step; m & 3 == s >> 2
        const int byte = 2 * (row0 + 16 * (blk & 1) + 4 * (s & 3));   // inside the 512-byte row
        return m * 512 + ((((byte >> 4) ^ (4 * (s >> 2))) << 4) | (byte & 15));
    }

    // Point the loads at tile (r0, c0).  Rows past the end are clamped to the last row: they are
    // loaded (valid memory) and their results discarded by the epilogue.
    // `kt`: first k-step that will be loaded from this tile.
    // (The caller flushes issue_loads_b() first: the pending B loads use the old tile's lane offsets.)
    __device__ void set_tile(const GemmOperands& g, int r0, int c0, int kt) {
        a_step = (g.layout & kBlockedA) ? kPanelBytes : Cfg::BK;
        b_step = (g.layout & kBlockedB) ? kPanelBytes : Cfg::BK;
        // a blocked operand's tile starts r0 / 256 * (K / 128) blocks in, which is r0 * K bytes
        a_next = g.A + (int64_t)r0 * ((g.layout & kBlockedA) ? (int64_t)g.K : g.lda) + (int64_t)kt * a_step;
        b_next = g.B + (int64_t)c0 * ((g.layout & kBlockedB) ? (int64_t)g.K : g.ldb) + (int64_t)kt * b_step;
        if (ATR) {
            // block (contraction / 256, output row / 128): the tile's two output-row blocks are adjacent
            a_next = g.A + (int64_t)(r0 >> 7) * kPanelBytes;
            a_pair_stride = (int64_t)(g.a_rows_pad >> 7) * kPanelBytes;
            a_kt = kt;
        }
        if (ATR16) {   // 64 contraction rows per k-step, the tile's rows start 2 * r0 bytes into each
            a_step = (int)(64 * g.lda);
            a_next = g.A + 2 * (int64_t)r0 + (int64_t)kt * a_step;
        }
        if (BTR16) {
            b_step = (int)(64 * g.ldb);
            b_next = g.B + 2 * (int64_t)c0 + (int64_t)kt * b_step;
        }
        const bool a_inner = g.R - r0 >= Cfg::BM, b_inner = g.C - c0 >= Cfg::BN;
        if (!(a_inner && (lo_state & 1))) lo.init_a(g, wave, lane, r0, ATR, ATR16);
        if (!(b_inner && (lo_state & 2))) lo.init_b(g, wave, lane, c0, BTR16);
        lo_state = (a_inner ? 1 : 0) | (b_inner ? 2 : 0);
    }

    // Loads the next k-step of the current tile into LDS slot `stage` and moves on to the one after: the A
    // slab now, the B slab when issue_loads_b() is called (behind the next k-step's first MFMAs, so that the
    // loads of one k-step do not leave the compute unit in a single burst).
    __device__ void issue_loads(uint8_t* smem, int stage) {
        uint8_t* s = smem + stage * Cfg::STAGE_BYTES;
        const uint8_t* ab = a_next;
        b_pending = b_next;
        pending_stage = stage;
        if (ATR) {   // contraction rows 128 * a_kt ..+127: block a_kt / 2, upper or lower half of its 256 rows
            ab = a_next + (int64_t)(a_kt >> 1) * a_pair_stride + (a_kt & 1) * (kPanelBytes / 2);
            ++a_kt;
        } else {
            a_next += a_step;
        }
        b_next += b_step;
#pragma unroll
        for (int i = 0; i < Cfg::A_LOADS; ++i)
            global_to_lds16(ab + lo.a_off[i], s + (wave + i * Cfg::NWAVES) * 1024);
    }
    __device__ void issue_loads_b(uint8_t* smem) {
        if (b_pending == nullptr) return;
        uint8_t* s = smem + pending_stage * Cfg::STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < Cfg::B_LOADS; ++i)
            global_to_lds16(b_pending + lo.b_off[i], s + Cfg::A_BYTES + (wave + i * Cfg::NWAVES) * 1024);
        b_pending = nullptr;
    }

    // Operand fragment of one 32-row MFMA tile for contraction sub-step ks (two 16-byte chunks).
    __device__ __forceinline__ v8i frag(const uint8_t* s, int off, int ks) const {
        int o = off ^ (ks * 64);
        v4i lo = *(const v4i*)(s + o);
        v4i hi = *(const v4i*)(s + (o ^ 16));
        return (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    }

    // A fragment through the transposing LDS read: four 8-byte reads, 8 contraction rows (1 KiB of LDS) apart.
    // Written as inline assembly: behind the builtin the compiler cannot tell these reads from the LDS
    // destinations of the direct-to-LDS loads still in flight and makes every one of them wait for
    // vmcnt(0), which serialises the operand prefetch.  The price is that the compiler does not count
    // them in lgkmcnt either: frag_fence() must stand between such a read and the first use of its result.
    template <int OFF>
    static __device__ __forceinline__ v2i read_tr8(uint32_t lds_addr) {
        v2i r;
        asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(r) : "v"(lds_addr), "n"(OFF));
        return r;
    }
    template <int KS>
    __device__ __forceinline__ v8i frag_a_tr(const uint8_t* s, int t) const {
        const uint32_t p = (uint32_t)(size_t)((const __attribute__((address_space(3))) uint8_t*)s) + (uint32_t)frag_a[t];
        v2i r0 = read_tr8<KS * 8192>(p), r1 = read_tr8<KS * 8192 + 1024>(p);
        v2i r2 = read_tr8<KS * 8192 + 2048>(p), r3 = read_tr8<KS * 8192 + 3072>(p);
        return (v8i){r0.x, r0.y, r1.x, r1.y, r2.x, r2.y, r3.x, r3.y};
    }
    __device__ __forceinline__ v8i frag_a_at(const uint8_t* s, int t, int ks) const {
        if constexpr (ATR) {
            static_assert(!ATR || Cfg::KSUB == 2, "two contraction sub-steps");
            return ks == 0 ? frag_a_tr<0>(s, t) : frag_a_tr<1>(s, t);
        } else {
            return frag(s, frag_a[t], ks);
        }
    }
    // All LDS reads issued so far have returned; ties the A fragments to that point.
    static __device__ __forceinline__ void frag_fence(v8i (&a)[Cfg::TM]) {
        if constexpr (ATR) {
            static_assert(!ATR || Cfg::TM == 2, "two A fragments");
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a[0]), "+v"(a[1]));
        }
    }

    // bf16 fragments (16 bytes per lane and MFMA tile) of contraction sub-step KS (16 elements) as inline assembly:
    // a transposed operand takes two transposing 8-byte reads 4 contraction rows (2 KiB) apart, a row-major one
    // one 16-byte read of chunk (2 KS + lane half) of its swizzled 128-byte row.
    template <int OFF>
    static __device__ __forceinline__ v2i read_tr16(uint32_t lds_addr) {
        v2i r;
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(r) : "v"(lds_addr), "n"(OFF));
        return r;
    }
    static __device__ __forceinline__ v4i read_b128(uint32_t lds_addr) {
        v4i r;
        asm volatile("ds_read_b128 %0, %1" : "=v"(r) : "v"(lds_addr));
        return r;
    }
    template <int KS>
    __device__ __forceinline__ void read_frags16(uint32_t sbase, v4i (&fa)[Cfg::TM], v4i (&fb)[Cfg::TN]) const {
        static_assert(Cfg::BK == 128 && 3 * 8192 + 2048 < 65536, "16-bit immediate offsets of the transposing reads");
#pragma unroll
        for (int t = 0; t < Cfg::TM; ++t) {
            if constexpr (ATR16) {
                const v2i lo = read_tr16<KS * 8192>(sbase + (uint32_t)frag_a[t]), hi = read_tr16<KS * 8192 + 2048>(sbase + (uint32_t)frag_a[t]);
                fa[t] = (v4i){lo.x, lo.y, hi.x, hi.y};
            } else {
                fa[t] = read_b128(sbase + (uint32_t)(frag_a[t] ^ (KS * 32)));
            }
        }
#pragma unroll
        for (int t = 0; t < Cfg::TN; ++t) {
            if constexpr (BTR16) {
                const v2i lo = read_tr16<KS * 8192>(sbase + (uint32_t)frag_b[t]), hi = read_tr16<KS * 8192 + 2048>(sbase + (uint32_t)frag_b[t]);
                fb[t] = (v4i){lo.x, lo.y, hi.x, hi.y};
            } else {
                fb[t] = read_b128(sbase + (uint32_t)(frag_b[t] ^ (KS * 32)));
            }
        }
    }
    // All LDS reads issued so far have returned; ties the fragments to that point.
    static __device__ __forceinline__ void frag16_fence(v4i (&fa)[Cfg::TM], v4i (&fb)[Cfg::TN]) {
        static_assert(Cfg::TM == 2 && Cfg::TN == 4, "fragment count of the fence");
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fa[0]), "+v"(fa[1]), "+v"(fb[0]), "+v"(fb[1]), "+v"(fb[2]), "+v"(fb[3]));
    }

    // One k-step of MFMAs on the operands in LDS slot `stage`, software-pipelined by hand.
    //  * Fragment reads run one MFMA group (TM MFMAs that share a B fragment) ahead of their use, and
    //    scheduling barriers keep the compiler from hoisting all reads to the top, which would leave
    //    the matrix pipe idle for an LDS round trip per sub-step.
    //  * `sync` (operand wait + workgroup barrier + issue of the next loads, supplied by the kernel) runs
    //    before the LAST group instead of between k-steps: at that point every LDS read of this slot
    //    has been issued, so after the barrier the slot may be refilled, and the first fragments of the
    //    next k-step (slot `next_stage`, if `want_next`) are read behind the last group's MFMAs.
    //    They are handed to the next call in a / b0 (`have` = they are valid on entry).
    //    `refill` (issue of the operand loads two k-steps ahead into the slot just freed) runs behind the
    //    last group's MFMAs, so that its address arithmetic is hidden too.
    //    FRESH: the caller knows at compile time that nothing was handed over (`have` is false).
    template <bool FIRST, bool FRESH, class Sync, class Refill>
    __device__ __forceinline__ void compute(uint8_t* smem, int stage, int next_stage, bool have, bool want_next,
                                            v16f (&acc)[Cfg::TM][Cfg::TN], v8i (&a)[Cfg::TM], v8i& b0, Sync&& sync,
                                            Refill&& refill) {
        const uint8_t* s = smem + stage * Cfg::STAGE_BYTES;
        const uint8_t* sn = smem + next_stage * Cfg::STAGE_BYTES;
        if constexpr ((AFMT & 3) == FMT_BF16) {
            // bf16 operands: 32 contraction bytes (16 elements) per MFMA, one 16-byte chunk per lane;
            // no fragment hand-over between k-steps
            constexpr int KS = Cfg::BK / 32;
            issue_loads_b(smem);
            if constexpr (kAsmFrags16) {
                // All fragment reads of this path are inline assembly (see read_tr8 for why), so the compiler does
                // not count them: frag16_fence() stands between a sub-step's reads and its MFMAs.  The reads of
                // sub-step ks + 1 are issued behind that fence and ahead of the MFMAs of ks, which cover their
                // latency; behind the barrier of the last sub-step the first fragments of the NEXT k-step (slot
                // `next_stage`) are read and handed to the next call in h16a / h16b[0] (`have`).
                const uint32_t sbase = (uint32_t)(size_t)((const __attribute__((address_space(3))) uint8_t*)s);
                const uint32_t nbase = (uint32_t)(size_t)((const __attribute__((address_space(3))) uint8_t*)sn);
                static_assert(KS == 4, "four sub-steps: the hand-over lands in fragment set 0 again");
                if (FRESH || !have) read_frags16<0>(sbase, h16a[0], h16b[0]);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    frag16_fence(h16a[ks & 1], h16b[ks & 1]);
                    if (ks == 0) read_frags16<1>(sbase, h16a[1], h16b[1]);
                    if (ks == 1) read_frags16<2>(sbase, h16a[0], h16b[0]);
                    if (ks == 2) read_frags16<3>(sbase, h16a[1], h16b[1]);
                    if (ks == KS - 1) {
                        sync();
                        if (want_next) read_frags16<0>(nbase, h16a[0], h16b[0]);
                    }
                    __builtin_amdgcn_s_setprio(1);
#pragma unroll
                    for (int tn = 0; tn < Cfg::TN; ++tn)
#pragma unroll
                        for (int tm = 0; tm < Cfg::TM; ++tm) {
                            const v16f zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                            acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                                __builtin_bit_cast(v8bf, h16a[ks & 1][tm]), __builtin_bit_cast(v8bf, h16b[ks & 1][tn]),
                                (FIRST && ks == 0) ? zero : acc[tm][tn], 0, 0, 0);
                        }
                    __builtin_amdgcn_s_setprio(0);
                    __builtin_amdgcn_sched_barrier(0);
                }
                refill();
                __builtin_amdgcn_sched_barrier(0);
                return;
            }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                v8bf fa[Cfg::TM], fb[Cfg::TN];
#pragma unroll
                for (int t = 0; t < Cfg::TM; ++t) fa[t] = *(const v8bf*)(s + (frag_a[t] ^ (ks * 32)));
#pragma unroll
                for (int t = 0; t < Cfg::TN; ++t) fb[t] = *(const v8bf*)(s + (frag_b[t] ^ (ks * 32)));
                if (ks == KS - 1) sync();
#pragma unroll
                for (int tm = 0; tm < Cfg::TM; ++tm)
#pragma unroll
                    for (int tn = 0; tn < Cfg::TN; ++tn) {
                        const v16f zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                        acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                            fa[tm], fb[tn], (FIRST && ks == 0) ? zero : acc[tm][tn], 0, 0, 0);
                    }
            }
            refill();
        } else {
            v8i bcur = b0;
            if (FRESH || !have) {
#pragma unroll
                for (int t = 0; t < Cfg::TM; ++t) a[t] = frag_a_at(s, t, 0);
                bcur = frag(s, frag_b[0], 0);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ks = 0; ks < Cfg::KSUB; ++ks) {
                frag_fence(a);
                v8i an[Cfg::TM];
#pragma unroll
                for (int tn = 0; tn < Cfg::TN; ++tn) {
                    v8i bnext;
                    if (tn + 1 < Cfg::TN) {
                        bnext = frag(s, frag_b[tn + 1], ks);
                    } else if (ks + 1 < Cfg::KSUB) {
                        if (!ATR) {
#pragma unroll
                            for (int t = 0; t < Cfg::TM; ++t) an[t] = frag_a_at(s, t, ks + 1);
                        }
                        bnext = frag(s, frag_b[0], ks + 1);
                    } else {
                        sync();
                        if (want_next) {
#pragma unroll
                            for (int t = 0; t < Cfg::TM; ++t) an[t] = frag_a_at(sn, t, 0);
                            bnext = frag(sn, frag_b[0], 0);
                        } else {
#pragma unroll
                            for (int t = 0; t < Cfg::TM; ++t) an[t] = a[t];
                            bnext = bcur;
                        }
                    }
                    __builtin_amdgcn_s_setprio(1);   // a wave about to feed the matrix pipe goes first (measured: 0.5 % of a GEMM)
#pragma unroll
                    for (int tm = 0; tm < Cfg::TM; ++tm) {
                        const v16f zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                        acc[tm][tn] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                            a[tm], bcur, (FIRST && ks == 0) ? zero : acc[tm][tn], AFMT & 1, BFMT & 1, 0, 0, 0, 0);
                    }
                    __builtin_amdgcn_s_setprio(0);
                    if (ks == 0 && tn == 0) issue_loads_b(smem);   // second half of the loads issued at the end of the previous k-step
                    // Transposing reads (twice as many instructions) of the next sub-step's A fragments: one
                    // fragment per group from the first on, issued behind the group's MFMAs and after its B
                    // read, so that the next group waits for that B fragment only (LDS reads return in order).
                    if (ATR && ks + 1 < Cfg::KSUB) {
#pragma unroll
                        for (int t = 0; t < Cfg::TM; ++t)
                            if (tn == (t < Cfg::TN - 1 ? t : Cfg::TN - 1)) an[t] = frag_a_at(s, t, ks + 1);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    bcur = bnext;
                }
#pragma unroll
                for (int t = 0; t < Cfg::TM; ++t) a[t] = an[t];
            }
            b0 = bcur;
            refill();
            __builtin_amdgcn_sched_barrier(0);
        }
    }
};

// Coordinates of accumulator element (tm, tn, v) of this lane inside the workgroup tile.
// `perm`: the kernel read its A operand transposed from a panel whose 128-byte rows hold the output rows
// of every 32-group in the order position 16h + 4g + i <-> row 8g + 4h + i (the order in which the producer's
// accumulator registers held them).  MFMA row 8a + 4H + b (register group a, lane half H) then is output
// row {0, 16, 4, 20}[a] + 8H + b of its 32-group.
template <class Cfg>
struct AccCoords {
    int wave_row0, wave_col0;   // origin of this wave's sub-tile
    int row_base, col_base;     // this lane's element for tm = tn = 0, v = 0
    bool perm;
    __device__ AccCoords(int wr, int wc, int lane, bool perm_ = false)
        : wave_row0(wr * Cfg::WTM), wave_col0(wc * Cfg::WTN),
          row_base(wr * Cfg::WTM + (perm_ ? 8 : 4) * (lane >> 5)), col_base(wc * Cfg::WTN + (lane & 31)), perm(perm_) {}
    // row of accumulator register v of MFMA tile tm, relative to row_base
    __device__ int dr(int tm, int v) const {
        const int a = v >> 2;
        return tm * 32 + (perm ? ((a & 1) * 16 + (a >> 1) * 4) : 8 * a) + (v & 3);
    }
    __device__ int row(int tm, int v) const { return row_base + dr(tm, v); }
    __device__ int col(int tn) const { return col_base + tn * 32; }
};

// Default job walk: the tiles of the R x C grid in TileOrder.  The first `full` tiles are one job
// each; every later tile is cut into `splits` jobs along the contraction (partial results, for an
// accumulating epilogue).  Split jobs are numbered split-major, so the workgroups that run together
// work on neighbouring tiles.  With full = tiles rounded down to a multiple of the grid and the
// remainder split to fill one more round, no workgroup idles while the last tiles finish.
struct GridIter {
    TileOrder order;
    int it, bid, G, seq, tr_, tc_, split_, splits, full, jobs, nk_, kt_lo_, kt_hi_;
    __device__ GridIter(const GemmOperands& g, int BM, int BN, int bid_, int G_)
        : order(g.R, g.C, BM, BN), it(0), bid(bid_), G(G_), tr_(0), tc_(0), split_(0),
          splits(g.splits < 1 ? 1 : g.splits), nk_(g.K / 128), kt_lo_(0), kt_hi_(0) {
        full = (splits == 1) ? order.total : min(max(g.full_tiles, 0), order.total);
        jobs = full + (order.total - full) * splits;
        seq = TileOrder::seq_of(0, bid, G);
        locate();
    }
    __device__ void locate() {
        if (seq < jobs) {
            int tile = seq;
            split_ = 0;
            kt_lo_ = 0;
            kt_hi_ = nk_;
            if (seq >= full) {
                const int rem = order.total - full, idx = seq - full;
                split_ = idx / rem;
                tile = full + idx - split_ * rem;
                split_ = __builtin_amdgcn_readfirstlane(split_);
                // contraction range of the job in units of 128 bytes
                kt_lo_ = __builtin_amdgcn_readfirstlane(nk_ * split_ / splits);
                kt_hi_ = __builtin_amdgcn_readfirstlane(nk_ * (split_ + 1) / splits);
            }
            order.coords(tile, tr_, tc_);
            // the walk depends on the workgroup id only: tell the compiler these are scalars
            tr_ = __builtin_amdgcn_readfirstlane(tr_);
            tc_ = __builtin_amdgcn_readfirstlane(tc_);
        }
    }
    __device__ bool valid() const { return seq < jobs; }
    __device__ int tr() const { return tr_; }
    __device__ int tc() const { return tc_; }
    // nk k-steps of BK bytes cover the same contraction as nk_ units of 128 bytes
    __device__ int kt_begin(int nk) const { return nk == nk_ ? kt_lo_ : 2 * kt_lo_; }
    __device__ int kt_end(int nk) const { return nk == nk_ ? kt_hi_ : 2 * kt_hi_; }
    __device__ bool partial() const { return seq >= full; }     // the job holds part of its tile's contraction
    // number of a partial job: split * (split tiles) + (index of its tile among the split tiles)
    __device__ int part_slot() const { return seq - full; }
    __device__ bool job_begin() const { return false; }
    __device__ bool job_end() const { return false; }
    __device__ int job_id() const { return 0; }
    __device__ void advance() {
        ++it;
        seq = TileOrder::seq_of(it, bid, G);
        locate();
    }
};

// GridIter over a list of tiles: tile_list[i] = (tile row << 16) | tile column, i < *tile_count (both written by an
// earlier kernel and read through the constant address space, i.e. as scalar loads that stay out of the vector memory
// counter); the base class then walks a 1 x count grid and its column index is the position in the list.  If the probe
// counts say so (GemmOperands::probe_hits) the walk covers the whole grid instead.
struct TileListIter : GridIter {
    const int* list;
    bool whole;
    static __device__ bool whole_grid(const GemmOperands& g) { return probe_total(g.probe_hits) > g.probe_limit; }
    static __device__ GemmOperands listed(GemmOperands g, int BM, int BN) {
        if (!whole_grid(g)) {
            g.R = BM;
            g.C = ((const __attribute__((address_space(4))) int*)(uintptr_t)g.tile_count)[0] * BN;
        }
        return g;
    }
    __device__ TileListIter(const GemmOperands& g, int BM, int BN, int bid_, int G_)
        : GridIter(listed(g, BM, BN), BM, BN, bid_, G_), list(g.tile_list), whole(whole_grid(g)) {}
    __device__ int entry() const { return ((const __attribute__((address_space(4))) int*)(uintptr_t)list)[tc_]; }
    __device__ int tr() const { return whole ? tr_ : entry() >> 16; }
    __device__ int tc() const { return whole ? tc_ : entry() & 0xffff; }
};

// The generic persistent kernel.  `Iter` walks the tiles of this workgroup (see GridIter).  `Epi` supplies
//   void begin(int bid, int nblocks)
//   void partial(bool, int slot)   -- before each tile(): the job holds only part of the tile's contraction; slot numbers such jobs
//   void tile(acc, r0, c0, coords, scratch /* wave-private LDS */, lane)
//   void job_begin(c0) / job_end(c0, job_id, coords, stage_scratch /* whole free LDS stage */)
//                                                              -- only if Iter reports job boundaries
//   void end(uint8_t* smem, int bid, int nblocks)
// `tile` runs after a workgroup barrier, so the just-consumed LDS stage is free for staging.
// Dynamic LDS: Epi::EXTRA_LDS bytes that the epilogue owns for the whole kernel (lookup tables; at
// offset 0 so their addresses fit the 16-bit offset field of LDS instructions), then
// Cfg::SMEM_BYTES for the operand stages.
// Walks (tile, k-step) pairs of one workgroup as one flat sequence, so the software pipeline of
// operand loads runs ahead across tile boundaries.
template <class Iter>
struct StepCursor {
    Iter it;
    int kt, kt_lo, kt_hi, nk;
    __device__ StepCursor(const Iter& i, int nk_) : it(i), kt(0), kt_lo(0), kt_hi(0), nk(nk_) { enter(); }
    __device__ void enter() {
        if (it.valid()) {
            kt_lo = it.kt_begin(nk);
            kt_hi = it.kt_end(nk);
        }
        kt = kt_lo;
    }
    __device__ bool valid() const { return it.valid(); }
    __device__ bool at_job_start() const { return kt == kt_lo; }
    __device__ void advance() {
        if (++kt == kt_hi) {
            asm volatile("; next job" ::: "memory");   // rare: keep it a branch, out of the k-loop's straight path
            it.advance();
            enter();
        }
    }
};

// Epilogues that declare `static constexpr int TILE_STORES = n` promise that every wave issues exactly n
// vector-memory instructions in each tile() call (and none in job_end).  The memory counter retires in
// issue order and the operand loads of a tile's first k-step are issued before the previous tile's
// epilogue, so that k-step may start while those n stores are still in flight.
template <class E, class = void>
struct EpiTileStores : std::integral_constant<int, 0> {};
template <class E>
struct EpiTileStores<E, std::void_t<decltype(E::TILE_STORES)>> : std::integral_constant<int, E::TILE_STORES> {};

// An epilogue whose number of stores depends on the tile (masked edges) has `bool all_stores_issued() const`:
// the relaxed wait after its tile is taken only if it returns true.
template <class E, class = void>
struct EpiReportsStores : std::false_type {};
template <class E>
struct EpiReportsStores<E, std::void_t<decltype(std::declval<const E&>().all_stores_issued())>> : std::true_type {};

// Epilogues with `static constexpr bool HAS_TILE_BEGIN = true` get tile_begin<Cfg>(r0, c0) before the
// k-loop of every job; LDS it fills (also through direct-to-LDS loads) is visible in tile().
template <class E, class = void>
struct EpiHasTileBegin : std::false_type {};
template <class E>
struct EpiHasTileBegin<E, std::void_t<decltype(E::HAS_TILE_BEGIN)>> : std::bool_constant<E::HAS_TILE_BEGIN> {};

// Epilogues with `static constexpr bool DROPS_FRAGMENTS = true` need the registers that would carry the next
// k-step's first operand fragments across tile(): the last k-step of a job then reads nothing ahead and the next
// job's first k-step fetches its own fragments (one LDS round trip per tile instead of spills in the epilogue).
template <class E, class = void>
struct EpiDropsFragments : std::false_type {};
template <class E>
struct EpiDropsFragments<E, std::void_t<decltype(E::DROPS_FRAGMENTS)>> : std::bool_constant<E::DROPS_FRAGMENTS> {};


template <class Cfg, int AFMT, int BFMT, class Epi, class Iter = GridIter>
__global__ __launch_bounds__(Cfg::THREADS, Cfg::WGS_PER_CU) void gemm_tn_kernel(GemmOperands g, Epi epi) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem_all[];
    static_assert(Epi::EXTRA_LDS % 1024 == 0, "epilogue LDS must keep the stages 1 KiB aligned");
    static_assert(Cfg::NSTAGES == 2, "the k-loop below alternates between two LDS slots");
    uint8_t* const smem = smem_all + Epi::EXTRA_LDS;      // operand slots
    TileMainloop<Cfg, AFMT, BFMT> ml;
    ml.init();
    const int bid = blockIdx.x, G = gridDim.x;
    const int nk = g.K / Cfg::BK;
    AccCoords<Cfg> coords(ml.wr, ml.wc, ml.lane, (g.layout & kRowsPermuted) != 0);
    Iter cur(g, Cfg::BM, Cfg::BN, bid, G);
    // a walk over listed tiles usually has no job at all: leave before the epilogue's set-up (other walks go on, their
    // epilogues may have something to write for a workgroup without work)
    if constexpr (std::is_same<Iter, TileListIter>::value) { if (!cur.valid()) return; }

    // `pre` walks the (job, k-step) sequence of this workgroup ahead of the MFMAs; `ahead` counts the
    // k-steps whose operand loads have been issued and not yet consumed (at most one per slot).
    StepCursor<Iter> pre(cur, nk);
    int ahead = 0;
    auto refill = [&](int into_slot) {
        if (pre.valid()) {
            if (pre.at_job_start()) {
                asm volatile("; new tile" ::: "memory");   // rare: keep it a branch, out of the k-loop's straight path
                ml.issue_loads_b(smem);
                ml.set_tile(g, pre.it.tr() * Cfg::BM, pre.it.tc() * Cfg::BN, pre.kt);
            }
            ml.issue_loads(smem, into_slot);
            pre.advance();
            ++ahead;
        }
    };
    refill(0);
    ml.issue_loads_b(smem);
    refill(1);
    ml.issue_loads_b(smem);
    epi.begin(bid, G, smem_all);
    // operands of the first k-step
    if (ahead == 2) wait_vmem_le<Cfg::LOADS>();
    else wait_vmem_le<0>();
    wg_barrier();

    v16f acc[Cfg::TM][Cfg::TN];     // the first k-step of a job overwrites them
    v8i fa[Cfg::TM], fb = {};      // first fragments of the upcoming k-step, when `have`
#pragma unroll
    for (int t = 0; t < Cfg::TM; ++t) fa[t] = (v8i){};
    bool have = false;
    int slot = 0;
    bool first_job = true;
    bool prev_deferred = false;    // the previous job's epilogue kept its slot: the refill went out after its stores
    while (cur.valid()) {
        const int r0 = cur.tr() * Cfg::BM, c0 = cur.tc() * Cfg::BN;
        if (cur.job_begin()) epi.template job_begin<Cfg>(c0);   // made visible by the k-loop's barriers
        const int kt0 = cur.kt_begin(nk), kt1 = cur.kt_end(nk);
        if constexpr (EpiHasTileBegin<Epi>::value) epi.template tile_begin<Cfg>(r0, c0);
        // the epilogue of this job reuses the slot of its last k-step as scratch: keep loads out of it
        const bool keep_slot = Epi::NEEDS_SCRATCH || (Epi::JOB_END_NEEDS_SCRATCH && cur.job_end());
        // One k-step.  sync() runs before its last MFMA group: the next k-step's operands must have
        // landed (its loads are the newest load group in flight; the memory counter retires in issue
        // order, so anything issued after them -- the previous epilogue's stores -- may still be
        // pending), the workgroup meets, and the slot just read is refilled two k-steps ahead.
        auto kstep = [&](auto first, bool relaxed, bool last_kt) {
            // a k-step follows this one (and its first fragments may be read ahead)
            const bool more = ahead >= 2 && !(EpiDropsFragments<Epi>::value && last_kt);
            auto sync = [&]() {
                // only the wait differs between the relaxed and the plain first k-step: a scalar branch around it
                // instead of a second copy of the k-step
                if (decltype(first)::value && EpiTileStores<Epi>::value > 0 && relaxed) wait_vmem_le<EpiTileStores<Epi>::value>();
                else wait_vmem_le<0>();
                wg_barrier();
            };
            auto refill_here = [&]() {
                if (!(last_kt && keep_slot)) refill(slot);
                // before an epilogue both halves go out at once: the relaxed wait of the next job's first
                // k-step counts on every operand load having been issued before the epilogue's stores
                if (last_kt) ml.issue_loads_b(smem);
            };
            ml.template compute<decltype(first)::value, decltype(first)::value && EpiDropsFragments<Epi>::value>(
                smem, slot, slot ^ 1, have, more, acc, fa, fb, sync, refill_here);
            have = more && (TileMainloop<Cfg, AFMT, BFMT>::kAsmFrags16 || (AFMT & 3) != FMT_BF16);
            --ahead;
            slot ^= 1;
        };
        // relaxed wait: only behind an epilogue that stored (not the first job), with a later k-step of
        // the same job to wait for tile_begin's load, and only if that epilogue's refill was not deferred
        constexpr bool kMayRelax = !Epi::NEEDS_SCRATCH && EpiTileStores<Epi>::value > 0;
        bool relax = kMayRelax && !first_job && !prev_deferred && kt1 - kt0 >= 2;
        if constexpr (EpiReportsStores<Epi>::value) relax = relax && epi.all_stores_issued();
        kstep(std::true_type{}, relax, kt0 + 1 == kt1);
        first_job = false;
        for (int kt = kt0 + 1; kt < kt1; ++kt) kstep(std::false_type{}, false, kt + 1 == kt1);
        // every wave passed the last k-step's barrier after its final read of slot ^ 1
        uint8_t* free_stage = smem + (slot ^ 1) * Cfg::STAGE_BYTES;
        epi.partial(cur.partial(), cur.part_slot());
        epi.template tile<Cfg>(acc, r0, c0, coords, free_stage + ml.wave * Cfg::WAVE_SCRATCH, ml.lane);
        if (cur.job_end()) epi.template job_end<Cfg>(c0, cur.job_id(), coords, free_stage);
        if (keep_slot) {
            wg_barrier();          // all waves are done with the scratch
            refill(slot ^ 1);
            ml.issue_loads_b(smem);
        }
        prev_deferred = keep_slot;
        cur.advance();
    }
    wg_barrier();
    epi.end(smem, bid, G);
}

}  // namespace ngpt
