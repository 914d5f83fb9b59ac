// Panel-blocked fp8 operands (see GemmOperands in gemm_tn.h) and the kernels that produce them.
#pragma once
#include "gemm_tn.h"
#include "host_util.h"

namespace ngpt {

// Order of the 128 contraction bytes of one k-step row when the producer is the accumulator layout of
// the logits-recompute kernel (a lane owns one vocabulary column and the rows 8g + 4h + i of every
// 32-row MFMA tile): position 16h + 4g + i of a 32-group holds row 8g + 4h + i.
// token tt of a k-step (0..127) sits at byte dw_pos(tt) of the row
__host__ __device__ inline int dw_pos(int tt) { return (tt & ~31) | (((tt >> 2) & 1) << 4) | (((tt >> 3) & 3) << 2) | (tt & 3); }
__host__ __device__ inline int dw_pos_inv(int p) { return (p & ~31) | (((p >> 2) & 3) << 3) | (((p >> 4) & 1) << 2) | (p & 3); }

__host__ __device__ inline int64_t panel_offset(int row, int kbyte, int nk /* k-steps per row */) {
    return ((int64_t)(row >> 8) * nk + (kbyte >> 7)) * kPanelBytes + (row & 255) * 128;
}


constexpr int kPanelRaw = -1;    // panel_transpose: the input is fp8 bytes already

// 4 x 4 byte transpose: r[i] holds bytes (columns) 0..3 of row i; afterwards r[j] holds rows 0..3 of column j.
__device__ __forceinline__ void transpose4x4_bytes(uint32_t (&r)[4]) {
    // v_perm_b32 D = bytes of {S0, S1} picked by the selector, S1 = bytes 0..3, S0 = bytes 4..7
    const uint32_t a0 = __builtin_amdgcn_perm(r[1], r[0], 0x05010400);   // r0.b0 r1.b0 r0.b1 r1.b1
    const uint32_t a1 = __builtin_amdgcn_perm(r[1], r[0], 0x07030602);   // r0.b2 r1.b2 r0.b3 r1.b3
    const uint32_t b0 = __builtin_amdgcn_perm(r[3], r[2], 0x05010400);
    const uint32_t b1 = __builtin_amdgcn_perm(r[3], r[2], 0x07030602);
    r[0] = __builtin_amdgcn_perm(b0, a0, 0x05040100);   // a0.lo16 b0.lo16
    r[1] = __builtin_amdgcn_perm(b0, a0, 0x07060302);   // a0.hi16 b0.hi16
    r[2] = __builtin_amdgcn_perm(b1, a1, 0x05040100);
    r[3] = __builtin_amdgcn_perm(b1, a1, 0x07060302);
}

// Panel-blocked transpose of a row-major matrix: out row = input column c (c < cols), contraction = input
// rows [row0, row0 + nrows) padded with zeros to nk * 128, contraction bytes of each k-step permuted by
// PERM (0 none, 2 dw_pos).  QFMT = kPanelRaw: fp8 input, `ld` in bytes.  QFMT = FMT_E4M3 / FMT_E5M2: bf16
// input (`ld` in elements) quantised on the way as fp8(bf16(x / scale)).
// One workgroup moves a 128 (rows = one k-step) x 128 (columns) tile: 16 KiB of one panel block, contiguous.
// The tile sits in LDS as fp8 rows of 33 words with the word index XORed by 4 * (row / 16 % 8), which makes
// the transposing reads below conflict-free.  A thread then owns 4 columns x 16 rows: four 4 x 4 byte
// blocks, transposed in registers, are the four words of one 16-byte piece of each column's panel row;
// the 8 threads that share a column group are adjacent lanes, so they write whole 128-byte rows.
// The work of one workgroup of 256 threads: column group cg, k-step kt (also called by kernels that do several jobs in one launch).
template <int PERM, int QFMT>
__device__ __forceinline__ void panel_transpose_block(const uint8_t* __restrict__ in, int64_t ld, int row0, int nrows, int cols,
                                                      int nk, float scale, uint8_t* __restrict__ out, int cg, int kt) {
    constexpr int kStride = 33;
    __shared__ uint32_t tile[128 * kStride];
    const int tid = threadIdx.x;
    auto word_at = [&](int r, int w) -> uint32_t& { return tile[r * kStride + (w ^ (((r >> 4) & 7) << 2))]; };
    if (QFMT == kPanelRaw) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = tid + 256 * j, r = i >> 3, ch = i & 7;   // 16 input bytes = 16 columns
            const int gr = kt * 128 + r;
            v4i v = {0, 0, 0, 0};
            if (gr < nrows && cg * 128 + ch * 16 < cols) v = *(const v4i*)(in + (int64_t)(row0 + gr) * ld + cg * 128 + ch * 16);
#pragma unroll
            for (int k = 0; k < 4; ++k) word_at(r, ch * 4 + k) = (uint32_t)v[k];
        }
    } else {
        const QuantScale qs(scale);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int i = tid + 256 * j, r = i >> 4, ch = i & 15;  // 16 input bytes = 8 columns
            const int gr = kt * 128 + r;
            v2i q = {0, 0};
            if (gr < nrows && cg * 128 + ch * 8 < cols)
                q = quant8<QFMT == kPanelRaw ? 0 : QFMT>(*(const v4i*)(in + ((int64_t)(row0 + gr) * ld + cg * 128 + ch * 8) * 2), qs);
            word_at(r, ch * 2) = (uint32_t)q[0];
            word_at(r, ch * 2 + 1) = (uint32_t)q[1];
        }
    }
    __syncthreads();
    const int sub = tid & 7, cgp = tid >> 3;      // 16-byte piece of the 128-byte panel row, group of 4 columns
    // rows whose bytes make up piece `sub`: positions 16 sub ..+15 of the k-step, position 16h + 4g + i of a 32-group
    // holding row 8g + 4h + i under dw_pos
    const int rbase = PERM == 2 ? 32 * (sub >> 1) + 4 * (sub & 1) : 16 * sub;
    uint32_t w[4][4];   // [g][column]
#pragma unroll
    for (int g = 0; g < 4; ++g) {
#pragma unroll
        for (int i = 0; i < 4; ++i) w[g][i] = word_at(rbase + (PERM == 2 ? 8 : 4) * g + i, cgp);
        transpose4x4_bytes(w[g]);
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int col = cg * 128 + cgp * 4 + c;
        if (col < cols)
            *(v4i*)(out + panel_offset(col, kt * 128, nk) + sub * 16) = (v4i){(int)w[0][c], (int)w[1][c], (int)w[2][c], (int)w[3][c]};
    }
}

template <int PERM, int QFMT>
__global__ __launch_bounds__(256) void panel_transpose_kernel(const uint8_t* __restrict__ in, int64_t ld, int row0, int nrows, int cols,
                                                              int nk, float scale, uint8_t* __restrict__ out) {
    // neighbouring workgroups take neighbouring column groups of the same rows: together they read whole rows
    panel_transpose_block<PERM, QFMT>(in, ld, row0, nrows, cols, nk, scale, out, blockIdx.x, blockIdx.y);
}

template <int PERM, int QFMT = kPanelRaw>
static int panel_transpose(const void* in, int64_t ld, int row0, int nrows, int cols, int nk, void* out, hipStream_t st,
                           float scale = 1.0f) {
    if (cols % 16 || ld % 16) return fail(NGPT_EALIGN, "panel_transpose: cols=%d ld=%lld", cols, (long long)ld);
    dim3 grid((cols + 127) / 128, nk);
    panel_transpose_kernel<PERM, QFMT><<<grid, 256, 0, st>>>((const uint8_t*)in, ld, row0, nrows, cols, nk, scale, (uint8_t*)out);
    return check_launch("panel_transpose_kernel");
}

// Panel-blocked copy (no transpose) of a row-major fp8 matrix [rows, cols], cols % 128 == 0: 16 bytes per thread.
template <int UNUSED = 0>   // a template only so that it may be defined in this header
__global__ __launch_bounds__(256) void panel_pack_kernel(const uint8_t* __restrict__ in, int64_t ld, int rows, int cols,
                                                         uint8_t* __restrict__ out) {
    const int chunks = cols / 16;
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)rows * chunks) return;
    int r = (int)(i / chunks), c = (int)(i % chunks) * 16;
    *(v4i*)(out + panel_offset(r, c, cols / 128) + (c & 127)) = *(const v4i*)(in + (int64_t)r * ld + c);
}

static int panel_pack(const void* in, int64_t ld, int rows, int cols, void* out, hipStream_t st) {
    if (cols % 128 || ld % 16) return fail(NGPT_EALIGN, "panel_pack: cols=%d ld=%lld", cols, (long long)ld);
    int64_t n = (int64_t)rows * (cols / 16);
    panel_pack_kernel<0><<<(int)((n + 255) / 256), 256, 0, st>>>((const uint8_t*)in, ld, rows, cols, (uint8_t*)out);
    return check_launch("panel_pack_kernel");
}

}  // namespace ngpt
