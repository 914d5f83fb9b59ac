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

// Panel-blocked transpose of a row-major matrix: out row = input column c (c < cols), contraction = input
// rows [row0, row0 + nrows) padded with zeros to nk * 128, contraction bytes of each k-step permuted by
// PERM (0 none, 2 dw_pos).  QFMT = kPanelRaw: fp8 input, `ld` in bytes.  QFMT = FMT_E4M3 / FMT_E5M2: bf16
// input (`ld` in elements) quantised on the way as fp8(bf16(x / scale)).  One workgroup moves a 128 (rows) x
// 64 (columns) tile.
template <int PERM, int QFMT>
__global__ __launch_bounds__(256) void panel_transpose_kernel(const uint8_t* __restrict__ in, int64_t ld, int row0, int nrows, int cols,
                                                              int nk, float scale, uint8_t* __restrict__ out) {
    __shared__ __attribute__((aligned(16))) uint8_t tile[128][80];
    const int kt = blockIdx.x, cg = blockIdx.y, tid = threadIdx.x;
    if (QFMT == kPanelRaw) {
        for (int i = tid; i < 512; i += 256) {
            int r = i >> 2, ch = i & 3;
            int gr = kt * 128 + r;
            v4i v = {0, 0, 0, 0};
            if (gr < nrows && cg * 64 + ch * 16 < cols) v = *(const v4i*)(in + (int64_t)(row0 + gr) * ld + cg * 64 + ch * 16);
            *(v4i*)&tile[r][ch * 16] = v;
        }
    } else {
        for (int i = tid; i < 1024; i += 256) {
            int r = i >> 3, ch = i & 7;
            int gr = kt * 128 + r;
            v2i q = {0, 0};
            if (gr < nrows && cg * 64 + ch * 8 < cols)
                q = quant8<QFMT == kPanelRaw ? 0 : QFMT>(*(const v4i*)(in + ((int64_t)(row0 + gr) * ld + cg * 64 + ch * 8) * 2), scale);
            *(v2i*)&tile[r][ch * 8] = q;
        }
    }
    __syncthreads();
    const int o = tid >> 2, part = tid & 3;
    const int c = cg * 64 + o;
    if (c >= cols) return;
    uint32_t w[8];
#pragma unroll
    for (int d = 0; d < 8; ++d) {
        uint32_t word = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            int p = part * 32 + d * 4 + b;
            int t = PERM == 2 ? dw_pos_inv(p) : p;
            word |= (uint32_t)tile[t][o] << (8 * b);
        }
        w[d] = word;
    }
    uint8_t* dst = out + panel_offset(c, kt * 128, nk) + part * 32;
    *(v4i*)dst = (v4i){(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
    *(v4i*)(dst + 16) = (v4i){(int)w[4], (int)w[5], (int)w[6], (int)w[7]};
}

template <int PERM, int QFMT = kPanelRaw>
static int panel_transpose(const void* in, int64_t ld, int row0, int nrows, int cols, int nk, void* out, hipStream_t st,
                           float scale = 1.0f) {
    if (cols % 16 || ld % 16) return fail(NGPT_EALIGN, "panel_transpose: cols=%d ld=%lld", cols, (long long)ld);
    dim3 grid(nk, (cols + 63) / 64);
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
