// bf16 -> fp8 quantisers and byte transposes (HBM-bound, one pass over the input).
#include "common.h"
#include "host_util.h"

namespace ngpt {

template <int FMT>
__global__ __launch_bounds__(256) void quant_kernel(const v4i* __restrict__ in, v2i* __restrict__ out,
                                                    int64_t n8, float s) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * 256;
    const QuantScale qs(s);
    for (; i < n8; i += stride) out[i] = quant8<FMT>(in[i], qs);
}

// Two tensors in one launch (activations and weights ahead of a GEMM): blocks [0, blocks0) take the first.
__global__ __launch_bounds__(256) void quant_pair_kernel(const v4i* __restrict__ in0, v2i* __restrict__ out0, int64_t n8_0, float s0,
                                                         const v4i* __restrict__ in1, v2i* __restrict__ out1, int64_t n8_1, float s1,
                                                         int blocks0) {
    const bool first = (int)blockIdx.x < blocks0;
    const v4i* in = first ? in0 : in1;
    v2i* out = first ? out0 : out1;
    const int64_t n8 = first ? n8_0 : n8_1;
    const int b = first ? blockIdx.x : blockIdx.x - blocks0, nb = first ? blocks0 : gridDim.x - blocks0;
    const QuantScale qs(first ? s0 : s1);
    for (int64_t i = (int64_t)b * 256 + threadIdx.x; i < n8; i += (int64_t)nb * 256) out[i] = quant8<FMT_E4M3>(in[i], qs);
}

// 64 x 64 tile: quantise, write the row-major bytes, and write the transposed bytes via LDS.
// IN_BYTES = 2: bf16 input quantised with scale s.  IN_BYTES = 1: plain byte transpose.
template <int FMT, int IN_BYTES>
__global__ __launch_bounds__(256) void tile_transpose_kernel(const uint8_t* __restrict__ in, int rows, int cols,
                                                             float s, uint8_t* __restrict__ out,
                                                             uint8_t* __restrict__ out_t) {
    __shared__ uint8_t tile[64][64 + 4];   // [col][row]
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    const int t = threadIdx.x;
    const QuantScale qs(s);
    // phase 1: each thread handles 8 consecutive columns of one row; 8 threads per row, 32 rows per pass
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        int rl = p * 32 + (t >> 3), cl = (t & 7) * 8;
        int r = r0 + rl, c = c0 + cl;
        v2i q = {0, 0};
        if (r < rows && c < cols) {
            if (IN_BYTES == 2) {
                v4i v = *(const v4i*)(in + ((int64_t)r * cols + c) * 2);
                q = quant8<FMT>(v, qs);
                if (out) *(v2i*)(out + (int64_t)r * cols + c) = q;
            } else {
                q = *(const v2i*)(in + (int64_t)r * cols + c);
            }
        }
        uint32_t lo = (uint32_t)q.x, hi = (uint32_t)q.y;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            tile[cl + i][rl] = (uint8_t)(lo >> (8 * i));
            tile[cl + 4 + i][rl] = (uint8_t)(hi >> (8 * i));
        }
    }
    __syncthreads();
    // phase 2: 64 transposed rows of 64 bytes = 256 pieces of 16 bytes
    if (out_t) {
        int cl = t >> 2, ch = (t & 3) * 16;
        int c = c0 + cl, r = r0 + ch;
        if (c < cols && r < rows) {
            uint32_t w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) w[i] = *(const uint32_t*)&tile[cl][ch + 4 * i];
            *(v4i*)(out_t + (int64_t)c * rows + r) = (v4i){(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
        }
    }
}

}  // namespace ngpt

using namespace ngpt;

namespace ngpt {
// e4m3 copies of two bf16 tensors (n0, n1 elements, multiples of 8) in one launch.
int quant_e4m3_pair(const void* in0, void* out0, int64_t n0, float s0, const void* in1, void* out1, int64_t n1, float s1,
                    hipStream_t st) {
    if (n0 % 8 || n1 % 8 || n0 <= 0 || n1 <= 0) return fail(NGPT_EALIGN, "quant_e4m3_pair: sizes %lld, %lld", (long long)n0, (long long)n1);
    const int64_t cap = (int64_t)num_cus() * 16;
    // blocks in proportion to the sizes, at least one each
    int64_t b0 = (n0 / 8 + 255) / 256, b1 = (n1 / 8 + 255) / 256;
    if (b0 + b1 > cap) {
        b0 = b0 * cap / (b0 + b1);
        if (b0 < 1) b0 = 1;
        b1 = cap - b0 < 1 ? 1 : cap - b0;
    }
    quant_pair_kernel<<<(int)(b0 + b1), 256, 0, st>>>((const v4i*)in0, (v2i*)out0, n0 / 8, s0, (const v4i*)in1, (v2i*)out1, n1 / 8, s1, (int)b0);
    return check_launch("quant_pair_kernel");
}
}  // namespace ngpt

extern "C" int ngpt_quant_fp8(const void* in_bf16, void* out_f8, int64_t n, float scale, int fmt, void* stream) {
    if (!in_bf16 || !out_f8 || n < 0) return fail(NGPT_EINVAL, "ngpt_quant_fp8: null pointer or negative size");
    if (n % 8) return fail(NGPT_EALIGN, "ngpt_quant_fp8: n=%lld must be a multiple of 8", (long long)n);
    if (fmt != NGPT_FMT_E4M3 && fmt != NGPT_FMT_E5M2) return fail(NGPT_EINVAL, "ngpt_quant_fp8: fmt=%d", fmt);
    if (n == 0) return NGPT_OK;
    int64_t n8 = n / 8;
    int grid = (int)((n8 + 255) / 256 < (int64_t)num_cus() * 16 ? (n8 + 255) / 256 : (int64_t)num_cus() * 16);
    hipStream_t st = (hipStream_t)stream;
    if (fmt == NGPT_FMT_E4M3)
        quant_kernel<FMT_E4M3><<<grid, 256, 0, st>>>((const v4i*)in_bf16, (v2i*)out_f8, n8, scale);
    else
        quant_kernel<FMT_E5M2><<<grid, 256, 0, st>>>((const v4i*)in_bf16, (v2i*)out_f8, n8, scale);
    return check_launch("quant_kernel");
}

extern "C" int ngpt_quant_fp8_2d(const void* in_bf16, int rows, int cols, float scale, int fmt,
                                 void* out_f8, void* out_f8_t, void* stream) {
    if (!in_bf16 || rows <= 0 || cols <= 0 || (!out_f8 && !out_f8_t))
        return fail(NGPT_EINVAL, "ngpt_quant_fp8_2d: null pointer or empty matrix");
    if (rows % 16 || cols % 16)
        return fail(NGPT_EALIGN, "ngpt_quant_fp8_2d: rows=%d and cols=%d must be multiples of 16", rows, cols);
    if (fmt != NGPT_FMT_E4M3 && fmt != NGPT_FMT_E5M2) return fail(NGPT_EINVAL, "ngpt_quant_fp8_2d: fmt=%d", fmt);
    hipStream_t st = (hipStream_t)stream;
    if (!out_f8_t) return ngpt_quant_fp8(in_bf16, out_f8, (int64_t)rows * cols, scale, fmt, stream);
    dim3 grid((cols + 63) / 64, (rows + 63) / 64);
    if (fmt == NGPT_FMT_E4M3)
        tile_transpose_kernel<FMT_E4M3, 2><<<grid, 256, 0, st>>>((const uint8_t*)in_bf16, rows, cols, scale,
                                                                (uint8_t*)out_f8, (uint8_t*)out_f8_t);
    else
        tile_transpose_kernel<FMT_E5M2, 2><<<grid, 256, 0, st>>>((const uint8_t*)in_bf16, rows, cols, scale,
                                                                (uint8_t*)out_f8, (uint8_t*)out_f8_t);
    return check_launch("tile_transpose_kernel(quant)");
}

extern "C" int ngpt_transpose_u8(const void* in, int rows, int cols, void* out, void* stream) {
    if (!in || !out || rows <= 0 || cols <= 0) return fail(NGPT_EINVAL, "ngpt_transpose_u8: null pointer or empty matrix");
    if (rows % 16 || cols % 16)
        return fail(NGPT_EALIGN, "ngpt_transpose_u8: rows=%d and cols=%d must be multiples of 16", rows, cols);
    dim3 grid((cols + 63) / 64, (rows + 63) / 64);
    tile_transpose_kernel<FMT_E4M3, 1><<<grid, 256, 0, (hipStream_t)stream>>>((const uint8_t*)in, rows, cols, 1.0f,
                                                                             nullptr, (uint8_t*)out);
    return check_launch("tile_transpose_kernel(u8)");
}
