// Small HBM-bound helpers around the FP8 MLP: delayed-scaling bookkeeping of the down projection
// and the tied-embedding gradient add.
#include "common.h"
#include "host_util.h"

namespace ngpt {

// scales[l] = max(max_i partial[l, i], 1e-12) * headroom / 448
__global__ __launch_bounds__(256) void reduce_scales_kernel(const float* __restrict__ partial, int64_t stride,
                                                            int count, float headroom, float* __restrict__ scales) {
    __shared__ float red[4];
    const int layer = blockIdx.x;
    float m = 0.0f;
    for (int i = threadIdx.x; i < count; i += 256) m = fmaxf(m, partial[layer * stride + i]);
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        float a = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        scales[layer] = fmaxf(a, 1.0e-12f) * (headroom / 448.0f);
    }
}

// 64 (hidden) x 64 (model) tile of layer l: out[l, d, h] = e4m3(clamp(w[l, h, d] / scale[l], +-448)),
// partial_amax[l, tile] = max |w| over the tile, used_scales[l] = scale[l].
__global__ __launch_bounds__(256) void quant_transpose_down_kernel(
    const uint16_t* __restrict__ w, int64_t layer_stride, int hidden, int model, const float* __restrict__ scales,
    uint8_t* __restrict__ out, float* __restrict__ used_scales, float* __restrict__ partial_amax, int tiles_d, int tiles) {
    __shared__ uint8_t tile[64][64 + 4];   // [d][h]
    __shared__ float red[4];
    const int layer = blockIdx.y, t = blockIdx.x;
    const int h0 = (t / tiles_d) * 64, d0 = (t % tiles_d) * 64;
    const float scale = scales[layer];
    const uint16_t* wl = w + layer * layer_stride;
    float amax = 0.0f;
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        int hl = p * 32 + (threadIdx.x >> 3), dl = (threadIdx.x & 7) * 8;
        int h = h0 + hl, d = d0 + dl;
        if (h < hidden && d < model) {
            v4i v = *(const v4i*)(wl + (int64_t)h * model + d);
            uint32_t u[4] = {(uint32_t)v.x, (uint32_t)v.y, (uint32_t)v.z, (uint32_t)v.w};
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float x = bf16_bits_to_f32((u[i >> 1] >> (16 * (i & 1))) & 0xffffu);
                amax = fmaxf(amax, fabsf(x));
                tile[dl + i][hl] = (uint8_t)f32_to_e4m3_sat(__fdiv_rn(x, scale));
            }
        }
    }
    amax = wave_max(amax);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
    __syncthreads();
    {
        int dl = threadIdx.x >> 2, ch = (threadIdx.x & 3) * 16;
        int d = d0 + dl, h = h0 + ch;
        if (d < model && h < hidden) {
            uint32_t q[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) q[i] = *(const uint32_t*)&tile[dl][ch + 4 * i];
            *(v4i*)(out + ((int64_t)layer * model + d) * hidden + h) = (v4i){(int)q[0], (int)q[1], (int)q[2], (int)q[3]};
        }
    }
    if (threadIdx.x == 0) {
        partial_amax[(int64_t)layer * tiles + t] = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        if (t == 0) used_scales[layer] = scale;
    }
}

// dst [cols, rows] += src [rows, cols]^T, 64 x 64 tiles through LDS; T = bf16 bits (fp32 add, one rounding) or float.
template <class T>
__global__ __launch_bounds__(256) void transpose_add_kernel(const T* __restrict__ src, int rows, int cols, T* __restrict__ dst) {
    __shared__ float tile[64][65];
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        int rl = i >> 6, cl = i & 63;
        int r = r0 + rl, c = c0 + cl;
        float v = 0.0f;
        if (r < rows && c < cols) {
            if constexpr (sizeof(T) == 2) v = bf16_bits_to_f32(src[(int64_t)r * cols + c]);
            else v = src[(int64_t)r * cols + c];
        }
        tile[rl][cl] = v;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        int cl = i >> 6, rl = i & 63;       // dst row = source column
        int r = r0 + rl, c = c0 + cl;
        if (r < rows && c < cols) {
            T* p = dst + (int64_t)c * rows + r;
            if constexpr (sizeof(T) == 2) *p = (T)f32_to_bf16_bits(bf16_bits_to_f32(*p) + tile[rl][cl]);
            else *p = *p + tile[rl][cl];
        }
    }
}

}  // namespace ngpt

using namespace ngpt;

extern "C" int ngpt_reduce_scales(const float* partial_amax, int64_t partial_stride, int num_layers, int partial_count,
                                  float headroom, float* scales, void* stream) {
    if (!partial_amax || !scales || num_layers <= 0 || partial_count <= 0)
        return fail(NGPT_EINVAL, "ngpt_reduce_scales: null pointer or empty input");
    reduce_scales_kernel<<<num_layers, 256, 0, (hipStream_t)stream>>>(partial_amax, partial_stride, partial_count, headroom, scales);
    return check_launch("reduce_scales_kernel");
}

extern "C" int ngpt_quant_transpose_down(const void* weights_bf16, int num_layers, int hidden, int model_dim,
                                         int64_t layer_stride, const float* scales, void* out_f8, float* used_scales,
                                         float* partial_amax, void* stream) {
    if (!weights_bf16 || !scales || !out_f8 || !used_scales || !partial_amax)
        return fail(NGPT_EINVAL, "ngpt_quant_transpose_down: null pointer");
    if (num_layers <= 0 || hidden <= 0 || model_dim <= 0) return fail(NGPT_EINVAL, "ngpt_quant_transpose_down: empty input");
    if (hidden % 16 || model_dim % 16)
        return fail(NGPT_EALIGN, "ngpt_quant_transpose_down: hidden=%d and model_dim=%d must be multiples of 16", hidden, model_dim);
    int tiles_d = (model_dim + 63) / 64, tiles_h = (hidden + 63) / 64;
    dim3 grid(tiles_d * tiles_h, num_layers);
    quant_transpose_down_kernel<<<grid, 256, 0, (hipStream_t)stream>>>(
        (const uint16_t*)weights_bf16, layer_stride, hidden, model_dim, scales, (uint8_t*)out_f8, used_scales,
        partial_amax, tiles_d, tiles_d * tiles_h);
    return check_launch("quant_transpose_down_kernel");
}

extern "C" int ngpt_transpose_add(const void* src, int rows, int cols, void* dst, int elem_bytes, void* stream) {
    if (!src || !dst || rows <= 0 || cols <= 0) return fail(NGPT_EINVAL, "ngpt_transpose_add: null pointer or empty matrix");
    dim3 grid((cols + 63) / 64, (rows + 63) / 64);
    if (elem_bytes == 2)
        transpose_add_kernel<uint16_t><<<grid, 256, 0, (hipStream_t)stream>>>((const uint16_t*)src, rows, cols, (uint16_t*)dst);
    else if (elem_bytes == 4)
        transpose_add_kernel<float><<<grid, 256, 0, (hipStream_t)stream>>>((const float*)src, rows, cols, (float*)dst);
    else
        return fail(NGPT_EINVAL, "ngpt_transpose_add: elem_bytes=%d (2 = bf16, 4 = fp32)", elem_bytes);
    return check_launch("transpose_add_kernel");
}
