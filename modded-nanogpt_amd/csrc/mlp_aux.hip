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

// dst [cols, rows] = src [rows, cols]^T for 2- and 4-byte elements, 64 x 64 tiles through LDS (the 1-byte
// case has its own kernel with 16-byte accesses, tile_transpose_kernel).
template <class T>
__global__ __launch_bounds__(256) void transpose_copy_kernel(const T* __restrict__ src, int rows, int cols, T* __restrict__ dst) {
    __shared__ T tile[64][64 + (sizeof(T) == 2 ? 2 : 1)];
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        const int rl = i >> 6, cl = i & 63;
        const int r = r0 + rl, c = c0 + cl;
        if (r < rows && c < cols) tile[rl][cl] = src[(int64_t)r * cols + c];
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        const int cl = i >> 6, rl = i & 63;       // dst row = source column
        const int r = r0 + rl, c = c0 + cl;
        if (r < rows && c < cols) dst[(int64_t)c * rows + r] = tile[rl][cl];
    }
}

// ---------------------------------------------------------------------------------------------
// MLP input producer: rms-norm, per-tensor amax and dynamic e4m3 quantisation (two passes over the
// activations instead of the two reductions plus two element-wise passes of the eager formulation).
constexpr int kNormPartials = 1024;      // per-workgroup running maxima of |normed|

// Pass 1.  One wave per row: normed = bf16(x * rsqrt(mean(x^2) + eps)) in fp32 like F.rms_norm on
// bf16 input with eps = None (machine epsilon of fp32); partial[bid] = max |normed| seen by the workgroup.
__global__ __launch_bounds__(256) void rmsnorm_amax_kernel(const uint16_t* __restrict__ x, int rows, int dim,
                                                           uint16_t* __restrict__ normed, float* __restrict__ partial) {
    __shared__ float red[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int chunks = dim / 8;              // 16-byte chunks per row
    float amax = 0.0f;
    for (int row = blockIdx.x * 4 + wave; row < rows; row += gridDim.x * 4) {
        const v4i* xr = (const v4i*)(x + (int64_t)row * dim);
        v4i buf[4];                          // up to 4 chunks per lane: dim <= 2048
        float ss = 0.0f;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            int ch = lane + 64 * c;
            if (ch < chunks) {
                buf[c] = xr[ch];
                const uint32_t u[4] = {(uint32_t)buf[c].x, (uint32_t)buf[c].y, (uint32_t)buf[c].z, (uint32_t)buf[c].w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float lo = bf16_bits_to_f32(u[i] & 0xffffu), hi = bf16_bits_to_f32(u[i] >> 16);
                    ss += lo * lo + hi * hi;
                }
            }
        }
        ss = wave_sum(ss);
        const float r = __fdiv_rn(1.0f, __fsqrt_rn(ss / (float)dim + 1.1920928955078125e-07f));
        v4i* nr = (v4i*)(normed + (int64_t)row * dim);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            int ch = lane + 64 * c;
            if (ch < chunks) {
                const uint32_t u[4] = {(uint32_t)buf[c].x, (uint32_t)buf[c].y, (uint32_t)buf[c].z, (uint32_t)buf[c].w};
                uint32_t o[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float lo = round_to_bf16(bf16_bits_to_f32(u[i] & 0xffffu) * r);
                    float hi = round_to_bf16(bf16_bits_to_f32(u[i] >> 16) * r);
                    amax = fmaxf(amax, fmaxf(fabsf(lo), fabsf(hi)));
                    o[i] = (__float_as_uint(lo) >> 16) | (__float_as_uint(hi) & 0xffff0000u);
                }
                nr[ch] = (v4i){(int)o[0], (int)o[1], (int)o[2], (int)o[3]};
            }
        }
    }
    amax = wave_max(amax);
    if (lane == 0) red[wave] = amax;
    __syncthreads();
    if (threadIdx.x == 0) partial[blockIdx.x] = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

__device__ __forceinline__ float block_max_of(const float* __restrict__ v, int n, float* red) {
    float m = 0.0f;
    for (int i = threadIdx.x; i < n; i += 256) m = fmaxf(m, v[i]);
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    return fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

// Pass 2.  amax = max(partials) clamped to bf16(1e-12); x_f8 = e4m3(bf16(normed * q)) with
// q = bf16(bf16(1 / amax) * 448): every bf16 operation of the eager expression rounds, and eager evaluates
// `448.0 / amax` (Python float over a bf16 tensor) as amax.reciprocal() * 448.0, not as one division -- the two
// differ in the last bf16 digit for about a quarter of all amax values.  dequant[0] = up_scale * amax / 448 in fp32.
__global__ __launch_bounds__(256) void amax_quant_kernel(const v4i* __restrict__ normed, int64_t n8, const float* __restrict__ partial,
                                                         int npartial, const float* __restrict__ up_scale,
                                                         v2i* __restrict__ x_f8, float* __restrict__ dequant) {
    __shared__ float red[4];
    float amax = fmaxf(block_max_of(partial, npartial, red), round_to_bf16(1.0e-12f));
    if (blockIdx.x == 0 && threadIdx.x == 0) dequant[0] = __fdiv_rn(up_scale[0] * amax, 448.0f);
    const float q = round_to_bf16(round_to_bf16(__fdiv_rn(1.0f, amax)) * 448.0f);
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += (int64_t)gridDim.x * 256) {
        v4i v = normed[i];
        const uint32_t u[4] = {(uint32_t)v.x, (uint32_t)v.y, (uint32_t)v.z, (uint32_t)v.w};
        uint32_t c[8];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            c[2 * k] = f32_to_e4m3_torch(round_to_bf16(bf16_bits_to_f32(u[k] & 0xffffu) * q));
            c[2 * k + 1] = f32_to_e4m3_torch(round_to_bf16(bf16_bits_to_f32(u[k] >> 16) * q));
        }
        x_f8[i] = (v2i){(int)(c[0] | c[1] << 8 | c[2] << 16 | c[3] << 24), (int)(c[4] | c[5] << 8 | c[6] << 16 | c[7] << 24)};
    }
}

// Up-projection weights, per layer: partial[l, b] = max |w| over a slice of layer l ...
__global__ __launch_bounds__(256) void layer_amax_kernel(const v4i* __restrict__ w, int64_t n8_per_layer, float* __restrict__ partial) {
    __shared__ float red[4];
    const int layer = blockIdx.y;
    const v4i* wl = w + layer * n8_per_layer;
    float m = 0.0f;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n8_per_layer; i += (int64_t)gridDim.x * 256) {
        v4i v = wl[i];
        const uint32_t u[4] = {(uint32_t)v.x, (uint32_t)v.y, (uint32_t)v.z, (uint32_t)v.w};
#pragma unroll
        for (int k = 0; k < 4; ++k)
            m = fmaxf(m, fmaxf(fabsf(bf16_bits_to_f32(u[k] & 0xffffu)), fabsf(bf16_bits_to_f32(u[k] >> 16))));
    }
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) partial[layer * gridDim.x + blockIdx.x] = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

// ... then scale[l] = bf16(max(amax_l, bf16(1e-12)) / 448) and w_f8 = e4m3(bf16(w / scale[l])).
__global__ __launch_bounds__(256) void layer_quant_kernel(const v4i* __restrict__ w, int64_t n8_per_layer, const float* __restrict__ partial,
                                                          int npartial, v2i* __restrict__ w_f8, float* __restrict__ scales) {
    __shared__ float red[4];
    const int layer = blockIdx.y;
    const float amax = fmaxf(block_max_of(partial + layer * npartial, npartial, red), round_to_bf16(1.0e-12f));
    const float scale = round_to_bf16(__fdiv_rn(amax, 448.0f));
    if (blockIdx.x == 0 && threadIdx.x == 0) scales[layer] = scale;
    const v4i* wl = w + layer * n8_per_layer;
    v2i* ol = w_f8 + layer * n8_per_layer;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n8_per_layer; i += (int64_t)gridDim.x * 256) {
        v4i v = wl[i];
        const uint32_t u[4] = {(uint32_t)v.x, (uint32_t)v.y, (uint32_t)v.z, (uint32_t)v.w};
        uint32_t c[8];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            c[2 * k] = f32_to_e4m3_torch(round_to_bf16(__fdiv_rn(bf16_bits_to_f32(u[k] & 0xffffu), scale)));
            c[2 * k + 1] = f32_to_e4m3_torch(round_to_bf16(__fdiv_rn(bf16_bits_to_f32(u[k] >> 16), scale)));
        }
        ol[i] = (v2i){(int)(c[0] | c[1] << 8 | c[2] << 16 | c[3] << 24), (int)(c[4] | c[5] << 8 | c[6] << 16 | c[7] << 24)};
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

extern "C" int ngpt_transpose_copy(const void* src, int rows, int cols, void* dst, int elem_bytes, void* stream) {
    if (!src || !dst || rows <= 0 || cols <= 0) return fail(NGPT_EINVAL, "ngpt_transpose_copy: null pointer or empty matrix");
    if (elem_bytes == 1 && rows % 16 == 0 && cols % 16 == 0) return ngpt_transpose_u8(src, rows, cols, dst, stream);
    dim3 grid((cols + 63) / 64, (rows + 63) / 64);
    if (elem_bytes == 1)
        transpose_copy_kernel<uint8_t><<<grid, 256, 0, (hipStream_t)stream>>>((const uint8_t*)src, rows, cols, (uint8_t*)dst);
    else if (elem_bytes == 2)
        transpose_copy_kernel<uint16_t><<<grid, 256, 0, (hipStream_t)stream>>>((const uint16_t*)src, rows, cols, (uint16_t*)dst);
    else if (elem_bytes == 4)
        transpose_copy_kernel<uint32_t><<<grid, 256, 0, (hipStream_t)stream>>>((const uint32_t*)src, rows, cols, (uint32_t*)dst);
    else
        return fail(NGPT_EINVAL, "ngpt_transpose_copy: elem_bytes=%d (1, 2 or 4)", elem_bytes);
    return check_launch("transpose_copy_kernel");
}

extern "C" int64_t ngpt_mlp_input_quant_workspace_bytes(void) { return kNormPartials * (int64_t)sizeof(float); }

extern "C" int ngpt_mlp_input_quant(const void* x_bf16, int rows, int dim, const float* up_scale, void* normed_bf16,
                                    void* x_f8, float* dequant, void* workspace, int64_t workspace_bytes, void* stream) {
    if (!x_bf16 || !up_scale || !normed_bf16 || !x_f8 || !dequant || !workspace)
        return fail(NGPT_EINVAL, "ngpt_mlp_input_quant: null pointer");
    if (rows <= 0 || dim <= 0) return fail(NGPT_EINVAL, "ngpt_mlp_input_quant: empty problem rows=%d dim=%d", rows, dim);
    if (dim % 8 || dim > 2048) return fail(NGPT_EALIGN, "ngpt_mlp_input_quant: dim=%d must be a multiple of 8 and at most 2048", dim);
    if (workspace_bytes < ngpt_mlp_input_quant_workspace_bytes())
        return fail(NGPT_EWORKSPACE, "ngpt_mlp_input_quant: workspace %lld < %lld bytes", (long long)workspace_bytes,
                    (long long)ngpt_mlp_input_quant_workspace_bytes());
    hipStream_t st = (hipStream_t)stream;
    ProfileScope prof(PROF_PRODUCERS, st);
    float* partial = (float*)workspace;
    int blocks = (rows + 3) / 4;
    if (blocks > kNormPartials) blocks = kNormPartials;
    rmsnorm_amax_kernel<<<blocks, 256, 0, st>>>((const uint16_t*)x_bf16, rows, dim, (uint16_t*)normed_bf16, partial);
    if (int e = check_launch("rmsnorm_amax_kernel")) return e;
    const int64_t n8 = (int64_t)rows * dim / 8;
    int grid = (int)((n8 + 255) / 256 < (int64_t)num_cus() * 8 ? (n8 + 255) / 256 : (int64_t)num_cus() * 8);
    amax_quant_kernel<<<grid, 256, 0, st>>>((const v4i*)normed_bf16, n8, partial, blocks, up_scale, (v2i*)x_f8, dequant);
    return check_launch("amax_quant_kernel");
}

// Backward of y = x * rsqrt(mean(x^2) + eps) (F.rms_norm on bf16 input, eps = fp32 machine epsilon):
// dx = r * g - x * r^3 * mean(g * x), r = rsqrt(mean(x^2) + eps), in fp32, rounded to bf16 once.
// One wave per row, the row's x and g stay in registers between the reduction and the output.
__global__ __launch_bounds__(256) void rmsnorm_bwd_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ g, int rows,
                                                          int dim, uint16_t* __restrict__ dx) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int chunks = dim / 8;              // 16-byte chunks per row
    for (int row = blockIdx.x * 4 + wave; row < rows; row += gridDim.x * 4) {
        const v4i* xr = (const v4i*)(x + (int64_t)row * dim);
        const v4i* gr = (const v4i*)(g + (int64_t)row * dim);
        v4i bx[4], bg[4];                    // up to 4 chunks per lane: dim <= 2048
        float ss = 0.0f, sg = 0.0f;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int ch = lane + 64 * c;
            if (ch < chunks) {
                bx[c] = xr[ch];
                bg[c] = gr[ch];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t ux = (uint32_t)bx[c][i], ug = (uint32_t)bg[c][i];
                    const float x0 = bf16_bits_to_f32(ux & 0xffffu), x1 = bf16_bits_to_f32(ux >> 16);
                    const float g0 = bf16_bits_to_f32(ug & 0xffffu), g1 = bf16_bits_to_f32(ug >> 16);
                    ss += x0 * x0 + x1 * x1;
                    sg += g0 * x0 + g1 * x1;
                }
            }
        }
        ss = wave_sum(ss);
        sg = wave_sum(sg);
        const float r = __fdiv_rn(1.0f, __fsqrt_rn(ss / (float)dim + 1.1920928955078125e-07f));
        const float k = r * r * r * (sg / (float)dim);
        v4i* out = (v4i*)(dx + (int64_t)row * dim);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int ch = lane + 64 * c;
            if (ch < chunks) {
                v4i o;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t ux = (uint32_t)bx[c][i], ug = (uint32_t)bg[c][i];
                    const float d0 = r * bf16_bits_to_f32(ug & 0xffffu) - k * bf16_bits_to_f32(ux & 0xffffu);
                    const float d1 = r * bf16_bits_to_f32(ug >> 16) - k * bf16_bits_to_f32(ux >> 16);
                    o[i] = (int)cvt_pk_bf16(d0, d1);
                }
                out[ch] = o;
            }
        }
    }
}

extern "C" int ngpt_rmsnorm_bwd(const void* x_bf16, const void* g_bf16, int rows, int dim, void* dx_bf16, void* stream) {
    if (!x_bf16 || !g_bf16 || !dx_bf16) return fail(NGPT_EINVAL, "ngpt_rmsnorm_bwd: null pointer");
    if (rows <= 0 || dim <= 0) return fail(NGPT_EINVAL, "ngpt_rmsnorm_bwd: empty problem");
    if (dim % 8 || dim > 2048) return fail(NGPT_EALIGN, "ngpt_rmsnorm_bwd: dim=%d must be a multiple of 8 and <= 2048", dim);
    int blocks = (rows + 3) / 4;
    const int cap = num_cus() * 16;
    if (blocks > cap) blocks = cap;
    ProfileScope prof(PROF_PRODUCERS, (hipStream_t)stream);
    rmsnorm_bwd_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>((const uint16_t*)x_bf16, (const uint16_t*)g_bf16, rows, dim, (uint16_t*)dx_bf16);
    return check_launch("rmsnorm_bwd_kernel");
}

constexpr int kLayerPartials = 64;
extern "C" int64_t ngpt_quant_up_weights_workspace_bytes(int layers) { return (int64_t)layers * kLayerPartials * sizeof(float); }

extern "C" int ngpt_quant_up_weights(const void* w_bf16, int layers, int64_t per_layer, void* w_f8, float* scales,
                                     void* workspace, int64_t workspace_bytes, void* stream) {
    if (!w_bf16 || !w_f8 || !scales || !workspace) return fail(NGPT_EINVAL, "ngpt_quant_up_weights: null pointer");
    if (layers <= 0 || per_layer <= 0) return fail(NGPT_EINVAL, "ngpt_quant_up_weights: empty problem");
    if (per_layer % 8) return fail(NGPT_EALIGN, "ngpt_quant_up_weights: elements per layer (%lld) must be a multiple of 8", (long long)per_layer);
    if (workspace_bytes < ngpt_quant_up_weights_workspace_bytes(layers))
        return fail(NGPT_EWORKSPACE, "ngpt_quant_up_weights: workspace %lld < %lld bytes", (long long)workspace_bytes,
                    (long long)ngpt_quant_up_weights_workspace_bytes(layers));
    hipStream_t st = (hipStream_t)stream;
    const int64_t n8 = per_layer / 8;
    layer_amax_kernel<<<dim3(kLayerPartials, layers), 256, 0, st>>>((const v4i*)w_bf16, n8, (float*)workspace);
    if (int e = check_launch("layer_amax_kernel")) return e;
    layer_quant_kernel<<<dim3(kLayerPartials, layers), 256, 0, st>>>((const v4i*)w_bf16, n8, (const float*)workspace, kLayerPartials,
                                                                    (v2i*)w_f8, scales);
    return check_launch("layer_quant_kernel");
}
