// Measurement build only (-DNGPT_BENCH_BUILD): a microbenchmark of the k-step skeleton of the fp8 GEMM, used to
// find what an MFMA-bound loop of this instruction mix can reach on a given machine (clock under load included).
// One workgroup per compute unit, 8 waves, each wave 2 x 4 MFMA tiles of v_mfma_f32_32x32x64_f8f6f4 per contraction
// sub-step, i.e. the tile shape of the shipped kernel.  MODE bits:
//   1  operand fragments are re-read from LDS in every sub-step (ds_read_b128, swizzled rows as in the kernel)
//   2  one workgroup barrier per k-step
//   4  64 KiB of operands per k-step arrive through direct-to-LDS loads (global_load_lds_dwordx4)
// MODE 0 is the matrix pipe alone.  The operands come from `src` (>= 64 KiB + 8 x 64 KiB per workgroup stride):
// zeros and random fp8 bytes draw very different power, and the shader clock follows.
#ifdef NGPT_BENCH_BUILD
#include "common.h"
#include "host_util.h"

namespace ngpt {

__device__ __forceinline__ v8i bench_frag(const uint8_t* s, int off, int ks) {
    const int o = off ^ (ks * 64);
    const v4i lo = *(const v4i*)(s + o), hi = *(const v4i*)(s + (o ^ 16));
    return (v8i){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
}

template <int MODE>
__global__ __launch_bounds__(512, 1) void kstep_rate_kernel(const uint8_t* __restrict__ src, int64_t src_stride, int iters,
                                                            float* __restrict__ sink, long long* __restrict__ ticks) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wr = wave / 2, wc = wave % 2, h = lane >> 5;
    const uint8_t* gsrc = src + (int64_t)blockIdx.x * src_stride;
    for (int i = threadIdx.x; i < 131072 / 16; i += 512) ((v4i*)smem)[i] = ((const v4i*)gsrc)[i & 4095];
    __syncthreads();
    int fa[2], fb[4];
    for (int t = 0; t < 2; ++t) { const int row = wr * 64 + t * 32 + (lane & 31); fa[t] = row * 128 + (((2 * h) ^ ((row >> 1) & 7)) << 4); }
    for (int t = 0; t < 4; ++t) { const int row = wc * 128 + t * 32 + (lane & 31); fb[t] = 32768 + row * 128 + (((2 * h) ^ ((row >> 1) & 7)) << 4); }
    v16f acc[2][4];
    for (int i = 0; i < 2; ++i) for (int j = 0; j < 4; ++j) for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    v8i a[2], b[4];
    for (int t = 0; t < 2; ++t) a[t] = bench_frag(smem, fa[t], 0);
    for (int t = 0; t < 4; ++t) b[t] = bench_frag(smem, fb[t], 0);
    uint32_t goff[8];
    for (int i = 0; i < 8; ++i) goff[i] = (wave + i * 8) * 1024 + lane * 16;
    if (MODE & 4) for (int i = 0; i < 8; ++i) global_to_lds16(gsrc + goff[i], smem + 65536 + (wave + i * 8) * 1024);
    const long long t0 = clock64(), w0 = wall_clock64();
    int slot = 0;
    for (int it = 0; it < iters; ++it) {
        const uint8_t* s = smem + slot * 65536;
        if (MODE & 4) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (MODE & 2) wg_barrier();
        if (MODE & 1) {
            // fragment reads one MFMA group ahead of their use, as in the shipped k-step
            v8i aa[2], bc;
            aa[0] = bench_frag(s, fa[0], 0); aa[1] = bench_frag(s, fa[1], 0); bc = bench_frag(s, fb[0], 0);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                v8i an[2];
#pragma unroll
                for (int tn = 0; tn < 4; ++tn) {
                    v8i bn;
                    if (tn + 1 < 4) bn = bench_frag(s, fb[tn + 1], ks);
                    else if (ks + 1 < 2) { an[0] = bench_frag(s, fa[0], 1); an[1] = bench_frag(s, fa[1], 1); bn = bench_frag(s, fb[0], 1); }
#pragma unroll
                    for (int tm = 0; tm < 2; ++tm)
                        acc[tm][tn] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(aa[tm], bc, acc[tm][tn], 0, 0, 0, 0, 0, 0);
                    if ((MODE & 4) && ks == 0 && tn == 0) {
                        const uint8_t* gs = gsrc + ((it & 7) << 16);
                        for (int i = 0; i < 8; ++i) global_to_lds16(gs + goff[i], smem + (slot ^ 1) * 65536 + (wave + i * 8) * 1024);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    if (tn + 1 < 4 || ks + 1 < 2) bc = bn;
                }
                if (ks + 1 < 2) { aa[0] = an[0]; aa[1] = an[1]; }
            }
        } else {
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int tm = 0; tm < 2; ++tm)
#pragma unroll
                    for (int tn = 0; tn < 4; ++tn)
                        acc[tm][tn] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[tm], b[tn], acc[tm][tn], 0, 0, 0, 0, 0, 0);
        }
        if (MODE & 4) slot ^= 1;
    }
    const long long t1 = clock64(), w1 = wall_clock64();
    float sum = 0.f;
    for (int i = 0; i < 2; ++i) for (int j = 0; j < 4; ++j) for (int v = 0; v < 16; ++v) sum += acc[i][j][v];
    if (sum == 123.456f) sink[threadIdx.x] = sum;
    if (threadIdx.x == 0) { ticks[2 * blockIdx.x] = t1 - t0; ticks[2 * blockIdx.x + 1] = w1 - w0; }
}

template <int MODE>
static int launch_kstep_rate(const void* src, int64_t stride, int iters, int grid, float* sink, long long* ticks, hipStream_t st) {
    auto kernel = kstep_rate_kernel<MODE>;
    if (int e = allow_lds(kernel, 131072)) return e;
    kernel<<<grid, 512, 131072, st>>>((const uint8_t*)src, stride, iters, sink, ticks);
    return check_launch("kstep_rate_kernel");
}

}  // namespace ngpt

using namespace ngpt;

// One launch of the k-step skeleton: `grid` workgroups x `iters` k-steps of 256 x 256 x 128 each.  src: fp8 bytes,
// at least 64 KiB + 8 * 64 KiB per workgroup at `src_stride` bytes apart (0 = all workgroups read the same bytes);
// sink: 512 floats; ticks: 2 x grid int64 = (shader-clock cycles, 100 MHz wall ticks) each workgroup spent in its loop.
extern "C" int ngpt_bench_kstep_rate(const void* src, int64_t src_stride, int mode, int iters, int grid, float* sink,
                                     long long* ticks, void* stream) {
    if (!src || !sink || !ticks || iters <= 0 || grid <= 0) return fail(NGPT_EINVAL, "ngpt_bench_kstep_rate: bad argument");
    hipStream_t st = (hipStream_t)stream;
    switch (mode) {
        case 0: return launch_kstep_rate<0>(src, src_stride, iters, grid, sink, ticks, st);
        case 1: return launch_kstep_rate<1>(src, src_stride, iters, grid, sink, ticks, st);
        case 3: return launch_kstep_rate<3>(src, src_stride, iters, grid, sink, ticks, st);
        case 7: return launch_kstep_rate<7>(src, src_stride, iters, grid, sink, ticks, st);
    }
    return fail(NGPT_EINVAL, "ngpt_bench_kstep_rate: mode=%d (0, 1, 3 or 7)", mode);
}
#endif  // NGPT_BENCH_BUILD
