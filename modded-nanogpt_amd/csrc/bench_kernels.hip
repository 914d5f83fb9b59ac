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

// Issue rate of single vector instructions: every wave runs `iters` x 32 instructions of one kind on eight independent
// registers and leaves its cycle count in ticks[wave] (workgroup 0 only).  With one wave per SIMD (256 threads) that is
// the rate at which a wave issues; with two or four (512 / 1024 threads) the slowest wave's count, divided by the waves
// per SIMD, is what the SIMD's vector pipe retires.
template <int KIND>
__global__ __launch_bounds__(1024) void valu_rate_kernel(uint32_t* out, int iters, uint32_t seed, long long* ticks) {
    uint32_t r[8];
    for (int i = 0; i < 8; ++i) r[i] = seed * (threadIdx.x + 1 + i) + i;
    const uint32_t c = seed | 3;
    const long long t0 = clock64();
    for (int it = 0; it < iters; ++it) {
#define NGPT_OP(i)                                                                                                              \
    if (KIND == 0) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(r[i]) : "v"(c));                                                   \
    if (KIND == 1) asm volatile("v_add_f32 %0, %0, %1" : "+v"(r[i]) : "v"(c));                                                   \
    if (KIND == 2) asm volatile("v_and_b32 %0, %0, %1" : "+v"(r[i]) : "v"(c));                                                   \
    if (KIND == 3) asm volatile("v_lshrrev_b32 %0, 1, %0" : "+v"(r[i]));                                                         \
    if (KIND == 4) asm volatile("v_max_f32 %0, %0, %1" : "+v"(r[i]) : "v"(c));                                                   \
    if (KIND == 5) asm volatile("v_fma_f32 %0, %0, %1, %1" : "+v"(r[i]) : "v"(c));                                               \
    if (KIND == 6) asm volatile("v_perm_b32 %0, %0, %1, %2" : "+v"(r[i]) : "v"(c), "s"(0x05010400));                             \
    if (KIND == 7) asm volatile("v_and_or_b32 %0, %0, %1, %2" : "+v"(r[i]) : "s"(0x40004000), "v"(c));                           \
    if (KIND == 8) asm volatile("v_cvt_pk_bf16_f32 %0, %0, %1" : "+v"(r[i]) : "v"(c));                                           \
    if (KIND == 9) asm volatile("v_pk_sub_u16 %0, %0, %1 clamp" : "+v"(r[i]) : "v"(c));                                          \
    if (KIND == 10) asm volatile("v_pk_min_u16 %0, %0, %1" : "+v"(r[i]) : "v"(c));                                               \
    if (KIND == 11) asm volatile("v_pk_lshlrev_b16 %0, 2, %0 op_sel_hi:[0,1]" : "+v"(r[i]));                                     \
    if (KIND == 12) asm volatile("v_mov_b32_dpp %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf" : "+v"(r[i]));            \
    if (KIND == 13) asm volatile("v_exp_f32 %0, %0" : "+v"(r[i]));
#define NGPT_OP8 NGPT_OP(0) NGPT_OP(1) NGPT_OP(2) NGPT_OP(3) NGPT_OP(4) NGPT_OP(5) NGPT_OP(6) NGPT_OP(7)
        NGPT_OP8 NGPT_OP8 NGPT_OP8 NGPT_OP8
#undef NGPT_OP8
#undef NGPT_OP
    }
    const long long t1 = clock64();
    uint32_t x = 0;
    for (int i = 0; i < 8; ++i) x ^= r[i];
    if (x == 0x12345678u) out[threadIdx.x] = x;
    if ((threadIdx.x & 63) == 0 && blockIdx.x == 0) ticks[threadIdx.x >> 6] = t1 - t0;
}
constexpr int kValuKinds = 14;

// Throughput of 64-lane LDS gathers (ds_read_b32) over a table of `entries` floats: every wave issues 16 reads with the
// byte offsets offs[(global thread) * 16 ..+15], waits for them, and repeats; ticks[wave] of workgroup 0 as above.
__global__ __launch_bounds__(512) void lds_gather_kernel(const uint32_t* __restrict__ offs, int entries, int iters, float* out, long long* ticks) {
    extern __shared__ float gather_tab[];
    for (int i = threadIdx.x; i < entries; i += blockDim.x) gather_tab[i] = (float)i;
    __syncthreads();
    uint32_t o[16];
    for (int i = 0; i < 16; ++i) o[i] = offs[((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 16 + i];
    float acc = 0.f;
    const long long t0 = clock64();
    for (int it = 0; it < iters; ++it) {
        float v[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) asm volatile("ds_read_b32 %0, %1" : "=v"(v[i]) : "v"(o[i]));
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]), "+v"(v[8]), "+v"(v[9]),
                       "+v"(v[10]), "+v"(v[11]), "+v"(v[12]), "+v"(v[13]), "+v"(v[14]), "+v"(v[15]));
#pragma unroll
        for (int i = 0; i < 16; ++i) acc += v[i];
    }
    const long long t1 = clock64();
    if (acc == 1.2345f) out[threadIdx.x] = acc;
    if ((threadIdx.x & 63) == 0 && blockIdx.x == 0) ticks[threadIdx.x >> 6] = t1 - t0;
}

}  // namespace ngpt

using namespace ngpt;

// kind: 0 v_mul_f32, 1 v_add_f32, 2 v_and_b32, 3 v_lshrrev_b32, 4 v_max_f32, 5 v_fma_f32, 6 v_perm_b32, 7 v_and_or_b32,
// 8 v_cvt_pk_bf16_f32, 9 v_pk_sub_u16 clamp, 10 v_pk_min_u16, 11 v_pk_lshlrev_b16, 12 v_mov_b32_dpp, 13 v_exp_f32.
// threads: 256, 512 or 1024 per workgroup (1, 2, 4 waves per SIMD), one workgroup per compute unit; iters x 32
// instructions per wave; sink: 1024 uint32; ticks: 16 int64 (cycles of each wave of workgroup 0).
extern "C" int ngpt_bench_valu_rate(int kind, int threads, int iters, void* sink, long long* ticks, void* stream) {
    if (kind < 0 || kind >= kValuKinds || (threads != 256 && threads != 512 && threads != 1024) || iters <= 0 || !sink || !ticks)
        return fail(NGPT_EINVAL, "ngpt_bench_valu_rate: bad argument");
    const int grid = num_cus();
    if (grid <= 0) return fail(NGPT_EINVAL, "no HIP device");
    hipStream_t st = (hipStream_t)stream;
    switch (kind) {
#define NGPT_CASE(K) case K: valu_rate_kernel<K><<<grid, threads, 0, st>>>((uint32_t*)sink, iters, 12345u, ticks); break;
        NGPT_CASE(0) NGPT_CASE(1) NGPT_CASE(2) NGPT_CASE(3) NGPT_CASE(4) NGPT_CASE(5) NGPT_CASE(6) NGPT_CASE(7) NGPT_CASE(8) NGPT_CASE(9)
        NGPT_CASE(10) NGPT_CASE(11) NGPT_CASE(12) NGPT_CASE(13)
#undef NGPT_CASE
    }
    return check_launch("valu_rate_kernel");
}

// offs: device array of (compute units x threads x 16) byte offsets below 4 * entries; threads 256 or 512 (4 or 8 waves
// per compute unit); sink: 512 floats; ticks: 8 int64.
extern "C" int ngpt_bench_lds_gather(const void* offs, int entries, int threads, int iters, void* sink, long long* ticks, void* stream) {
    if (!offs || entries <= 0 || entries > 16384 || (threads != 256 && threads != 512) || iters <= 0 || !sink || !ticks)
        return fail(NGPT_EINVAL, "ngpt_bench_lds_gather: bad argument");
    const int grid = num_cus();
    if (grid <= 0) return fail(NGPT_EINVAL, "no HIP device");
    lds_gather_kernel<<<grid, threads, entries * 4, (hipStream_t)stream>>>((const uint32_t*)offs, entries, iters, (float*)sink, ticks);
    return check_launch("lds_gather_kernel");
}

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
