// Host-side helpers shared by the C-ABI entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>
#include "../../include/ngpt_fp8.h"

namespace ngpt {

char* last_error_buf();

inline int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(last_error_buf(), 512, fmt, ap);
    va_end(ap);
    return code;
}

inline int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail((int)e, "%s: %s", what, hipGetErrorString(e));
    return NGPT_OK;
}

// e4m3 copies of two bf16 tensors in one launch (quant.hip).
int quant_e4m3_pair(const void* in0, void* out0, int64_t n0, float s0, const void* in1, void* out1, int64_t n1, float s1,
                    hipStream_t st);

// fp8 GEMM with a row-major bf16 output on the token-stationary kernel (ce.hip, token_stationary.h): out [M, N] = x [M, K] . w [N, K]^T,
// w given in fragment order (xs_gemm_frag_bytes bytes, written by xs_gemm_make_frag from the row-major e4m3 matrix or by
// xs_gemm_quant_pair_frag together with the e4m3 copies of both bf16 operands).  mode: 3 = bf16(acc * scale), 4 = the
// ReLU^2 epilogue of c_fc, 5 = the same with the e4m3 copy and per-workgroup maxima; the scale is `scale` times
// *dscale (device, nullable).  `slot`: profile slot of the launch.
bool xs_gemm_eligible(int M, int N, int K);
int64_t xs_gemm_frag_bytes(int N, int K);
int xs_gemm_make_frag(const void* w_f8, int N, int K, void* w_frag, hipStream_t st);
int xs_gemm_quant_pair_frag(const void* x_bf16, void* x_f8, int64_t nx, float x_s, const void* w_bf16, void* w_f8, int N, int K, float w_s,
                            void* w_frag, hipStream_t st);
int xs_gemm_lines(int mode, const void* x_f8, const void* w_frag, int M, int N, int K, float scale, const float* dscale,
                  void* out_bf16, int64_t ld_out, void* out_f8, int64_t ld_f8, const float* act_scale, float* partial_amax, int n_partials,
                  int slot, hipStream_t st);

// Index of the current HIP device (-1 if there is none) and its number of compute units (cached per device).
constexpr int kMaxDevices = 64;
int current_device();
int num_cus();

// Allow a kernel to use `bytes` of dynamic LDS (needed above 64 KiB); cached per kernel.
template <class K>
inline int allow_lds(K kernel, int bytes) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute(%d B LDS): %s", bytes, hipGetErrorString(e));
    return NGPT_OK;
}

// Optional per-kernel timing with HIP events on the launch stream (off by default).
// Slots name the heavy kernels of the fused lm_head + CE path.
enum ProfileSlot : int {
    PROF_CE_FWD = 0,      // lm_head GEMM + softcap + row statistics
    PROF_CE_DLOGITS = 1,  // logits recompute + e5m2 dlogits
    PROF_CE_DX = 2,       // dx GEMM
    PROF_CE_DW = 3,       // dW GEMM
    PROF_GEMM = 4,        // any other fp8 GEMM launch (nanogpt::mm forward / backward, the FP8 down projection)
    PROF_FC_RELU2 = 5,    // up projection with the ReLU^2 epilogue (fp8 or bf16 operands)
    PROF_DPRE = 6,        // dpre GEMM of the MLP backward
    PROF_GEMM_BF16 = 7,   // plain bf16 GEMMs of the MLP (c_proj, dx, dW1, dW2), their summing pass included
    PROF_PRODUCERS = 8,   // rms-norm + amax + quantise of the MLP input, the norm's backward
    PROF_SLOTS = 9
};
bool profiling_on();
void profile_begin(int slot, hipStream_t st);
void profile_end(int slot, hipStream_t st);

struct ProfileScope {
    int slot;
    hipStream_t st;
    bool on;
    ProfileScope(int s, hipStream_t stream, bool enable = true) : slot(s), st(stream), on(enable && profiling_on()) {
        if (on) profile_begin(slot, st);
    }
    ~ProfileScope() {
        if (on) profile_end(slot, st);
    }
};

// Which profile slot the balanced GEMM launches inside a scope are booked under (per host thread: entry points may
// be called concurrently).
extern thread_local int g_gemm_slot;
struct GemmSlot {
    int saved;
    explicit GemmSlot(int s) : saved(g_gemm_slot) { g_gemm_slot = s; }
    ~GemmSlot() { g_gemm_slot = saved; }
};

inline int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

}  // namespace ngpt
