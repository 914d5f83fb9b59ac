// C-ABI entry points built on the persistent FP8 TN GEMM: the raw GEMM, nanogpt::mm(_t)
// forward/backward and the fused up-projection + ReLU^2.
#include "epilogues.h"
#include "host_util.h"
#include "launch.h"
#include "panel.h"
#include <atomic>
#include <algorithm>
#include <mutex>
#include <vector>

namespace ngpt {

// ---------------------------------------------------------------- per-kernel event timing
namespace {
struct EventPair {
    hipEvent_t a, b;
};
std::mutex g_prof_mu;
bool g_prof_on = false;
std::vector<EventPair> g_prof_pending[PROF_SLOTS];
std::vector<EventPair> g_prof_free;
hipEvent_t g_prof_open[PROF_SLOTS];
}  // namespace

bool profiling_on() { return g_prof_on; }

void profile_begin(int slot, hipStream_t st) {
    std::lock_guard<std::mutex> lk(g_prof_mu);
    EventPair p;
    if (!g_prof_free.empty()) {
        p = g_prof_free.back();
        g_prof_free.pop_back();
    } else if (hipEventCreate(&p.a) != hipSuccess || hipEventCreate(&p.b) != hipSuccess) {
        (void)hipGetLastError();
        return;
    }
    (void)hipEventRecord(p.a, st);
    g_prof_pending[slot].push_back(p);
    g_prof_open[slot] = p.b;
}

void profile_end(int slot, hipStream_t st) {
    std::lock_guard<std::mutex> lk(g_prof_mu);
    if (!g_prof_pending[slot].empty()) (void)hipEventRecord(g_prof_open[slot], st);
}

char* last_error_buf() {
    static thread_local char buf[512];
    return buf;
}

int current_device() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return -1;
    }
    return dev;
}

// Compute units of the CURRENT device; one relaxed atomic per device caches the query (two threads that
// race on the first call both store the same value).
int num_cus() {
    static std::atomic<int> cached[kMaxDevices];
    const int dev = current_device();
    if (dev < 0) return 0;
    if (dev < kMaxDevices) {
        const int c = cached[dev].load(std::memory_order_relaxed);
        if (c > 0) return c;
    }
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    if (dev < kMaxDevices) cached[dev].store(n, std::memory_order_relaxed);
    return n;
}

static int check_gemm_dims(const char* who, int R, int C, int K, int64_t lda, int64_t ldb) {
    if (R <= 0 || C <= 0 || K <= 0) return fail(NGPT_EINVAL, "%s: empty problem R=%d C=%d K=%d", who, R, C, K);
    if (K % 128) return fail(NGPT_EALIGN, "%s: contraction length %d must be a multiple of 128", who, K);
    if (lda % 16 || ldb % 16 || lda < K || ldb < K)
        return fail(NGPT_EALIGN, "%s: operand row strides (%lld, %lld) must be multiples of 16 and >= K",
                    who, (long long)lda, (long long)ldb);
    return NGPT_OK;
}

thread_local int g_gemm_slot = PROF_GEMM;

// ---------------------------------------------------------------------------------------------
// Balanced walk.  A persistent grid of G workgroups finishes `tiles` tiles in ceil(tiles / G) rounds,
// and in the last round tiles % G workgroups work while the others idle (dx of the lm_head backward:
// 576 tiles on 256 CUs = 2.25 rounds, paid as 3).  Instead the first floor(tiles / G) * G tiles run as
// whole tiles and each of the remaining ones is cut along the contraction into as many jobs as fill
// one more round; every part goes to its own fp32 scratch tile and a summing pass adds a tile's parts up in a fixed order.
struct BalancePlan {
    int tiles, full, rem, splits;
};
static BalancePlan plan_balance(int R, int C, int K) {
    BalancePlan p{};
    p.tiles = ((R + MainCfg::BM - 1) / MainCfg::BM) * ((C + MainCfg::BN - 1) / MainCfg::BN);
    int G = num_cus() * MainCfg::WGS_PER_CU;
    if (G <= 0) G = 1;
    p.full = p.tiles / G * G;
    p.rem = p.tiles - p.full;
    p.splits = 1;
    if (p.rem > 0) {
        int s = G / p.rem;                       // jobs of the last round: rem * s <= G
        int max_s = K / MainCfg::BK / 8;          // a job keeps at least 8 k-steps
        if (s > max_s) s = max_s;
        if (s > 1) p.splits = s;
    }
    if (p.splits == 1) { p.full = p.tiles; p.rem = 0; }
    return p;
}

// Adds up the parts of the split tiles and writes them out.  Tile number first + blockIdx.x of the walk order is the
// blockIdx.x-th split tile; its `splits` parts are the fp32 tiles number s * gridDim.x + blockIdx.x of `part32`
// (GridIter::part_slot), summed in the order of the contraction.  T = uint16_t: bf16 output, T = float: fp32.
constexpr int kRemSlices = 8;
static_assert(MainCfg::BM % kRemSlices == 0, "row slices of a tile");
template <class T>
__global__ __launch_bounds__(256) void rem_tiles_kernel(const float* __restrict__ part32, int splits, T* __restrict__ out, int64_t ldo,
                                                        int R, int C, int first) {
    TileOrder order(R, C, MainCfg::BM, MainCfg::BN);
    int tr, tc;
    order.coords(first + blockIdx.x, tr, tc);
    // blockIdx.y: which slice of the tile's rows (a few dozen tiles alone would leave most of the chip idle)
    constexpr int rows = MainCfg::BM / kRemSlices, cols4 = MainCfg::BN / 4, tile_elems = MainCfg::BM * MainCfg::BN;
    const int rl0 = blockIdx.y * rows;
    const int64_t part_stride = (int64_t)gridDim.x * tile_elems;
    for (int i = threadIdx.x; i < rows * cols4; i += blockDim.x) {
        const int rl = rl0 + i / cols4, cl = (i % cols4) * 4;
        const int r = tr * MainCfg::BM + rl, c = tc * MainCfg::BN + cl;
        if (r >= R || c >= C) continue;          // C % 4 == 0 is checked by the caller
        const float* p = part32 + (int64_t)blockIdx.x * tile_elems + rl * MainCfg::BN + cl;
        v4f v = *(const v4f*)p;
        for (int s_ = 1; s_ < splits; ++s_) v += *(const v4f*)(p + s_ * part_stride);
        if constexpr (sizeof(T) == 2) *(v2i*)(out + (int64_t)r * ldo + c) = (v2i){(int)cvt_pk_bf16(v[0], v[1]), (int)cvt_pk_bf16(v[2], v[3])};
        else *(v4f*)(out + (int64_t)r * ldo + c) = v;
    }
}

// Bytes of fp32 scratch a balanced GEMM may need for the parts of its split tiles, whatever the device: at most one
// part per workgroup of the last round (kMaxGrid bounds the grid) and never more than tiles x splits.
constexpr int kMaxGrid = 512;
int64_t balanced_part_bytes(int R, int C, int K) {
    const int64_t tiles = (int64_t)((R + MainCfg::BM - 1) / MainCfg::BM) * ((C + MainCfg::BN - 1) / MainCfg::BN);
    int64_t max_s = K / MainCfg::BK / 8;
    if (max_s < 1) max_s = 1;
    int64_t parts = tiles * max_s;
    if (parts > kMaxGrid) parts = kMaxGrid;
    return parts * MainCfg::BM * MainCfg::BN * 4;
}

// C[R, C] = scale * A . B^T with the balanced walk.  `layout`: kBlockedA | kBlockedB.
// part32: balanced_part_bytes(R, C, K) bytes of scratch for the split tiles.
// fa may carry FMT_TRANSPOSED (A = panel of the transpose, a_rows_pad = R rounded up to 256).
int gemm_balanced_bf16(const void* A, int fa, int64_t lda, const void* B, int fb, int64_t ldb, int layout, int R, int C, int K,
                       float scale, void* out_bf16, int64_t ldc, float* part32, int a_rows_pad, hipStream_t st,
                       const float* dscale_a = nullptr, const float* dscale_b = nullptr) {
    if (R <= 0 || C <= 0 || K <= 0 || K % 128 || C % 4 || ldc % 4)
        return fail(NGPT_EALIGN, "gemm_balanced_bf16: R=%d C=%d K=%d ldc=%lld", R, C, K, (long long)ldc);
    BalancePlan p = plan_balance(R, C, K);
    if (p.splits > 1 && (!part32 || p.rem * p.splits > kMaxGrid)) return fail(NGPT_EINVAL, "gemm_balanced_bf16: split tiles need the fp32 scratch tiles");
    ProfileScope prof(g_gemm_slot, st);
    GemmOperands g{(const uint8_t*)A, (const uint8_t*)B, lda, ldb, R, C, K, p.splits, layout, p.full, a_rows_pad};
    EpiStoreBf16 epi{(uint16_t*)out_bf16, ldc, scale, R, C, part32, false, 0, dscale_a, dscale_b};
    if (int e = launch_gemm<MainCfg>(g, fa, fb, epi, st)) return e;
    if (p.splits > 1) rem_tiles_kernel<uint16_t><<<dim3(p.rem, kRemSlices), 256, 0, st>>>(part32, p.splits, (uint16_t*)out_bf16, ldc, R, C, p.full);
    return check_launch("gemm_balanced_bf16");
}

// fp32 output.  accumulate: every tile adds into `out` (which the caller initialised) with atomics; otherwise whole
// tiles are stored and the split tiles are added up from their parts in part32.
int gemm_balanced_f32(const void* A, int fa, int64_t lda, const void* B, int fb, int64_t ldb, int layout, int R, int C, int K,
                      float scale, float* out, int64_t ldc, bool accumulate, float* part32, hipStream_t st) {
    if (R <= 0 || C <= 0 || K <= 0 || K % 128 || C % 4 || ldc % 4)
        return fail(NGPT_EALIGN, "gemm_balanced_f32: R=%d C=%d K=%d ldc=%lld", R, C, K, (long long)ldc);
    BalancePlan p = plan_balance(R, C, K);
    ProfileScope prof(g_gemm_slot, st);
    GemmOperands g{(const uint8_t*)A, (const uint8_t*)B, lda, ldb, R, C, K, p.splits, layout, p.full};
    if (accumulate) {
        EpiStoreF32<true> epi{out, ldc, scale, R, C, nullptr, false, 0};
        return launch_gemm<MainCfg>(g, fa, fb, epi, st);
    }
    if (p.splits > 1 && (!part32 || p.rem * p.splits > kMaxGrid)) return fail(NGPT_EINVAL, "gemm_balanced_f32: split tiles need the fp32 scratch tiles");
    EpiStoreF32<false> epi{out, ldc, scale, R, C, part32, false, 0};
    if (int e = launch_gemm<MainCfg>(g, fa, fb, epi, st)) return e;
    if (p.splits > 1) rem_tiles_kernel<float><<<dim3(p.rem, kRemSlices), 256, 0, st>>>(part32, p.splits, out, ldc, R, C, p.full);
    return check_launch("gemm_balanced_f32");
}

// out_kind: 0 bf16, 1 fp32, 2 fp32 accumulate (atomic), 3 discard.  splits > 1 cuts each tile's
// contraction into that many jobs and needs out_kind 2 on a buffer the caller has zeroed or wants added to.
int gemm_store(const void* A, int fa, int64_t lda, const void* B, int fb, int64_t ldb, int R, int C, int K,
               float scale, void* out, int64_t ldc, int out_kind, hipStream_t st, int splits) {
    if (int e = check_gemm_dims("gemm_fp8_tn", R, C, K, lda, ldb)) return e;
    if (splits < 1) splits = 1;
    if (splits > K / 128) splits = K / 128;
    if (splits > 1 && out_kind != 2) return fail(NGPT_EINVAL, "gemm_fp8_tn: split-K needs the accumulating fp32 output");
    GemmOperands g{(const uint8_t*)A, (const uint8_t*)B, lda, ldb, R, C, K, splits};
    ProfileScope prof(g_gemm_slot, st);
    if (out_kind == 0) {
        EpiStoreBf16 epi{(uint16_t*)out, ldc, scale, R, C, nullptr, false, 0};
        const int tiles = ((R + MainCfg::BM - 1) / MainCfg::BM) * ((C + MainCfg::BN - 1) / MainCfg::BN);
        if (fa == FMT_E4M3 && fb == FMT_E4M3 && splits == 1 && 2 * tiles <= num_cus())
            return launch_gemm_fmt<SmallCfg, FMT_E4M3, FMT_E4M3>(g, epi, st, 0);
        return launch_gemm<MainCfg>(g, fa, fb, epi, st);
    }
    if (out_kind == 3) {
#ifdef NGPT_BENCH_BUILD
        EpiDiscard epi{(float*)out, 0, 0};
        return launch_gemm<MainCfg>(g, fa, fb, epi, st);
#else
        return fail(NGPT_EINVAL, "gemm_fp8_tn: out_kind 3 (discard) exists in the measurement build of the library only");
#endif
    }
    if (out_kind == 2) {
        EpiStoreF32<true> epi{(float*)out, ldc, scale, R, C, nullptr, false, 0};
        return launch_gemm<MainCfg>(g, fa, fb, epi, st);
    }
    EpiStoreF32<false> epi{(float*)out, ldc, scale, R, C, nullptr, false, 0};
    return launch_gemm<MainCfg>(g, fa, fb, epi, st);
}

}  // namespace ngpt

using namespace ngpt;

extern "C" int ngpt_abi_version(void) { return 1; }
extern "C" const char* ngpt_last_error(void) { return last_error_buf(); }
extern "C" int ngpt_num_cus(void) { return num_cus(); }

extern "C" int ngpt_profile_enable(int on) {
    std::lock_guard<std::mutex> lk(g_prof_mu);
    g_prof_on = on != 0;
    return NGPT_OK;
}

// Waits for the recorded launches of `slot`, adds up their durations and forgets them.
extern "C" int ngpt_profile_read(int slot, double* total_ms, int* launches) {
    if (slot < 0 || slot >= PROF_SLOTS || !total_ms || !launches)
        return fail(NGPT_EINVAL, "ngpt_profile_read: slot=%d", slot);
    std::lock_guard<std::mutex> lk(g_prof_mu);
    double sum = 0.0;
    int n = 0;
    for (EventPair& p : g_prof_pending[slot]) {
        float ms = 0.0f;
        if (hipEventSynchronize(p.b) == hipSuccess && hipEventElapsedTime(&ms, p.a, p.b) == hipSuccess) {
            sum += ms;
            ++n;
        } else {
            (void)hipGetLastError();
        }
        g_prof_free.push_back(p);
    }
    g_prof_pending[slot].clear();
    *total_ms = sum;
    *launches = n;
    return NGPT_OK;
}

extern "C" int ngpt_gemm_fp8_tn(const void* A, int fmt_a, int64_t lda, const void* B, int fmt_b, int64_t ldb,
                                int R, int C, int K, float scale, void* out, int64_t ldc, int out_kind,
                                void* stream) {
    if (!A || !B || !out) return fail(NGPT_EINVAL, "ngpt_gemm_fp8_tn: null pointer");
    if ((fmt_a | fmt_b) & ~1) return fail(NGPT_EINVAL, "ngpt_gemm_fp8_tn: fmt_a=%d fmt_b=%d", fmt_a, fmt_b);
    if (out_kind < 0 || out_kind > 3) return fail(NGPT_EINVAL, "ngpt_gemm_fp8_tn: out_kind=%d", out_kind);
    if (ldc < C) return fail(NGPT_EINVAL, "ngpt_gemm_fp8_tn: ldc=%lld < C=%d", (long long)ldc, C);
    const int splits = 1;
    return gemm_store(A, fmt_a, lda, B, fmt_b, ldb, R, C, K, scale, out, ldc, out_kind, (hipStream_t)stream, splits);
}

// ------------------------------------------------------------------------------------------ mm forward
// The token-stationary kernel (128-token jobs x up to 4 output shares) needs about one job per compute unit to pay.
static bool mm_fwd_xs(int M, int N, int K) { return xs_gemm_eligible(M, N, K) && (int64_t)(M / 128) * 4 >= num_cus(); }
// [N, K] e4m3 copy of (in, out) weights | fragment-ordered weights (token-stationary kernel)
extern "C" int64_t ngpt_mm_fwd_workspace_bytes(int M, int N, int K, int w_layout) {
    return (w_layout == NGPT_W_IN_OUT ? align_up((int64_t)N * K, 256) : 0) + (mm_fwd_xs(M, N, K) ? xs_gemm_frag_bytes(N, K) : 0);
}

extern "C" int ngpt_mm_fwd(const void* x_bf16, const void* w_bf16, int M, int N, int K, float x_s, float w_s,
                           void* out_bf16, void* x_f8, void* w_f8, int w_layout,
                           void* workspace, int64_t workspace_bytes, void* stream) {
    if (!x_bf16 || !w_bf16 || !out_bf16 || !x_f8 || !w_f8) return fail(NGPT_EINVAL, "ngpt_mm_fwd: null pointer");
    if (M <= 0 || N <= 0 || K <= 0) return fail(NGPT_EINVAL, "ngpt_mm_fwd: empty problem M=%d N=%d K=%d", M, N, K);
    if (K % 128 || M % 16 || N % 16)
        return fail(NGPT_EALIGN, "ngpt_mm_fwd: need K %% 128 == 0, M %% 16 == 0, N %% 16 == 0 (M=%d N=%d K=%d)", M, N, K);
    if (w_layout != NGPT_W_OUT_IN && w_layout != NGPT_W_IN_OUT) return fail(NGPT_EINVAL, "ngpt_mm_fwd: w_layout=%d", w_layout);
    // needed: the [N, K] copy of (in, out) weights; with room for the fragment-ordered weights as well the product runs
    // on the token-stationary kernel
    const int64_t need = w_layout == NGPT_W_IN_OUT ? align_up((int64_t)N * K, 256) : 0;
    if (need > 0 && (!workspace || workspace_bytes < need))
        return fail(NGPT_EWORKSPACE, "ngpt_mm_fwd: workspace %lld < %lld bytes", (long long)workspace_bytes, (long long)need);
    hipStream_t st = (hipStream_t)stream;
    const void* w_nk = w_f8;
    const bool xs = mm_fwd_xs(M, N, K) && workspace && workspace_bytes >= ngpt_mm_fwd_workspace_bytes(M, N, K, w_layout);
    uint8_t* w_frag = (uint8_t*)workspace + (w_layout == NGPT_W_IN_OUT ? align_up((int64_t)N * K, 256) : 0);
    if (w_layout == NGPT_W_OUT_IN) {
        if (xs) {
            if (int e = xs_gemm_quant_pair_frag(x_bf16, x_f8, (int64_t)M * K, x_s, w_bf16, w_f8, N, K, w_s, w_frag, st)) return e;
        } else if (int e = quant_e4m3_pair(x_bf16, x_f8, (int64_t)M * K, x_s, w_bf16, w_f8, (int64_t)N * K, w_s, st)) return e;
    } else {
        if (int e = ngpt_quant_fp8(x_bf16, x_f8, (int64_t)M * K, x_s, NGPT_FMT_E4M3, stream)) return e;
        // w is [K, N]: one pass writes w_f8 [K, N] and the [N, K] copy the GEMM reads
        if (int e = ngpt_quant_fp8_2d(w_bf16, K, N, w_s, NGPT_FMT_E4M3, w_f8, workspace, stream)) return e;
        w_nk = workspace;
        if (xs)
            if (int e = xs_gemm_make_frag(w_nk, N, K, w_frag, st)) return e;
    }
    if (xs) return xs_gemm_lines(3, x_f8, w_frag, M, N, K, x_s * w_s, nullptr, out_bf16, N, nullptr, 0, nullptr, nullptr, 0, PROF_GEMM, st);
    return gemm_store(x_f8, FMT_E4M3, K, w_nk, FMT_E4M3, K, M, N, K, x_s * w_s, out_bf16, N, 0, st, 1);
}

// ------------------------------------------------------------------------------------------ mm backward
// The incoming gradient is quantised ONCE, into a panel-blocked e5m2 matrix with rows = N and 128-byte
// rows = 128 consecutive rows of g (tokens): dW = x^T . g consumes it directly as its B operand, dx = g . w
// reads it as the transpose of its A operand (transposed on the way from LDS to the MFMA registers).
// Both GEMMs use the balanced walk.
// workspace: g^T panel [Np, Mt] | x_f8^T panel [Kp, Mt] | w^T panel [Kp, N] | fp32 parts of the split tiles of dx, then of dW   (p / t = rounded up to 256)
static int64_t round256(int64_t n) { return (n + 255) / 256 * 256; }
extern "C" int64_t ngpt_mm_bwd_workspace_bytes(int M, int N, int K, int w_layout) {
    (void)w_layout;
    const int64_t Mt = round256(M), Np = round256(N), Kp = round256(K);
    const int64_t parts = std::max(balanced_part_bytes(M, K, N), balanced_part_bytes(K, N, (int)Mt));
    return Np * Mt + Kp * Mt + Kp * (int64_t)N + parts;
}

extern "C" int ngpt_mm_bwd(const void* g_bf16, const void* x_f8, const void* w_f8, int M, int N, int K,
                           float x_s, float w_s, float grad_s, void* dx_bf16, void* dw_kn_f32, int w_layout,
                           void* workspace, int64_t workspace_bytes, void* stream) {
    if (!g_bf16 || !x_f8 || !w_f8 || !dx_bf16 || !dw_kn_f32 || !workspace) return fail(NGPT_EINVAL, "ngpt_mm_bwd: null pointer");
    if (M <= 0 || N <= 0 || K <= 0) return fail(NGPT_EINVAL, "ngpt_mm_bwd: empty problem M=%d N=%d K=%d", M, N, K);
    if (M % 128 || N % 128 || K % 16)
        return fail(NGPT_EALIGN, "ngpt_mm_bwd: need M %% 128 == 0, N %% 128 == 0, K %% 16 == 0 (M=%d N=%d K=%d)", M, N, K);
    if (w_layout != NGPT_W_OUT_IN && w_layout != NGPT_W_IN_OUT) return fail(NGPT_EINVAL, "ngpt_mm_bwd: w_layout=%d", w_layout);
    int64_t need = ngpt_mm_bwd_workspace_bytes(M, N, K, w_layout);
    if (workspace_bytes < need)
        return fail(NGPT_EWORKSPACE, "ngpt_mm_bwd: workspace %lld < %lld bytes", (long long)workspace_bytes, (long long)need);
    hipStream_t st = (hipStream_t)stream;
    const int64_t Mt = round256(M), Np = round256(N), Kp = round256(K);
    const int nkt = (int)(Mt / 128), nkn = N / 128;
    uint8_t* ws = (uint8_t*)workspace;
    uint8_t* g_panel = ws;
    uint8_t* x_t = g_panel + Np * Mt;
    uint8_t* w_t = x_t + Kp * Mt;
    float* parts = (float*)(w_t + Kp * (int64_t)N);
    if (int e = (panel_transpose<0, FMT_E5M2>(g_bf16, N, 0, M, N, nkt, g_panel, st, grad_s))) return e;
    if (int e = panel_transpose<0>(x_f8, K, 0, M, K, nkt, x_t, st)) return e;
    if (w_layout == NGPT_W_OUT_IN) {   // w [N, K]  ->  rows = K, contraction = N
        if (int e = panel_transpose<0>(w_f8, K, 0, N, K, nkn, w_t, st)) return e;
    } else {                           // w [K, N] already has the contraction contiguous
        if (int e = panel_pack(w_f8, N, K, N, w_t, st)) return e;
    }
    // dx [M,K] = g [M,N] . (w^T [K,N])^T, contraction over N, g read transposed from the panel
    if (int e = gemm_balanced_bf16(g_panel, FMT_E5M2 | FMT_TRANSPOSED, 0, w_t, FMT_E4M3, 0, kBlockedB, M, K, N, grad_s * w_s,
                                   dx_bf16, K, parts, (int)Mt, st)) return e;
    // dw [K,N] = x_f8^T [K,Mt] . (g^T [N,Mt])^T, contraction over the (zero padded) rows of g
    return gemm_balanced_f32(x_t, FMT_E4M3, 0, g_panel, FMT_E5M2, 0, kBlockedA | kBlockedB, K, N, (int)Mt, x_s * grad_s,
                             (float*)dw_kn_f32, N, false, parts, st);
}

// ------------------------------------------------------------------------------------------ dpre (bf16)
extern "C" int ngpt_fc_relu2_bwd_dpre(const void* dy_bf16, const void* w2_bf16, const void* post_bf16, int M, int H, int D,
                                      void* dpre_bf16, void* stream) {
    if (!dy_bf16 || !w2_bf16 || !post_bf16 || !dpre_bf16) return fail(NGPT_EINVAL, "ngpt_fc_relu2_bwd_dpre: null pointer");
    if (M <= 0 || H <= 0 || D <= 0) return fail(NGPT_EINVAL, "ngpt_fc_relu2_bwd_dpre: empty problem M=%d H=%d D=%d", M, H, D);
    if (D % 64 || H % 8) return fail(NGPT_EALIGN, "ngpt_fc_relu2_bwd_dpre: need D %% 64 == 0 and H %% 8 == 0 (D=%d H=%d)", D, H);
    // bf16 operands: the loader works in bytes, so the contraction length and row strides are 2 * D.
    // Transposed product (tile rows = hidden units, tile columns = tokens), see EpiDpre.
    GemmOperands g{(const uint8_t*)w2_bf16, (const uint8_t*)dy_bf16, 2 * (int64_t)D, 2 * (int64_t)D, H, M, 2 * D, 1};
    EpiDpre epi{(uint16_t*)dpre_bf16, (const uint16_t*)post_bf16, H, H, M};
    ProfileScope prof(PROF_DPRE, (hipStream_t)stream);
    return launch_gemm_fmt<MainCfg, FMT_BF16, FMT_BF16>(g, epi, (hipStream_t)stream, 0);
}

// ------------------------------------------------------------------------------------------ fp8 GEMM with device-side scales
// torch._scaled_mm(post_f8, W2_f8, scale_a = activation_scale, scale_b = W2_scale, out_dtype = bf16): the FP8 down
// projection of FusedLinearReLUSquareFunction.forward (triton_kernels.py:706-713).  Both scales are 1-element fp32
// device buffers; the epilogue multiplies by their product, so nothing of size [R, C] but the bf16 result is written.
extern "C" int64_t ngpt_gemm_fp8_scaled_workspace_bytes(int R, int C, int K) { return balanced_part_bytes(R, C, K); }

extern "C" int ngpt_gemm_fp8_scaled(const void* A, int fa, int64_t lda, const void* B, int fb, int64_t ldb, int R, int C, int K,
                                    const float* scale_a, const float* scale_b, void* out_bf16, int64_t ldc,
                                    void* workspace, int64_t workspace_bytes, void* stream) {
    if (!A || !B || !out_bf16 || !scale_a || !scale_b || !workspace) return fail(NGPT_EINVAL, "ngpt_gemm_fp8_scaled: null pointer");
    if ((fa != NGPT_FMT_E4M3 && fa != NGPT_FMT_E5M2) || (fb != NGPT_FMT_E4M3 && fb != NGPT_FMT_E5M2))
        return fail(NGPT_EINVAL, "ngpt_gemm_fp8_scaled: fa=%d fb=%d", fa, fb);
    if (int e = check_gemm_dims("ngpt_gemm_fp8_scaled", R, C, K, lda, ldb)) return e;
    if (C % 4 || ldc % 4 || ldc < C) return fail(NGPT_EALIGN, "ngpt_gemm_fp8_scaled: C=%d ldc=%lld must be multiples of 4, ldc >= C", C, (long long)ldc);
    if (workspace_bytes < ngpt_gemm_fp8_scaled_workspace_bytes(R, C, K))
        return fail(NGPT_EWORKSPACE, "ngpt_gemm_fp8_scaled: workspace %lld < %lld bytes", (long long)workspace_bytes,
                    (long long)ngpt_gemm_fp8_scaled_workspace_bytes(R, C, K));
    GemmSlot slot(PROF_GEMM);
    return gemm_balanced_bf16(A, fa, lda, B, fb, ldb, 0, R, C, K, 1.0f, out_bf16, ldc, (float*)workspace, 0, (hipStream_t)stream,
                              scale_a, scale_b);
}

// ------------------------------------------------------------------------------------------ plain bf16 GEMM
// The four bf16 products of FusedLinearReLUSquareFunction besides dpre (triton_kernels.py:715, 723, 727, 728).
extern "C" int64_t ngpt_gemm_bf16_workspace_bytes(int R, int C, int K) { return balanced_part_bytes(R, C, 2 * K); }

extern "C" int ngpt_gemm_bf16(const void* A, int a_layout, int64_t lda, const void* B, int b_layout, int64_t ldb,
                              int R, int C, int K, void* out_bf16, int64_t ldc, void* workspace, int64_t workspace_bytes,
                              void* stream) {
    if (!A || !B || !out_bf16 || !workspace) return fail(NGPT_EINVAL, "ngpt_gemm_bf16: null pointer");
    if (R <= 0 || C <= 0 || K <= 0) return fail(NGPT_EINVAL, "ngpt_gemm_bf16: empty problem R=%d C=%d K=%d", R, C, K);
    if ((a_layout | b_layout) & ~1) return fail(NGPT_EINVAL, "ngpt_gemm_bf16: a_layout=%d b_layout=%d", a_layout, b_layout);
    if (K % 64 || R % 8 || C % 8)
        return fail(NGPT_EALIGN, "ngpt_gemm_bf16: need K %% 64 == 0, R %% 8 == 0, C %% 8 == 0 (R=%d C=%d K=%d)", R, C, K);
    const int64_t min_lda = a_layout == NGPT_K_CONTIGUOUS ? K : R, min_ldb = b_layout == NGPT_K_CONTIGUOUS ? K : C;
    if (lda % 8 || ldb % 8 || lda < min_lda || ldb < min_ldb || ldc < C || ldc % 4)
        return fail(NGPT_EALIGN, "ngpt_gemm_bf16: leading dimensions lda=%lld ldb=%lld ldc=%lld", (long long)lda, (long long)ldb, (long long)ldc);
    if (workspace_bytes < ngpt_gemm_bf16_workspace_bytes(R, C, K))
        return fail(NGPT_EWORKSPACE, "ngpt_gemm_bf16: workspace %lld < %lld bytes", (long long)workspace_bytes,
                    (long long)ngpt_gemm_bf16_workspace_bytes(R, C, K));
    // the loader works in bytes: contraction length and row strides are 2 x the element counts
    const int fa = a_layout == NGPT_K_CONTIGUOUS ? FMT_BF16 : (FMT_BF16 | FMT_TRANSPOSED);
    const int fb = b_layout == NGPT_K_CONTIGUOUS ? FMT_BF16 : (FMT_BF16 | FMT_TRANSPOSED);
    GemmSlot slot(PROF_GEMM_BF16);
    return gemm_balanced_bf16(A, fa, 2 * lda, B, fb, 2 * ldb, 0, R, C, 2 * K, 1.0f, out_bf16, ldc, (float*)workspace, 0,
                              (hipStream_t)stream);
}

// post [M, N] = bf16(max(bf16(x . w^T), 0)^2) on bf16 operands: linear_relu_square_kernel FORWARD without USE_FP8
// (triton_kernels.py:402-499 as launched at :716-718 when no fp8 copies are passed).  Same transposed product and
// whole-line stores as the FP8 c_fc.
extern "C" int ngpt_linear_relu2_bf16(const void* x_bf16, const void* w_bf16, int M, int N, int K, void* post_bf16, void* stream) {
    if (!x_bf16 || !w_bf16 || !post_bf16) return fail(NGPT_EINVAL, "ngpt_linear_relu2_bf16: null pointer");
    if (M <= 0 || N <= 0 || K <= 0) return fail(NGPT_EINVAL, "ngpt_linear_relu2_bf16: empty problem M=%d N=%d K=%d", M, N, K);
    if (K % 64 || N % 8) return fail(NGPT_EALIGN, "ngpt_linear_relu2_bf16: need K %% 64 == 0 and N %% 8 == 0 (N=%d K=%d)", N, K);
    GemmOperands gt{(const uint8_t*)w_bf16, (const uint8_t*)x_bf16, 2 * (int64_t)K, 2 * (int64_t)K, N, M, 2 * K, 1};
    EpiRelu2Lines epi{(uint16_t*)post_bf16, N, nullptr, N, M};
    ProfileScope prof(PROF_FC_RELU2, (hipStream_t)stream);
    return launch_gemm_fmt<MainCfg, FMT_BF16, FMT_BF16>(gt, epi, (hipStream_t)stream, 0);
}

// ------------------------------------------------------------------------------------------ fc + relu^2
extern "C" int64_t ngpt_fc_relu2_fwd_workspace_bytes(int M, int N, int K) { return mm_fwd_xs(M, N, K) ? xs_gemm_frag_bytes(N, K) : 0; }

extern "C" int ngpt_fc_relu2_fwd(const void* x_f8, const void* w_f8, const float* dequant, int M, int N, int K,
                                 void* post_bf16, void* post_f8, const float* act_scale,
                                 float* partial_amax, int n_partials, void* stream) {
    return ngpt_fc_relu2_fwd_ws(x_f8, w_f8, dequant, M, N, K, post_bf16, post_f8, act_scale, partial_amax, n_partials, nullptr, 0, stream);
}

extern "C" int ngpt_fc_relu2_fwd_ws(const void* x_f8, const void* w_f8, const float* dequant, int M, int N, int K,
                                    void* post_bf16, void* post_f8, const float* act_scale,
                                    float* partial_amax, int n_partials, void* workspace, int64_t workspace_bytes, void* stream) {
    if (!x_f8 || !w_f8 || !dequant || !post_bf16) return fail(NGPT_EINVAL, "ngpt_fc_relu2_fwd: null pointer");
    if (post_f8 && (!act_scale || !partial_amax || n_partials <= 0))
        return fail(NGPT_EINVAL, "ngpt_fc_relu2_fwd: post_f8 needs act_scale and partial_amax");
    if (int e = check_gemm_dims("ngpt_fc_relu2_fwd", M, N, K, K, K)) return e;
    if (N % 16) return fail(NGPT_EALIGN, "ngpt_fc_relu2_fwd: N=%d must be a multiple of 16", N);
    // with room for the weights in fragment order: the token-stationary kernel (the partial maxima then are one per
    // workgroup of its grid, at most one per compute unit)
    if (mm_fwd_xs(M, N, K) && workspace && workspace_bytes >= xs_gemm_frag_bytes(N, K) && (!post_f8 || n_partials >= num_cus())) {
        ProfileScope prof(PROF_FC_RELU2, (hipStream_t)stream);
        if (int e = xs_gemm_make_frag(w_f8, N, K, workspace, (hipStream_t)stream)) return e;
        return xs_gemm_lines(post_f8 ? 5 : 4, x_f8, workspace, M, N, K, 1.0f, dequant, post_bf16, N, post_f8, N, act_scale, partial_amax, n_partials,
                             -2, (hipStream_t)stream);
    }
    ProfileScope prof(PROF_FC_RELU2, (hipStream_t)stream);
    // transposed product (tile rows = hidden units, tile columns = tokens): whole-line stores of post
    GemmOperands gt{(const uint8_t*)w_f8, (const uint8_t*)x_f8, K, K, N, M, K, 1};
    if (post_f8) {
        EpiRelu2LinesT<true> epi{(uint16_t*)post_bf16, N, dequant, N, M, (uint8_t*)post_f8, N, act_scale, partial_amax, n_partials};
        // one partial-amax slot per persistent workgroup
        return launch_gemm_fmt<MainCfg, FMT_E4M3, FMT_E4M3>(gt, epi, (hipStream_t)stream, n_partials);
    }
    EpiRelu2Lines epi{(uint16_t*)post_bf16, N, dequant, N, M};
    return launch_gemm_fmt<MainCfg, FMT_E4M3, FMT_E4M3>(gt, epi, (hipStream_t)stream, 0);
}
