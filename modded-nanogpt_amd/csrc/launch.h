// Host-side launcher of gemm_tn_kernel: picks the fp8 format instantiation and the grid.
#pragma once
#include "gemm_tn.h"
#include "host_util.h"
#include <atomic>

namespace ngpt {

// 256 x 256 tile, 8 waves as 4 (rows) x 2 (cols): each wave owns 64 x 128 = 2 x 4 MFMA tiles.
using MainCfg = TileCfg<256, 256, 4, 2, 128, 2>;
// Small problems (fewer 256 x 256 tiles than half the compute units): 128 x 128 tiles, 4 waves of 64 x 64, two
// workgroups per compute unit, so that four times as many workgroups share the work.
using SmallCfg = TileCfg<128, 128, 2, 2, 128, 2, 2>;
// (Measured slower on MI355X for the shapes of this path: four 32 KiB stages of 64-byte k-steps, and a
// 256 x 128 tile with two 4-wave workgroups per CU.  The kernel stays generic over TileCfg.)


// hipFuncSetAttribute applies to the device that is current when it is called: one flag per kernel
// instantiation and device.  Racing first calls both set the attribute, which is harmless.
struct PerDeviceOnce {
    std::atomic<bool> done[kMaxDevices];
    template <class F>
    int run(F&& f) {
        const int dev = current_device();
        if (dev >= 0 && dev < kMaxDevices && done[dev].load(std::memory_order_acquire)) return NGPT_OK;
        if (int e = f()) return e;
        if (dev >= 0 && dev < kMaxDevices) done[dev].store(true, std::memory_order_release);
        return NGPT_OK;
    }
};

template <class Cfg, int FA, int FB, class Epi>
int launch_gemm_fmt(const GemmOperands& g, const Epi& epi, hipStream_t st, int max_grid) {
    auto kernel = gemm_tn_kernel<Cfg, FA, FB, Epi, GridIter>;
    constexpr int LDS = Cfg::SMEM_BYTES + Epi::EXTRA_LDS;
    static PerDeviceOnce configured;
    if (int e = configured.run([&] { return allow_lds(kernel, LDS); })) return e;
    int tiles = ((g.R + Cfg::BM - 1) / Cfg::BM) * ((g.C + Cfg::BN - 1) / Cfg::BN) * (g.splits < 1 ? 1 : g.splits);
    int cus = num_cus();
    if (cus <= 0) return fail(NGPT_EINVAL, "no HIP device");
    int slots = cus * Cfg::WGS_PER_CU;      // as many workgroups as can be resident at once
    int grid = tiles < slots ? tiles : slots;
    // a multiple of 8 keeps the walk's XCD-aware numbering (TileOrder::seq_of); surplus workgroups find no job and leave
    if (grid % 8 && (grid + 7) / 8 * 8 <= slots) grid = (grid + 7) / 8 * 8;
    if (max_grid > 0 && grid > max_grid) grid = max_grid;
    kernel<<<grid, Cfg::THREADS, LDS, st>>>(g, epi);
    return check_launch("gemm_tn_kernel");
}

struct EpiStoreBf16;
template <class Epi> constexpr bool kBf16Epi = std::is_same<Epi, EpiStoreBf16>::value;

template <class Cfg, class Epi>
int launch_gemm_cfg(const GemmOperands& g, int fa, int fb, const Epi& epi, hipStream_t st, int max_grid = 0) {
    if ((fa & 3) == FMT_BF16 || (fb & 3) == FMT_BF16) {   // bf16 x bf16 -> bf16: row-major or contraction-major operands
        if constexpr (kBf16Epi<Epi> && std::is_same<Cfg, MainCfg>::value) {
            constexpr int N = FMT_BF16, T = FMT_BF16 | FMT_TRANSPOSED;
            if (fa == N && fb == N) return launch_gemm_fmt<Cfg, N, N>(g, epi, st, max_grid);
            if (fa == N && fb == T) return launch_gemm_fmt<Cfg, N, T>(g, epi, st, max_grid);
            if (fa == T && fb == T) return launch_gemm_fmt<Cfg, T, T>(g, epi, st, max_grid);
            if (fa == T && fb == N) return launch_gemm_fmt<Cfg, T, N>(g, epi, st, max_grid);
        }
        return fail(NGPT_EINVAL, "bf16 operands: unsupported format / output combination");
    }
    if (fa & FMT_TRANSPOSED) {   // only the combination the fused CE backward uses is instantiated
        if constexpr (std::is_same<Epi, EpiStoreBf16>::value) {
            if (fa == (FMT_E5M2 | FMT_TRANSPOSED) && fb == FMT_E4M3)
                return launch_gemm_fmt<Cfg, FMT_E5M2 | FMT_TRANSPOSED, FMT_E4M3>(g, epi, st, max_grid);
        }
        return fail(NGPT_EINVAL, "transposed A operand: unsupported format / output combination");
    }
    if (fa == FMT_E4M3 && fb == FMT_E4M3) return launch_gemm_fmt<Cfg, FMT_E4M3, FMT_E4M3>(g, epi, st, max_grid);
    if (fa == FMT_E5M2 && fb == FMT_E4M3) return launch_gemm_fmt<Cfg, FMT_E5M2, FMT_E4M3>(g, epi, st, max_grid);
    if (fa == FMT_E4M3 && fb == FMT_E5M2) return launch_gemm_fmt<Cfg, FMT_E4M3, FMT_E5M2>(g, epi, st, max_grid);
    return launch_gemm_fmt<Cfg, FMT_E5M2, FMT_E5M2>(g, epi, st, max_grid);
}

template <class Cfg, class Epi>
int launch_gemm(const GemmOperands& g, int fa, int fb, const Epi& epi, hipStream_t st, int max_grid = 0) {
    return launch_gemm_cfg<Cfg>(g, fa, fb, epi, st, max_grid);
}

}  // namespace ngpt
