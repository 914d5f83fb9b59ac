// Host-side launcher of gemm_tn_kernel: picks the fp8 format instantiation and the grid.
#pragma once
#include "gemm_tn.h"
#include "host_util.h"

namespace ngpt {

// 256 x 256 tile, 8 waves as 4 (rows) x 2 (cols): each wave owns 64 x 128 = 2 x 4 MFMA tiles.
using MainCfg = TileCfg<256, 256, 4, 2, 128, 2>;
// Alternatives selectable at run time through ngpt_tuning_set(0, id) (tuning aid; slower on MI355X
// for the shapes of this path).
using Cfg256x256k64s4 = TileCfg<256, 256, 4, 2, 64, 4>;     // id 1: four 32 KiB stages
using Cfg256x128k64s2 = TileCfg<256, 128, 2, 2, 64, 2, 2>;  // id 5: 4 waves, 48 KiB: two workgroups per CU

// Tuning keys: [0] GEMM tile config id, [2] ablation bits (timing aid),
// [4] split-K factor of ngpt_gemm_fp8_tn, [5] fused CE kernels: 1 = id 5 tile, 2 = id 1 tile,
// [6] 1 = split-K in the CE backward GEMMs
extern int g_tuning[8];

template <class Cfg, int FA, int FB, class Epi>
int launch_gemm_fmt(const GemmOperands& g, const Epi& epi, hipStream_t st, int max_grid) {
    auto kernel = gemm_tn_kernel<Cfg, FA, FB, Epi, GridIter>;
    constexpr int LDS = Cfg::SMEM_BYTES + Epi::EXTRA_LDS;
    static bool configured = false;
    if (!configured) {
        if (int e = allow_lds(kernel, LDS)) return e;
        configured = true;
    }
    int tiles = ((g.R + Cfg::BM - 1) / Cfg::BM) * ((g.C + Cfg::BN - 1) / Cfg::BN) * (g.splits < 1 ? 1 : g.splits);
    int cus = num_cus();
    if (cus <= 0) return fail(NGPT_EINVAL, "no HIP device");
    int slots = cus * Cfg::WGS_PER_CU;      // as many workgroups as can be resident at once
    int grid = tiles < slots ? tiles : slots;
    if (max_grid > 0 && grid > max_grid) grid = max_grid;
    kernel<<<grid, Cfg::THREADS, LDS, st>>>(g, epi);
    return check_launch("gemm_tn_kernel");
}

template <class Cfg, class Epi>
int launch_gemm_cfg(const GemmOperands& g, int fa, int fb, const Epi& epi, hipStream_t st, int max_grid = 0) {
    if (fa == FMT_E4M3 && fb == FMT_E4M3) return launch_gemm_fmt<Cfg, FMT_E4M3, FMT_E4M3>(g, epi, st, max_grid);
    if (fa == FMT_E5M2 && fb == FMT_E4M3) return launch_gemm_fmt<Cfg, FMT_E5M2, FMT_E4M3>(g, epi, st, max_grid);
    if (fa == FMT_E4M3 && fb == FMT_E5M2) return launch_gemm_fmt<Cfg, FMT_E4M3, FMT_E5M2>(g, epi, st, max_grid);
    return launch_gemm_fmt<Cfg, FMT_E5M2, FMT_E5M2>(g, epi, st, max_grid);
}

// Dispatch on the run-time tile configuration (default MainCfg).
template <class Cfg /* default */, class Epi>
int launch_gemm(const GemmOperands& g, int fa, int fb, const Epi& epi, hipStream_t st, int max_grid = 0) {
    switch (g_tuning[0]) {
        case 1: return launch_gemm_cfg<Cfg256x256k64s4>(g, fa, fb, epi, st, max_grid);
        case 5: return launch_gemm_cfg<Cfg256x128k64s2>(g, fa, fb, epi, st, max_grid);
        default: return launch_gemm_cfg<Cfg>(g, fa, fb, epi, st, max_grid);
    }
}

}  // namespace ngpt
