// Launch planning of the FP32 MFMA products: host arithmetic only (see csrc/gemm_plan.hpp).  Kept apart from the
// kernels so that a change of the planner never touches a kernel source.
#include <cstdlib>

#include "../csrc/dlmi_common.hpp"
#include "../csrc/gemm_plan.hpp"

namespace dlmi {

struct TileCfg {
  int bm, bn, bk;
};

// Tuning aid: DLMI_GEMM_SPLIT=<n> forces the number of K slices (1 = none).
static int split_choice() {
  static int const c = [] {
    char const *e = std::getenv("DLMI_GEMM_SPLIT");
    return e != nullptr ? std::atoi(e) : 0;  // 0: choose by shape
  }();
  return c;
}

// Tuning aid: DLMI_GEMM_TILE=<index> forces a tile shape (0: 128x128, 1: 256x128, 2: 256x256, 3: 64x64 with 4
// wavefronts; 4: 128x128 with 8 wavefronts).
static int tile_choice() {
  static int const c = [] {
    char const *e = std::getenv("DLMI_GEMM_TILE");
    return e != nullptr ? std::atoi(e) : -1;  // -1: choose by shape
  }();
  return c;
}

GemmPlan plan_gemm(int const num_cu, size_t M, size_t N, size_t K) {
  static TileCfg const cfgs[] = {{128, 128, 16}, {256, 128, 16}, {256, 256, 16}, {64, 64, 16}, {128, 128, 16}};
  int choice = tile_choice();
  if (choice < 0 || choice >= static_cast<int>(sizeof(cfgs) / sizeof(cfgs[0]))) {
    // default: the shape with the smallest estimated time.  Main loop: rounds of workgroups over the CUs x
    // work of one workgroup x workgroups sharing a CU / measured relative efficiency of the shape (256 x 256
    // runs one workgroup per CU, 128-wide shapes two, 64 x 64 four).  Epilogue: storing a tile costs about as
    // much as 32 k of its main loop, and it is exposed once per CU - workgroups that share a CU or follow each
    // other on it store while another one multiplies.  (Measured on 65536 x 256 x 256, where the 256 x 256 shape
    // is one round of 16 K tiles: its 7.4 us of stores are 10 % of the launch; 128-wide tiles run 4 % faster.)
    // A small output picks small tiles: a workgroup's time is its own MFMA count as long as it has a CU to itself.
    static int const per_cu[] = {2, 2, 1, 4};
    static double const eff[] = {0.95, 0.97, 1.0, 0.8};
    double const epilogue_k = 32.0;
    double best = 0.0;
    for (int c = 0; c < 4; ++c) {
      size_t const tiles = dlmi_ceil_div(M, cfgs[c].bm) * dlmi_ceil_div(N, cfgs[c].bn);
      size_t const slots = static_cast<size_t>(num_cu) * per_cu[c];
      size_t const rounds = dlmi_ceil_div(tiles, slots);
      size_t const sharing = dlmi_ceil_div(tiles < slots ? tiles : slots, static_cast<size_t>(num_cu));
      double const per_k = static_cast<double>(cfgs[c].bm) * cfgs[c].bn * sharing;
      double const t = per_k * (static_cast<double>(rounds) * K / eff[c] + epilogue_k / (rounds * sharing));
      if (c == 0 || t < best) {
        best = t;
        choice = c;
      }
    }
  }
  // A small output behind a very long reduction (the weight gradient of a narrow layer on a tall batch) is
  // split over K anyway; its slices then run best as 128 x 128 tiles, one workgroup per CU (measured on
  // 256 x 256 x 65536: 92 us against 98 us with 64 x 64 tiles and 32 slices).
  size_t const tiles_128 = dlmi_ceil_div(M, 128) * dlmi_ceil_div(N, 128);
  bool const long_k = tile_choice() < 0 && split_choice() <= 0 && K >= 8192 && tiles_128 * 8 <= static_cast<size_t>(num_cu);
  if (long_k) choice = 0;
  // 128 x 128 tiles that come to at most one workgroup per CU: four wavefronts would leave every SIMD with one,
  // which cannot hide its own LDS and memory latencies.  The same tile as 8 wavefronts (4 x 2, each 32 x 64) puts
  // two on every SIMD (2048 x 2048 x 1024: 68.6 -> 65.9 us).  More than one workgroup per CU is better served by
  // independent 4-wavefront workgroups, which fill each other's barrier waits (measured: 128 x 64 and 256 x 128
  // tiles of 8 wavefronts lose 3-6 % against two workgroups of half the tile).  DLMI_GEMM_WAVES8=0 switches it off.
  static bool const waves8 = [] { char const *e = std::getenv("DLMI_GEMM_WAVES8"); return e == nullptr || std::atoi(e) != 0; }();
  if (choice == 0 && waves8 && tile_choice() < 0) {
    size_t const tiles0 = dlmi_ceil_div(M, 128) * dlmi_ceil_div(N, 128);
    size_t const slices = long_k ? static_cast<size_t>(num_cu) / tiles_128 : 1;
    if (tiles0 * (slices > 0 ? slices : 1) <= static_cast<size_t>(num_cu)) choice = 4;
  }
  GemmPlan p;
  p.choice = choice; p.bm = cfgs[choice].bm; p.bn = cfgs[choice].bn; p.bk = cfgs[choice].bk;
  p.waves = choice >= 4 ? 8 : 4;
  p.splits = 1;
  p.scratch_bytes = 0;
  if (long_k) {
    size_t s = static_cast<size_t>(num_cu) / tiles_128;
    size_t const max_s = dlmi_ceil_div(K, p.bk) / 8;
    if (s > max_s) s = max_s;
    if (s > 1) {
      p.splits = static_cast<unsigned>(s);
      p.scratch_bytes = s * M * N * sizeof(float);
    }
    return p;
  }
  // Split K when the output alone cannot fill the machine (few tiles, long K):
  // each slice writes its partial product, a second kernel adds them in order.
  size_t const tiles = dlmi_ceil_div(M, p.bm) * dlmi_ceil_div(N, p.bn);
  size_t const ktiles = dlmi_ceil_div(K, p.bk);
  size_t const target = static_cast<size_t>(num_cu) * 2;
  if ((tiles < target / 2 && ktiles >= 16) || split_choice() > 1) {
    size_t s = dlmi_ceil_div(target, tiles);
    size_t const max_s = ktiles / 8;  // at least 8 K tiles per slice
    if (s > max_s) s = max_s;
    if (split_choice() > 0) s = static_cast<size_t>(split_choice());
    if (s > 1) {
      p.splits = static_cast<unsigned>(s);
      p.scratch_bytes = s * M * N * sizeof(float);
    }
  }
  return p;
}

// Register stages of the K loop (see the launch switch of gemm() in csrc/gemm_f32_mfma.hip): two for the small tiles
// from 32 K tiles per slice on, one otherwise.
int gemm_register_stages(int bm, int bn, size_t kt_per_split) {
  return bm * bn <= 128 * 128 && kt_per_split >= 32 ? 2 : 1;
}

// Scratch the three products of a layer [B, K] -> [B, H] may ask for (K splits, epilogue statistics).
size_t fc_scratch_bytes(dlmi_ctx const *ctx, size_t B, size_t K, size_t H) {
  size_t need = 2 * 2 * 64 * H * sizeof(float);  // epilogue statistics: at most B / 64 ... 64 tile rows reserved
  size_t const rows = dlmi_ceil_div(B, 64);
  if (2 * 2 * rows * H * sizeof(float) > need) need = 2 * 2 * rows * H * sizeof(float);
  size_t const shapes[3][3] = {{B, H, K}, {B, K, H}, {H, K, B}};
  for (auto const &sh : shapes) {
    GemmPlan const p = plan_gemm(ctx->num_cu, sh[0], sh[1], sh[2]);
    // (behind the partial products of a split: the slices' shares of a bias gradient, [splits][M])
    size_t const b = p.scratch_bytes + (p.splits > 1 ? static_cast<size_t>(p.splits) * sh[0] * sizeof(float) : 0);
    if (b > need) need = b;
  }
  return need;
}

}  // namespace dlmi

using namespace dlmi;

extern "C" {

int dlmi_gemm_plan(int compute_units, size_t M, size_t N, size_t K, int *tile_m, int *tile_n, unsigned *k_slices,
                   int *register_stages) {
  if (compute_units <= 0 || M == 0 || N == 0 || K == 0) return DLMI_E_INVALID;
  GemmPlan const p = plan_gemm(compute_units, M, N, K);  // only the CU count enters the plan
  size_t const ktiles = dlmi_ceil_div(K, p.bk);
  size_t const kt_per_split = dlmi_ceil_div(ktiles, p.splits);
  if (tile_m != nullptr) *tile_m = p.bm;
  if (tile_n != nullptr) *tile_n = p.bn;
  if (k_slices != nullptr) *k_slices = static_cast<unsigned>(dlmi_ceil_div(ktiles, kt_per_split));
  if (register_stages != nullptr) *register_stages = gemm_register_stages(p.bm, p.bn, kt_per_split);
  return DLMI_OK;
}

}  // extern "C"
