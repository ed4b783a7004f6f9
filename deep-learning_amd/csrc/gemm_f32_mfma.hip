// FP32 matrix-core (MFMA) contractions of the fully-connected layer for gfx950:
//
//   forward  Z  = X   * W^T   M=B, N=H,  K=K    A k-contiguous, B k-contiguous
//   dX       dY = dZn * Wn    M=B, N=H,  K=Hn   A k-contiguous, B n-contiguous
//   dW       dW = dZ^T * Xin  M=H, N=K,  K=B    A m-contiguous, B n-contiguous
//
// (reference leaves: v1/learner/fwp_st.cpp:4518-4555, bwp_st.cpp:1009-1045,
//  update_derivative_fwp_st.cpp:246-281 under /root/reference/lib/deep-learning.)
//
// One kernel template covers the three operand layouts.  A workgroup of 4
// wavefronts (2 x 2) or 8 (4 along M x 2 along N) owns a BM x BN tile of C; each
// wavefront owns its share as a grid of 32x32 v_mfma_f32_32x32x2_f32 blocks whose
// accumulators stay in registers for the whole K loop.  Why 8: two 4-wavefront
// workgroups that share a CU do not advance alike - the scheduler favours the
// older wavefronts, so one workgroup finishes early and the other runs its last
// sixth alone, on a matrix pipe it cannot keep fed (measured on 1024 x 2048 x 2048
// with 64 x 64 tiles: half the workgroups end after 56 us, the other half after
// 66 us).  Eight wavefronts behind one barrier stay together and share the B tile.  Operand tiles are
// staged through LDS (two stages, one barrier per K tile) behind one register
// stage (the global loads run two tiles ahead of the MFMAs) or, for the small
// tiles on a long reduction, two (three tiles ahead); the LDS writes, the
// global loads and the fragment reads of a tile are spread between the MFMAs
// of the previous one with scheduling-group hints.  Three edge treatments:
// none (shapes that are multiples of the tile), clamped rows (ragged M or N),
// guarded element by element (anything else).
//
// The MFMA consumes two k per instruction: lanes 0-31 supply k_lo, lanes 32-63
// k_hi.  Because the sum over k is order-free inside a tile, the kernel feeds
// k = {s, s+4} (s = 0..3) of every group of 8 instead of {2s, 2s+1}: a lane
// then needs 4 CONSECUTIVE k of one row, i.e. one ds_read_b128 per 4 MFMAs for
// either operand (one whose row index is contiguous in memory is transposed on
// its way into LDS).  Rows are padded by 4 floats so that those 16-byte reads
// (served 8 lanes at a time: 8 rows, 20 words apart) hit 32 distinct banks.  The
// stores into LDS are not conflict-free with that stride - a 16-byte store of a
// k-contiguous operand puts 4 lanes on a row, and the two rows of an 8-lane group
// overlap in 4 banks; the 4-byte stores of a transposed operand pair up row groups
// two apart - both two-way.  A stride that clears the stores (16 or 48 words)
// would put the reads four-way; the reads are three quarters of the LDS cycles.
// Counters: conflict cycles / LDS active = 0.33, 0.8 % of wave cycles wait on LDS.
//
// Workgroup ids are remapped so that (a) the ids that land on one XCD (id % 8)
// cover a compact block of tiles and (b) tiles are walked in groups of 8 rows
// of tiles, which keeps the A and B panels of concurrently running workgroups
// resident in that XCD's L2.
#include <cstdlib>
#include <type_traits>

#include "dlmi_common.hpp"
#include "gemm_plan.hpp"

namespace dlmi {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kGemmThreads = 256;  // of the 4-wavefront workgroups; the 8-wavefront ones have twice as many
constexpr int kXcds = 8;
constexpr int kGroupM = 8;
constexpr unsigned kClockWgs = 4096;  // workgroups whose time stamps a clocked launch keeps

struct GemmArgs {
  float const *A;
  float const *B;
  float *C;
  float const *bias;  // per-n, may be null
  size_t M, N, K;
  size_t lda, ldb, ldc;
  size_t k_per_split;  // K range of one blockIdx.z slice (multiple of BK)
  float *split_out;    // when gridDim.z > 1: [splits][M][N] partial products
  float *stats_out;    // optional [2][tiles_m][N]: per tile-row column sums of C and C^2 (gridDim.z == 1)
  // with stats_out, optional: the first tile row copies two per-column vectors [N] (the moving statistics of the
  // normalization that follows, before it updates them) to snap_out [2][N]
  float const *snap_a, *snap_b;
  float *snap_out;
  // optional: the workgroup of tile 0 / slice 0 stores {engine clock ticks, 100 MHz reference ticks} it spent from
  // entry to its last store (measurement aid: the engine clock inside this very launch, no profiler attached);
  // behind these two words every workgroup of slice 0 (the first kClockWgs) leaves four more: the 100 MHz counter
  // at its entry, after its last store was issued and after that store was acknowledged, and where it ran
  // (XCC_ID << 32 | HW_ID)
  unsigned long long *clock_out;
  int accumulate;      // C += result (only when gridDim.z == 1)
  int a_vec, b_vec;    // operand base and leading dimension allow 16-byte loads (ragged variant)
  unsigned tiles_m, tiles_n;
  // DB variants (a weight gradient dW = dZ^T X split over K): [gridDim.z][M], the sums over this slice's K range of
  // the A operand's rows - the slice's share of the bias gradient, taken from the registers the A tiles pass through
  float *db_out;
};

// LDS tile of either operand: [ROWS][BK+4], k contiguous, so that the MFMA
// fragments of both operands are 16-byte LDS reads whatever the layout in
// memory.  An operand whose row (m or n) index is contiguous in memory is
// transposed on its way into LDS.
template <int ROWS, int BK, bool KCONTIG, int THREADS = kGemmThreads>
struct TileShape {
  static constexpr int kStride = BK + 4;
  static constexpr int kFloats = ROWS * (BK + 4);
  static constexpr int kVec4 = ROWS * BK / 4;             // 16-byte pieces per tile
  // pieces per thread; a tile of fewer pieces than threads is moved by the first kVec4 threads (whole wavefronts)
  static constexpr int kPerThread = kVec4 >= THREADS ? kVec4 / THREADS : 1;
  static constexpr bool kSomeIdle = kVec4 < THREADS;
  static_assert(kVec4 % THREADS == 0 || (kVec4 < THREADS && kVec4 % 64 == 0), "tile must divide evenly over the workgroup");
  static_assert(ROWS % 32 == 0 && BK % 8 == 0, "tile shape");
  // the prefetch registers of one thread as ONE vector value (a first-class
  // SSA value: it can neither be spilled to scratch nor be promoted to LDS the
  // way a local array can)
  typedef float Regs __attribute__((ext_vector_type(4 * kPerThread)));

  // Which 16-byte piece thread-slot f (0 .. kVec4-1) moves: `row` and `k` are
  // relative to the tile; the piece covers 4 consecutive k (KCONTIG) or 4
  // consecutive rows (!KCONTIG).
  // !KCONTIG: a wavefront covers 8 k x 8 row groups, i.e. 8 segments of 128
  // contiguous bytes in memory; its transposed 4-byte LDS stores then fall
  // into 32 distinct banks (stride 20: row groups 4 apart share a bank).
  __device__ static __forceinline__ void piece(int f, int &row, int &k) {
    if constexpr (KCONTIG) {
      row = f / (BK / 4);
      k = (f % (BK / 4)) * 4;
    } else {
      int const kl = f & 7, rl = (f >> 3) & 7, rest = f >> 6;
      int const rh = rest % (ROWS / 32), kh = rest / (ROWS / 32);
      k = kh * 8 + kl;
      row = (rh * 8 + rl) * 4;
    }
  }
};

// How a kernel variant treats the edges of its operands.
//   kGuarded  any shape and alignment: every piece checked, element by element where it crosses an edge
//   kFast     M, N, K multiples of the tile, 16-byte aligned operands: no checks at all
//   kClamped  K a multiple of BK and aligned operands, but M or N ragged (a layer of 784 or 10 units): the loads
//             of rows beyond the operand are redirected to its last rows (always in bounds, still one 16-byte
//             load each, so the K loop is the fast one) and their products are dropped by the guarded stores
enum : int { kGuarded = 0, kFast = 1, kClamped = 2 };

// Global -> registers for one operand tile.  `row0` is the tile's first row
// (m or n), `k0` its first k.
template <int ROWS, int BK, bool KCONTIG, int MODE, int THREADS>
__device__ __forceinline__ typename TileShape<ROWS, BK, KCONTIG, THREADS>::Regs tile_load(float const *__restrict__ P,
                                                                                        size_t ld, size_t row0, size_t k0,
                                                                                        size_t rows_total, size_t k_end,
                                                                                        bool vec_ok) {
  using T = TileShape<ROWS, BK, KCONTIG, THREADS>;
  typename T::Regs regs;
  if constexpr (T::kSomeIdle) {
    if (static_cast<int>(threadIdx.x) >= T::kVec4) {
#pragma unroll
      for (int e = 0; e < 4 * T::kPerThread; ++e) regs[e] = 0.0f;
      return regs;
    }
  }
#pragma unroll
  for (int i = 0; i < T::kPerThread; ++i) {
    int tr, tk;
    T::piece(threadIdx.x + i * THREADS, tr, tk);
    size_t row = row0 + tr;
    size_t const k = k0 + tk;
    if constexpr (MODE == kClamped) {
      // a k-contiguous piece lies in one row, the other kind covers 4 consecutive rows (rows_total % 4 == 0)
      size_t const last = KCONTIG ? rows_total - 1 : rows_total - 4;
      row = row < last ? row : last;
    }
    float const *src = KCONTIG ? P + row * ld + k : P + k * ld + row;
    v4f t;
    if constexpr (MODE != kGuarded) {
      (void)vec_ok;
      t = *reinterpret_cast<v4f const *>(src);
    } else {
      // ragged shape: a piece that lies wholly inside the operand still moves as
      // one 16-byte load when the operand's alignment allows (vec_ok); only the
      // pieces on the edge go element by element, zero-filled outside
      bool const whole = KCONTIG ? (row < rows_total && k + 3 < k_end) : (row + 3 < rows_total && k < k_end);
      if (vec_ok && whole) {
        t = *reinterpret_cast<v4f const *>(src);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          size_t const rr = KCONTIG ? row : row + e;
          size_t const kk = KCONTIG ? k + e : k;
          t[e] = (rr < rows_total && kk < k_end) ? (KCONTIG ? P[rr * ld + kk] : P[kk * ld + rr]) : 0.0f;
        }
      }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) regs[4 * i + e] = t[e];
  }
  return regs;
}

template <int ROWS, int BK, bool KCONTIG, int THREADS>
__device__ __forceinline__ void tile_store(float *__restrict__ lds,
                                           typename TileShape<ROWS, BK, KCONTIG, THREADS>::Regs const &regs) {
  using T = TileShape<ROWS, BK, KCONTIG, THREADS>;
  if constexpr (T::kSomeIdle) {
    if (static_cast<int>(threadIdx.x) >= T::kVec4) return;
  }
#pragma unroll
  for (int i = 0; i < T::kPerThread; ++i) {
    int tr, tk;
    T::piece(threadIdx.x + i * THREADS, tr, tk);
    if constexpr (KCONTIG) {
      v4f t;
#pragma unroll
      for (int e = 0; e < 4; ++e) t[e] = regs[4 * i + e];
      *reinterpret_cast<v4f *>(lds + tr * T::kStride + tk) = t;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) lds[(tr + e) * T::kStride + tk] = regs[4 * i + e];
    }
  }
}

// Fragment for 4 consecutive MFMA steps of one 32-row block: element s feeds
// step s.  `r` = row inside the tile (block base + lane % 32), `kk` = first k
// of this lane's 4 (group base + (lane / 32) * 4).
template <int ROWS, int BK, bool KCONTIG>
__device__ __forceinline__ v4f frag_load(float const *__restrict__ lds, int r, int kk) {
  using T = TileShape<ROWS, BK, KCONTIG>;
  return *reinterpret_cast<v4f const *>(lds + r * T::kStride + kk);
}

// Instruction-order hints for the software pipeline (scheduling group masks:
// 0x008 MFMA, 0x020 vector-memory read, 0x100 LDS read, 0x200 LDS write).
template <int MASK, int N>
__device__ __forceinline__ void sched_group() {
  if constexpr (N > 0) __builtin_amdgcn_sched_group_barrier(MASK, N, 0);
}
// CNT instructions of kind MASK spread evenly behind NMF consecutive MFMAs.
template <int NMF, int MASK, int CNT, int M = 0>
__device__ __forceinline__ void sched_spread() {
  if constexpr (M < NMF) {
    sched_group<0x008, 1>();
    sched_group<MASK, ((M + 1) * CNT) / NMF - (M * CNT) / NMF>();
    sched_spread<NMF, MASK, CNT, M + 1>();
  }
}

// XCD-aware order of a launch's workgroups: the ids that land on one XCD (id % 8) walk one compact eighth of
// the tiles.
__device__ __forceinline__ unsigned xcd_order(unsigned id, unsigned ntiles) {
  return ntiles % kXcds == 0 ? (id % kXcds) * (ntiles / kXcds) + id / kXcds : id;
}

// One tile of one product: tile number `lid` (in the grouped order below) of K slice `zslice` of `nslices`.
template <int BM, int BN, int BK, bool A_KCONTIG, bool B_KCONTIG, int MODE, int RST, int WVM = 2, bool DB = false>
__device__ __forceinline__ void gemm_tile(GemmArgs const &g, unsigned const lid, unsigned const zslice, unsigned const nslices,
                                          float *__restrict__ lds) {
  constexpr bool FAST = MODE == kFast;          // no edge anywhere: unguarded stores
  constexpr bool FAST_LOOP = MODE != kGuarded;  // the scheduled K loop
  constexpr int THREADS = 128 * WVM;            // WVM wavefronts along M x 2 along N
  using TA = TileShape<BM, BK, A_KCONTIG, THREADS>;
  using TB = TileShape<BN, BK, B_KCONTIG, THREADS>;
  constexpr int WM = BM / WVM, WN = BN / 2;  // wavefront tile
  constexpr int TM = WM / 32, TN = WN / 32;
  static_assert(BK % 8 == 0, "K tile is consumed in groups of 8");
  constexpr int kStage = TA::kFloats + TB::kFloats;  // lds: 2 stages of (A tile, B tile)

  bool const clocked = g.clock_out != nullptr && lid == 0 && zslice == 0;
  unsigned long long c0 = 0, r0 = 0;
  if (clocked) {
    c0 = __builtin_amdgcn_s_memtime();
    r0 = __builtin_amdgcn_s_memrealtime();
  }
  // ---- which tile: walked in groups of 8 rows of tiles -----------------------
  unsigned const per_group = kGroupM * g.tiles_n;
  unsigned const first_m = (lid / per_group) * kGroupM;
  unsigned const gsize = (g.tiles_m - first_m) < kGroupM ? (g.tiles_m - first_m) : kGroupM;
  unsigned const tile_m = first_m + (lid % per_group) % gsize;
  unsigned const tile_n = (lid % per_group) / gsize;
  size_t const m0 = static_cast<size_t>(tile_m) * BM;
  size_t const n0 = static_cast<size_t>(tile_n) * BN;

  size_t const k_begin = zslice * g.k_per_split;
  size_t const k_end = (k_begin + g.k_per_split < g.K) ? k_begin + g.k_per_split : g.K;
  int const ktiles = static_cast<int>((k_end - k_begin + BK - 1) / BK);

  int const lane = threadIdx.x & 63;
  int const wave = threadIdx.x >> 6;
  int const wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;
  int const lr = lane & 31;        // row inside a 32-block (A: m, B: n)
  int const lk = (lane >> 5) * 4;  // this lane's k offset inside a group of 8

  v16f acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  // Fragments of K group `kk` (8 consecutive k) of the tile staged at sa / sb.
  auto frags = [&](float const *__restrict__ sa, float const *__restrict__ sb, int kk, v4f (&fa)[TM], v4f (&fb)[TN]) {
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[i] = frag_load<BM, BK, A_KCONTIG>(sa, wm0 + i * 32 + lr, kk + lk);
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[j] = frag_load<BN, BK, B_KCONTIG>(sb, wn0 + j * 32 + lr, kk + lk);
  };
  // MFMA steps s0 .. s1-1 (of 4) of one K group for every block of the wavefront.
  auto steps = [&](v4f const (&fa)[TM], v4f const (&fb)[TN], int s0, int s1) {
#pragma unroll
    for (int s = s0; s < s1; ++s)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][s], fb[j][s], acc[i][j], 0, 0, 0);
  };

  // DB: every A tile goes through this thread's registers once, on its way to LDS; what it holds of each - 4
  // consecutive rows at one k - is added up per thread over the K tiles and combined at the end of the tile.
  static_assert(!DB || (!A_KCONTIG && MODE == kFast), "the bias gradient rides along in the fast weight-gradient variants");
  bool const db_here = DB && tile_n == 0;  // one column of tiles reports the sums
  float dbacc[DB ? 4 * TA::kPerThread : 1];
#pragma unroll
  for (int e = 0; e < (DB ? 4 * TA::kPerThread : 1); ++e) dbacc[e] = 0.0f;
  auto db_add = [&](typename TA::Regs const &r) {  // (every workgroup adds: a branch would cut the K loop's schedule in two)
    if constexpr (DB) {
#pragma unroll
      for (int e = 0; e < 4 * TA::kPerThread; ++e) dbacc[e] += r[e];
    }
  };
  static_assert(BK == 16, "the pipeline below is written for two K groups per tile");
  constexpr int NM = TM * TN * (BK / 2);                                     // MFMAs per K tile
  constexpr int NFR = TM + TN;                                               // LDS reads per K group
  constexpr int NWR = (A_KCONTIG ? 1 : 4) * TA::kPerThread + (B_KCONTIG ? 1 : 4) * TB::kPerThread;  // LDS writes
  constexpr int NLD = TA::kPerThread + TB::kPerThread;                       // global loads

  if (ktiles > 0) {
    // Software pipeline over the K tiles: two LDS stages, one or two register stages.
    // During tile kt (LDS stage kt&1): tile kt+1, fetched from memory during
    // tile kt-1, moves from registers into the other stage, the global loads of
    // tile kt+2 are issued, and after the barrier - placed three quarters into
    // the tile's MFMAs, when every wavefront is done with both the reads of this
    // stage and the writes of the next - the first fragments of tile kt+1 are
    // read.  LDS and memory traffic is spread between the MFMAs, so the matrix
    // pipe only waits at the barrier itself.
    // RST == 2: TWO register stages.  A K tile of a small tile lasts a quarter of a microsecond, less than a
    // load from the memory side takes, so the loads run three tiles ahead of the MFMAs (tile kt+3 is fetched
    // during tile kt and moves to LDS during tile kt+2); the stages alternate with the tile's parity.
    static_assert(RST == 1 || RST == 2, "one or two register stages");
    auto load_a = [&](int t) {
      return tile_load<BM, BK, A_KCONTIG, MODE, THREADS>(g.A, g.lda, m0, k_begin + static_cast<size_t>(t) * BK, g.M, k_end, g.a_vec != 0);
    };
    auto load_b = [&](int t) {
      return tile_load<BN, BK, B_KCONTIG, MODE, THREADS>(g.B, g.ldb, n0, k_begin + static_cast<size_t>(t) * BK, g.N, k_end, g.b_vec != 0);
    };
    // The loads of the first two (with two register stages: three) K tiles are issued back to back and only
    // the first is waited for before it goes to LDS: a workgroup's start costs one trip to memory, not two
    // (the loads of a wavefront return in the order of their issue).
    // One register stage: ra/rb hold tile kt+1 at the start of tile kt.  Two: tile kt+1 is in ra/rb for even
    // kt and in ra2/rb2 for odd kt, tile kt+2 in the other pair.
    typename TA::Regs const r0a = load_a(0);
    typename TB::Regs const r0b = load_b(0);
    typename TA::Regs ra = {}, ra2 = {};
    typename TB::Regs rb = {}, rb2 = {};
    if (ktiles > 1) {
      ra = load_a(1);
      rb = load_b(1);
    }
    if constexpr (RST == 2) {
      if (ktiles > 2) {
        ra2 = load_a(2);
        rb2 = load_b(2);
      }
    }
    tile_store<BM, BK, A_KCONTIG, THREADS>(lds, r0a);
    tile_store<BN, BK, B_KCONTIG, THREADS>(lds + TA::kFloats, r0b);
    db_add(r0a);
    __syncthreads();
    v4f f0a[TM], f0b[TN];
    frags(lds, lds + TA::kFloats, 0, f0a, f0b);

    // one K tile; STORE: a next tile exists (in the registers xa / xb), LOAD: a tile RST further on exists and
    // is fetched into the same registers
    auto tile_step = [&](int kt, auto store_c, auto load_c, typename TA::Regs &xa, typename TB::Regs &xb) {
      constexpr bool STORE = decltype(store_c)::value, LOAD = decltype(load_c)::value;
      float const *const sa = lds + (kt & 1) * kStage;
      float *const na = lds + ((kt & 1) ^ 1) * kStage;
      v4f f1a[TM], f1b[TN];
      frags(sa, sa + TA::kFloats, 8, f1a, f1b);
      steps(f0a, f0b, 0, 4);
      if constexpr (STORE) {
        tile_store<BM, BK, A_KCONTIG, THREADS>(na, xa);
        tile_store<BN, BK, B_KCONTIG, THREADS>(na + TA::kFloats, xb);
        db_add(xa);
      }
      if constexpr (LOAD) {
        xa = load_a(kt + 1 + RST);
        xb = load_b(kt + 1 + RST);
      }
      steps(f1a, f1b, 0, 2);
      if constexpr (FAST_LOOP) {
        sched_spread<NM / 8, 0x100, NFR>();
        sched_spread<NM / 4, 0x200, STORE ? NWR : 0>();
        sched_spread<NM / 4, 0x020, LOAD ? NLD : 0>();
        sched_group<0x008, NM / 8>();
      }
      if constexpr (STORE) {
        __syncthreads();
        frags(na, na + TA::kFloats, 0, f0a, f0b);
      }
      steps(f1a, f1b, 2, 4);
      if constexpr (FAST_LOOP && STORE) {
        sched_group<0x100, NFR>();
        sched_group<0x008, NM / 4>();
      }
    };
    using std::false_type;
    using std::true_type;
    int kt = 0;
    if constexpr (RST == 1) {
      for (; kt + 2 < ktiles; ++kt) tile_step(kt, true_type{}, true_type{}, ra, rb);
      if (kt + 1 < ktiles) {
        tile_step(kt, true_type{}, false_type{}, ra, rb);
        ++kt;
      }
      tile_step(kt, false_type{}, false_type{}, ra, rb);
    } else {
      // pairs of tiles while both still fetch (the second of a pair fetches tile kt+4)
      for (; kt + 4 < ktiles; kt += 2) {
        tile_step(kt, true_type{}, true_type{}, ra, rb);
        tile_step(kt + 1, true_type{}, true_type{}, ra2, rb2);
      }
      // the last (at most four) tiles: kt is even here
      for (; kt < ktiles; ++kt) {
        bool const store = kt + 1 < ktiles, load = kt + 3 < ktiles;
        typename TA::Regs &xa = (kt & 1) ? ra2 : ra;
        typename TB::Regs &xb = (kt & 1) ? rb2 : rb;
        if (load) tile_step(kt, true_type{}, true_type{}, xa, xb);
        else if (store) tile_step(kt, true_type{}, false_type{}, xa, xb);
        else tile_step(kt, false_type{}, false_type{}, xa, xb);
      }
    }
  }

  // ---- epilogue: accumulator register e of lane l holds
  //      row (e/4)*8 + (l/32)*4 + e%4, column l%32 of its 32x32 block
  bool const split = nslices > 1;
  float *const out = split ? g.split_out + static_cast<size_t>(zslice) * g.M * g.N : g.C;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      size_t const col = n0 + wn0 + j * 32 + lr;
      float const bv = (!split && g.bias != nullptr && (FAST || col < g.N)) ? g.bias[col] : 0.0f;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        size_t const row = m0 + wm0 + i * 32 + (e / 4) * 8 + (lane >> 5) * 4 + (e % 4);
        if (FAST || (row < g.M && col < g.N)) {
          float *p = out + row * g.ldc + col;
          float v = acc[i][j][e] + bv;
          if (!split && g.accumulate) v += *p;
          *p = v;
        }
      }
    }

  // ---- optional fused epilogue: column sums of this tile's outputs and of
  // their squares, the batch-chunk partials the batch-(re)norm finalize kernel
  // consumes (chunk = tile row).  Fixed order: rows of a lane, the two lane
  // halves, the two wavefronts stacked along M.
  if (g.stats_out != nullptr) {
    __syncthreads();  // every wavefront is done reading the operand tiles: reuse that LDS
    float *const sl = lds;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      size_t const col = n0 + wn0 + j * 32 + lr;
      float const bv = (g.bias != nullptr && (FAST || col < g.N)) ? g.bias[col] : 0.0f;
      float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          size_t const row = m0 + wm0 + i * 32 + (e / 4) * 8 + (lane >> 5) * 4 + (e % 4);
          float const v = (FAST || row < g.M) ? acc[i][j][e] + bv : 0.0f;
          s1 += v;
          s2 += v * v;
        }
      s1 += __shfl_xor(s1, 32, 64);
      s2 += __shfl_xor(s2, 32, 64);
      if (lane < 32) {
        sl[((wave >> 1) * BN + wn0 + j * 32 + lr) * 2 + 0] = s1;
        sl[((wave >> 1) * BN + wn0 + j * 32 + lr) * 2 + 1] = s2;
      }
    }
    __syncthreads();
    for (int c = threadIdx.x; c < BN; c += THREADS) {
      size_t const col = n0 + c;
      if (FAST || col < g.N) {
        float t1 = sl[(0 * BN + c) * 2 + 0] + sl[(1 * BN + c) * 2 + 0];
        float t2 = sl[(0 * BN + c) * 2 + 1] + sl[(1 * BN + c) * 2 + 1];
#pragma unroll
        for (int w = 2; w < WVM; ++w) {  // the wavefronts stacked along M, top to bottom
          t1 += sl[(w * BN + c) * 2 + 0];
          t2 += sl[(w * BN + c) * 2 + 1];
        }
        g.stats_out[(0 * static_cast<size_t>(g.tiles_m) + tile_m) * g.N + col] = t1;
        g.stats_out[(1 * static_cast<size_t>(g.tiles_m) + tile_m) * g.N + col] = t2;
        if (g.snap_out != nullptr && tile_m == 0) {
          g.snap_out[col] = g.snap_a[col];
          g.snap_out[g.N + col] = g.snap_b[col];
        }
      }
    }
  }
  if constexpr (DB) {
    if (db_here) {
      // a piece's k is (f & 7) + 8 * kh: the 8 lanes that share a row group first (xor tree), then the halves kh
      // through LDS, kh = 0 first
      __syncthreads();  // every wavefront is done reading the operand tiles: reuse that LDS
#pragma unroll
      for (int i = 0; i < TA::kPerThread; ++i) {
        int const f = threadIdx.x + i * THREADS;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] = dbacc[4 * i + e];
          v[e] += __shfl_xor(v[e], 1, 64);
          v[e] += __shfl_xor(v[e], 2, 64);
          v[e] += __shfl_xor(v[e], 4, 64);
        }
        if ((f & 7) == 0 && (!TA::kSomeIdle || f < TA::kVec4)) {
          int tr, tk;
          TA::piece(f, tr, tk);
#pragma unroll
          for (int e = 0; e < 4; ++e) lds[(tk >> 3) * BM + tr + e] = v[e];
        }
      }
      __syncthreads();
      for (int r = threadIdx.x; r < BM; r += THREADS) {
        float t = lds[r];
#pragma unroll
        for (int kh = 1; kh < BK / 8; ++kh) t += lds[kh * BM + r];
        g.db_out[static_cast<size_t>(zslice) * g.M + m0 + r] = t;
      }
    }
  }
  if (clocked && threadIdx.x == 0) {
    g.clock_out[0] = __builtin_amdgcn_s_memtime() - c0;
    g.clock_out[1] = __builtin_amdgcn_s_memrealtime() - r0;
  }
}

// The workgroup of a product launch: which tile and slice it computes, and the time stamps of a clocked launch.
template <int BM, int BN, int BK, bool A_KCONTIG, bool B_KCONTIG, int MODE, int RST, int WVM, bool DB>
__device__ __forceinline__ void gemm_workgroup(GemmArgs const &g, float *__restrict__ lds) {
  unsigned const ntiles = g.tiles_m * g.tiles_n;
  unsigned lid = xcd_order(blockIdx.x, ntiles), zslice = blockIdx.z;
  if (gridDim.z % kXcds == 0 && ntiles % kXcds != 0) {
    // A split product of few tiles (dW of a wide-batch, narrow layer: 2 x 2 tiles, 64 slices): the tiles of one
    // K slice read the same rows of both operands.  Workgroups go to the XCDs in turn by their linear number
    // (x fastest, z slowest), which would put a slice's tiles on different XCDs and fetch every operand row once
    // per tile.  Renumbered so that a slice's tiles are consecutive workgroups of ONE XCD: they run at the same
    // time and the second and later readers hit that XCD's L2.  Which workgroup computes which (tile, slice)
    // changes, the sums do not.
    unsigned const linear = blockIdx.z * ntiles + blockIdx.x;
    unsigned const on_xcd = linear / kXcds;
    lid = on_xcd % ntiles;
    zslice = (on_xcd / ntiles) * kXcds + linear % kXcds;
  }
  bool const stamp = g.clock_out != nullptr && blockIdx.z == 0 && blockIdx.x < kClockWgs;
  unsigned long long ts = 0;
  if (stamp) ts = __builtin_amdgcn_s_memrealtime();
  gemm_tile<BM, BN, BK, A_KCONTIG, B_KCONTIG, MODE, RST, WVM, DB>(g, lid, zslice, gridDim.z, lds);
  if (stamp && threadIdx.x == 0) {
    unsigned long long const te = __builtin_amdgcn_s_memrealtime();
    __builtin_amdgcn_s_waitcnt(0);
    unsigned long long const td = __builtin_amdgcn_s_memrealtime();
    unsigned hw, xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw));
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    unsigned long long *o = g.clock_out + 2 + 4 * static_cast<size_t>(blockIdx.x);
    o[0] = ts; o[1] = te; o[2] = td; o[3] = (static_cast<unsigned long long>(xcc) << 32) | hw;
  }
}

template <int BM, int BN, int BK, bool A_KCONTIG, bool B_KCONTIG, int MODE, int WAVES_PER_EU, int RST, int WVM = 2>
__global__ __launch_bounds__(128 * WVM) __attribute__((amdgpu_waves_per_eu(WAVES_PER_EU, WAVES_PER_EU)))
void k_gemm_f32(GemmArgs g) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  gemm_workgroup<BM, BN, BK, A_KCONTIG, B_KCONTIG, MODE, RST, WVM, false>(g, lds);
}

// The fast weight-gradient variant whose K slices also leave their shares of the bias gradient (GemmArgs::db_out).
template <int BM, int BN, int BK, bool A_KCONTIG, bool B_KCONTIG, int WAVES_PER_EU, int RST, int WVM = 2>
__global__ __launch_bounds__(128 * WVM) __attribute__((amdgpu_waves_per_eu(WAVES_PER_EU, WAVES_PER_EU)))
void k_gemm_f32_db(GemmArgs g) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  gemm_workgroup<BM, BN, BK, A_KCONTIG, B_KCONTIG, kFast, RST, WVM, true>(g, lds);
}

// Several independent products of one kernel variant in ONE launch (the weight gradients of a network's layers:
// every layer's dZ exists once the backward pass has run).  The workgroups walk the concatenated tile lists in
// the XCD-aware order, so each XCD works on whole products and keeps their operands in its L2; a launch of
// many rounds of tiles runs at the rate of one large product instead of paying every product's start and tail.
constexpr int kGroupMax = 32;
struct GemmGroupProblem {
  float const *A, *B;
  float *C;
  unsigned M, N, K;
  unsigned tiles_n;
  unsigned tile_end;  // tiles of this and all earlier problems
};
struct GemmGroupArgs {
  GemmGroupProblem p[kGroupMax];
  unsigned n, total_tiles;
  int accumulate;
};
template <int BM, int BN, int BK, bool A_KCONTIG, bool B_KCONTIG, int WAVES_PER_EU, int RST>
__global__ __launch_bounds__(kGemmThreads) __attribute__((amdgpu_waves_per_eu(WAVES_PER_EU, WAVES_PER_EU)))
void k_gemm_f32_group(GemmGroupArgs a) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  unsigned const t = xcd_order(blockIdx.x, a.total_tiles);
  unsigned pi = 0;
  while (pi + 1 < a.n && t >= a.p[pi].tile_end) ++pi;
  GemmGroupProblem const &q = a.p[pi];
  GemmArgs g;
  g.A = q.A; g.B = q.B; g.C = q.C; g.bias = nullptr;
  g.M = q.M; g.N = q.N; g.K = q.K;
  g.lda = A_KCONTIG ? q.K : q.M; g.ldb = B_KCONTIG ? q.K : q.N; g.ldc = q.N;
  g.k_per_split = q.K; g.split_out = nullptr; g.stats_out = nullptr; g.clock_out = nullptr; g.db_out = nullptr;
  g.snap_a = nullptr; g.snap_b = nullptr; g.snap_out = nullptr;
  g.accumulate = a.accumulate; g.a_vec = 1; g.b_vec = 1;
  g.tiles_n = q.tiles_n; g.tiles_m = (q.M + BM - 1) / BM;
  gemm_tile<BM, BN, BK, A_KCONTIG, B_KCONTIG, kFast, RST>(g, t - (pi == 0 ? 0u : a.p[pi - 1].tile_end), 0u, 1u, lds);
}

// Fixed-order sum of the split-K partial products (+ bias, + previous C): slice 0, 1, 2, ... as before, with
// the loads of eight slices in flight at a time (one thread per element would otherwise walk the slices one
// memory latency after the other: 17 us for 64 slices of a 256 x 256 product).
// db_part != nullptr: also db[m] (+)= the slices' sums [splits][M] of the A operand's rows (the bias gradient that a
// split weight gradient formed on its way), slice 0 first.
__global__ __launch_bounds__(256) void k_splitk_reduce(float const *__restrict__ part, unsigned splits, size_t mn,
                                                        size_t N, float const *__restrict__ bias,
                                                        float *__restrict__ C, int accumulate,
                                                        float const *__restrict__ db_part, float *__restrict__ db,
                                                        size_t M) {
  size_t const stride = static_cast<size_t>(gridDim.x) * 256;
  if (db_part != nullptr) {
    for (size_t m = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; m < M; m += stride) {
      float s = 0.0f;
      unsigned z = 0;
      for (; z + 8 <= splits; z += 8) {  // (eight loads in flight, added in slice order)
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = db_part[(z + u) * M + m];
#pragma unroll
        for (int u = 0; u < 8; ++u) s += v[u];
      }
      for (; z < splits; ++z) s += db_part[z * M + m];
      db[m] = accumulate ? db[m] + s : s;
    }
  }
  for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < mn; i += stride) {
    float s = 0.0f;
    unsigned z = 0;
    for (; z + 8 <= splits; z += 8) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = part[(z + u) * mn + i];
#pragma unroll
      for (int u = 0; u < 8; ++u) s += v[u];
    }
    for (; z < splits; ++z) s += part[z * mn + i];
    if (bias != nullptr) s += bias[i % N];
    if (accumulate) s += C[i];
    C[i] = s;
  }
}

// ---------------------------------------------------------------- host side
template <int BM, int BN, int BK, bool AK, bool BKC, int WPE, bool HAS_CLAMPED, int RST, int WVM = 2, bool DB = false>
static int launch_gemm(dlmi_ctx *ctx, GemmArgs g, unsigned splits, int mode) {
  if (DB && mode != kFast) return dlmi_fail(ctx, DLMI_E_INVALID, "launch_gemm: the bias-gradient variant is a fast-path kernel");
  using TA = TileShape<BM, BK, AK, 128 * WVM>;
  using TB = TileShape<BN, BK, BKC, 128 * WVM>;
  constexpr size_t lds_bytes = 2 * (TA::kFloats + TB::kFloats) * sizeof(float);
  g.tiles_m = static_cast<unsigned>(dlmi_ceil_div(g.M, BM));
  g.tiles_n = static_cast<unsigned>(dlmi_ceil_div(g.N, BN));
  dim3 const grid(g.tiles_m * g.tiles_n, 1, splits);
  void (*kfast)(GemmArgs);
  if constexpr (DB) kfast = k_gemm_f32_db<BM, BN, BK, AK, BKC, WPE, RST, WVM>;
  else kfast = k_gemm_f32<BM, BN, BK, AK, BKC, kFast, WPE, RST, WVM>;
  auto const kslow = k_gemm_f32<BM, BN, BK, AK, BKC, kGuarded, WPE, 1, WVM>;
  // the clamped variant exists for the small tiles, which are the ones ragged layers run
  auto const kclamp = k_gemm_f32<BM, BN, BK, AK, BKC, HAS_CLAMPED ? kClamped : kGuarded, WPE, HAS_CLAMPED ? RST : 1, WVM>;
  if (!HAS_CLAMPED && mode == kClamped) mode = kGuarded;
  // more than 64 KB of LDS has to be asked for once per kernel and device
  static bool attr_set_on[64] = {false};
  bool &attr_set = attr_set_on[ctx->device >= 0 && ctx->device < 64 ? ctx->device : 0];
  if (!attr_set) {
    DLMI_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<void const *>(kfast),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
    DLMI_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<void const *>(kslow),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
    DLMI_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<void const *>(kclamp),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
    attr_set = true;
  }
  if (mode == kFast)
    hipLaunchKernelGGL(kfast, grid, dim3(128 * WVM), lds_bytes, ctx->stream, g);
  else if (mode == kClamped)
    hipLaunchKernelGGL(kclamp, grid, dim3(128 * WVM), lds_bytes, ctx->stream, g);
  else
    hipLaunchKernelGGL(kslow, grid, dim3(128 * WVM), lds_bytes, ctx->stream, g);
  DLMI_LAUNCH_CHECK(ctx, "k_gemm_f32");
  return DLMI_OK;
}

// C[M,N] (+)= A . B with the operand layouts given by the two flags.
// stats_chunks != nullptr: also write the column-sum partials [2][*stats_chunks][N]
// of C into the first half of the context's scratch (no split-K then).
template <bool AK, bool BKC>
static int gemm(dlmi_ctx *ctx, size_t M, size_t N, size_t K, float const *A, size_t lda, float const *B, size_t ldb,
                float *C, float const *bias, int accumulate, unsigned *stats_chunks = nullptr,
                unsigned *defer_slices = nullptr, float const *snap_a = nullptr, float const *snap_b = nullptr,
                float const **snap_out = nullptr, float *db = nullptr, bool *db_done = nullptr) {
  GemmPlan const plan = plan_gemm(ctx->num_cu, M, N, K);
  int const choice = plan.choice;
  int const bm = plan.bm, bn = plan.bn, bk = plan.bk;

  GemmArgs g;
  g.A = A; g.B = B; g.C = C; g.bias = bias; g.M = M; g.N = N; g.K = K; g.lda = lda; g.ldb = ldb; g.ldc = N;
  g.accumulate = accumulate; g.split_out = nullptr; g.stats_out = nullptr;
  g.snap_a = g.snap_b = nullptr; g.snap_out = nullptr;
  g.clock_out = ctx->gemm_clock;
  g.db_out = nullptr;
  if (db_done != nullptr) *db_done = false;
  if (snap_out != nullptr) *snap_out = nullptr;
  g.a_vec = (lda % 4 == 0 && dlmi_aligned16(A)) ? 1 : 0;
  g.b_vec = (ldb % 4 == 0 && dlmi_aligned16(B)) ? 1 : 0;
  int mode = kGuarded;
  if (K % bk == 0 && g.a_vec && g.b_vec) {
    if (M % bm == 0 && N % bn == 0)
      mode = kFast;
    else if ((AK || M % 4 == 0) && (BKC || N % 4 == 0) && M >= 4 && N >= 4)
      mode = kClamped;
  }
  size_t const ktiles = dlmi_ceil_div(K, bk);
  unsigned splits = plan.splits;
  if (splits > 1) {
    // (room for the slices' shares of a bias gradient behind the partial products)
    int rc = dlmi_scratch_reserve(ctx, plan.scratch_bytes + static_cast<size_t>(splits) * M * sizeof(float));
    if (rc != DLMI_OK) return rc;
  }
  if (stats_chunks != nullptr) {
    if (splits > 1) {
      *stats_chunks = 0;  // the slices hold partial products: the caller takes the statistics from C itself
    } else {
      *stats_chunks = static_cast<unsigned>(dlmi_ceil_div(M, bm));
      // also what the normalization tail reserves itself: it must not have to grow
      // (and thereby free) the block while these partials sit in it
      size_t const chunks_reserved = *stats_chunks > 32 ? *stats_chunks : 32;
      int rc = dlmi_scratch_reserve(ctx, 2 * 2 * static_cast<size_t>(chunks_reserved) * N * sizeof(float));
      if (rc != DLMI_OK) return rc;
      g.stats_out = reinterpret_cast<float *>(dlmi_scratch_data(ctx));
      if (snap_out != nullptr && snap_a != nullptr && snap_b != nullptr) {
        // the second half of what was reserved: the partial sums fill the first
        g.snap_a = snap_a; g.snap_b = snap_b;
        g.snap_out = g.stats_out + 2 * static_cast<size_t>(chunks_reserved) * N;
        *snap_out = g.snap_out;
      }
    }
  }
  size_t const kt_per_split = dlmi_ceil_div(ktiles, splits);
  g.k_per_split = kt_per_split * bk;
  splits = static_cast<unsigned>(dlmi_ceil_div(ktiles, kt_per_split));
  if (splits > 1) g.split_out = reinterpret_cast<float *>(dlmi_scratch_data(ctx));
  // A weight gradient that is split over K and runs the fast 128 x 128 kernels forms the bias gradient on its way:
  // the slices leave their shares behind the partial products, and the slice sum below adds them up too.  (Such a
  // product never shares a launch with others, so the grouped entry point takes this same path for it.)
  bool db_in_product = false;
  if constexpr (!AK) {
    db_in_product = db != nullptr && defer_slices == nullptr && splits > 1 && mode == kFast && (choice == 0 || choice == 4) &&
                    ctx->tune.db_in_product != 0;
    if (db_in_product) g.db_out = g.split_out + static_cast<size_t>(splits) * M * N;
  }
  int rc;
  switch (choice) {
    case 1: rc = launch_gemm<256, 128, 16, AK, BKC, 2, false, 1>(ctx, g, splits, mode); break;
    case 2: rc = launch_gemm<256, 256, 16, AK, BKC, 1, false, 1>(ctx, g, splits, mode); break;
    // The small tiles keep two register stages on a long reduction: a K tile of 64 x 64 is shorter than a load
    // takes (1024 x 2048 x 2048: forward 70.9 -> 67.7 us, dX 75.5 -> 69.9 us), and 128 x 128 gains too
    // (2048 x 2048 x 1024: 69.8 -> 68.5 us; at 8192 x 4096 x 4096 it reaches 145 TFLOP/s with them, 140
    // without).  A short reduction (16 K tiles) loses 2.5 % to the longer start.
    case 3:
      if (gemm_register_stages(bm, bn, kt_per_split) == 2)
        rc = launch_gemm<64, 64, 16, AK, BKC, 4, true, 2>(ctx, g, splits, mode);
      else
        rc = launch_gemm<64, 64, 16, AK, BKC, 4, true, 1>(ctx, g, splits, mode);
      break;
    // 8 wavefronts (4 along M x 2 along N) behind one barrier, one workgroup per CU, two wavefronts per SIMD
    case 4:
      if constexpr (!AK) {
        if (db_in_product) {
          if (gemm_register_stages(bm, bn, kt_per_split) == 2)
            rc = launch_gemm<128, 128, 16, AK, BKC, 2, false, 2, 4, true>(ctx, g, splits, mode);
          else
            rc = launch_gemm<128, 128, 16, AK, BKC, 2, false, 1, 4, true>(ctx, g, splits, mode);
          break;
        }
      }
      if (gemm_register_stages(bm, bn, kt_per_split) == 2)
        rc = launch_gemm<128, 128, 16, AK, BKC, 2, false, 2, 4>(ctx, g, splits, mode);
      else
        rc = launch_gemm<128, 128, 16, AK, BKC, 2, false, 1, 4>(ctx, g, splits, mode);
      break;
    default:
      if constexpr (!AK) {
        if (db_in_product) {
          if (gemm_register_stages(bm, bn, kt_per_split) == 2)
            rc = launch_gemm<128, 128, 16, AK, BKC, 2, true, 2, 2, true>(ctx, g, splits, mode);
          else
            rc = launch_gemm<128, 128, 16, AK, BKC, 2, true, 1, 2, true>(ctx, g, splits, mode);
          break;
        }
      }
      if (gemm_register_stages(bm, bn, kt_per_split) == 2)
        rc = launch_gemm<128, 128, 16, AK, BKC, 2, true, 2>(ctx, g, splits, mode);
      else
        rc = launch_gemm<128, 128, 16, AK, BKC, 2, true, 1>(ctx, g, splits, mode);
      break;
  }
  if (rc != DLMI_OK) return rc;
  if (defer_slices != nullptr) {
    // the caller adds the slices itself ([splits][M][N] at the start of the scratch block, slice order)
    *defer_slices = splits > 1 ? splits : 0;
    if (splits > 1) return DLMI_OK;
  }
  if (splits > 1) {
    size_t const mn = M * N;
    size_t blocks = dlmi_ceil_div(mn, 256);
    size_t const cap = static_cast<size_t>(ctx->num_cu) * 16;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(k_splitk_reduce, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, ctx->stream,
                       g.split_out, splits, mn, N, bias, C, accumulate, static_cast<float const *>(g.db_out), db, M);
    DLMI_LAUNCH_CHECK(ctx, "k_splitk_reduce");
    if (db_in_product && db_done != nullptr) *db_done = true;
  }
  return DLMI_OK;
}

// ---- several products in one launch
struct GroupItem {
  size_t M, N, K;
  float const *A, *B;
  float *C;
};
template <int BM, int BN, int BK, bool AK, bool BKC, int WPE, int RST>
static int launch_group(dlmi_ctx *ctx, GroupItem const *items, size_t n, int accumulate) {
  using TA = TileShape<BM, BK, AK>;
  using TB = TileShape<BN, BK, BKC>;
  constexpr size_t lds_bytes = 2 * (TA::kFloats + TB::kFloats) * sizeof(float);
  auto const kern = k_gemm_f32_group<BM, BN, BK, AK, BKC, WPE, RST>;
  static bool attr_set_on[64] = {false};
  bool &attr_set = attr_set_on[ctx->device >= 0 && ctx->device < 64 ? ctx->device : 0];
  if (!attr_set) {
    DLMI_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<void const *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      static_cast<int>(lds_bytes)));
    attr_set = true;
  }
  for (size_t first = 0; first < n; first += kGroupMax) {
    GemmGroupArgs a;
    a.n = static_cast<unsigned>(n - first < static_cast<size_t>(kGroupMax) ? n - first : kGroupMax);
    a.accumulate = accumulate;
    unsigned total = 0;
    for (unsigned i = 0; i < a.n; ++i) {
      GroupItem const &it = items[first + i];
      GemmGroupProblem &q = a.p[i];
      q.A = it.A; q.B = it.B; q.C = it.C;
      q.M = static_cast<unsigned>(it.M); q.N = static_cast<unsigned>(it.N); q.K = static_cast<unsigned>(it.K);
      q.tiles_n = static_cast<unsigned>(it.N / BN);
      total += static_cast<unsigned>(it.M / BM) * q.tiles_n;
      q.tile_end = total;
    }
    for (unsigned i = a.n; i < static_cast<unsigned>(kGroupMax); ++i) a.p[i] = a.p[a.n - 1];
    a.total_tiles = total;
    hipLaunchKernelGGL(kern, dim3(total), dim3(kGemmThreads), lds_bytes, ctx->stream, a);
    DLMI_LAUNCH_CHECK(ctx, "k_gemm_f32_group");
  }
  return DLMI_OK;
}

// Whether a product may join a grouped launch, and which kernel variant it would run there: shapes that are
// multiples of their tile, 16-byte aligned operands, no K split.  Returns the variant key (tile choice * 4 +
// register stages), or -1.
template <bool AK, bool BKC>
static int group_variant(dlmi_ctx const *ctx, GroupItem const &it) {
  GemmPlan const plan = plan_gemm(ctx->num_cu, it.M, it.N, it.K);
  if (plan.splits != 1 || plan.choice == 1) return -1;
  size_t const lda = AK ? it.K : it.M, ldb = BKC ? it.K : it.N;
  bool const vec = lda % 4 == 0 && ldb % 4 == 0 && dlmi_aligned16(it.A) && dlmi_aligned16(it.B);
  if (!vec || it.K % plan.bk != 0 || it.M % plan.bm != 0 || it.N % plan.bn != 0) return -1;
  if (it.M > 0xffffffffull || it.N > 0xffffffffull || it.K > 0xffffffffull) return -1;
  int const rst = plan.choice == 2 ? 1 : gemm_register_stages(plan.bm, plan.bn, dlmi_ceil_div(it.K, plan.bk));
  // (the 8-wavefront 128 x 128 variant is for launches of one workgroup per CU; a group has many per CU)
  return (plan.choice == 4 ? 0 : plan.choice) * 4 + rst;
}
template <bool AK, bool BKC>
static int launch_group_variant(dlmi_ctx *ctx, int variant, GroupItem const *items, size_t n, int accumulate) {
  switch (variant) {
    case 0 * 4 + 1: return launch_group<128, 128, 16, AK, BKC, 2, 1>(ctx, items, n, accumulate);
    case 0 * 4 + 2: return launch_group<128, 128, 16, AK, BKC, 2, 2>(ctx, items, n, accumulate);
    case 2 * 4 + 1: return launch_group<256, 256, 16, AK, BKC, 1, 1>(ctx, items, n, accumulate);
    case 3 * 4 + 1: return launch_group<64, 64, 16, AK, BKC, 4, 1>(ctx, items, n, accumulate);
    case 3 * 4 + 2: return launch_group<64, 64, 16, AK, BKC, 4, 2>(ctx, items, n, accumulate);
    default: return dlmi_fail(ctx, DLMI_E_INVALID, "no grouped kernel for variant %d", variant);
  }
}

}  // namespace dlmi

using namespace dlmi;

extern "C" {

int dlmi_fc_fwd(dlmi_ctx *ctx, size_t B, size_t K, size_t H, float const *X, float const *W, float const *bias,
                float *Z) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, X && W && Z, "null pointer");
  DLMI_REQUIRE(ctx, B > 0 && K > 0 && H > 0, "empty operand");
  if (narrow_fc_fwd_eligible(ctx, B, H)) return narrow_fc_fwd(ctx, B, K, H, X, W, bias, Z, nullptr);
  return gemm<true, true>(ctx, B, H, K, X, K, W, K, Z, bias, 0);
}

int dlmi_fc_softmax_fwd(dlmi_ctx *ctx, size_t B, size_t K, size_t H, float const *X, float const *W, float const *bias,
                        float *Z, float *Q) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, X && W && Z && Q, "null pointer");
  DLMI_REQUIRE(ctx, B > 0 && K > 0 && H > 0, "empty operand");
  if (narrow_fc_fwd_eligible(ctx, B, H)) return narrow_fc_fwd(ctx, B, K, H, X, W, bias, Z, Q);
  int const rc = gemm<true, true>(ctx, B, H, K, X, K, W, K, Z, bias, 0);
  return rc != DLMI_OK ? rc : dlmi_softmax_fwd(ctx, B, H, Z, Q);
}

static int fc_norm_act_fwd(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t K, size_t H, float const *X,
                           float const *W, float const *gamma, float const *beta, uint8_t const *mask,
                           float const *shortcut, float *Z, float *mean, float *stdv, float *mov_mean, float *mov_std,
                           float *r, float *d, float *y) {
  unsigned chunks = 0, slices = 0;
  // a mini-batch: the normalization kernel that follows owns whole columns and adds the K slices itself
  bool const defer = small_norm_eligible(ctx, B, H);
  float const *snapshot = nullptr;  // the moving statistics before this step, copied by the product's epilogue
  int rc = gemm<true, true>(ctx, B, H, K, X, K, W, K, Z, nullptr, 0, &chunks, defer ? &slices : nullptr, mov_mean, mov_std,
                            &snapshot);
  if (rc != DLMI_OK) return rc;
  float const *const scratch = reinterpret_cast<float const *>(dlmi_scratch_data(ctx));
  if (slices != 0)
    return fused_fwd_from_partials(ctx, desc, B, H, Z, gamma, beta, mask, shortcut, mean, stdv, mov_mean, mov_std, r, d, y,
                                   nullptr, 0, scratch, slices);
  // a small output runs split over K, where no slice sees whole sums: the
  // statistics then come from a pass over Z (nullptr / 0)
  return fused_fwd_from_partials(ctx, desc, B, H, Z, gamma, beta, mask, shortcut, mean, stdv, mov_mean, mov_std, r, d, y,
                                 chunks != 0 ? scratch : nullptr, chunks, nullptr, 0, snapshot);
}

int dlmi_fc_norm_act_fwd(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t K, size_t H, float const *X,
                         float const *W, float const *gamma, float const *beta, uint8_t const *mask, float *Z,
                         float *mean, float *stdv, float *mov_mean, float *mov_std, float *r, float *d, float *y) {
  if (ctx == nullptr || desc == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, X && W && Z, "null pointer");
  DLMI_REQUIRE(ctx, B > 0 && K > 0 && H > 0, "empty operand");
  return fc_norm_act_fwd(ctx, desc, B, K, H, X, W, gamma, beta, mask, nullptr, Z, mean, stdv, mov_mean, mov_std, r, d, y);
}

int dlmi_fc_norm_act_residual_fwd(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t K, size_t H,
                                  float const *X, float const *W, float const *gamma, float const *beta,
                                  uint8_t const *mask, float const *shortcut, float *Z, float *mean, float *stdv,
                                  float *mov_mean, float *mov_std, float *r, float *d, float *y) {
  if (ctx == nullptr || desc == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, X && W && Z && shortcut, "null pointer");
  DLMI_REQUIRE(ctx, B > 0 && K > 0 && H > 0, "empty operand");
  return fc_norm_act_fwd(ctx, desc, B, K, H, X, W, gamma, beta, mask, shortcut, Z, mean, stdv, mov_mean, mov_std, r, d, y);
}

int dlmi_fc_bwd_dx(dlmi_ctx *ctx, size_t B, size_t Hn, size_t H, float const *dZn, float const *Wn, float *dY,
                   int accumulate) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, dZn && Wn && dY, "null pointer");
  DLMI_REQUIRE(ctx, B > 0 && Hn > 0 && H > 0, "empty operand");
  return gemm<true, false>(ctx, B, H, Hn, dZn, Hn, Wn, H, dY, nullptr, accumulate);
}

int dlmi_fc_bwd_dx_norm_act_bwd(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t Hn, size_t H,
                                float const *dZn, float const *Wn, float const *x, float const *gamma, float const *beta,
                                uint8_t const *mask, float const *mean, float const *stdv, float const *r, float const *d,
                                float *dgamma, float *dbeta, float *dX) {
  if (ctx == nullptr || desc == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, dZn && Wn && dX, "null pointer");
  DLMI_REQUIRE(ctx, B > 0 && Hn > 0 && H > 0, "empty operand");
  // a mini-batch: the normalization kernel owns whole columns and adds the K slices of dY = dZn . Wn itself
  unsigned slices = 0;
  bool const defer = small_norm_eligible(ctx, B, H);
  // ... and below a narrow layer (an output layer of a few units) it forms dY itself: no product launch
  if (defer && Hn <= fused_bwd_narrow_max() && ctx->tune.narrow_dx_fused && x && gamma && beta && mean && stdv && r && d && dgamma && dbeta)
    return fused_bwd_from_narrow(ctx, desc, B, H, x, gamma, beta, mask, mean, stdv, r, d, dZn, Wn, Hn, dgamma, dbeta, dX);
  int rc = gemm<true, false>(ctx, B, H, Hn, dZn, Hn, Wn, H, dX, nullptr, 0, nullptr, defer ? &slices : nullptr);
  if (rc != DLMI_OK) return rc;
  if (slices != 0)
    return fused_bwd_from_slices(ctx, desc, B, H, x, gamma, beta, mask, mean, stdv, r, d,
                                 reinterpret_cast<float const *>(dlmi_scratch_data(ctx)), slices, dgamma, dbeta, dX);
  return dlmi_fused_norm_act_bwd(ctx, desc, B, H, x, gamma, beta, mask, mean, stdv, r, d, dX, dgamma, dbeta, dX);
}

int dlmi_fc_bwd_dw(dlmi_ctx *ctx, size_t B, size_t K, size_t H, float const *Xin, float const *dZ, float *dW,
                   float *db, int accumulate) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, Xin && dZ && dW, "null pointer");
  DLMI_REQUIRE(ctx, B > 0 && K > 0 && H > 0, "empty operand");
  // a narrow layer on a mini-batch: dW and db in one launch
  if (int const took = narrow_dw_try(ctx, B, K, H, Xin, dZ, dW, db, accumulate); took != 0) return took < 0 ? took : DLMI_OK;
  // any layer on a mini-batch: the reduction is the batch, a handful of K tiles; a kernel that stages it whole
  int rc = minibatch_dw_try(ctx, B, K, H, Xin, dZ, dW, accumulate);
  bool db_done = false;  // a product split over K brings the bias gradient along
  if (rc == 0)
    rc = gemm<false, false>(ctx, H, K, B, dZ, H, Xin, K, dW, nullptr, accumulate, nullptr, nullptr, nullptr, nullptr, nullptr,
                            db, &db_done);
  else rc = rc < 0 ? rc : DLMI_OK;
  if (rc != DLMI_OK || db == nullptr || db_done) return rc;
  // db[h] (+)= sum_b dZ[b,h] (update_derivative_fwp_st.cpp:283-302)
  return column_sums(ctx, B, H, dZ, db, accumulate);
}

int dlmi_fc_bwd_dw_grouped(dlmi_ctx *ctx, size_t n, dlmi_dw_problem const *problems, int accumulate) {
  if (ctx == nullptr) return DLMI_E_INVALID;
  DLMI_REQUIRE(ctx, n == 0 || problems != nullptr, "null pointer");
  // products of one kernel variant share a launch (from two on); everything else goes one by one
  constexpr size_t kMaxProblems = 256;
  for (size_t first = 0; first < n; first += kMaxProblems) {
    size_t const m = n - first < kMaxProblems ? n - first : kMaxProblems;
    dlmi_dw_problem const *pr = problems + first;
    int variant[kMaxProblems];
    GroupItem item[kMaxProblems];
    for (size_t i = 0; i < m; ++i) {
      DLMI_REQUIRE(ctx, pr[i].Xin && pr[i].dZ && pr[i].dW, "null pointer");
      DLMI_REQUIRE(ctx, pr[i].B > 0 && pr[i].K > 0 && pr[i].H > 0, "empty operand");
      item[i] = GroupItem{pr[i].H, pr[i].K, pr[i].B, pr[i].dZ, pr[i].Xin, pr[i].dW};
      variant[i] = group_variant<false, false>(ctx, item[i]);  // (a narrow layer is no multiple of a tile: -1)
      if (minibatch_dw_eligible(ctx, pr[i].B, pr[i].K, pr[i].H, pr[i].Xin, pr[i].dZ, pr[i].dW)) variant[i] = -1;  // its own kernel
    }
    // the mini-batch products that are not narrow layers: one launch for all of them, from two on; the first
    // narrow layer (at most 16 units: its kernel forms the bias gradient too) rides along in that launch
    {
      MinibatchDwProblem mb[kMaxProblems];
      size_t which[kMaxProblems], nmb = 0, narrow_at = m;
      for (size_t i = 0; i < m; ++i) {
        if (variant[i] == -1 && pr[i].H > 16 &&
            minibatch_dw_eligible(ctx, pr[i].B, pr[i].K, pr[i].H, pr[i].Xin, pr[i].dZ, pr[i].dW)) {
          which[nmb] = i;
          mb[nmb++] = MinibatchDwProblem{pr[i].B, pr[i].K, pr[i].H, pr[i].Xin, pr[i].dZ, pr[i].dW};
        } else if (narrow_at == m && pr[i].H <= 16 && narrow_dw_eligible(ctx, pr[i].B, pr[i].H)) {
          narrow_at = i;
        }
      }
      if (nmb >= 2 || (nmb == 1 && narrow_at < m)) {
        NarrowDwProblem nw{};
        if (narrow_at < m) {
          dlmi_dw_problem const &q = pr[narrow_at];
          nw = NarrowDwProblem{q.B, q.K, q.H, q.Xin, q.dZ, q.dW, q.db};
        }
        int rc = minibatch_dw_group(ctx, nmb, mb, accumulate, narrow_at < m ? &nw : nullptr);
        if (rc != DLMI_OK) return rc;
        for (size_t j = 0; j < nmb; ++j) variant[which[j]] = -2;  // done; the bias gradients follow below
        if (narrow_at < m) variant[narrow_at] = -3;                // done, bias gradient included
      }
    }
    for (size_t i = 0; i < m; ++i) {
      if (variant[i] == -2 || variant[i] == -3) continue;  // went with an earlier one
      GroupItem same[kMaxProblems];
      size_t ns = 0;
      if (variant[i] >= 0)
        for (size_t j = i; j < m; ++j)
          if (variant[j] == variant[i]) same[ns++] = item[j];
      if (ns >= 2) {
        int const v = variant[i];
        for (size_t j = i; j < m; ++j)
          if (variant[j] == v) variant[j] = -2;
        int rc = launch_group_variant<false, false>(ctx, v, same, ns, accumulate);
        if (rc != DLMI_OK) return rc;
        continue;  // (the bias gradients of grouped products follow below)
      }
      int rc = dlmi_fc_bwd_dw(ctx, pr[i].B, pr[i].K, pr[i].H, pr[i].Xin, pr[i].dZ, pr[i].dW, pr[i].db, accumulate);
      if (rc != DLMI_OK) return rc;
      variant[i] = -3;  // done, bias gradient included
    }
    for (size_t i = 0; i < m; ++i)
      if (variant[i] == -2 && pr[i].db != nullptr) {
        int rc = column_sums(ctx, pr[i].B, pr[i].H, pr[i].dZ, pr[i].db, accumulate);
        if (rc != DLMI_OK) return rc;
      }
  }
  return DLMI_OK;
}

}  // extern "C"
