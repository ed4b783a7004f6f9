// Single-launch batch-(re)normalization for tensors of a few thousand rows: the column panel scheme.
//
// MI355X has 8 XCDs of 32 CUs, each XCD with an L2 of its own; whatever misses an L2 crosses the fabric to
// the memory side at about 6.5 TB/s in total, so a kernel pair that reads a tensor twice (statistics, then
// apply) cannot move its 12 B/element (forward) faster than that.  Here the tensor is read ONCE: the
// launch has one workgroup per CU; the 32 workgroups that run on one XCD own H/8 columns together and walk
// them in panels of P columns.  Per panel every workgroup loads its own B/32 rows of the panel into
// registers, forms the column sums of those rows, publishes them as one chunk partial, waits until the
// other 31 workgroups of the XCD have published theirs, adds the 32 partials in rank order (the same
// fixed-order, atomic-free sum as the multi-launch path), and applies the result to the rows it still
// holds in registers.  Three panels are in flight per workgroup (loading p+2, published p+1, applying p), so
// the wait for the other workgroups overlaps the memory stream.
//
// The exchange among the 32 workgroups never leaves their XCD: the partials are written with ordinary
// stores (write-through to the L2), completed with s_waitcnt before the workgroup's arrival is counted, and
// both the arrival counter and its polling are read-modify-write atomics, which execute in the L2 itself
// (a plain or workgroup-scope atomic LOAD may be served by the CU's own L1 and never see the other CUs'
// arrivals).  Which XCD a workgroup runs on is read from the XCC_ID hardware register, its rank among the
// workgroups of that XCD from a ticket counter in the same L2; nothing is assumed about the dispatch order
// except that every XCD receives 32 of the 256 workgroups, which dlmi_ctx_create checks with a probe
// launch.  Every wait is bounded: a workgroup that does not see its XCD complete within the context's spin
// limit (kPanelSpinLimit polls unless DLMI_PANEL_SPIN_LIMIT says otherwise) raises the abort word and leaves,
// the others follow, and the give-up is written to a word of pinned host memory, which the host reads after
// every synchronization of the context's stream at no cost: dlmi_ctx_synchronize then reports the failure
// once, clears the barrier words and keeps the context on the multi-launch path from then on.  A launch that
// finds the words of an earlier give-up still in place (more tickets than workgroups) leaves at once and
// says so in a second host word, so every call whose results are not valid is reported.  Two panel kernels
// side by side could starve each other, so launches on different streams of one process are ordered with an
// event, and once a stream has recorded a panel kernel into a HIP graph (whose replays this library does not
// see) every other stream of that device takes the multi-launch kernels.  Other kernels may hold CUs when a
// panel kernel starts: its workgroups then start late, the ones already running wait for them (a product
// lasts milliseconds at most, the limit is about a second), and the arrival words are kept so that being
// late is harmless (see kPanelStateStride below).
#ifndef DLMI_NORM_PANEL_COMMON_HPP
#define DLMI_NORM_PANEL_COMMON_HPP

#include "norm_shared.hpp"

namespace dlmi {

constexpr int kPanelRanks = 32;   // workgroups per XCD
constexpr int kPanelXcds = 8;
constexpr int kPanelThreads = 512;
constexpr int kPanelSpinLimit = 1 << 20;
// words of the barrier state: [xcd][16] = { rank ticket, arrivals at even panels, departures, abort, arrivals
// at odd panels }.  Every word is only ever touched by the workgroups of its own XCD (the L2s of different XCDs
// are not coherent inside a kernel).
// Why two arrival words: a workgroup counts itself in for panel p+1 before it waits for panel p, so one
// running total could reach 32 (p+1) on the arrivals of the workgroups that are ahead while another has not
// arrived for p at all (one that started late because its CU was still held by another kernel).  With one word
// per panel parity an arrival for p+2 can only come from a workgroup that has finished p+1, i.e. after all 32
// have arrived for p+1 and therefore for p: the first 32 (p/2+1) arrivals on a word are those for panels <= p.
constexpr int kPanelStateStride = 16;
constexpr int kPanelStateWords = kPanelXcds * kPanelStateStride;

typedef float pv4f __attribute__((ext_vector_type(4)));

__device__ __forceinline__ unsigned panel_xcc_id() {
  unsigned x;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(x));
  return x & 0xfu;
}
// the counter's value as the L2 holds it
__device__ __forceinline__ unsigned panel_poll(unsigned *p) {
  unsigned r, zero = 0;
  asm volatile("global_atomic_add %0, %1, %2, off sc0\n\ts_waitcnt vmcnt(0)" : "=v"(r) : "v"(p), "v"(zero) : "memory");
  return r;
}
__device__ __forceinline__ unsigned panel_ticket(unsigned *p) {
  unsigned r, one = 1;
  asm volatile("global_atomic_add %0, %1, %2, off sc0\n\ts_waitcnt vmcnt(0)" : "=v"(r) : "v"(p), "v"(one) : "memory");
  return r;
}
__device__ __forceinline__ void panel_count(unsigned *p) {
  unsigned one = 1;
  asm volatile("global_atomic_add %0, %1, off" ::"v"(p), "v"(one) : "memory");
}

// Loads whose completion the panel kernels wait for themselves.  A wavefront's loads return in the order they were issued, and
// the compiler, which must assume the fewest younger loads over every path to a use, would wait for ALL loads in
// flight before the first use of a panel fetched two steps earlier (it does: vmcnt(0) in the steady state) - the
// panels just asked for would never be in flight while this one is worked on.  So the bulk loads and the loads of
// the other workgroups' sums are issued as explicit instructions, invisible to the compiler's bookkeeping, and
// every use is preceded by an explicit wait that names the number of younger memory operations of the wavefront
// that may still be outstanding; the registers pass through that wait as in/out operands, so no use can be
// scheduled before it.
__device__ __forceinline__ void issue_load(pv4f &dst, float const *p) {
  asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(dst) : "v"(p) : "memory");
}
__device__ __forceinline__ void issue_load(float &dst, float const *p) {
  asm volatile("global_load_dword %0, %1, off nt" : "=v"(dst) : "v"(p) : "memory");
}
__device__ __forceinline__ void issue_load(unsigned &dst, uint8_t const *p) {  // four mask bytes
  asm volatile("global_load_dword %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}
// Waits until at most n memory operations of this wavefront are outstanding, i.e. for everything but the n
// youngest.  n is a run-time value (the same in all lanes), clamped to 0 .. 47 (a smaller count only waits for
// more): a jump into a table of 48 waits, 8 bytes of code each (a chain of compares would cost several scalar
// instructions per candidate and a kilobyte of code per wait, and these kernels hold dozens of them)
__device__ __forceinline__ void wait_younger_n(int n) {
  int t = __builtin_amdgcn_readfirstlane(n < 0 ? 0 : (n > 47 ? 47 : n));
  asm volatile("s_getpc_b64 vcc\n"            // the address of the next instruction; the table starts 20 bytes
               "s_lshl_b32 %0, %0, 3\n"       // (five 4-byte instructions) after it
               "s_add_u32 %0, %0, 20\n"
               "s_add_u32 vcc_lo, vcc_lo, %0\n"
               "s_addc_u32 vcc_hi, vcc_hi, 0\n"
               "s_setpc_b64 vcc\n"
               "s_waitcnt vmcnt(0)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(1)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(2)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(3)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(4)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(5)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(6)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(7)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(8)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(9)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(10)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(11)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(12)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(13)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(14)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(15)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(16)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(17)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(18)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(19)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(20)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(21)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(22)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(23)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(24)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(25)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(26)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(27)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(28)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(29)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(30)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(31)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(32)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(33)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(34)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(35)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(36)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(37)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(38)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(39)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(40)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(41)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(42)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(43)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(44)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(45)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(46)\n s_branch .Lwait_done_%=\n"
               "s_waitcnt vmcnt(47)\n s_branch .Lwait_done_%=\n"
               ".Lwait_done_%=:\n"
               : "+s"(t)
               :
               : "vcc", "scc", "memory");
}

// Entry of a panel kernel: the workgroup's XCD and its rank there.  false: more than 32 workgroups on this
// XCD (abort word set).
struct PanelWho {
  unsigned xcd, rank;
  unsigned *st;
  unsigned *flag;  // pinned host memory: [0] a wait gave up, [1] a launch found an earlier give-up's words
  int spin_limit;
};
// What every panel kernel receives about the barrier besides its operands.
struct PanelSync {
  unsigned *state;  // kPanelStateWords words of device memory
  unsigned *flag;   // two words of pinned host memory
  int spin_limit;
};
__device__ __forceinline__ bool panel_enter(PanelSync const &sy, PanelWho &w, unsigned *s_rank) {
  unsigned *const state = sy.state;
  w.flag = sy.flag;
  w.spin_limit = sy.spin_limit;
  w.xcd = panel_xcc_id();
  if (w.xcd >= static_cast<unsigned>(kPanelXcds)) w.xcd = 0;  // the probe at context creation rules this out
  w.st = state + w.xcd * kPanelStateStride;
  if (threadIdx.x == 0) *s_rank = panel_ticket(w.st + 0);
  __syncthreads();
  w.rank = *s_rank;
  if (w.rank >= static_cast<unsigned>(kPanelRanks)) {
    if (threadIdx.x == 0) {
      w.st[3] = 1;
      *reinterpret_cast<unsigned volatile *>(w.flag + 1) = 1u;
    }
    return false;
  }
  return true;
}
__device__ __forceinline__ unsigned *panel_arrivals(PanelWho const &w, int p) { return w.st + ((p & 1) ? 4 : 1); }
// Thread 0 waits until all workgroups of this XCD have arrived for panel p.  Returns false after the spin limit.
__device__ __forceinline__ bool panel_wait(PanelWho const &w, int p) {
  unsigned const target = static_cast<unsigned>(kPanelRanks) * static_cast<unsigned>(p / 2 + 1);
  unsigned *const word = panel_arrivals(w, p);
  int spins = 0;
  while (panel_poll(word) < target) {
    if (++spins > w.spin_limit || (spins % 1024 == 0 && panel_poll(w.st + 3) != 0)) {
      panel_count(w.st + 3);
      *reinterpret_cast<unsigned volatile *>(w.flag) = 1u;
      return false;
    }
  }
  return true;
}
// Exit: the last workgroup of an XCD to leave puts the three words back to zero for the next launch.
__device__ __forceinline__ void panel_leave(PanelWho const &w) {
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned const d = panel_ticket(w.st + 2);
    if (d == static_cast<unsigned>(kPanelRanks) - 1) {
      w.st[0] = 0;
      w.st[1] = 0;
      w.st[2] = 0;
      w.st[4] = 0;
    }
  }
}

// host side (norm_panel_fwd.hip; panel_init / panel_check / panel_scratch_bytes are declared in dlmi_common.hpp)
// Before a panel launch: 1 = go (ordered behind the last panel kernel of another stream where needed),
// 0 = this launch must take the multi-launch kernels (see panel_admit), < 0 = failure.
int panel_admit(dlmi_ctx *ctx);
void panel_launched(dlmi_ctx *ctx);            // after it
inline PanelSync panel_sync_of(dlmi_ctx const *ctx) { return PanelSync{ctx->panel_state, ctx->panel_flag_dev, ctx->panel_spin_limit}; }

}  // namespace dlmi

#endif  // DLMI_NORM_PANEL_COMMON_HPP
