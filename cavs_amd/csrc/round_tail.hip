// The rounds of a batch of trees near the roots -- the last forward rounds and the first backward
// rounds, a few vertices each -- in ONE launch per direction instead of one launch per round.
//
// A round of thirty vertices is 0.08 GFLOP; as a launch of its own it costs the 4-5 us every
// dependent launch costs plus a pass of the recurrent weights (160 KB per workgroup) through the
// texture path, and two dozen such launches are a quarter of a training step.  Here the rows of
// those rounds are dealt to up to eight GROUPS such that no message crosses from one group to
// another (the caller's job: whole trees of the message flow per group), and each group is run by
// the H / 16 workgroups of one XCD, which stay resident and walk the group's rounds behind a
// barrier of their own:
//   * workgroup ids are dealt to the eight XCDs round-robin, so the workgroups b with b % 8 == g
//     all sit on one XCD and share one L2: what one of them writes is in that L2 once its stores
//     are acknowledged, and the others read it there (their L1 cannot hold a line of a row before
//     the barrier that follows the row's round).  No L2 write-back or invalidate is involved,
//     which is what makes an agent-scope barrier across XCDs cost as much as a launch (the
//     invalidate alone, buffer_inv sc1, was measured at 15 us for 32 workgroups).  Groups never
//     wait for each other;
//   * arrival is one atomic add per workgroup and round on the group's counter in that L2; the wait
//     polls it with a bound and gives up into a status word the host reads (every wave then leaves);
//   * the weights never move again: a wavefront owns one eighth of K (64 k at H = 512) of its
//     workgroup's sixteen columns, i.e. sixteen float4 of the tile-major weights, and keeps them in
//     registers for the whole launch.  A round then fetches only its operand rows;
//   * the index lists of a group (slab rows, children, destination rows) are fetched once, into a
//     table in LDS, while the weights arrive.
// The arithmetic is that of the four-row tiles of the per-round kernels (treelstm_round_fwd_kernel
// / treelstm_round_bwd_children_kernel with ROWS4): the same MFMAs on the same operands in the
// same order, the same order of sums, the same gate function -- and a row's result does not
// depend on which rows share its tile -- so the results equal the per-round launches' bit for bit.
#include "round_common.h"

namespace cavs {

constexpr int kTailH = 512;        // K / 8 per wavefront = 64 k = one float4 per lane and operand row
constexpr int kTailRows = 32;      // at most eight tiles of four rows per group and round
constexpr int kTailGroups = 8;     // one per XCD
constexpr int kTailMaxRounds = 32; // lists per group

// LDS of the two kernels: the parked partial sums (floats), then five index tables of one int per list position
constexpr int kTailFwdRed = 8 * 8 * 20 * 16, kTailBwdRed = 8 * 8 * 12 * 16;
constexpr size_t kTailTabBytes = 5 * sizeof(int) * kTailMaxRounds * kTailRows;

// What each group does: nrounds[g] lists of slab rows, list i = rows[start[g][i] .. + count[g][i]).
// flags[g][i]: bit 0 -- the group's workgroups tell each other when the list is done (an arrival);
// the rest -- how many of the group's arrivals must be in before the list starts (0: none, e.g. the
// second slice of a round that does not fit one list).
struct TailPlan {
  int nrounds[kTailGroups], arrivals[kTailGroups];
  int start[kTailGroups][kTailMaxRounds];
  short count[kTailGroups][kTailMaxRounds], flags[kTailGroups][kTailMaxRounds];
};

// The sync block: word 1 = status (all groups); group g owns the 32 words from 32 (g + 1): arrivals,
// then the XCDs its workgroups saw (bit mask).  A cache line per group: they live in different L2s.
enum { TAIL_STATUS = 1, TAIL_GROUP_WORDS = 32, TAIL_ARRIVALS = 0, TAIL_XCC = 1 };

__device__ inline int xcc_id() { return __builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11)) & 15; }  // HW_REG_XCC_ID[3:0]

// This workgroup's results of a round are written: tell the others of the group.  The last
// arrival of the launch leaves the group's words as the next launch expects them.
__device__ inline void tail_arrive(unsigned *gsync, unsigned total) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's stores are acknowledged by the L2
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned old = __hip_atomic_fetch_add(gsync + TAIL_ARRIVALS, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (old + 1 == total) {
      __hip_atomic_store(gsync + TAIL_XCC, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(gsync + TAIL_ARRIVALS, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// Waits until `target` arrivals of the group are in.  False when the wait gave up (spin_max polls,
// or another workgroup already did, or the group's workgroups turned out to sit on more than one
// XCD): the status word says why and the caller returns.  Ends with a workgroup barrier either way.
__device__ inline bool tail_wait(unsigned *status, unsigned *gsync, unsigned target, int spin_max, bool check_xcc, int *s_bail) {
  if (threadIdx.x == 0) {
    int bail = 0, tries = 0;
    while (__hip_atomic_load(gsync + TAIL_ARRIVALS, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
      if (++tries > spin_max) {
        __hip_atomic_store(status, (unsigned)CAVS_TAIL_TIMEOUT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        bail = 1;
        break;
      }
      if ((tries & 15) == 0 && __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
        bail = 1;
        break;
      }
    }
    if (!bail && check_xcc) {
      const unsigned seen = __hip_atomic_load(gsync + TAIL_XCC, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (seen & (seen - 1)) {  // more than one XCD: the L2 is not shared, nothing read here can be trusted
        __hip_atomic_store(status, (unsigned)CAVS_TAIL_SPREAD, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        bail = 1;
      }
    }
    *s_bail = bail;
  }
  __syncthreads();
  asm volatile("buffer_inv sc0" ::: "memory");  // nothing this CU cached before the barrier is used after it
  return *s_bail == 0;
}

// A row another workgroup of the group wrote in an earlier round.  No line of such a row can be in
// this CU's L1 when the load is issued: the L1 starts a kernel empty, rows are whole cache lines,
// and a row is first read after the barrier that follows its round (tail_wait also invalidates
// the L1, for good measure).  So an ordinary load is served by the L2 the writers share.  (Loads
// that bypass the L1 by scope -- agent-scope atomic loads -- were measured at about sixty cycles per
// wavefront and access here, one request per lane: three times the MFMA time of a tile.)
__device__ inline float ld_row(const float *p) { return *p; }

// The four k slots of an element added up across the wavefront, for the four rows of NP products
// at once: afterwards the lanes of k slot s hold, in r[p][0], the sum of row s of product p --
// (v[x] + v[x+16]) + (v[x+32] + v[x+48]) with v = that row's accumulator, the order in which the
// per-round kernels add the slots up.  v_permlane16_swap exchanges the odd 16-lane rows of its first
// operand with the even rows of its second, v_permlane32_swap the upper half of the first with the
// lower half of the second; swapping two rows' accumulators and adding puts both partial sums into
// one register, a butterfly of three swaps and three adds per product on the vector ALU (a shuffle
// through the LDS crossbar costs eight cycles of a unit all eight wavefronts share).  Spelled out
// as instructions because the compiler's builtins for the two swaps return the first result twice.
// The compiler does not look inside such a statement, so the waits an instruction needs after the
// one that produced its operand are the caller's: all() carries its own (twelve cycles cover the
// six a two-pass MFMA asks for before a vector-ALU read, two between an add and the swap that reads
// it); the stages are for callers that put at least that many instructions between them.
template <int NP>
struct SlotSums;
template <>
struct SlotSums<5> {
  float r[5][4];
  __device__ inline void take(const floatx4 (&acc)[5]) {
#pragma unroll
    for (int p = 0; p < 5; p++)
#pragma unroll
      for (int k = 0; k < 4; k++) r[p][k] = acc[p][k];
  }
  // the stages one at a time, for a caller that puts other work (MFMAs of the next tile) between them
  __device__ inline void stage_a() {
    asm volatile(
        "v_permlane16_swap_b32 %0, %1\n\tv_permlane16_swap_b32 %2, %3\n\t"
        "v_permlane16_swap_b32 %4, %5\n\tv_permlane16_swap_b32 %6, %7\n\t"
        "v_permlane16_swap_b32 %8, %9\n\tv_permlane16_swap_b32 %10, %11\n\t"
        "v_permlane16_swap_b32 %12, %13\n\tv_permlane16_swap_b32 %14, %15\n\t"
        "v_permlane16_swap_b32 %16, %17\n\tv_permlane16_swap_b32 %18, %19"
        : "+v"(r[0][0]), "+v"(r[0][1]), "+v"(r[0][2]), "+v"(r[0][3]), "+v"(r[1][0]), "+v"(r[1][1]), "+v"(r[1][2]), "+v"(r[1][3]), "+v"(r[2][0]), "+v"(r[2][1]), "+v"(r[2][2]), "+v"(r[2][3]), "+v"(r[3][0]), "+v"(r[3][1]), "+v"(r[3][2]), "+v"(r[3][3]), "+v"(r[4][0]), "+v"(r[4][1]), "+v"(r[4][2]), "+v"(r[4][3]));
  }
  __device__ inline void stage_b() {
    asm volatile(
        "v_add_f32 %0, %0, %1\n\tv_add_f32 %2, %2, %3\n\t"
        "v_add_f32 %4, %4, %5\n\tv_add_f32 %6, %6, %7\n\t"
        "v_add_f32 %8, %8, %9\n\tv_add_f32 %10, %10, %11\n\t"
        "v_add_f32 %12, %12, %13\n\tv_add_f32 %14, %14, %15\n\t"
        "v_add_f32 %16, %16, %17\n\tv_add_f32 %18, %18, %19"
        : "+v"(r[0][0]), "+v"(r[0][1]), "+v"(r[0][2]), "+v"(r[0][3]), "+v"(r[1][0]), "+v"(r[1][1]), "+v"(r[1][2]), "+v"(r[1][3]), "+v"(r[2][0]), "+v"(r[2][1]), "+v"(r[2][2]), "+v"(r[2][3]), "+v"(r[3][0]), "+v"(r[3][1]), "+v"(r[3][2]), "+v"(r[3][3]), "+v"(r[4][0]), "+v"(r[4][1]), "+v"(r[4][2]), "+v"(r[4][3]));
  }
  __device__ inline void stage_c() {
    asm volatile(
        "v_permlane32_swap_b32 %0, %2\n\t"
        "v_permlane32_swap_b32 %4, %6\n\t"
        "v_permlane32_swap_b32 %8, %10\n\t"
        "v_permlane32_swap_b32 %12, %14\n\t"
        "v_permlane32_swap_b32 %16, %18"
        : "+v"(r[0][0]), "+v"(r[0][1]), "+v"(r[0][2]), "+v"(r[0][3]), "+v"(r[1][0]), "+v"(r[1][1]), "+v"(r[1][2]), "+v"(r[1][3]), "+v"(r[2][0]), "+v"(r[2][1]), "+v"(r[2][2]), "+v"(r[2][3]), "+v"(r[3][0]), "+v"(r[3][1]), "+v"(r[3][2]), "+v"(r[3][3]), "+v"(r[4][0]), "+v"(r[4][1]), "+v"(r[4][2]), "+v"(r[4][3]));
  }
  __device__ inline void stage_d() {
    asm volatile(
        "v_add_f32 %0, %0, %2\n\t"
        "v_add_f32 %4, %4, %6\n\t"
        "v_add_f32 %8, %8, %10\n\t"
        "v_add_f32 %12, %12, %14\n\t"
        "v_add_f32 %16, %16, %18"
        : "+v"(r[0][0]), "+v"(r[0][1]), "+v"(r[0][2]), "+v"(r[0][3]), "+v"(r[1][0]), "+v"(r[1][1]), "+v"(r[1][2]), "+v"(r[1][3]), "+v"(r[2][0]), "+v"(r[2][1]), "+v"(r[2][2]), "+v"(r[2][3]), "+v"(r[3][0]), "+v"(r[3][1]), "+v"(r[3][2]), "+v"(r[3][3]), "+v"(r[4][0]), "+v"(r[4][1]), "+v"(r[4][2]), "+v"(r[4][3]));
  }
  // all of it at once, right after the MFMAs that produced the accumulators
  __device__ inline void all() {
    asm volatile(
      "s_nop 7\n\ts_nop 3\n\t"
      "v_permlane16_swap_b32 %0, %1\n\tv_permlane16_swap_b32 %2, %3\n\t"
      "v_permlane16_swap_b32 %4, %5\n\tv_permlane16_swap_b32 %6, %7\n\t"
      "v_permlane16_swap_b32 %8, %9\n\tv_permlane16_swap_b32 %10, %11\n\t"
      "v_permlane16_swap_b32 %12, %13\n\tv_permlane16_swap_b32 %14, %15\n\t"
      "v_permlane16_swap_b32 %16, %17\n\tv_permlane16_swap_b32 %18, %19\n\t"
      "s_nop 1\n\t"
      "v_add_f32 %0, %0, %1\n\tv_add_f32 %2, %2, %3\n\t"
      "v_add_f32 %4, %4, %5\n\tv_add_f32 %6, %6, %7\n\t"
      "v_add_f32 %8, %8, %9\n\tv_add_f32 %10, %10, %11\n\t"
      "v_add_f32 %12, %12, %13\n\tv_add_f32 %14, %14, %15\n\t"
      "v_add_f32 %16, %16, %17\n\tv_add_f32 %18, %18, %19\n\t"
      "s_nop 1\n\t"
      "v_permlane32_swap_b32 %0, %2\n\t"
      "v_permlane32_swap_b32 %4, %6\n\t"
      "v_permlane32_swap_b32 %8, %10\n\t"
      "v_permlane32_swap_b32 %12, %14\n\t"
      "v_permlane32_swap_b32 %16, %18\n\t"
      "s_nop 1\n\t"
      "v_add_f32 %0, %0, %2\n\t"
      "v_add_f32 %4, %4, %6\n\t"
      "v_add_f32 %8, %8, %10\n\t"
      "v_add_f32 %12, %12, %14\n\t"
      "v_add_f32 %16, %16, %18"
        : "+v"(r[0][0]), "+v"(r[0][1]), "+v"(r[0][2]), "+v"(r[0][3]), "+v"(r[1][0]), "+v"(r[1][1]), "+v"(r[1][2]), "+v"(r[1][3]), "+v"(r[2][0]), "+v"(r[2][1]), "+v"(r[2][2]), "+v"(r[2][3]), "+v"(r[3][0]), "+v"(r[3][1]), "+v"(r[3][2]), "+v"(r[3][3]), "+v"(r[4][0]), "+v"(r[4][1]), "+v"(r[4][2]), "+v"(r[4][3]));
  }
};
template <>
struct SlotSums<3> {
  float r[3][4];
  __device__ inline void take(const floatx4 (&acc)[3]) {
#pragma unroll
    for (int p = 0; p < 3; p++)
#pragma unroll
      for (int k = 0; k < 4; k++) r[p][k] = acc[p][k];
  }
  // the stages one at a time, for a caller that puts other work (MFMAs of the next tile) between them
  __device__ inline void stage_a() {
    asm volatile(
        "v_permlane16_swap_b32 %0, %1\n\tv_permlane16_swap_b32 %2, %3\n\t"
        "v_permlane16_swap_b32 %4, %5\n\tv_permlane16_swap_b32 %6, %7\n\t"
        "v_permlane16_swap_b32 %8, %9\n\tv_permlane16_swap_b32 %10, %11"
        : "+v"(r[0][0]), "+v"(r[0][1]), "+v"(r[0][2]), "+v"(r[0][3]), "+v"(r[1][0]), "+v"(r[1][1]), "+v"(r[1][2]), "+v"(r[1][3]), "+v"(r[2][0]), "+v"(r[2][1]), "+v"(r[2][2]), "+v"(r[2][3]));
  }
  __device__ inline void stage_b() {
    asm volatile(
        "v_add_f32 %0, %0, %1\n\tv_add_f32 %2, %2, %3\n\t"
        "v_add_f32 %4, %4, %5\n\tv_add_f32 %6, %6, %7\n\t"
        "v_add_f32 %8, %8, %9\n\tv_add_f32 %10, %10, %11"
        : "+v"(r[0][0]), "+v"(r[0][1]), "+v"(r[0][2]), "+v"(r[0][3]), "+v"(r[1][0]), "+v"(r[1][1]), "+v"(r[1][2]), "+v"(r[1][3]), "+v"(r[2][0]), "+v"(r[2][1]), "+v"(r[2][2]), "+v"(r[2][3]));
  }
  __device__ inline void stage_c() {
    asm volatile(
        "v_permlane32_swap_b32 %0, %2\n\t"
        "v_permlane32_swap_b32 %4, %6\n\t"
        "v_permlane32_swap_b32 %8, %10"
        : "+v"(r[0][0]), "+v"(r[0][1]), "+v"(r[0][2]), "+v"(r[0][3]), "+v"(r[1][0]), "+v"(r[1][1]), "+v"(r[1][2]), "+v"(r[1][3]), "+v"(r[2][0]), "+v"(r[2][1]), "+v"(r[2][2]), "+v"(r[2][3]));
  }
  __device__ inline void stage_d() {
    asm volatile(
        "v_add_f32 %0, %0, %2\n\t"
        "v_add_f32 %4, %4, %6\n\t"
        "v_add_f32 %8, %8, %10"
        : "+v"(r[0][0]), "+v"(r[0][1]), "+v"(r[0][2]), "+v"(r[0][3]), "+v"(r[1][0]), "+v"(r[1][1]), "+v"(r[1][2]), "+v"(r[1][3]), "+v"(r[2][0]), "+v"(r[2][1]), "+v"(r[2][2]), "+v"(r[2][3]));
  }
  // all of it at once, right after the MFMAs that produced the accumulators
  __device__ inline void all() {
    asm volatile(
      "s_nop 7\n\ts_nop 3\n\t"
      "v_permlane16_swap_b32 %0, %1\n\tv_permlane16_swap_b32 %2, %3\n\t"
      "v_permlane16_swap_b32 %4, %5\n\tv_permlane16_swap_b32 %6, %7\n\t"
      "v_permlane16_swap_b32 %8, %9\n\tv_permlane16_swap_b32 %10, %11\n\t"
      "s_nop 1\n\t"
      "v_add_f32 %0, %0, %1\n\tv_add_f32 %2, %2, %3\n\t"
      "v_add_f32 %4, %4, %5\n\tv_add_f32 %6, %6, %7\n\t"
      "v_add_f32 %8, %8, %9\n\tv_add_f32 %10, %10, %11\n\t"
      "s_nop 1\n\t"
      "v_permlane32_swap_b32 %0, %2\n\t"
      "v_permlane32_swap_b32 %4, %6\n\t"
      "v_permlane32_swap_b32 %8, %10\n\t"
      "s_nop 1\n\t"
      "v_add_f32 %0, %0, %2\n\t"
      "v_add_f32 %4, %4, %6\n\t"
      "v_add_f32 %8, %8, %10"
        : "+v"(r[0][0]), "+v"(r[0][1]), "+v"(r[0][2]), "+v"(r[0][3]), "+v"(r[1][0]), "+v"(r[1][1]), "+v"(r[1][2]), "+v"(r[1][3]), "+v"(r[2][0]), "+v"(r[2][1]), "+v"(r[2][2]), "+v"(r[2][3]));
  }
};

// One k-group of four-row tiles is four MFMAs of sixteen 4 x 4 x 1 blocks each; block l / 4 of
// lane l is (column group (l / 4) % 4, k slot l / 16).  An MFMA can take its A operand, for the four
// blocks of a k slot, from one of them (A broadcast inside groups of four blocks: CBSZ = 2, ABID =
// which).  So lane l = 16 slot + 4 j + r fetches ONE float4 per operand row and tile: tile row r at
// k = 16 j + 4 slot .. + 3 of the wavefront's 64 k -- the wavefront's 64 float4 are the whole
// 4 x 64 piece of the operand, nothing is fetched twice and nothing crosses lanes -- and the MFMA
// of k-group g, step c reads component c with ABID = g: the operands the per-round kernels feed the
// same MFMAs after moving them across lanes.
#define CAVS_MMA4(acc, a, b, abid) acc = __builtin_amdgcn_mfma_f32_4x4x1f32(a, b, acc, 2, abid, 0)

// ------------------------------------------------------------------ forward
struct TailFwdArgs {
  float *pool;          // [*, 2H]
  const int *child;     // [2N] by slab row
  const int *pair;      // [N]
  const float *xW;      // [N, 4H] (ld_xw)
  long ld_xw;
  const float *Upk;     // tile-major U_iou [H, 3H], then U_f [H, H]
  const float *bias;    // [4H]
  float *G, *hlr, *gates, *msg, *go;  // whole-batch slabs (msg, go may be null)
  const int *out_rows;  // [N]
  const int *rows;      // the groups' lists of slab rows
  unsigned *sync;
  int spin_max, expect;
  TailPlan plan;
};

__global__ __launch_bounds__(512, 1) void treelstm_tail_fwd_kernel(TailFwdArgs a) {
  const int grp = blockIdx.x & 7;  // the group = the XCD this workgroup landed on
  const int nrounds = a.plan.nrounds[grp];
  if (nrounds == 0) return;
  unsigned *status = a.sync + TAIL_STATUS, *gsync = a.sync + TAIL_GROUP_WORDS * (grp + 1);
  // (an earlier launch on this block gave up and nobody has cleared it: nothing here can be trusted)
  if (__hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) return;
  constexpr int H = kTailH, H2 = 2 * H, NP = 5;
  const int ct = blockIdx.x >> 3;  // column tile
  extern __shared__ float red[];   // [tile][wavefront][product * 4 + row][column]: 8 * 8 * 20 * 16 floats, then the index table
  __shared__ int s_bail;
  const int tid = threadIdx.x, lane = tid & 63, ks = tid >> 6;
  const int x = lane & 15, slot = lane >> 4;
  const int j0 = ct * 16, kb = ks * (H / 8);

  // The group's index table, [what][list][position]: slab row, left and right child, the row of the
  // pool the message goes to, the row of the graph output (-1 = none, also past a list's end).  Read
  // from global memory where a round needs them these are chains of two and three dependent loads
  // on every workgroup's way to the round's barrier; here they are fetched once, under the weights.
  constexpr int TAB = kTailMaxRounds * kTailRows;
  int *tab = reinterpret_cast<int *>(red + kTailFwdRed);
  for (int e = tid; e < nrounds * kTailRows; e += 512) {
    const int r = e / kTailRows, i = e % kTailRows;
    int row = -1, cl = -1, cr = -1, dst = -1, out = -1;
    if (i < a.plan.count[grp][r]) {
      row = a.rows[a.plan.start[grp][r] + i];
      cl = a.child[2L * row];
      cr = a.child[2L * row + 1];
      dst = a.pair[row];
      if (a.go) out = a.out_rows[row];
    }
    tab[e] = row;
    tab[TAB + e] = cl;
    tab[2 * TAB + e] = cr;
    tab[3 * TAB + e] = dst;
    tab[4 * TAB + e] = out;
  }

  // this wavefront's weights: k-groups kb/16 .. kb/16 + 3 of column tile ct, four gates
  float4 wi[4], wo[4], wu[4], wf[4];
  {
    const float4 *pio = reinterpret_cast<const float4 *>(a.Upk) + ((long)(kb / 16) * (3 * H / 16) + ct) * 64 + slot * 16 + x;
    const float4 *pf = reinterpret_cast<const float4 *>(a.Upk) + 3L * H * H / 4 + ((long)(kb / 16) * (H / 16) + ct) * 64 + slot * 16 + x;
    constexpr int gate4 = H * 4;
#pragma unroll
    for (int g = 0; g < 4; g++) {
      wi[g] = pio[0];
      wo[g] = pio[gate4];
      wu[g] = pio[2 * gate4];
      wf[g] = *pf;
      pio += 3 * gate4;
      pf += gate4;
    }
  }
  // Wavefronts w and w + 4 share a SIMD and would run their MFMA and vector-ALU phases in step,
  // each at half speed with the matrix pipe idle in between: one of them goes first.
  if (ks < 4) __builtin_amdgcn_s_setprio(2);
  // the element of a tile this thread finishes: wavefront ks does tile ks, row lane / 16, column x
  const int ej = j0 + x;
  float bias[4];
#pragma unroll
  for (int k = 0; k < 4; k++) bias[k] = a.bias[k * H + ej];
  const unsigned total = (unsigned)a.plan.arrivals[grp] * a.expect;
  if (tid == 0 && total > 0) __hip_atomic_fetch_or(gsync + TAIL_XCC, 1u << xcc_id(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  bool first_wait = true;
  __syncthreads();

  for (int r = 0; r < nrounds; r++) {
    const int n = a.plan.count[grp][r], T = (n + 3) >> 2;
    const int need = a.plan.flags[grp][r] >> 1;
    const bool arrives = a.plan.flags[grp][r] & 1;
    const int *rtab = tab + r * kTailRows;
    // what does not depend on the rounds before: the epilogue's x * W
    const int eb = 4 * ks + (lane >> 4);
    const bool eon = eb < n;
    const long erow = eon ? rtab[eb] : 0;
    float xw[4] = {0.f, 0.f, 0.f, 0.f};
    if (eon) {
      const float *p = a.xW + erow * a.ld_xw + ej;
#pragma unroll
      for (int k = 0; k < 4; k++) xw[k] = p[k * H];
    }
    if (need > 0) {
      if (!tail_wait(status, gsync, (unsigned)need * a.expect, a.spin_max, first_wait, &s_bail)) return;
      first_wait = false;
    } else {
      __syncthreads();
    }

    // the epilogue's children
    int e_cl = -1, e_cr = -1, e_dst = -1, e_out = -1;
    float e_hl = 0.f, e_cl_c = 0.f, e_hr = 0.f, e_cr_c = 0.f;
    if (eon) {
      e_cl = rtab[TAB + eb];
      e_cr = rtab[2 * TAB + eb];
      e_dst = rtab[3 * TAB + eb];
      e_out = rtab[4 * TAB + eb];
      if (e_cl >= 0) { e_hl = ld_row(a.pool + (long)e_cl * H2 + ej); e_cl_c = ld_row(a.pool + (long)e_cl * H2 + H + ej); }
      if (e_cr >= 0) { e_hr = ld_row(a.pool + (long)e_cr * H2 + ej); e_cr_c = ld_row(a.pool + (long)e_cr * H2 + H + ej); }
    }

    // Operand rows: one float4 per child and tile (see CAVS_MMA4), unconditionally (a missing child
    // reads row 0 and is masked where the operand is used; past the last tile the last one is fetched
    // again).  A tile's instruction stream carries, between the four k-groups of its MFMAs, the two
    // loads of the next tile and the slot sums of the tile before it: a wavefront stalled in a load's
    // issue or busy on the vector ALU issues no MFMAs, and with every wavefront of the CU in the
    // same phase the matrix pipes idled through both (measured: the three costs simply added up).
    const int ka = kb + 16 * ((lane >> 2) & 3) + 4 * slot;
    struct Opnd {
      float4 l, r;
      int cl, cr;
    };
    auto child_of = [&](int t, int side) { return rtab[(1 + side) * TAB + 4 * (t < T ? t : T - 1) + (lane & 3)]; };
    SlotSums<NP> sums;
    auto park = [&](int t) {
      float *dst = red + ((t * 8 + ks) * (NP * 4)) * 16 + x;
#pragma unroll
      for (int p = 0; p < NP; p++) dst[(p * 4 + slot) * 16] = sums.r[p][0];
    };
    // tile t from `o`, fetching tile t + 1 into `nx`; PREV: tile t - 1 waits in `sums`
    auto tile = [&](auto prev, int t, const Opnd &o, Opnd &nx) {
      constexpr bool PREV = decltype(prev)::value;
      const float4 hl4 = o.cl >= 0 ? o.l : zero4(), hr4 = o.cr >= 0 ? o.r : zero4();
      floatx4 acc[NP];
#pragma unroll
      for (int p = 0; p < NP; p++) acc[p] = floatx4{0.f, 0.f, 0.f, 0.f};
      const float4 hs4 = make_float4(hl4.x + hr4.x, hl4.y + hr4.y, hl4.z + hr4.z, hl4.w + hr4.w);
      // (k-group g, step c: k = 16 g + 4 slot + c; the five products take turns as in the per-round kernels)
#define CAVS_FWD_STEP(g, comp)                    \
      CAVS_MMA4(acc[0], hs4.comp, wi[g].comp, g); \
      CAVS_MMA4(acc[1], hs4.comp, wo[g].comp, g); \
      CAVS_MMA4(acc[2], hs4.comp, wu[g].comp, g); \
      CAVS_MMA4(acc[3], hl4.comp, wf[g].comp, g); \
      CAVS_MMA4(acc[4], hr4.comp, wf[g].comp, g);
#define CAVS_FWD_GROUP(g) CAVS_FWD_STEP(g, x) CAVS_FWD_STEP(g, y) CAVS_FWD_STEP(g, z) CAVS_FWD_STEP(g, w)
      nx.cl = child_of(t + 1, 0);
      nx.cr = child_of(t + 1, 1);
      CAVS_FWD_GROUP(0)
      __builtin_amdgcn_sched_barrier(0);
      nx.l = ld4(a.pool + (long)(nx.cl >= 0 ? nx.cl : 0) * H2 + ka);
      if constexpr (PREV) sums.stage_a();
      __builtin_amdgcn_sched_barrier(0);
      CAVS_FWD_GROUP(1)
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (PREV) sums.stage_b();
      __builtin_amdgcn_sched_barrier(0);
      CAVS_FWD_GROUP(2)
      __builtin_amdgcn_sched_barrier(0);
      nx.r = ld4(a.pool + (long)(nx.cr >= 0 ? nx.cr : 0) * H2 + ka);
      if constexpr (PREV) sums.stage_c();
      __builtin_amdgcn_sched_barrier(0);
      CAVS_FWD_GROUP(3)
      __builtin_amdgcn_sched_barrier(0);
#undef CAVS_FWD_GROUP
#undef CAVS_FWD_STEP
      if constexpr (PREV) {
        sums.stage_d();
        park(t - 1);  // lanes of slot s park row s
      }
      sums.take(acc);
      __builtin_amdgcn_sched_barrier(0);
    };
    {
      Opnd oa, ob;
      oa.cl = child_of(0, 0);
      oa.cr = child_of(0, 1);
      oa.l = ld4(a.pool + (long)(oa.cl >= 0 ? oa.cl : 0) * H2 + ka);
      oa.r = ld4(a.pool + (long)(oa.cr >= 0 ? oa.cr : 0) * H2 + ka);
      tile(std::false_type{}, 0, oa, ob);
      for (int t = 1; t < T; t += 2) {
        tile(std::true_type{}, t, ob, oa);
        if (t + 1 < T) tile(std::true_type{}, t + 1, oa, ob);
      }
      sums.all();
      park(T - 1);
    }
    __syncthreads();

    TreeLstmCell q{};
    if (eon) {
      const float *pre = red + (ks * 8 * (NP * 4) + (lane >> 4)) * 16 + x;  // tile ks, wavefront 0, row lane / 16
      float v[NP];
#pragma unroll
      for (int p = 0; p < NP; p++) {
        float s = 0.f;
#pragma unroll
        for (int g = 0; g < 8; g++) s += pre[(g * NP * 4 + p * 4) * 16];
        v[p] = s;
      }
      q = treelstm_cell(xw, v, bias, e_cl_c, e_cr_c);
      // the message first: it is all a later round of this launch reads
      if (e_dst >= 0) {
        a.pool[(long)e_dst * H2 + ej] = q.h;
        a.pool[(long)e_dst * H2 + H + ej] = q.c;
      }
    }
    if (arrives) tail_arrive(gsync, total);
    else __syncthreads();
    if (eon) {  // what the backward pass and the caller read: on its way while the next round starts
      const long b = erow;
      float *g = a.gates + b * 6 * H + ej;
      g[0] = q.i; g[H] = q.o; g[2 * H] = q.u; g[3 * H] = q.f_l; g[4 * H] = q.f_r; g[5 * H] = q.tc;
      if (a.msg) {
        float *m = a.msg + b * H2 + ej;
        m[0] = q.h; m[H] = q.c;
      }
      if (e_out >= 0) a.go[(long)e_out * H + ej] = q.h;
      float *gl = a.G + (2 * b) * H2 + ej, *gr = gl + H2;
      gl[0] = e_hl; gl[H] = e_cl_c; gr[0] = e_hr; gr[H] = e_cr_c;
      a.hlr[b * H + ej] = e_hl + e_hr;
    }
  }
}

// ------------------------------------------------------------------ backward
struct TailBwdArgs {
  float *dxW;           // [N, 4H] (ld_dxw) whole batch
  long ld_dxw;
  float *dF, *dc;       // [2N, H], [N, H]
  const float *UTp;     // tile-major U_iou^T [3H, H], then U_f^T [H, H]
  const int *kids;      // [2N] children by slab row
  const float *gates, *G, *dret;
  const int *dret_rows;
  const int *rows;      // the groups' lists of slab rows
  unsigned *sync;
  int leaf_rows, spin_max, expect;
  TailPlan plan;
};

__global__ __launch_bounds__(512, 1) void treelstm_tail_bwd_kernel(TailBwdArgs a) {
  const int grp = blockIdx.x & 7;
  const int nrounds = a.plan.nrounds[grp];
  if (nrounds == 0) return;
  unsigned *status = a.sync + TAIL_STATUS, *gsync = a.sync + TAIL_GROUP_WORDS * (grp + 1);
  if (__hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) return;
  constexpr int H = kTailH, H2 = 2 * H, NP = 3;
  const int ct = blockIdx.x >> 3;
  extern __shared__ float red[];  // [tile][wavefront][product * 4 + row][column]: 8 * 8 * 12 * 16 floats, then the index table
  __shared__ int s_bail;
  const int tid = threadIdx.x, lane = tid & 63, ks = tid >> 6;
  const int x = lane & 15, slot = lane >> 4;
  const int j0 = ct * 16;

  // the group's index table (see the forward kernel): slab row, its two children, the rows of
  // `dret` that hold the children's gradients from outside (-1 = none, also past a list's end)
  constexpr int TAB = kTailMaxRounds * kTailRows;
  int *tab = reinterpret_cast<int *>(red + kTailBwdRed);
  for (int e = tid; e < nrounds * kTailRows; e += 512) {
    const int r = e / kTailRows, i = e % kTailRows;
    int row = -1, k0 = -1, k1 = -1, d0 = -1, d1 = -1;
    if (i < a.plan.count[grp][r]) {
      row = a.rows[a.plan.start[grp][r] + i];
      k0 = a.kids[2L * row];
      k1 = a.kids[2L * row + 1];
      if (k0 >= 0) d0 = a.dret_rows[k0];
      if (k1 >= 0) d1 = a.dret_rows[k1];
    }
    tab[e] = row;
    tab[TAB + e] = k0;
    tab[2 * TAB + e] = k1;
    tab[3 * TAB + e] = d0;
    tab[4 * TAB + e] = d1;
  }

  // weights: twelve k-groups of U_iou^T (K = 3H) and four of U_f^T (K = H) per wavefront
  float4 w0[12], w1[4];
  {
    const float4 *base = reinterpret_cast<const float4 *>(a.UTp) + ct * 64 + slot * 16 + x;
    constexpr int gstep4 = (H / 16) * 64;  // float4 between the blocks of consecutive k-groups
    const float4 *p0 = base + (long)(ks * (3 * H / 8) / 16) * gstep4;
    const float4 *p1 = base + 3L * H * H / 4 + (long)(ks * (H / 8) / 16) * gstep4;
#pragma unroll
    for (int g = 0; g < 12; g++) w0[g] = p0[(long)g * gstep4];
#pragma unroll
    for (int g = 0; g < 4; g++) w1[g] = p1[(long)g * gstep4];
  }
  const int ej = j0 + x;
  if (ks < 4) __builtin_amdgcn_s_setprio(2);  // (see the forward kernel)
  const unsigned total = (unsigned)a.plan.arrivals[grp] * a.expect;
  if (tid == 0 && total > 0) __hip_atomic_fetch_or(gsync + TAIL_XCC, 1u << xcc_id(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  bool first_wait = true;
  __syncthreads();

  for (int r = 0; r < nrounds; r++) {
    const int n = a.plan.count[grp][r], T = (n + 3) >> 2;
    const int need = a.plan.flags[grp][r] >> 1;
    const bool arrives = a.plan.flags[grp][r] & 1;
    const int *rtab = tab + r * kTailRows;
    // the operands of the children's gate gradients: everything except d c of the parent was
    // written before this launch
    const int eb = 4 * ks + (lane >> 4);
    const bool eon = eb < n;
    const long erow = eon ? rtab[eb] : 0;
    int kc[2] = {-1, -1}, kdr[2] = {-1, -1};
    float pf[2] = {0.f, 0.f};
    struct Kid {
      float g[6], dr, cl, cr;
    } kid[2];
    if (eon) {
      kc[0] = rtab[TAB + eb];
      kc[1] = rtab[2 * TAB + eb];
      kdr[0] = rtab[3 * TAB + eb];
      kdr[1] = rtab[4 * TAB + eb];
      pf[0] = a.gates[erow * 6 * H + 3 * H + ej];
      pf[1] = a.gates[erow * 6 * H + 4 * H + ej];
    }
#pragma unroll
    for (int s = 0; s < 2; s++) {
      Kid &kd = kid[s];
#pragma unroll
      for (int t = 0; t < 6; t++) kd.g[t] = 0.f;
      kd.dr = kd.cl = kd.cr = 0.f;
      const long v = kc[s];
      if (v >= 0) {
        const float *g = a.gates + v * 6 * H + ej;
#pragma unroll
        for (int t = 0; t < 6; t++) kd.g[t] = g[(long)t * H];
        kd.dr = a.dret[(long)kdr[s] * H + ej];
        if (v >= a.leaf_rows) {
          kd.cl = a.G[(2 * v) * H2 + H + ej];
          kd.cr = a.G[(2 * v + 1) * H2 + H + ej];
        }
      }
    }
    if (need > 0) {
      if (!tail_wait(status, gsync, (unsigned)need * a.expect, a.spin_max, first_wait, &s_bail)) return;
      first_wait = false;
    } else {
      __syncthreads();
    }
    const float pdc = eon ? ld_row(a.dc + erow * H + ej) : 0.f;

    // Per tile five float4 per lane (see CAVS_MMA4): three of [d_i|d_o|d_u] (K = 3H: twelve k-groups
    // per wavefront), one each of d_fl, d_fr (K = H).  As in the forward kernel a tile's instruction
    // stream carries the five loads of the next tile (past the last tile the last one is fetched
    // again) and the slot sums of the tile before it between its MFMAs; the K = H products' MFMAs
    // stand between those of the K = 3H product, whose single accumulator makes every one of them
    // wait for the one before.
    const int kq = 16 * ((lane >> 2) & 3) + 4 * slot;
    struct Opnd {
      float4 x[3], fl, fr;
    };
    // (rows past the list's end stand for its first row; their results are not written)
    auto row_of = [&](int t) {
      const int i = 4 * (t < T ? t : T - 1) + (lane & 3);
      return (long)rtab[i < n ? i : 0];
    };
    SlotSums<NP> sums;
    auto park = [&](int t) {
      float *dst = red + ((t * 8 + ks) * (NP * 4)) * 16 + x;
#pragma unroll
      for (int p = 0; p < NP; p++) dst[(p * 4 + slot) * 16] = sums.r[p][0];
    };
    auto tile = [&](auto prev, int t, const Opnd &o, Opnd &nx) {
      constexpr bool PREV = decltype(prev)::value;
      floatx4 acc[NP];
#pragma unroll
      for (int p = 0; p < NP; p++) acc[p] = floatx4{0.f, 0.f, 0.f, 0.f};
      const long nrow = row_of(t + 1);
      const float *px = a.dxW + nrow * a.ld_dxw + ks * (3 * H / 8) + kq;
      const float *pl = a.dF + 2 * nrow * H + ks * (H / 8) + kq;
      // (k-group 4 q + g of the K = 3H product: component by component of o.x[q], broadcast from block g)
#define CAVS_P0_GROUP(q, g)                            \
      CAVS_MMA4(acc[0], o.x[q].x, w0[4 * (q) + (g)].x, g); \
      CAVS_MMA4(acc[0], o.x[q].y, w0[4 * (q) + (g)].y, g); \
      CAVS_MMA4(acc[0], o.x[q].z, w0[4 * (q) + (g)].z, g); \
      CAVS_MMA4(acc[0], o.x[q].w, w0[4 * (q) + (g)].w, g);
#define CAVS_P12_STEP(g, comp)                     \
      CAVS_MMA4(acc[1], o.fl.comp, w1[g].comp, g); \
      CAVS_MMA4(acc[2], o.fr.comp, w1[g].comp, g);
      // one quarter of the tile: three k-groups of the long product around one of the short ones
#define CAVS_BWD_QUARTER(g)                                                             \
      CAVS_P0_GROUP((3 * g) / 4, (3 * g) % 4) CAVS_P12_STEP(g, x)                        \
      CAVS_P0_GROUP((3 * g + 1) / 4, (3 * g + 1) % 4) CAVS_P12_STEP(g, y) CAVS_P12_STEP(g, z) \
      CAVS_P0_GROUP((3 * g + 2) / 4, (3 * g + 2) % 4) CAVS_P12_STEP(g, w)
      CAVS_BWD_QUARTER(0)
      __builtin_amdgcn_sched_barrier(0);
      nx.x[0] = ld4(px);
      nx.x[1] = ld4(px + 64);
      if constexpr (PREV) sums.stage_a();
      __builtin_amdgcn_sched_barrier(0);
      CAVS_BWD_QUARTER(1)
      __builtin_amdgcn_sched_barrier(0);
      nx.x[2] = ld4(px + 128);
      if constexpr (PREV) sums.stage_b();
      __builtin_amdgcn_sched_barrier(0);
      CAVS_BWD_QUARTER(2)
      __builtin_amdgcn_sched_barrier(0);
      nx.fl = ld4(pl);
      nx.fr = ld4(pl + H);
      if constexpr (PREV) sums.stage_c();
      __builtin_amdgcn_sched_barrier(0);
      CAVS_BWD_QUARTER(3)
      __builtin_amdgcn_sched_barrier(0);
#undef CAVS_BWD_QUARTER
#undef CAVS_P12_STEP
#undef CAVS_P0_GROUP
      if constexpr (PREV) {
        sums.stage_d();
        park(t - 1);
      }
      sums.take(acc);
      __builtin_amdgcn_sched_barrier(0);
    };
    {
      Opnd oa, ob;
      {
        const long row = row_of(0);
        const float *px = a.dxW + row * a.ld_dxw + ks * (3 * H / 8) + kq;
        const float *pl = a.dF + 2 * row * H + ks * (H / 8) + kq;
#pragma unroll
        for (int q = 0; q < 3; q++) oa.x[q] = ld4(px + 64 * q);
        oa.fl = ld4(pl);
        oa.fr = ld4(pl + H);
      }
      tile(std::false_type{}, 0, oa, ob);
      for (int t = 1; t < T; t += 2) {
        tile(std::true_type{}, t, ob, oa);
        if (t + 1 < T) tile(std::true_type{}, t + 1, oa, ob);
      }
      sums.all();
      park(T - 1);
    }
    __syncthreads();

    if (eon) {
      const float *pre = red + (ks * 8 * (NP * 4) + (lane >> 4)) * 16 + x;
      float v[NP];
#pragma unroll
      for (int p = 0; p < NP; p++) {
        float s = 0.f;
#pragma unroll
        for (int g = 0; g < 8; g++) s += pre[(g * NP * 4 + p * 4) * 16];
        v[p] = s;
      }
#pragma unroll
      for (int s = 0; s < 2; s++) {
        const long c = kc[s];
        if (c < 0) continue;
        const Kid &kd = kid[s];
        const GateGrad gg = gate_grad(kd.g[0], kd.g[1], kd.g[2], kd.g[3], kd.g[4], kd.g[5], v[0] + v[1 + s], pdc * pf[s], kd.dr, kd.cl, kd.cr);
        float *dx = a.dxW + c * a.ld_dxw + ej;
        dx[0] = gg.di; dx[H] = gg.d_o; dx[2 * H] = gg.du; dx[3 * H] = gg.dfl + gg.dfr;
        if (c >= a.leaf_rows) {
          a.dF[(2 * c) * H + ej] = gg.dfl;
          a.dF[(2 * c + 1) * H + ej] = gg.dfr;
          a.dc[c * H + ej] = gg.dc;
        }
      }
    }
    if (arrives) tail_arrive(gsync, total);
    else __syncthreads();
  }
}

// the barrier alone, on the footprint of the kernels above (one workgroup per CU: the LDS sees to that)
__global__ __launch_bounds__(512, 1) void tail_probe_kernel(unsigned *sync, int spin_max, int expect) {
  extern __shared__ float red[];
  __shared__ int s_bail;
  unsigned *status = sync + TAIL_STATUS, *gsync = sync + TAIL_GROUP_WORDS * ((blockIdx.x & 7) + 1);
  red[threadIdx.x] = 0.f;
  if (threadIdx.x == 0) __hip_atomic_fetch_or(gsync + TAIL_XCC, 1u << xcc_id(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const unsigned total = 3u * expect;
  for (int r = 0; r < 3; r++) {
    if (r > 0 && !tail_wait(status, gsync, (unsigned)r * expect, spin_max, r == 1, &s_bail)) return;
    tail_arrive(gsync, total);
  }
}

// Copies the caller's description of the groups and checks it (host arrays: group g runs
// nrounds[g] lists, list i of group g is rows[start[g * max_rounds + i] .. + count[g * max_rounds + i]);
// flags as in TailPlan, or null: every list waits for all the lists before it and arrives).
static int tail_plan(const char *who, int ngroups, const int *nrounds, const int *start, const int *count, const int *flags,
                     int max_rounds, TailPlan *out) {
  CAVS_REQUIRE(ngroups >= 1 && ngroups <= kTailGroups && nrounds && start && count && max_rounds >= 1,
               "%s: bad plan (1..%d groups)", who, kTailGroups);
  *out = TailPlan{};
  int any = 0;
  for (int g = 0; g < ngroups; g++) {
    CAVS_REQUIRE(nrounds[g] >= 0 && nrounds[g] <= kTailMaxRounds && nrounds[g] <= max_rounds, "%s: group %d has %d lists, at most %d", who, g,
                 nrounds[g], kTailMaxRounds < max_rounds ? kTailMaxRounds : max_rounds);
    out->nrounds[g] = nrounds[g];
    any += nrounds[g];
    int arrived = 0;
    for (int i = 0; i < nrounds[g]; i++) {
      const int s = start[g * max_rounds + i], c = count[g * max_rounds + i];
      CAVS_REQUIRE(s >= 0 && c >= 1 && c <= kTailRows, "%s: group %d list %d: %d rows from %d (1..%d rows)", who, g, i, c, s, kTailRows);
      const int f = flags ? flags[g * max_rounds + i] : ((i << 1) | 1);
      CAVS_REQUIRE(f >= 0 && (f >> 1) <= arrived, "%s: group %d list %d waits for %d arrivals, %d lists before it arrive", who, g, i, f >> 1,
                   arrived);
      out->start[g][i] = s;
      out->count[g][i] = (short)c;
      out->flags[g][i] = (short)f;
      arrived += f & 1;
    }
    // (the last arrival of a launch clears the counter: nobody may still be waiting on it then)
    for (int i = nrounds[g] - 1; i >= 0 && !(out->flags[g][i] & 1); i--)
      CAVS_REQUIRE((out->flags[g][i] >> 1) == 0, "%s: group %d list %d waits, but no list from it on arrives", who, g, i);
    out->arrivals[g] = arrived;
  }
  return any > 0 ? 1 : 0;  // 0: nothing to do
}

static int tail_lds_attr(const void *kernel, size_t bytes) {
  CAVS_HIP_TRY(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
  return CAVS_OK;
}

}  // namespace cavs

using namespace cavs;

extern "C" {

int cavs_tail_rounds_ok(int n, int H) { return (H == kTailH && n >= 1 && n <= kTailRows) ? 1 : 0; }
int cavs_tail_max_rounds(void) { return kTailMaxRounds; }
int cavs_tail_max_groups(void) { return kTailGroups; }
size_t cavs_tail_sync_bytes(void) { return (size_t)TAIL_GROUP_WORDS * (kTailGroups + 1) * sizeof(unsigned); }

int cavs_tail_probe(unsigned *sync, int H, int spin_max, void *stream) {
  CAVS_REQUIRE(sync && H == kTailH && spin_max >= 0, "cavs_tail_probe: bad arguments (H = %d only)", kTailH);
  constexpr size_t lds = kTailFwdRed * sizeof(float) + kTailTabBytes;
  static int attr = tail_lds_attr(reinterpret_cast<const void *>(tail_probe_kernel), lds);
  if (attr != CAVS_OK) return attr;
  launch(tail_probe_kernel, dim3(8 * (H / 16)), 512, lds, as_stream(stream), sync, spin_max, H / 16);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_treelstm_tail_fwd(float *pool, const int *child, const int *pair, const float *xW, int ld_xw, const float *Upk,
                           const float *bias, float *G, float *hlr, float *gates, float *msg, float *graph_out,
                           const int *out_rows, const int *rows, int ngroups, const int *nrounds, const int *start,
                           const int *count, const int *flags, int max_rounds, int H, unsigned *sync, int spin_max,
                           int extra_arrivals, void *stream) {
  CAVS_REQUIRE(H == kTailH && ld_xw >= 4 * H && ld_xw % 4 == 0, "cavs_treelstm_tail_fwd: bad shape H=%d ld_xw=%d (H = %d only)", H, ld_xw,
               kTailH);
  CAVS_REQUIRE(pool && child && pair && xW && Upk && bias && G && hlr && gates && rows && sync, "cavs_treelstm_tail_fwd: null pointer");
  CAVS_REQUIRE(aligned16(pool) && aligned16(Upk), "cavs_treelstm_tail_fwd: pool and Upk must be 16-byte aligned");
  CAVS_REQUIRE(!graph_out || out_rows, "cavs_treelstm_tail_fwd: graph_out needs out_rows");
  CAVS_REQUIRE(spin_max >= 0 && extra_arrivals >= 0, "cavs_treelstm_tail_fwd: bad wait bound");
  TailFwdArgs a{pool, child, pair, xW, ld_xw, Upk, bias, G, hlr, gates, msg, graph_out, out_rows, rows, sync, spin_max,
                H / 16 + extra_arrivals, {}};
  const int todo = tail_plan("cavs_treelstm_tail_fwd", ngroups, nrounds, start, count, flags, max_rounds, &a.plan);
  if (todo <= 0) return todo;
  constexpr size_t lds = kTailFwdRed * sizeof(float) + kTailTabBytes;
  static int attr = tail_lds_attr(reinterpret_cast<const void *>(treelstm_tail_fwd_kernel), lds);
  if (attr != CAVS_OK) return attr;
  launch(treelstm_tail_fwd_kernel, dim3(8 * (H / 16)), 512, lds, as_stream(stream), a);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_treelstm_tail_bwd(float *dxW, int ld_dxw, float *dF, float *dc, const float *UTp, const int *child_rows,
                           const float *gates, const float *G, const float *dret, const int *dret_rows, int leaf_rows,
                           const int *rows, int ngroups, const int *nrounds, const int *start, const int *count,
                           const int *flags, int max_rounds, int H, unsigned *sync, int spin_max, int extra_arrivals,
                           void *stream) {
  CAVS_REQUIRE(H == kTailH && ld_dxw >= 4 * H && ld_dxw % 4 == 0 && leaf_rows >= 0,
               "cavs_treelstm_tail_bwd: bad shape H=%d ld=%d leaf_rows=%d (H = %d only)", H, ld_dxw, leaf_rows, kTailH);
  CAVS_REQUIRE(dxW && dF && dc && UTp && child_rows && gates && G && dret && dret_rows && rows && sync,
               "cavs_treelstm_tail_bwd: null pointer");
  CAVS_REQUIRE(aligned16(dxW) && aligned16(dF) && aligned16(UTp), "cavs_treelstm_tail_bwd: dxW, dF and UTp must be 16-byte aligned");
  CAVS_REQUIRE(spin_max >= 0 && extra_arrivals >= 0, "cavs_treelstm_tail_bwd: bad wait bound");
  TailBwdArgs a{dxW, ld_dxw, dF, dc, UTp, child_rows, gates, G, dret, dret_rows, rows, sync, leaf_rows, spin_max,
                H / 16 + extra_arrivals, {}};
  const int todo = tail_plan("cavs_treelstm_tail_bwd", ngroups, nrounds, start, count, flags, max_rounds, &a.plan);
  if (todo <= 0) return todo;
  constexpr size_t lds = kTailBwdRed * sizeof(float) + kTailTabBytes;
  static int attr = tail_lds_attr(reinterpret_cast<const void *>(treelstm_tail_bwd_kernel), lds);
  if (attr != CAVS_OK) return attr;
  launch(treelstm_tail_bwd_kernel, dim3(8 * (H / 16)), 512, lds, as_stream(stream), a);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

}  // extern "C"
