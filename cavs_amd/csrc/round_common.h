// Shared pieces of the fused round kernels: the two MFMA tile shapes, operand helpers, the
// per-wavefront partial-tile reduction through LDS, and the tile / wavefront plan.
#ifndef CAVS_CSRC_ROUND_COMMON_H_
#define CAVS_CSRC_ROUND_COMMON_H_

#include <type_traits>

#include "common.h"

namespace cavs {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

template <int TILE>
struct Mma;

// 32x32x2: lane l supplies A[row l%32][k l/32] and B[k l/32][col l%32]; accumulator
// element r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32.
template <>
struct Mma<32> {
  static constexpr int NR = 16, NSLOT = 2;
  typedef floatx16 Acc;
  static __device__ inline Acc mma(float a, float b, Acc c) { return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0); }
  static __device__ inline int row(int r, int lane) { return 8 * (r / 4) + 4 * (lane >> 5) + (r % 4); }
};

// 16x16x4: lane l supplies A[row l%16][k l/16] and B[k l/16][col l%16]; accumulator
// element r of lane l is row 4*(l/16) + r, column l%16.
template <>
struct Mma<16> {
  static constexpr int NR = 4, NSLOT = 4;
  typedef floatx4 Acc;
  static __device__ inline Acc mma(float a, float b, Acc c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
  static __device__ inline int row(int r, int lane) { return 4 * (lane >> 4) + r; }
};

// 4x4x1, sixteen blocks per instruction: lane l supplies A[row l%4] and B[col l%4] of block l/4;
// accumulator element r of lane l is row r, column l%4 of block l/4.  The round kernels use it for
// tiles of four rows by sixteen columns: block l/4 = (column group (l/4)%4, k slot l/16), so the
// operand fragments are those of the 16x16x4 shape with the A row taken modulo four, and the four
// k slots of an element (lanes x, x+16, x+32, x+48) are added up after the loop.
struct Mma4 {
  static constexpr int NR = 4, NSLOT = 4;
  typedef floatx4 Acc;
  static __device__ inline Acc mma(float a, float b, Acc c) { return __builtin_amdgcn_mfma_f32_4x4x1f32(a, b, c, 0, 0, 0); }
  static __device__ inline int row(int r, int lane) { return r; }
};

__device__ inline float4 ld4(const float *p) { return *reinterpret_cast<const float4 *>(p); }
__device__ inline float4 zero4() { return make_float4(0.f, 0.f, 0.f, 0.f); }
__device__ inline float elem(const float4 &v, int c) { return c == 0 ? v.x : c == 1 ? v.y : c == 2 ? v.z : v.w; }
// The gates of the fused round kernels: exp through v_exp_f32 and the reciprocal through
// v_rcp_f32 (1 ulp each; 4 and 6 instructions against the 26 and 28 of 1.f / (1.f + expf(-x)) and
// tanhf, of which a thread's epilogue has six).  Saturation comes out right without special
// cases: exp overflows to inf, whose reciprocal is 0, and underflows to 0.  tanh_r is accurate to
// 1e-7 absolute; near zero that is a large relative error of a tiny number.
// (No multiply-add contraction in these and in the gate functions below: whether the compiler
// fuses a product into a following sum depends on the code around it, and kernels that inline the
// same function must produce the same bits.)
__device__ inline float exp_r(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }
__device__ inline float sigm_r(float x) { return __builtin_amdgcn_rcpf(1.f + exp_r(-x)); }
__device__ inline float tanh_r(float x) {
#pragma clang fp contract(off)
  return 1.f - 2.f * __builtin_amdgcn_rcpf(1.f + exp_r(2.f * x));
}


// The gates of one hidden unit of one vertex (apps/paper/tree-lstm-cavs.cc:132-171): xw = the unit's
// four columns of x * W ([i|o|u|f]), v = its five recurrent pre-activations (i, o, u, f_l, f_r),
// bias = its four bias entries in the bias's own block order ([i|f|u|o]), c_left / c_right = the
// children's c.  One function for every kernel that finishes a forward round, so that they all
// evaluate the same expressions in the same association: (x * W + h * U) + bias.
struct TreeLstmCell {
  float i, o, u, f_l, f_r, tc, h, c;
};
__device__ inline TreeLstmCell treelstm_cell(const float (&xw)[4], const float (&v)[5], const float (&bias)[4], float c_left,
                                             float c_right) {
#pragma clang fp contract(off)
  TreeLstmCell q;
  q.i = sigm_r((xw[0] + v[0]) + bias[0]);
  q.o = sigm_r((xw[1] + v[1]) + bias[3]);
  q.u = tanh_r((xw[2] + v[2]) + bias[2]);
  q.f_l = sigm_r((xw[3] + v[3]) + bias[1]);
  q.f_r = sigm_r((xw[3] + v[4]) + bias[1]);
  q.c = (q.i * q.u + q.f_l * c_left) + q.f_r * c_right;
  q.tc = tanh_r(q.c);
  q.h = q.o * q.tc;
  return q;
}

// Gate gradients of one hidden unit of one vertex.  mh, mc: gradient of the vertex's message
// ([h|c] halves); dr: gradient of its pushed return value; c_left, c_right: the children's c
// (zero for a leaf).
struct GateGrad {
  float di, d_o, du, dfl, dfr, dc;
};
__device__ inline GateGrad gate_grad(float i, float o, float u, float f_l, float f_r, float tc, float mh, float mc, float dr,
                                     float c_left, float c_right) {
#pragma clang fp contract(off)
  GateGrad g;
  const float dh = mh + dr;
  const float d_o = dh * tc;
  const float dc = mc + (dh * o) * (1.f - tc * tc);
  g.dfl = (dc * c_left) * (f_l * (1.f - f_l));
  g.dfr = (dc * c_right) * (f_r * (1.f - f_r));
  g.di = (dc * u) * (i * (1.f - i));
  g.d_o = d_o * (o * (1.f - o));
  g.du = (dc * i) * (1.f - u * u);
  g.dc = dc;
  return g;
}

// The same for the vertices nobody sends a message gradient to (the roots), named by a list of
// slab rows over whole-batch slabs: d c of a vertex goes to row v of `dc`, from where the launch
// of the vertex's own round hands it on to the children.
struct BwdGatesRowsArgs {
  const int *rows;       // [n] slab rows
  const float *dret;     // gradient of the pushed return value: row dret_rows[v]
  const int *dret_rows;  // [*] by slab row
  const float *gates;    // [*, 6H]
  const float *G;        // [2*, 2H]
  float *dxW;            // [*, 4H] (ld_dxw)
  long ld_dxw;
  float *dF;             // [2*, H]
  float *dc;             // [*, H]
  int n, H, leaf_rows;   // slab rows below leaf_rows are leaves
};

// element idx of the launch: W consecutive hidden units of one listed vertex
template <int W>
__device__ inline void treelstm_gates_rows_at(const BwdGatesRowsArgs &a, long idx) {
  const int H = a.H, hw = H / W;
  const long H2 = 2L * H;
  if (idx >= (long)a.n * hw) return;
  const int j = (int)(idx % hw) * W;
  const long v = a.rows[idx / hw];
  const bool internal = v >= a.leaf_rows;
  const float *g = a.gates + v * 6 * H + j;
  const float *dr = a.dret + (long)a.dret_rows[v] * H + j;
  const float *cl = a.G + (2 * v) * H2 + H + j, *cr = cl + H2;
  float *dx = a.dxW + v * a.ld_dxw + j;
#pragma unroll
  for (int k = 0; k < W; k++) {
    const GateGrad q = gate_grad(g[k], g[H + k], g[2 * H + k], g[3 * H + k], g[4 * H + k], g[5 * H + k], 0.f, 0.f, dr[k],
                                 internal ? cl[k] : 0.f, internal ? cr[k] : 0.f);
    dx[k] = q.di; dx[H + k] = q.d_o; dx[2 * H + k] = q.du; dx[3 * H + k] = q.dfl + q.dfr;
    if (internal) {
      a.dF[(2 * v) * H + j + k] = q.dfl;
      a.dF[(2 * v + 1) * H + j + k] = q.dfr;
      a.dc[v * H + j + k] = q.dc;
    }
  }
}


// Parks the per-wavefront partial tiles of NP products in LDS as
// [region][row tile][product][accumulator element][lane].  There are NREG regions: the
// wavefronts with k-split index below NREG write theirs, the others add onto region
// ks % NREG in a second, third ... step, so that the reader only has to sum NREG values
// per element, always in the same order (deterministic).
template <int TILE, int NP, int KS, int NREG, int RT>
__device__ inline void park_partials(float *red, const typename Mma<TILE>::Acc (&acc)[NP], int rt, int ks, int lane) {
  constexpr int NR = Mma<TILE>::NR;
  static_assert(KS % NREG == 0, "k-splits must fill whole steps");
  for (int step = 0; step < KS / NREG; step++) {
    if (ks / NREG == step) {
      float *base = red + (ks % NREG) * (RT * NP * NR * 64);
#pragma unroll
      for (int p = 0; p < NP; p++)
#pragma unroll
        for (int r = 0; r < NR; r++) {
          float *q = base + ((rt * NP + p) * NR + r) * 64 + lane;
          *q = (step == 0) ? acc[p][r] : *q + acc[p][r];
        }
    }
    __syncthreads();
  }
}

// regions for a tile shape: all eight for the small tile (40 KB for five products), four for
// the large one (80 KB)
template <int TILE, int KS>
struct Regions {
  static constexpr int N = TILE == 16 ? KS : (KS >= 4 ? 4 : KS);
};

inline bool round_shape_ok(int H) { return H > 0 && H % 32 == 0; }

// tile shape and wavefronts per workgroup for a round of n rows
struct RoundPlan {
  int tile, waves;
};
// Measured on MI355X at H=512: the 16x16 tile wins while a round is too small to give every
// CU several 32x32 tiles (600 rows: 32 us against 40).  Eight wavefronts per workgroup for the
// smallest rounds (shortest latency chain); four beyond, compiled for four workgroups per CU so that
// their latency chains overlap; 32x32 tiles above a thousand rows, where operand reuse counts.
// Packed Tree-LSTM launches of at most this many rows use tiles of four rows (Mma4): measured in
// the C3 step, 0.4206 ms with sixteen-row tiles throughout, 0.4160 with four-row tiles up to 16
// rows, 0.4137 up to 32; a forward launch of 64 rows takes 11.4 us that way against 8.4 (every
// row tile streams the whole weight panel).
constexpr int kRows4Max = 32;

// Eight wavefronts reach up to 128 rows where H lets them keep their exact loops (a multiple of
// 512): C3 step 0.4135 ms with the limit at 64, 0.4114 at 96, 0.4101 at 128, 0.4143 at 192.
inline RoundPlan plan_round(int n, int H) {
  if (n <= (H % 512 == 0 ? 128 : 64)) return {16, 8};
  if (n <= 1024) return {16, 4};
  return {32, 8};
}

// The product loop of the fused round kernels when the wavefront's k range is an even number of
// whole pipeline stages (exact_stages below): acc[i] += A_i[row, k) * B[k, col] for NA operands
// A_i that share one B.  B comes through buffer loads -- a descriptor in scalar registers, a
// scalar byte offset that advances with k, and this lane's byte offsets vb[c] of column col in
// row 4 * slot + c of a k-group, fixed before the loop -- so no address arithmetic runs on the
// vector ALU (spelled out per load, its 64-bit row * stride products cost as much time as the
// MFMAs).  A rows are per-lane pointers (already at this wavefront's first k plus 4 * slot),
// bumped once per k-group.  Nothing in the loop is conditional, so the wait counts of the two
// stage buffers come out exact and one stage's loads are in flight under the other's MFMAs; the
// scheduler barriers keep that order (left alone, the compiler sinks every load to its use).
// PACKED (16x16 tiles): B is in the tile-major layout CAVS_TASK_PACK_T writes -- the lane's four k
// of a k-group are one float4, number slot * 16 + x of the 1 KB block of the k-group and column
// tile; bpk points at this lane's float4 of the wavefront's first block and b_row_bytes is the
// distance to the next k-group's block -- so a wavefront's B fragment is one load of a
// contiguous kilobyte instead of four loads of four 64-byte pieces each (the texture-address
// unit charges per piece).
// QUAD (16x16 tiles): arow[i] is the pointer of lane l into tile row l / 4 at k = 4 * (l % 4), so
// that the four lanes of a quad read 64 consecutive bytes of one row -- the texture-address unit
// works through a 16-byte-per-lane load a quad at a time, and a quad that spans four rows costs
// it four cache lines where this costs one.  The MFMA wants row x = l % 16, k-slot l / 16; the
// fragment crosses lanes (from lane 4 * x + slot) through the LDS crossbar just before it is used.
// ROWS4 (with QUAD): tiles of four rows on the 4x4x1 shape (Mma4); arow[i] then belongs to tile row
// (l / 4) % 4.
template <int TILE, int UG, int NA, bool PACKED = false, bool QUAD = false, bool ROWS4 = false>
__device__ inline void exact_products(typename Mma<TILE>::Acc *acc, const float *(&arow)[NA], __amdgpu_buffer_rsrc_t bbuf,
                                      const int (&vb)[4], int sb, int b_row_bytes, int nst, const float4 *bpk = nullptr) {
  using M = std::conditional_t<ROWS4, Mma4, Mma<TILE>>;
  static_assert(!ROWS4 || (QUAD && TILE == 16), "the four-row tiles go with the quad-contiguous loads of the 16-column tile");
  constexpr int GK = 4 * M::NSLOT;
  static_assert(!PACKED || TILE == 16, "the packed layout is for 16x16 tiles");
  static_assert(!QUAD || TILE == 16, "the quad-contiguous A loads are for 16x16 tiles");
  const int lane_ = threadIdx.x & 63, from4 = 4 * (4 * (lane_ & (ROWS4 ? 3 : 15)) + (lane_ >> 4));
  struct Frag {
    float4 a[UG][NA];
    float b[UG][4];
  };
  auto fetch = [&](Frag &f) {
#pragma unroll
    for (int u = 0; u < UG; u++) {
      if constexpr (PACKED) {
        const float4 v = *bpk;
        bpk = reinterpret_cast<const float4 *>(reinterpret_cast<const char *>(bpk) + b_row_bytes);
#pragma unroll
        for (int c = 0; c < 4; c++) f.b[u][c] = elem(v, c);
      } else {
#pragma unroll
        for (int c = 0; c < 4; c++) f.b[u][c] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(bbuf, vb[c], sb, 0));
      }
#pragma unroll
      for (int i = 0; i < NA; i++) {
        f.a[u][i] = ld4(arow[i]);
        arow[i] += GK;
      }
      if constexpr (!PACKED) sb += GK * b_row_bytes;
    }
  };
  auto multiply = [&](const Frag &f) {
    if constexpr (QUAD) {
      float av[UG][NA][4];
#pragma unroll
      for (int u = 0; u < UG; u++)
#pragma unroll
        for (int i = 0; i < NA; i++)
#pragma unroll
          for (int c = 0; c < 4; c++)
            av[u][i][c] = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(from4, __builtin_bit_cast(int, elem(f.a[u][i], c))));
#pragma unroll
      for (int u = 0; u < UG; u++)
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
          for (int i = 0; i < NA; i++) acc[i] = M::mma(av[u][i][c], f.b[u][c], acc[i]);
    } else {
#pragma unroll
      for (int u = 0; u < UG; u++)
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
          for (int i = 0; i < NA; i++) acc[i] = M::mma(elem(f.a[u][i], c), f.b[u][c], acc[i]);
    }
  };
  Frag f0, f1;
  fetch(f0);
  for (int st = 0; st + 2 < nst; st += 2) {
    fetch(f1);
    __builtin_amdgcn_sched_barrier(0);
    multiply(f0);
    __builtin_amdgcn_sched_barrier(0);
    fetch(f0);
    __builtin_amdgcn_sched_barrier(0);
    multiply(f1);
    __builtin_amdgcn_sched_barrier(0);
  }
  fetch(f1);
  __builtin_amdgcn_sched_barrier(0);
  multiply(f0);
  multiply(f1);
}

// K = H splits into an even number of whole pipeline stages for every wavefront of the plan's
// kernels (K-splits = wavefronts; a k-group is 16 k for either MFMA shape; one group per stage for
// the four-wavefront 16x16 kernels, two otherwise), and the weights' byte offsets fit 31 bits
inline bool exact_stages(int H, const RoundPlan &p) {
  const int ug = (p.tile == 16 && p.waves == 4) ? 1 : 2;
  return H % (p.waves * 16 * ug * 2) == 0 && H <= 8192;
}

}  // namespace cavs
#endif
