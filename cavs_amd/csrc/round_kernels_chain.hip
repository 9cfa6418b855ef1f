// Fused rounds of the chain LSTM (apps/paper/seq-lstm-cavs.cc:62-86) and of Tree-FC
// (apps/paper/tree-fc-cavs.cc:28-36): the same construction as the Tree-LSTM round kernels --
// a workgroup owns TILE rows x TILE hidden columns, its wavefronts split K and feed the MFMA
// straight from global memory with the gather as the operand fetch, partial tiles are
// parked per wavefront in LDS, and the epilogue applies the pointwise part of the vertex
// function and scatters the message.  A chain round is one sequence step for all live
// sequences (n <= batch size): without fusion it is four dependent launches of latency.
#include "round_common.h"

namespace cavs {

// One product chain: acc[p] += A[row, kb:ke) * B_p[kb:ke, col] for NB B operands that share A.
// a_row: the lane's A row (k-contiguous, 16-byte aligned) or nullptr for a zero row;
// b[p]: the lane's column of B operand p at k = 0, row stride ldb.
template <int TILE, int NB>
__device__ inline void product_chain(typename Mma<TILE>::Acc (&acc)[NB], const float *a_row, const float *const (&b)[NB],
                                     long ldb, int kb, int ke, int slot) {
  using M = Mma<TILE>;
  constexpr int GK = 4 * M::NSLOT, UG = 2, S = GK * UG;
  struct Frag {
    float4 a[UG];
    float b[UG][NB][4];
  };
  auto fetch = [&](int k0, Frag &f) {
#pragma unroll
    for (int u = 0; u < UG; u++) {
      const int kk = k0 + GK * u + 4 * slot;
      const bool kin = kk < ke;
#pragma unroll
      for (int p = 0; p < NB; p++)
#pragma unroll
        for (int c = 0; c < 4; c++) f.b[u][p][c] = kin ? b[p][(long)(kk + c) * ldb] : 0.f;
      f.a[u] = (kin && a_row) ? ld4(a_row + kk) : zero4();
    }
  };
  auto multiply = [&](const Frag &f) {
#pragma unroll
    for (int u = 0; u < UG; u++)
#pragma unroll
      for (int c = 0; c < 4; c++)
#pragma unroll
        for (int p = 0; p < NB; p++) acc[p] = M::mma(elem(f.a[u], c), f.b[u][p][c], acc[p]);
  };
  Frag f0, f1;
  if (kb < ke) fetch(kb, f0);
  for (int k0 = kb; k0 < ke; k0 += 2 * S) {
    if (k0 + S < ke) fetch(k0 + S, f1);
    multiply(f0);
    if (k0 + S < ke) {
      if (k0 + 2 * S < ke) fetch(k0 + 2 * S, f0);
      multiply(f1);
    }
  }
}

// The same chain when the wavefront's k range is an even number of whole stages of 32 k
// (chain_exact): the B operands come through buffer loads -- descriptor and k offset in scalar
// registers, this lane's byte offsets fixed before the loop -- so that no address arithmetic
// runs on the vector ALU, nothing in the loop is conditional and the wait counts come out exact
// (see exact_products).  B operand p is the block of columns [p * blk, p * blk + H) of the
// row-major matrix `bmat` (`bfloats` floats, row stride ldb); the chain covers its rows
// [krow, krow + 32 * nst).  a_row is already at this wavefront's first k; a lane without a row
// passes any readable address and has = false.
// PACKED: `bmat` is the same matrix tile-major (a CAVS_TASK_PACK_T / CAVS_TASK_SGD_PACK job
// writes it): float4 (slot, x) of the 16 x 16 tile (k-group, column tile) holds this lane's four
// k, so a wavefront's fragment is one contiguous kilobyte.  `ldb` is the matrix's column count.
template <int TILE, int NB, bool PACKED = false>
__device__ inline void product_chain_exact(typename Mma<TILE>::Acc (&acc)[NB], const float *a_row, bool has, const float *bmat,
                                           int bfloats, int col, int blk, int ldb, int krow, int nst, int slot) {
  using M = Mma<TILE>;
  constexpr int GK = 4 * M::NSLOT, UG = 2;
  static_assert(!PACKED || TILE == 16, "the packed layout is for 16x16 tiles");
  const float4 *bpk = reinterpret_cast<const float4 *>(bmat) + ((long)(krow / 16) * (ldb / 16) + col / 16) * 64 + slot * 16 + (col & 15);
  const int pstep = blk * 4, gstep = ldb * 4;  // float4 between column blocks, between k-groups
  const __amdgpu_buffer_rsrc_t bbuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(bmat), 0, bfloats * 4, 0x00020000);
  int vb[4];
#pragma unroll
  for (int c = 0; c < 4; c++) vb[c] = ((4 * slot + c) * ldb + col) * 4;
  int sb = krow * ldb * 4;
  a_row += 4 * slot;
  struct Frag {
    float4 a[UG];
    float b[UG][NB][4];
  };
  auto fetch = [&](Frag &f) {
#pragma unroll
    for (int u = 0; u < UG; u++) {
      if constexpr (PACKED) {
#pragma unroll
        for (int p = 0; p < NB; p++) {
          const float4 v = bpk[p * pstep];
#pragma unroll
          for (int c = 0; c < 4; c++) f.b[u][p][c] = elem(v, c);
        }
        bpk += gstep;
      } else {
#pragma unroll
        for (int p = 0; p < NB; p++)
#pragma unroll
          for (int c = 0; c < 4; c++)
            f.b[u][p][c] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(bbuf, vb[c], sb + p * blk * 4, 0));
        sb += GK * ldb * 4;
      }
      f.a[u] = ld4(a_row);
      a_row += GK;
    }
  };
  auto multiply = [&](const Frag &f) {
#pragma unroll
    for (int u = 0; u < UG; u++)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const float av = has ? elem(f.a[u], c) : 0.f;
#pragma unroll
        for (int p = 0; p < NB; p++) acc[p] = M::mma(av, f.b[u][p][c], acc[p]);
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

// K rows of B split over `waves` wavefronts into an even number of whole stages each, and the
// byte offsets into B fit 31 bits
inline bool chain_exact(long K, int waves, long bfloats) { return K > 0 && K % (waves * 64) == 0 && bfloats < (1L << 28); }

// element (q-th of this thread) of the workgroup's tile: slab row, column, LDS offset
template <int TILE, int NP, int THREADS>
struct TileElems {
  using M = Mma<TILE>;
  static constexpr int NR = M::NR, EPT = (NR * 64 + THREADS - 1) / THREADS;
  bool on[EPT];
  int b[EPT], j[EPT], lds[EPT];
  __device__ inline void init(int tid, int row0, int j0, int n) {
#pragma unroll
    for (int q = 0; q < EPT; q++) {
      const int e = tid + q * THREADS;
      const int l2 = e & 63, r = (e >> 6) % NR;
      b[q] = row0 + M::row(r, l2);
      j[q] = j0 + (l2 & (TILE - 1));
      lds[q] = r * 64 + l2;
      on[q] = e < NR * 64 && b[q] < n;
    }
  }
};

template <int NP, int NR, int NREG>
__device__ inline void sum_regions(float (&v)[NP], const float *red, int lds, int rsz) {
#pragma unroll
  for (int p = 0; p < NP; p++) {
    float s = red[lds + p * NR * 64];
#pragma unroll
    for (int g = 1; g < NREG; g++) s += red[g * rsz + lds + p * NR * 64];
    v[p] = s;
  }
}

template <int W>
__device__ inline void stw(float *p, const float (&v)[W]) {
  if constexpr (W == 4) {
    *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
#pragma unroll
    for (int k = 0; k < W; k++) p[k] = v[k];
  }
}
template <int W>
__device__ inline void ldw(const float *p, float (&v)[W]) {
  if constexpr (W == 4) {
    const float4 t = ld4(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  } else {
#pragma unroll
    for (int k = 0; k < W; k++) v[k] = p[k];
  }
}

// ================================================================== chain LSTM
struct LstmFwdArgs {
  const float *pool;    // [*, 2H] rows [h|c]
  const int *child;     // [n] pool row of the predecessor (-1: none) or nullptr (first step of every sequence)
  const int *pair;      // [n]
  const float *xW;      // [n, 4H] (ld) blocks [i|f|u|o]
  long ld_xw;
  const float *Wh;      // [H, 4H]
  const float *bias;    // [4H]
  float *G;             // [n, 2H] gathered predecessor
  float *gates;         // [n, 5H] = [i|f|u|o|tanh c]
  float *msg;           // [n, 2H]
  float *pool_out;
  float *go;
  const int *out_rows;
  int n, H;
};

template <int TILE, int WAVES, bool EXACT, bool PACKED = false>
__global__ __launch_bounds__(WAVES * 64) void lstm_round_fwd_kernel(LstmFwdArgs a) {
  using M = Mma<TILE>;
  using Acc = typename M::Acc;
  constexpr int THREADS = WAVES * 64, KS = WAVES, GK = 4 * M::NSLOT, NP = 4, NR = M::NR;
  constexpr int NREG = Regions<TILE, KS>::N, RSZ = NP * NR * 64;
  __shared__ float red[NREG * RSZ];
  const int tid = threadIdx.x, lane = tid & 63, ks = tid >> 6;
  const int x = lane & (TILE - 1), slot = lane / TILE;
  const int H = a.H;
  const long H2 = 2L * H, H4 = 4L * H;
  const int j0 = blockIdx.x * TILE, row0 = blockIdx.y * TILE;
  const int row = row0 + x;
  const int kper = ((H + KS - 1) / KS + GK - 1) / GK * GK;
  const int kb = ks * kper, ke = min(H, kb + kper);

  int cp = -1;
  if (row < a.n) cp = a.child[row];
  TileElems<TILE, NP, THREADS> el;
  el.init(tid, row0, j0, a.n);
  constexpr int EPT = TileElems<TILE, NP, THREADS>::EPT;
  int ecp[EPT], edst[EPT], eout[EPT];
  float exw[EPT][4], ebias[EPT][4];
#pragma unroll
  for (int q = 0; q < EPT; q++) {
    ecp[q] = edst[q] = eout[q] = -1;
    if (el.on[q]) {
      ecp[q] = a.child[el.b[q]];
      edst[q] = a.pair[el.b[q]];
      if (a.go) eout[q] = a.out_rows[el.b[q]];
      const float *xw = a.xW + el.b[q] * a.ld_xw + el.j[q];
#pragma unroll
      for (int k = 0; k < 4; k++) { exw[q][k] = xw[k * H]; ebias[q][k] = a.bias[k * H + el.j[q]]; }
    }
  }

  Acc acc[NP];
#pragma unroll
  for (int p = 0; p < NP; p++)
#pragma unroll
    for (int r = 0; r < NR; r++) acc[p][r] = 0.f;
  const float *bcol[NP];
#pragma unroll
  for (int p = 0; p < NP; p++) bcol[p] = a.Wh + p * H + j0 + x;
  if constexpr (EXACT) {
    const int kbu = __builtin_amdgcn_readfirstlane(ks) * (H / KS);
    product_chain_exact<TILE, NP, PACKED>(acc, a.pool + (cp >= 0 ? cp : 0) * H2 + kbu, cp >= 0, a.Wh, 4 * H * H, j0 + x, H, 4 * H, kbu,
                                          H / KS / 32, slot);
  } else {
    product_chain<TILE, NP>(acc, cp >= 0 ? a.pool + cp * H2 : nullptr, bcol, H4, kb, ke, slot);
  }

  float ehp[EPT], ecprev[EPT];
#pragma unroll
  for (int q = 0; q < EPT; q++) {
    ehp[q] = ecprev[q] = 0.f;
    if (ecp[q] >= 0) { ehp[q] = a.pool[ecp[q] * H2 + el.j[q]]; ecprev[q] = a.pool[ecp[q] * H2 + H + el.j[q]]; }
  }
  park_partials<TILE, NP, KS, NREG, 1>(red, acc, 0, ks, lane);

#pragma unroll
  for (int q = 0; q < EPT; q++) {
    if (!el.on[q]) continue;
    float v[NP];
    sum_regions<NP, NR, NREG>(v, red, el.lds[q], RSZ);
    const int b = el.b[q], j = el.j[q];
    // same association as the separate path: (x*W + h*W') + bias
    const float i = sigm_r((exw[q][0] + v[0]) + ebias[q][0]);
    const float f = sigm_r((exw[q][1] + v[1]) + ebias[q][1]);
    const float u = tanh_r((exw[q][2] + v[2]) + ebias[q][2]);
    const float o = sigm_r((exw[q][3] + v[3]) + ebias[q][3]);
    const float c = i * u + f * ecprev[q];
    const float tc = tanh_r(c);
    const float h = o * tc;
    float *g = a.gates + (long)b * 5 * H + j;
    g[0] = i; g[H] = f; g[2 * H] = u; g[3 * H] = o; g[4 * H] = tc;
    float *m = a.msg + b * H2 + j;
    m[0] = h; m[H] = c;
    if (edst[q] >= 0) { a.pool_out[edst[q] * H2 + j] = h; a.pool_out[edst[q] * H2 + H + j] = c; }
    if (eout[q] >= 0) a.go[(long)eout[q] * H + j] = h;
    float *gp = a.G + b * H2 + j;
    gp[0] = ehp[q]; gp[H] = ecprev[q];
  }
}

// first step of every sequence (no predecessor), and the gate gradients of any round:
// elementwise, with the row movement folded in
struct LstmLeavesArgs {
  const float *xW;
  long ld_xw;
  const float *bias;
  const int *pair;
  float *gates, *msg, *pool, *go;
  const int *out_rows;
  int n, H;
};

template <int W>
__global__ void lstm_round_leaves_fwd_kernel(LstmLeavesArgs a) {
  const int H = a.H, hw = H / W;
  const long H2 = 2L * H;
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)a.n * hw) return;
  const int r = (int)(idx / hw), j = (int)(idx % hw) * W;
  const int dst = a.pair[r], out = a.go ? a.out_rows[r] : -1;
  const float *xw = a.xW + r * a.ld_xw + j;
  float gi[W], gf[W], gu[W], go[W], gtc[W], mh[W], mc[W];
#pragma unroll
  for (int k = 0; k < W; k++) {
    const float i = sigm_r((xw[k] + 0.f) + a.bias[j + k]);
    const float f = sigm_r((xw[H + k] + 0.f) + a.bias[H + j + k]);
    const float u = tanh_r((xw[2 * H + k] + 0.f) + a.bias[2 * H + j + k]);
    const float o = sigm_r((xw[3 * H + k] + 0.f) + a.bias[3 * H + j + k]);
    const float c = i * u + f * 0.f;
    const float tc = tanh_r(c);
    gi[k] = i; gf[k] = f; gu[k] = u; go[k] = o; gtc[k] = tc; mh[k] = o * tc; mc[k] = c;
  }
  float *g = a.gates + (long)r * 5 * H + j;
  stw<W>(g, gi); stw<W>(g + H, gf); stw<W>(g + 2 * H, gu); stw<W>(g + 3 * H, go); stw<W>(g + 4 * H, gtc);
  float *m = a.msg + r * H2 + j;
  stw<W>(m, mh); stw<W>(m + H, mc);
  if (dst >= 0) { stw<W>(a.pool + dst * H2 + j, mh); stw<W>(a.pool + dst * H2 + H + j, mc); }
  if (out >= 0) stw<W>(a.go + (long)out * H + j, mh);
}

// Gate gradients of one hidden unit of one chain vertex.  mh, mc: gradient of its message
// ([h|c] halves); dr: gradient of its pushed return value; cprev: the predecessor's c (zero at
// the first step).
struct LstmGateGrad {
  float di, df, du, d_o, dc;
};
__device__ inline LstmGateGrad lstm_gate_grad(float i, float f, float u, float o, float tc, float mh, float mc, float dr,
                                              float cprev) {
  LstmGateGrad g;
  const float dh = mh + dr;
  const float d_o = dh * tc;
  const float dc = mc + (dh * o) * (1.f - tc * tc);
  g.di = (dc * u) * (i * (1.f - i));
  g.df = (dc * cprev) * (f * (1.f - f));
  g.du = (dc * i) * (1.f - u * u);
  g.d_o = d_o * (o * (1.f - o));
  g.dc = dc;
  return g;
}
__device__ inline float treefc_dz(float dh, float y, int act) { return act ? dh * (1.f - y * y) : (y > 0.f ? dh : 0.f); }

struct LstmBwdGatesArgs {
  const float *dpool;
  const int *pair;
  const int *child;      // [n] or nullptr (first step)
  const float *dret;
  const int *dret_rows;  // or nullptr
  const float *gates;    // [n, 5H]
  const float *G;        // [n, 2H] or nullptr
  float *da;             // [n, 4H] (ld) blocks [i|f|u|o]
  long ld_da;
  float *dpool_out;
  int n, H;
};

template <int W>
__global__ void lstm_round_bwd_gates_kernel(LstmBwdGatesArgs a) {
  const int H = a.H, hw = H / W;
  const long H2 = 2L * H;
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)a.n * hw) return;
  const int r = (int)(idx / hw), j = (int)(idx % hw) * W;
  const int src = a.pair[r];
  const int dr_row = a.dret_rows ? a.dret_rows[r] : r;
  const int cp = a.child ? a.child[r] : -1;
  const float *g = a.gates + (long)r * 5 * H + j;
  float gi[W], gf[W], gu[W], go[W], gtc[W], dmh[W], dmc[W], dr[W], cprev[W];
  ldw<W>(g, gi); ldw<W>(g + H, gf); ldw<W>(g + 2 * H, gu); ldw<W>(g + 3 * H, go); ldw<W>(g + 4 * H, gtc);
  ldw<W>(a.dret + (long)dr_row * H + j, dr);
  if (src >= 0) { ldw<W>(a.dpool + src * H2 + j, dmh); ldw<W>(a.dpool + src * H2 + H + j, dmc); }
  if (a.G) ldw<W>(a.G + r * H2 + H + j, cprev);
  float di[W], df[W], du[W], dvo[W], dcp[W];
#pragma unroll
  for (int k = 0; k < W; k++) {
    const float mh = src >= 0 ? dmh[k] : 0.f, mc = src >= 0 ? dmc[k] : 0.f, cpv = a.G ? cprev[k] : 0.f;
    const LstmGateGrad q = lstm_gate_grad(gi[k], gf[k], gu[k], go[k], gtc[k], mh, mc, dr[k], cpv);
    di[k] = q.di; df[k] = q.df; du[k] = q.du; dvo[k] = q.d_o;
    dcp[k] = q.dc * gf[k];
  }
  float *d = a.da + r * a.ld_da + j;
  stw<W>(d, di); stw<W>(d + H, df); stw<W>(d + 2 * H, du); stw<W>(d + 3 * H, dvo);
  if (cp >= 0) stw<W>(a.dpool_out + cp * H2 + H + j, dcp);
}

// The pointwise backward part for the vertices nobody sends a message gradient to (the last step
// of every sequence, the roots of the trees), named by a list of slab rows over whole-batch slabs.
struct LstmBwdRowsArgs {
  const int *rows;
  const float *dret;
  const int *dret_rows;  // [*] by slab row
  const float *gates;    // [*, 5H]
  const float *G;        // [*, 2H]
  float *da;             // [*, 4H] (ld)
  long ld_da;
  float *dc;             // [*, H]
  int n, H, leaf_rows;
};

template <int W>
__global__ void lstm_bwd_gates_rows_kernel(LstmBwdRowsArgs a) {
  const int H = a.H, hw = H / W;
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)a.n * hw) return;
  const int j = (int)(idx % hw) * W;
  const long v = a.rows[idx / hw];
  const bool later = v >= a.leaf_rows;
  const float *g = a.gates + v * 5 * H + j, *dr = a.dret + (long)a.dret_rows[v] * H + j, *cp = a.G + v * 2 * H + H + j;
  float *d = a.da + v * a.ld_da + j;
#pragma unroll
  for (int k = 0; k < W; k++) {
    const LstmGateGrad q = lstm_gate_grad(g[k], g[H + k], g[2 * H + k], g[3 * H + k], g[4 * H + k], 0.f, 0.f, dr[k], later ? cp[k] : 0.f);
    d[k] = q.di; d[H + k] = q.df; d[2 * H + k] = q.du; d[3 * H + k] = q.d_o;
    if (later) a.dc[v * H + j + k] = q.dc;
  }
}

struct TreeFcBwdRowsArgs {
  const int *rows;
  const float *dret;
  const int *dret_rows;
  const float *h;  // [*, H]
  float *dz;       // [*, H]
  int n, H, act;
};

template <int W>
__global__ void treefc_bwd_rows_kernel(TreeFcBwdRowsArgs a) {
  const int H = a.H, hw = H / W;
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)a.n * hw) return;
  const int j = (int)(idx % hw) * W;
  const long v = a.rows[idx / hw];
  const float *dr = a.dret + (long)a.dret_rows[v] * H + j, *y = a.h + v * H + j;
#pragma unroll
  for (int k = 0; k < W; k++) a.dz[v * H + j + k] = treefc_dz(0.f + dr[k], y[k], a.act);
}

// Gradient of the gathered children's h: for child p of slab row b,
//   dpool[child[b*NB + p]][0:H) = dA[b, 0:K) * BT[0:K, p*H : (p+1)*H)
// (grad of Gather is Scatter, folded into the product's epilogue).  Chain LSTM: NB = 1,
// dA = da [n,4H], BT = W'^T [4H,H].  Tree-FC: NB = 2, dA = dz [n,H], BT = W^T [H,2H].
//
// FOLD 1 (chain LSTM) and 2 (Tree-FC): the launch goes on to the pointwise backward part of the
// children.  `child` then names them by slab row over whole-batch slabs, and the thread that
// holds d h of hidden unit j of a child writes the child's row of dA (and d c) directly; the
// message gradient never passes through the pool.
struct ChildBwdArgs {
  const float *dA;    // [n, K] (ld)
  long ld;
  const float *BT;    // [K, ldb]
  long ldb;
  const int *child;   // [n * NB]
  float *dpool;       // [*, mw]
  long mw;            // row width of the pool
  int n, H, K;
  // FOLD only; whole-batch slabs, the round starts at slab row row0
  float *dA_all, *dc_all;
  const float *gates_all, *G_all, *h_all, *dret;
  const int *dret_rows;
  int row0, leaf_rows, act;
};

template <int TILE, int WAVES, bool EXACT, int NB, int FOLD, bool PACKED = false>
__global__ __launch_bounds__(WAVES * 64) void round_bwd_children_kernel(ChildBwdArgs a) {
  using M = Mma<TILE>;
  using Acc = typename M::Acc;
  constexpr int THREADS = WAVES * 64, KS = WAVES, GK = 4 * M::NSLOT, NR = M::NR;
  constexpr int NREG = Regions<TILE, KS>::N, RSZ = NB * NR * 64;
  __shared__ float red[NREG * RSZ];
  // A round of the backward chain is latency, not work: where it shares CUs with a long product on
  // another stream, its wavefronts go first.
  __builtin_amdgcn_s_setprio(3);
  const int tid = threadIdx.x, lane = tid & 63, ks = tid >> 6;
  const int x = lane & (TILE - 1), slot = lane / TILE;
  const int H = a.H, K = a.K;
  const int j0 = blockIdx.x * TILE, row0 = blockIdx.y * TILE;
  const int row = row0 + x;
  const int kper = ((K + KS - 1) / KS + GK - 1) / GK * GK;
  const int kb = ks * kper, ke = min(K, kb + kper);
  TileElems<TILE, NB, THREADS> el;
  el.init(tid, row0, j0, a.n);
  constexpr int EPT = TileElems<TILE, NB, THREADS>::EPT;
  int ecp[EPT][NB];
#pragma unroll
  for (int q = 0; q < EPT; q++)
#pragma unroll
    for (int p = 0; p < NB; p++) ecp[q][p] = el.on[q] ? a.child[el.b[q] * NB + p] : -1;
  // FOLD: what the children's pointwise part needs besides d h, fetched while the product runs
  struct Kid {
    float g[FOLD == 1 ? 5 : 1], dr, cp;
  };
  Kid kid[FOLD ? EPT : 1][NB];
  float pdc[FOLD ? EPT : 1];
  if constexpr (FOLD != 0) {
#pragma unroll
    for (int q = 0; q < EPT; q++) {
      const int j = el.j[q];
      pdc[q] = 0.f;
      if constexpr (FOLD == 1) {
        const long gb = a.row0 + el.b[q];
        if (el.on[q]) pdc[q] = a.dc_all[gb * H + j] * a.gates_all[gb * 5 * H + H + j];  // d c handed on: d c * f
      }
#pragma unroll
      for (int p = 0; p < NB; p++) {
        const long v = ecp[q][p];
        Kid &kd = kid[q][p];
        kd.dr = kd.cp = 0.f;
#pragma unroll
        for (int t = 0; t < (FOLD == 1 ? 5 : 1); t++) kd.g[t] = 0.f;
        if (v < 0) continue;
        kd.dr = a.dret[(long)a.dret_rows[v] * H + j];
        if constexpr (FOLD == 1) {
#pragma unroll
          for (int t = 0; t < 5; t++) kd.g[t] = a.gates_all[v * 5 * H + (long)t * H + j];
          if (v >= a.leaf_rows) kd.cp = a.G_all[v * 2 * H + H + j];
        } else {
          kd.g[0] = a.h_all[v * H + j];
        }
      }
    }
  }
  Acc acc[NB];
  const float *bcol[NB];
#pragma unroll
  for (int p = 0; p < NB; p++) {
    bcol[p] = a.BT + (long)p * H + j0 + x;
#pragma unroll
    for (int r = 0; r < NR; r++) acc[p][r] = 0.f;
  }
  if constexpr (EXACT) {
    const int kbu = __builtin_amdgcn_readfirstlane(ks) * (K / KS);
    product_chain_exact<TILE, NB, PACKED>(acc, a.dA + (row < a.n ? row : 0) * a.ld + kbu, row < a.n, a.BT, K * (int)a.ldb, j0 + x, H,
                                          (int)a.ldb, kbu, K / KS / 32, slot);
  } else {
    product_chain<TILE, NB>(acc, row < a.n ? a.dA + row * a.ld : nullptr, bcol, a.ldb, kb, ke, slot);
  }
  park_partials<TILE, NB, KS, NREG, 1>(red, acc, 0, ks, lane);
#pragma unroll
  for (int q = 0; q < EPT; q++) {
    if (!el.on[q]) continue;
    float v[NB];
    sum_regions<NB, NR, NREG>(v, red, el.lds[q], RSZ);
#pragma unroll
    for (int p = 0; p < NB; p++) {
      const long c = ecp[q][p];
      if (c < 0) continue;
      const int j = el.j[q];
      if constexpr (FOLD == 1) {
        const Kid &kd = kid[q][p];
        const LstmGateGrad gg = lstm_gate_grad(kd.g[0], kd.g[1], kd.g[2], kd.g[3], kd.g[4], v[p], pdc[q], kd.dr, kd.cp);
        float *d = a.dA_all + c * a.ld + j;
        d[0] = gg.di; d[H] = gg.df; d[2 * H] = gg.du; d[3 * H] = gg.d_o;
        if (c >= a.leaf_rows) a.dc_all[c * H + j] = gg.dc;
      } else if constexpr (FOLD == 2) {
        a.dA_all[c * a.ld + j] = treefc_dz(v[p] + kid[q][p].dr, kid[q][p].g[0], a.act);
      } else {
        a.dpool[c * a.mw + j] = v[p];
      }
    }
  }
}

// ================================================================== Tree-FC
// h = act(W^T [h_l ; h_r] + b + x): one product whose A row is the concatenation of the two
// children's rows (k < H from the left child, k >= H from the right one).
struct TreeFcFwdArgs {
  const float *pool;    // [*, H]
  const int *child;     // [2n]
  const int *pair;      // [n]
  const float *W;       // [2H, H]
  const float *bias;    // [H] or nullptr
  const float *x;       // [n, H] or nullptr
  float *G;             // [n, 2H] gathered children [h_l | h_r]
  float *msg;           // [n, H]
  float *pool_out;
  float *go;
  const int *out_rows;
  int n, H, act;
};

template <int TILE, int WAVES, bool EXACT>
__global__ __launch_bounds__(WAVES * 64) void treefc_round_fwd_kernel(TreeFcFwdArgs a) {
  using M = Mma<TILE>;
  using Acc = typename M::Acc;
  constexpr int THREADS = WAVES * 64, KS = WAVES, GK = 4 * M::NSLOT, NP = 1, NR = M::NR;
  constexpr int NREG = Regions<TILE, KS>::N, RSZ = NP * NR * 64;
  __shared__ float red[NREG * RSZ];
  const int tid = threadIdx.x, lane = tid & 63, ks = tid >> 6;
  const int x = lane & (TILE - 1), slot = lane / TILE;
  const int H = a.H;
  const int j0 = blockIdx.x * TILE, row0 = blockIdx.y * TILE;
  const int row = row0 + x;
  // the wavefronts split each half of K (one half per child) between them
  const int kper = ((H + KS - 1) / KS + GK - 1) / GK * GK;
  const int kb = ks * kper, ke = min(H, kb + kper);
  int cl = -1, cr = -1;
  if (row < a.n) { cl = a.child[2 * row]; cr = a.child[2 * row + 1]; }
  TileElems<TILE, NP, THREADS> el;
  el.init(tid, row0, j0, a.n);
  constexpr int EPT = TileElems<TILE, NP, THREADS>::EPT;
  int ecl[EPT], ecr[EPT], edst[EPT], eout[EPT];
  float eb[EPT], ex[EPT];
#pragma unroll
  for (int q = 0; q < EPT; q++) {
    ecl[q] = ecr[q] = edst[q] = eout[q] = -1;
    eb[q] = ex[q] = 0.f;
    if (el.on[q]) {
      ecl[q] = a.child[2 * el.b[q]];
      ecr[q] = a.child[2 * el.b[q] + 1];
      edst[q] = a.pair[el.b[q]];
      if (a.go) eout[q] = a.out_rows[el.b[q]];
      if (a.bias) eb[q] = a.bias[el.j[q]];
      if (a.x) ex[q] = a.x[(long)el.b[q] * H + el.j[q]];
    }
  }
  Acc acc[NP];
#pragma unroll
  for (int r = 0; r < NR; r++) acc[0][r] = 0.f;
  const float *bl[NP] = {a.W + j0 + x};
  const float *br[NP] = {a.W + (long)H * H + j0 + x};
  if constexpr (EXACT) {
    const int kbu = __builtin_amdgcn_readfirstlane(ks) * (H / KS);
    product_chain_exact<TILE, NP>(acc, a.pool + (long)(cl >= 0 ? cl : 0) * H + kbu, cl >= 0, a.W, 2 * H * H, j0 + x, 0, H, kbu,
                                  H / KS / 32, slot);
    product_chain_exact<TILE, NP>(acc, a.pool + (long)(cr >= 0 ? cr : 0) * H + kbu, cr >= 0, a.W, 2 * H * H, j0 + x, 0, H, H + kbu,
                                  H / KS / 32, slot);
  } else {
    product_chain<TILE, NP>(acc, cl >= 0 ? a.pool + (long)cl * H : nullptr, bl, H, kb, ke, slot);
    product_chain<TILE, NP>(acc, cr >= 0 ? a.pool + (long)cr * H : nullptr, br, H, kb, ke, slot);
  }
  float ehl[EPT], ehr[EPT];
#pragma unroll
  for (int q = 0; q < EPT; q++) {
    ehl[q] = ecl[q] >= 0 ? a.pool[(long)ecl[q] * H + el.j[q]] : 0.f;
    ehr[q] = ecr[q] >= 0 ? a.pool[(long)ecr[q] * H + el.j[q]] : 0.f;
  }
  park_partials<TILE, NP, KS, NREG, 1>(red, acc, 0, ks, lane);
#pragma unroll
  for (int q = 0; q < EPT; q++) {
    if (!el.on[q]) continue;
    float v[NP];
    sum_regions<NP, NR, NREG>(v, red, el.lds[q], RSZ);
    const int b = el.b[q], j = el.j[q];
    float t = v[0];
    if (a.bias) t += eb[q];
    if (a.x) t += ex[q];
    const float h = a.act ? tanh_r(t) : (t > 0.f ? t : 0.f);
    a.msg[(long)b * H + j] = h;
    if (edst[q] >= 0) a.pool_out[(long)edst[q] * H + j] = h;
    if (eout[q] >= 0) a.go[(long)eout[q] * H + j] = h;
    float *gp = a.G + (long)b * 2 * H + j;
    gp[0] = ehl[q]; gp[H] = ehr[q];
  }
}

// leaves forward and the pointwise gradient of any round, with the row movement folded in
struct TreeFcLeavesArgs {
  const float *bias, *x;
  const int *pair;
  float *msg, *pool, *go;
  const int *out_rows;
  int n, H, act;
};

template <int W>
__global__ void treefc_round_leaves_fwd_kernel(TreeFcLeavesArgs a) {
  const int H = a.H, hw = H / W;
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)a.n * hw) return;
  const int r = (int)(idx / hw), j = (int)(idx % hw) * W;
  const int dst = a.pair[r], out = a.go ? a.out_rows[r] : -1;
  float h[W];
#pragma unroll
  for (int k = 0; k < W; k++) {
    float t = 0.f;
    if (a.bias) t += a.bias[j + k];
    if (a.x) t += a.x[(long)r * H + j + k];
    h[k] = a.act ? tanh_r(t) : (t > 0.f ? t : 0.f);
  }
  stw<W>(a.msg + (long)r * H + j, h);
  if (dst >= 0) stw<W>(a.pool + (long)dst * H + j, h);
  if (out >= 0) stw<W>(a.go + (long)out * H + j, h);
}

struct TreeFcBwdArgs {
  const float *dpool;
  const int *pair;
  const float *dret;
  const int *dret_rows;
  const float *h;   // [n, H] forward output of the round
  float *dz;        // [n, H]
  int n, H, act;
};

template <int W>
__global__ void treefc_round_bwd_kernel(TreeFcBwdArgs a) {
  const int H = a.H, hw = H / W;
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)a.n * hw) return;
  const int r = (int)(idx / hw), j = (int)(idx % hw) * W;
  const int src = a.pair[r];
  const int dr_row = a.dret_rows ? a.dret_rows[r] : r;
  float y[W], dm[W], dr[W], o[W];
  ldw<W>(a.h + (long)r * H + j, y);
  ldw<W>(a.dret + (long)dr_row * H + j, dr);
  if (src >= 0) ldw<W>(a.dpool + (long)src * H + j, dm);
#pragma unroll
  for (int k = 0; k < W; k++) {
    o[k] = treefc_dz((src >= 0 ? dm[k] : 0.f) + dr[k], y[k], a.act);
  }
  stw<W>(a.dz + (long)r * H + j, o);
}

// KERNEL<tile, wavefronts, exact, ...> for a round of n rows whose products run over K rows of a
// B matrix of BFLOATS floats
#define CAVS_LAUNCH_ROUND(KERNEL, a, n, H, K, BFLOATS, st, ...)                                                  \
  do {                                                                                                           \
    const RoundPlan p_ = plan_round(n, H);                                                                          \
    const dim3 grid_((H) / p_.tile, ((n) + p_.tile - 1) / p_.tile);                                              \
    const bool ex_ = chain_exact(K, p_.waves, BFLOATS);                                                          \
    if (p_.tile == 16 && p_.waves == 8) {                                                                        \
      if (ex_) launch(KERNEL<16, 8, true, ##__VA_ARGS__>, grid_, 512, 0, st, a);                                 \
      else launch(KERNEL<16, 8, false, ##__VA_ARGS__>, grid_, 512, 0, st, a);                                    \
    } else if (p_.tile == 16) {                                                                                  \
      if (ex_) launch(KERNEL<16, 4, true, ##__VA_ARGS__>, grid_, 256, 0, st, a);                                 \
      else launch(KERNEL<16, 4, false, ##__VA_ARGS__>, grid_, 256, 0, st, a);                                    \
    } else {                                                                                                     \
      launch(KERNEL<32, 8, false, ##__VA_ARGS__>, grid_, 512, 0, st, a);                                         \
    }                                                                                                            \
  } while (0)

template <typename A, typename K4, typename K1>
static void launch_pointwise(const A &a, int n, int H, bool vec, hipStream_t st, K4 k4, K1 k1) {
  if (vec) {
    long total = (long)n * (H / 4);
    launch(k4, (unsigned)((total + 255) / 256), 256, 0, st, a);
  } else {
    long total = (long)n * H;
    launch(k1, (unsigned)((total + 255) / 256), 256, 0, st, a);
  }
}

static bool all16(std::initializer_list<const void *> ps) {
  for (const void *p : ps)
    if (p && !aligned16(p)) return false;
  return true;
}

}  // namespace cavs

using namespace cavs;

extern "C" {

int cavs_lstm_round_fwd(float *pool, const int *child, const int *pair, const float *xW, int ld_xw, const float *Wh,
                        const float *bias, float *G, float *gates, float *msg, float *graph_out, const int *out_rows,
                        int n, int H, void *stream) {
  CAVS_REQUIRE(n >= 0 && round_shape_ok(H) && ld_xw >= 4 * H, "cavs_lstm_round_fwd: bad shape n=%d H=%d ld=%d (H must be a multiple of 32)", n, H, ld_xw);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(pool && child && pair && xW && Wh && bias && G && gates && msg, "cavs_lstm_round_fwd: null pointer");
  CAVS_REQUIRE(aligned16(pool), "cavs_lstm_round_fwd: pool must be 16-byte aligned");
  CAVS_REQUIRE(!graph_out || out_rows, "cavs_lstm_round_fwd: graph_out needs out_rows");
  LstmFwdArgs a{pool, child, pair, xW, ld_xw, Wh, bias, G, gates, msg, pool, graph_out, out_rows, n, H};
  CAVS_LAUNCH_ROUND(lstm_round_fwd_kernel, a, n, H, H, 4L * H * H, as_stream(stream));
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_lstm_round_packed_ok(int n, int H) {
  if (n < 0 || !round_shape_ok(H)) return 0;
  const RoundPlan p = plan_round(n > 0 ? n : 1, H);
  return p.tile == 16 && chain_exact(H, p.waves, 4L * H * H) ? 1 : 0;  // K = H forward; K = 4H backward follows
}

int cavs_lstm_round_fwd_packed(float *pool, const int *child, const int *pair, const float *xW, int ld_xw, const float *Whp,
                               const float *bias, float *G, float *gates, float *msg, float *graph_out, const int *out_rows,
                               int n, int H, void *stream) {
  CAVS_REQUIRE(n >= 0 && ld_xw >= 4 * H && cavs_lstm_round_packed_ok(n, H),
               "cavs_lstm_round_fwd_packed: bad shape n=%d H=%d ld=%d (see cavs_lstm_round_packed_ok)", n, H, ld_xw);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(pool && child && pair && xW && Whp && bias && G && gates && msg, "cavs_lstm_round_fwd_packed: null pointer");
  CAVS_REQUIRE(aligned16(pool) && aligned16(Whp), "cavs_lstm_round_fwd_packed: pool and Whp must be 16-byte aligned");
  CAVS_REQUIRE(!graph_out || out_rows, "cavs_lstm_round_fwd_packed: graph_out needs out_rows");
  LstmFwdArgs a{pool, child, pair, xW, ld_xw, Whp, bias, G, gates, msg, pool, graph_out, out_rows, n, H};
  const dim3 grid(H / 16, (n + 15) / 16);
  if (plan_round(n, H).waves == 8) launch(lstm_round_fwd_kernel<16, 8, true, true>, grid, 512, 0, as_stream(stream), a);
  else launch(lstm_round_fwd_kernel<16, 4, true, true>, grid, 256, 0, as_stream(stream), a);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_lstm_round_leaves_fwd(float *pool, const int *pair, const float *xW, int ld_xw, const float *bias, float *gates,
                               float *msg, float *graph_out, const int *out_rows, int n, int H, void *stream) {
  CAVS_REQUIRE(n >= 0 && H > 0 && ld_xw >= 4 * H, "cavs_lstm_round_leaves_fwd: bad shape n=%d H=%d ld=%d", n, H, ld_xw);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(pool && pair && xW && bias && gates && msg, "cavs_lstm_round_leaves_fwd: null pointer");
  CAVS_REQUIRE(!graph_out || out_rows, "cavs_lstm_round_leaves_fwd: graph_out needs out_rows");
  LstmLeavesArgs a{xW, ld_xw, bias, pair, gates, msg, pool, graph_out, out_rows, n, H};
  const bool vec = H % 4 == 0 && ld_xw % 4 == 0 && all16({pool, xW, bias, gates, msg, graph_out});
  launch_pointwise(a, n, H, vec, as_stream(stream), lstm_round_leaves_fwd_kernel<4>, lstm_round_leaves_fwd_kernel<1>);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_lstm_round_bwd_gates(float *dpool, const int *pair, const int *child, const float *dret, const int *dret_rows,
                              const float *gates, const float *G, float *da, int ld_da, int n, int H, void *stream) {
  CAVS_REQUIRE(n >= 0 && H > 0 && ld_da >= 4 * H, "cavs_lstm_round_bwd_gates: bad shape n=%d H=%d ld=%d", n, H, ld_da);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(dpool && pair && dret && gates && da, "cavs_lstm_round_bwd_gates: null pointer");
  CAVS_REQUIRE((child && G) || (!child && !G), "cavs_lstm_round_bwd_gates: child and G must be both set or both null");
  LstmBwdGatesArgs a{dpool, pair, child, dret, dret_rows, gates, G, da, ld_da, dpool, n, H};
  const bool vec = H % 4 == 0 && ld_da % 4 == 0 && all16({dpool, dret, gates, G, da});
  launch_pointwise(a, n, H, vec, as_stream(stream), lstm_round_bwd_gates_kernel<4>, lstm_round_bwd_gates_kernel<1>);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_round_bwd_children(const float *dA, int ld, int K, const float *BT, int ldb, int nchild, const int *child,
                            float *dpool, int pool_width, int n, int H, void *stream) {
  CAVS_REQUIRE(n >= 0 && round_shape_ok(H) && K > 0 && K % 4 == 0 && ld >= K && ld % 4 == 0 && pool_width >= H &&
                   (nchild == 1 || nchild == 2) && ldb >= nchild * H,
               "cavs_round_bwd_children: bad shape n=%d H=%d K=%d ld=%d ldb=%d nchild=%d pool_width=%d", n, H, K, ld, ldb, nchild, pool_width);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(dA && BT && child && dpool, "cavs_round_bwd_children: null pointer");
  CAVS_REQUIRE(aligned16(dA), "cavs_round_bwd_children: dA must be 16-byte aligned");
  ChildBwdArgs a{dA, ld, BT, ldb, child, dpool, pool_width, n, H, K, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0, 0};
  hipStream_t st = as_stream(stream);
  if (nchild == 1)
    CAVS_LAUNCH_ROUND(round_bwd_children_kernel, a, n, H, K, (long)K * ldb, st, 1, 0);
  else
    CAVS_LAUNCH_ROUND(round_bwd_children_kernel, a, n, H, K, (long)K * ldb, st, 2, 0);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_lstm_round_bwd_children_gates(float *da, int ld_da, float *dc, const float *WhT, const int *child_rows,
                                       const float *gates, const float *G, const float *dret, const int *dret_rows, int row0,
                                       int n, int leaf_rows, int H, void *stream) {
  CAVS_REQUIRE(n >= 0 && row0 >= 0 && leaf_rows >= 0 && round_shape_ok(H) && ld_da >= 4 * H && ld_da % 4 == 0,
               "cavs_lstm_round_bwd_children_gates: bad shape row0=%d n=%d leaf_rows=%d H=%d ld=%d (H must be a multiple of 32)", row0, n,
               leaf_rows, H, ld_da);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(da && dc && WhT && child_rows && gates && G && dret && dret_rows, "cavs_lstm_round_bwd_children_gates: null pointer");
  CAVS_REQUIRE(aligned16(da), "cavs_lstm_round_bwd_children_gates: da must be 16-byte aligned");
  ChildBwdArgs a{da + (long)row0 * ld_da, ld_da, WhT, H, child_rows, nullptr, 0, n, H, 4 * H, da, dc, gates, G, nullptr, dret, dret_rows, row0, leaf_rows, 0};
  CAVS_LAUNCH_ROUND(round_bwd_children_kernel, a, n, H, 4 * H, 4L * H * H, as_stream(stream), 1, 1);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_lstm_round_bwd_children_gates_packed(float *da, int ld_da, float *dc, const float *WhTp, const int *child_rows,
                                              const float *gates, const float *G, const float *dret, const int *dret_rows,
                                              int row0, int n, int leaf_rows, int H, void *stream) {
  CAVS_REQUIRE(n >= 0 && row0 >= 0 && leaf_rows >= 0 && ld_da >= 4 * H && ld_da % 4 == 0 && cavs_lstm_round_packed_ok(n, H),
               "cavs_lstm_round_bwd_children_gates_packed: bad shape row0=%d n=%d leaf_rows=%d H=%d ld=%d (see cavs_lstm_round_packed_ok)",
               row0, n, leaf_rows, H, ld_da);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(da && dc && WhTp && child_rows && gates && G && dret && dret_rows, "cavs_lstm_round_bwd_children_gates_packed: null pointer");
  CAVS_REQUIRE(aligned16(da) && aligned16(WhTp), "cavs_lstm_round_bwd_children_gates_packed: da and WhTp must be 16-byte aligned");
  ChildBwdArgs a{da + (long)row0 * ld_da, ld_da, WhTp, H, child_rows, nullptr, 0, n, H, 4 * H, da, dc, gates, G, nullptr, dret, dret_rows, row0, leaf_rows, 0};
  const dim3 grid(H / 16, (n + 15) / 16);
  if (plan_round(n, H).waves == 8) launch(round_bwd_children_kernel<16, 8, true, 1, 1, true>, grid, 512, 0, as_stream(stream), a);
  else launch(round_bwd_children_kernel<16, 4, true, 1, 1, true>, grid, 256, 0, as_stream(stream), a);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_lstm_bwd_gates_rows(const int *rows, int n, const float *dret, const int *dret_rows, const float *gates, const float *G,
                             float *da, int ld_da, float *dc, int leaf_rows, int H, void *stream) {
  CAVS_REQUIRE(n >= 0 && H > 0 && leaf_rows >= 0 && ld_da >= 4 * H, "cavs_lstm_bwd_gates_rows: bad shape n=%d H=%d ld=%d", n, H, ld_da);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(rows && dret && dret_rows && gates && G && da && dc, "cavs_lstm_bwd_gates_rows: null pointer");
  LstmBwdRowsArgs a{rows, dret, dret_rows, gates, G, da, ld_da, dc, n, H, leaf_rows};
  launch_pointwise(a, n, H, H % 4 == 0, as_stream(stream), lstm_bwd_gates_rows_kernel<4>, lstm_bwd_gates_rows_kernel<1>);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_treefc_round_bwd_children_act(float *dz, const float *WT, const int *child_rows, const float *h, const float *dret,
                                       const int *dret_rows, int row0, int n, int H, int act, void *stream) {
  CAVS_REQUIRE(n >= 0 && row0 >= 0 && round_shape_ok(H) && (act == 0 || act == 1),
               "cavs_treefc_round_bwd_children_act: bad argument row0=%d n=%d H=%d act=%d (H must be a multiple of 32)", row0, n, H, act);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(dz && WT && child_rows && h && dret && dret_rows, "cavs_treefc_round_bwd_children_act: null pointer");
  CAVS_REQUIRE(aligned16(dz), "cavs_treefc_round_bwd_children_act: dz must be 16-byte aligned");
  ChildBwdArgs a{dz + (long)row0 * H, H, WT, 2L * H, child_rows, nullptr, 0, n, H, H, dz, nullptr, nullptr, nullptr, h, dret, dret_rows, row0, 0, act};
  CAVS_LAUNCH_ROUND(round_bwd_children_kernel, a, n, H, H, 2L * H * H, as_stream(stream), 2, 2);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_treefc_bwd_rows(const int *rows, int n, const float *dret, const int *dret_rows, const float *h, float *dz, int H,
                         int act, void *stream) {
  CAVS_REQUIRE(n >= 0 && H > 0 && (act == 0 || act == 1), "cavs_treefc_bwd_rows: bad argument n=%d H=%d act=%d", n, H, act);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(rows && dret && dret_rows && h && dz, "cavs_treefc_bwd_rows: null pointer");
  TreeFcBwdRowsArgs a{rows, dret, dret_rows, h, dz, n, H, act};
  launch_pointwise(a, n, H, H % 4 == 0, as_stream(stream), treefc_bwd_rows_kernel<4>, treefc_bwd_rows_kernel<1>);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_treefc_round_fwd(float *pool, const int *child, const int *pair, const float *W, const float *bias,
                          const float *x, float *G, float *msg, float *graph_out, const int *out_rows, int n, int H,
                          int act, void *stream) {
  CAVS_REQUIRE(n >= 0 && round_shape_ok(H) && (act == 0 || act == 1), "cavs_treefc_round_fwd: bad argument n=%d H=%d act=%d (H must be a multiple of 32)", n, H, act);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(pool && child && pair && W && G && msg, "cavs_treefc_round_fwd: null pointer");
  CAVS_REQUIRE(aligned16(pool), "cavs_treefc_round_fwd: pool must be 16-byte aligned");
  CAVS_REQUIRE(!graph_out || out_rows, "cavs_treefc_round_fwd: graph_out needs out_rows");
  TreeFcFwdArgs a{pool, child, pair, W, bias, x, G, msg, pool, graph_out, out_rows, n, H, act};
  CAVS_LAUNCH_ROUND(treefc_round_fwd_kernel, a, n, H, H, 2L * H * H, as_stream(stream));
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_treefc_round_leaves_fwd(float *pool, const int *pair, const float *bias, const float *x, float *msg,
                                 float *graph_out, const int *out_rows, int n, int H, int act, void *stream) {
  CAVS_REQUIRE(n >= 0 && H > 0 && (act == 0 || act == 1), "cavs_treefc_round_leaves_fwd: bad argument n=%d H=%d act=%d", n, H, act);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(pool && pair && msg, "cavs_treefc_round_leaves_fwd: null pointer");
  CAVS_REQUIRE(!graph_out || out_rows, "cavs_treefc_round_leaves_fwd: graph_out needs out_rows");
  TreeFcLeavesArgs a{bias, x, pair, msg, pool, graph_out, out_rows, n, H, act};
  const bool vec = H % 4 == 0 && all16({pool, bias, x, msg, graph_out});
  launch_pointwise(a, n, H, vec, as_stream(stream), treefc_round_leaves_fwd_kernel<4>, treefc_round_leaves_fwd_kernel<1>);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_treefc_round_bwd(const float *dpool, const int *pair, const float *dret, const int *dret_rows, const float *h,
                          float *dz, int n, int H, int act, void *stream) {
  CAVS_REQUIRE(n >= 0 && H > 0 && (act == 0 || act == 1), "cavs_treefc_round_bwd: bad argument n=%d H=%d act=%d", n, H, act);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(dpool && pair && dret && h && dz, "cavs_treefc_round_bwd: null pointer");
  TreeFcBwdArgs a{dpool, pair, dret, dret_rows, h, dz, n, H, act};
  const bool vec = H % 4 == 0 && all16({dpool, dret, h, dz});
  launch_pointwise(a, n, H, vec, as_stream(stream), treefc_round_bwd_kernel<4>, treefc_round_bwd_kernel<1>);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

}  // extern "C"
