// One round of the Tree-LSTM vertex function in one launch (forward) or two (backward).
//
// A round of n vertices is n rows times five products against slices of the recurrent
// weights (h_l+h_r with the i, o, u blocks of U_iou; h_l and h_r with U_f), the gate
// arithmetic, and row movement through the child and scatter lists.  As separate kernels
// that is a chain of five launches whose intermediates make a round trip through HBM; for
// the rounds of a batch of parse trees (a few hundred rows down to one) the chain is
// bound by launch latency, not by the matrix cores.  Here one workgroup owns a
// (RT*TILE rows) x (TILE columns of H) piece of the round's output:
//   * its eight wavefronts split the K range of the products between them and feed the
//     MFMA straight from global memory -- the A operand rows are read through the child
//     list (the gather is the operand fetch), B is TILE consecutive floats per k, so
//     neither needs staging through LDS;
//   * the five partial tiles are summed through LDS in wavefront order (deterministic),
//     which leaves all five pre-activations of an output element in one thread;
//   * the epilogue applies the gates and writes the message into the pool row named by
//     the scatter list, plus everything the backward pass reads again (gates, gathered
//     children, h_l+h_r).
// TILE is 32 (v_mfma_f32_32x32x2_f32) or, for rounds of a few rows near the roots, 16
// (v_mfma_f32_16x16x4_f32), which spreads a tiny round over four times as many CUs.
#include <type_traits>

#include "round_common.h"

namespace cavs {

// ------------------------------------------------------------------ forward
struct RoundFwdArgs {
  const float *pool;   // [*, 2H] message pool, rows [h|c]
  const int *child;    // [2n] pool rows of the children of slab row b at 2b, 2b+1 (-1: none)
  const int *pair;     // [n] pool row the message of slab row b goes to (-1: nowhere)
  const float *xW;     // [n, 4H] (ld_xw) blocks [i|o|u|f]
  long ld_xw;
  const float *U;      // [H, 3H] blocks [i|o|u], then [H, H] (forget gate)
  const float *Upk;    // PACKED: the same two matrices tile-major (a CAVS_TASK_SGD_PACK job writes them)
  const float *bias;   // [4H] blocks [i|f|u|o]
  float *G;            // [2n, 2H] gathered children (saved for backward)
  float *hlr;          // [n, H] h_l + h_r (saved for the weight gradient)
  float *gates;        // [n, 6H]
  float *msg;          // [n, 2H]
  float *pool_out;     // same buffer as pool: rows of this round are written, rows of earlier rounds read
  float *go;           // [*, H] or nullptr: the pushed return value h of slab row b goes to row out_rows[b]
  const int *out_rows; // [n] (FunctionPopRet folded in)
  int n, H;
};

// EXACT: H splits into an even number of whole pipeline stages for every wavefront.  The product
// loop then has no ragged end and no conditions: the weights come through buffer loads whose
// address is a descriptor of U in scalar registers, a scalar offset that advances with k and a
// per-lane offset fixed before the loop (no address arithmetic on the vector ALU, whose 64-bit
// row * stride products otherwise cost as much time as the MFMAs), the rows of A through
// per-lane pointers that are bumped once per k-group, and the wait counts of the two stage
// buffers come out exact, so the loads of one stage are in flight under the MFMAs of the other.
// PACKED: the loop reads the weights from the tile-major copy, one float4 per lane, gate and
// k-group -- a wavefront's fragment is one contiguous kilobyte instead of four 64-byte pieces per
// dword load (the texture-address unit charges per piece).
// ROWS4 (with PACKED): tiles of four rows by sixteen columns on the 4x4x1 MFMA shape -- a round of
// a few rows spends a quarter of the matrix-pipe time per tile and spreads over four times as
// many CUs.
template <int TILE, int WAVES, bool EXACT, bool PACKED = false, bool ROWS4 = false>
__global__ __launch_bounds__(WAVES * 64, (TILE == 16 && WAVES == 4) ? 4 : 1) void treelstm_round_fwd_kernel(RoundFwdArgs a) {
  static_assert(!PACKED || (EXACT && TILE == 16), "the packed layout is for the exact loops over 16x16 tiles");
  static_assert(!ROWS4 || PACKED, "the four-row tiles read packed weights");
  using M = std::conditional_t<ROWS4, Mma4, Mma<TILE>>;
  constexpr int TR = ROWS4 ? 4 : TILE;  // rows of a tile
  using Acc = typename M::Acc;
  constexpr int RT = 1, kRoundThreads = WAVES * 64;
  constexpr int KS = WAVES / RT, GK = 4 * M::NSLOT, NP = 5, NR = M::NR;
  // k-groups per pipeline stage; the four-wavefront 16x16 variant keeps one, to stay within the
  // registers of four workgroups per CU
  constexpr int UG = (TILE == 16 && WAVES == 4) ? 1 : 2;
  constexpr int NREG = Regions<TILE, KS>::N, RSZ = RT * NP * NR * 64;
  __shared__ float red[NREG * RSZ];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rt = wave / KS, ks = wave % KS;
  const int x = lane & (TILE - 1), slot = lane / TILE;
  const int xr = x & (TR - 1);  // tile row of this lane's A operand
  const int H = a.H;
  const long H2 = 2L * H, H3 = 3L * H;
  const int j0 = blockIdx.x * TILE;
  const int row = (blockIdx.y * RT + rt) * TR + xr;
  const int kper = ((H + KS - 1) / KS + GK - 1) / GK * GK;
  const int kb = ks * kper, ke = min(H, kb + kper);
  const float *Uio = a.U + j0 + x, *Uf = a.U + H3 * H + j0 + x;

  // Issue order of the prologue: (1) every row id this thread needs, (2) what does not depend
  // on them -- the first B fragments and the x*W / bias operands of the epilogue -- so that it
  // travels while the ids do, (3) the rows the ids name.
  int cl = -1, cr = -1;
  if (row < a.n) {
    cl = a.child[2 * row];
    cr = a.child[2 * row + 1];
  }
  // PACKED: A is read a quad of lanes per row piece (lane l: tile row l / 4, k = 4 * (l % 4); see
  // exact_products) and crosses to the MFMA's lanes just before use
  constexpr bool QUAD = PACKED;
  const int from4 = 4 * (4 * xr + slot);
  // (the child ids of tile row l / 4 are with lane l / 4, whose x is that row: no second fetch)
  int qcl = -1, qcr = -1;
  if constexpr (QUAD) {
    qcl = __builtin_amdgcn_ds_bpermute(4 * ((lane >> 2) & (TR - 1)), cl);
    qcr = __builtin_amdgcn_ds_bpermute(4 * ((lane >> 2) & (TR - 1)), cr);
  }
  constexpr int EPT = (RT * NR * 64 + kRoundThreads - 1) / kRoundThreads;
  struct Epi {
    bool on;
    int b, j, dst, lds, c_l, c_r, out;
    float xw[4], bias[4], hl, cl, hr, cr;
  } epi[EPT];
#pragma unroll
  for (int q = 0; q < EPT; q++) {
    Epi &ep = epi[q];
    const int e = tid + q * kRoundThreads;
    const int l2 = e & 63, r = (e >> 6) % NR, t = e / (64 * NR);
    ep.b = (blockIdx.y * RT + t) * TILE + M::row(r, l2);
    ep.j = j0 + (l2 & (TILE - 1));
    ep.lds = (t * NP * NR + r) * 64 + l2;
    ep.on = e < RT * NR * 64 && ep.b < a.n;
    if constexpr (ROWS4) {  // sixty-four elements: row e / 16, column e % 16, four k slots each
      ep.b = blockIdx.y * TR + (e >> 4);
      ep.j = j0 + (e & 15);
      ep.lds = (e >> 4) * 64 + (e & 15);
      ep.on = e < TR * 16 && ep.b < a.n;
    }
    ep.c_l = ep.c_r = ep.dst = ep.out = -1;
    if (ep.on) {
      ep.c_l = a.child[2 * ep.b];
      ep.c_r = a.child[2 * ep.b + 1];
      ep.dst = a.pair[ep.b];
      if (a.go) ep.out = a.out_rows[ep.b];
    }
  }

  Acc acc[NP];
#pragma unroll
  for (int p = 0; p < NP; p++)
#pragma unroll
    for (int r = 0; r < NR; r++) acc[p][r] = 0.f;

  struct Frag {
    float4 hl[UG], hr[UG];
    float b[UG][4][4];
  };
  auto fetch_b = [&](int k0, Frag &f) {
#pragma unroll
    for (int u = 0; u < UG; u++) {
      const int kk = k0 + GK * u + 4 * slot;
      const bool kin = kk < ke;  // H is a multiple of 4: a group of 4 k is wholly in or out
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const float *ui = Uio + (long)(kin ? kk + c : 0) * H3;
        f.b[u][0][c] = kin ? ui[0] : 0.f;
        f.b[u][1][c] = kin ? ui[H] : 0.f;
        f.b[u][2][c] = kin ? ui[2 * H] : 0.f;
        f.b[u][3][c] = kin ? Uf[(long)(kk + c) * H] : 0.f;
      }
    }
  };
  const float *pl = nullptr, *pr = nullptr;
  auto fetch_a = [&](int k0, Frag &f) {
#pragma unroll
    for (int u = 0; u < UG; u++) {
      const int kk = k0 + GK * u + 4 * slot;
      const bool kin = kk < ke;
      f.hl[u] = (kin && cl >= 0) ? ld4(pl + kk) : zero4();
      f.hr[u] = (kin && cr >= 0) ? ld4(pr + kk) : zero4();
    }
  };
  auto fetch = [&](int k0, Frag &f) {
    fetch_b(k0, f);
    fetch_a(k0, f);
  };
  auto multiply = [&](const Frag &f) {
#pragma unroll
    for (int u = 0; u < UG; u++)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const float hl = elem(f.hl[u], c), hr = elem(f.hr[u], c), hs = hl + hr;
        acc[0] = M::mma(hs, f.b[u][0][c], acc[0]);
        acc[1] = M::mma(hs, f.b[u][1][c], acc[1]);
        acc[2] = M::mma(hs, f.b[u][2][c], acc[2]);
        acc[3] = M::mma(hl, f.b[u][3][c], acc[3]);
        acc[4] = M::mma(hr, f.b[u][3][c], acc[4]);
      }
  };
  Frag f0, f1;
  constexpr int S = GK * UG;
  // EXACT: a missing child (no message to gather) is masked where the operand is used
  const bool has_l = cl >= 0, has_r = cr >= 0;
  auto xmultiply = [&](const Frag &f) {
#pragma unroll
    for (int u = 0; u < UG; u++)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        float hl = elem(f.hl[u], c), hr = elem(f.hr[u], c);
        if constexpr (QUAD) {
          hl = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(from4, __builtin_bit_cast(int, hl)));
          hr = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(from4, __builtin_bit_cast(int, hr)));
        }
        hl = has_l ? hl : 0.f;
        hr = has_r ? hr : 0.f;
        const float hs = hl + hr;
        acc[0] = M::mma(hs, f.b[u][0][c], acc[0]);
        acc[1] = M::mma(hs, f.b[u][1][c], acc[1]);
        acc[2] = M::mma(hs, f.b[u][2][c], acc[2]);
        acc[3] = M::mma(hl, f.b[u][3][c], acc[3]);
        acc[4] = M::mma(hr, f.b[u][3][c], acc[4]);
      }
  };
  // PACKED: float4 (slot, x) of tile (k-group, column tile); gates i, o, u are column tiles
  // H/16 apart in the [H, 3H] matrix's packing, the forget gate's matrix follows it
  const float4 *pio = reinterpret_cast<const float4 *>(a.Upk) + ((long)(kb / GK) * (3 * H / 16) + blockIdx.x) * 64 + slot * 16 + x;
  const float4 *pf = reinterpret_cast<const float4 *>(a.Upk) + 3L * H * H / 4 + ((long)(kb / GK) * (H / 16) + blockIdx.x) * 64 + slot * 16 + x;
  const int gate4 = H * 4;  // float4 between the gates' column tiles
  auto pfetch_b = [&](Frag &f) {  // a stage's weights from the packed copy; moves on to the next stage
#pragma unroll
    for (int u = 0; u < UG; u++) {
      const float4 bi = pio[0], bo = pio[gate4], bu = pio[2 * gate4], bf = *pf;
#pragma unroll
      for (int c = 0; c < 4; c++) {
        f.b[u][0][c] = elem(bi, c);
        f.b[u][1][c] = elem(bo, c);
        f.b[u][2][c] = elem(bu, c);
        f.b[u][3][c] = elem(bf, c);
      }
      pio += 3 * gate4;
      pf += gate4;
    }
  };
  if constexpr (PACKED) {
    pfetch_b(f0);
  } else {
    if (kb < ke) fetch_b(kb, f0);
  }
#pragma unroll
  for (int q = 0; q < EPT; q++) {
    Epi &ep = epi[q];
    if (!ep.on) continue;
    const float *xw = a.xW + ep.b * a.ld_xw + ep.j;
#pragma unroll
    for (int k = 0; k < 4; k++) { ep.xw[k] = xw[k * H]; ep.bias[k] = a.bias[k * H + ep.j]; }
  }
  if constexpr (QUAD) {  // a missing child reads row 0 and is masked where the operand is used
    pl = a.pool + (qcl >= 0 ? qcl : 0) * H2 + 4 * (lane & 3) - 4 * slot;
    pr = a.pool + (qcr >= 0 ? qcr : 0) * H2 + 4 * (lane & 3) - 4 * slot;
#pragma unroll
    for (int u = 0; u < UG; u++) {
      f0.hl[u] = ld4(pl + kb + GK * u + 4 * slot);
      f0.hr[u] = ld4(pr + kb + GK * u + 4 * slot);
    }
  } else {
    pl = a.pool + (cl >= 0 ? cl : 0) * H2;
    pr = a.pool + (cr >= 0 ? cr : 0) * H2;
    if (kb < ke) fetch_a(kb, f0);
  }
#pragma unroll
  for (int q = 0; q < EPT; q++) {
    Epi &ep = epi[q];
    ep.hl = ep.cl = ep.hr = ep.cr = 0.f;
    if (ep.c_l >= 0) { ep.hl = a.pool[ep.c_l * H2 + ep.j]; ep.cl = a.pool[ep.c_l * H2 + H + ep.j]; }
    if (ep.c_r >= 0) { ep.hr = a.pool[ep.c_r * H2 + ep.j]; ep.cr = a.pool[ep.c_r * H2 + H + ep.j]; }
  }

  if constexpr (EXACT) {
    const __amdgpu_buffer_rsrc_t ubuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(a.U), 0, 4 * H * H * 4, 0x00020000);
    int vio[4], vf[4];  // byte offsets of this lane's column in row 4 * slot + c of a k-group
#pragma unroll
    for (int c = 0; c < 4; c++) {
      vio[c] = ((4 * slot + c) * 3 * H + j0 + x) * 4;
      vf[c] = ((4 * slot + c) * H + j0 + x) * 4;
    }
    const int kbu = __builtin_amdgcn_readfirstlane(kb), nst = __builtin_amdgcn_readfirstlane((ke - kb) / S);
    int sio = (kbu + S) * 3 * H * 4, sf = (3 * H * H + (kbu + S) * H) * 4;  // scalar byte offsets of the next k-group
    const float *al = pl + kb + S + 4 * slot, *ar = pr + kb + S + 4 * slot;
    auto xfetch = [&](Frag &f) {
      if constexpr (PACKED) pfetch_b(f);
#pragma unroll
      for (int u = 0; u < UG; u++) {
        if constexpr (!PACKED) {
#pragma unroll
          for (int c = 0; c < 4; c++) {
            f.b[u][0][c] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(ubuf, vio[c], sio, 0));
            f.b[u][1][c] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(ubuf, vio[c], sio + H * 4, 0));
            f.b[u][2][c] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(ubuf, vio[c], sio + H * 8, 0));
            f.b[u][3][c] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(ubuf, vf[c], sf, 0));
          }
          sio += GK * 3 * H * 4;
          sf += GK * H * 4;
        }
        f.hl[u] = ld4(al);
        f.hr[u] = ld4(ar);
        al += GK;
        ar += GK;
      }
    };
    // (the first stage was fetched above through the general path; nst is even)
    // (the scheduler barriers keep a stage's loads ahead of the other stage's MFMAs; left alone,
    // the compiler sinks every load to just before its use)
    for (int st = 0; st + 2 < nst; st += 2) {
      xfetch(f1);
      __builtin_amdgcn_sched_barrier(0);
      xmultiply(f0);
      __builtin_amdgcn_sched_barrier(0);
      xfetch(f0);
      __builtin_amdgcn_sched_barrier(0);
      xmultiply(f1);
      __builtin_amdgcn_sched_barrier(0);
    }
    xfetch(f1);
    __builtin_amdgcn_sched_barrier(0);
    xmultiply(f0);
    xmultiply(f1);
  } else {
    for (int k0 = kb; k0 < ke; k0 += 2 * S) {
      if (k0 + S < ke) fetch(k0 + S, f1);
      multiply(f0);
      if (k0 + S < ke) {
        if (k0 + 2 * S < ke) fetch(k0 + 2 * S, f0);
        multiply(f1);
      }
    }
  }

  park_partials<TILE, NP, KS, NREG, RT>(red, acc, rt, ks, lane);

  // epilogue: element (t, r, l2) of the workgroup's tiles is slab row b, column j; its
  // operands were fetched before the products started
#pragma unroll
  for (int q = 0; q < EPT; q++) {
    const Epi &ep = epi[q];
    if (!ep.on) continue;
    const float *pre = red + ep.lds;
    float v[NP];
#pragma unroll
    for (int p = 0; p < NP; p++) {
      float s;
      if constexpr (ROWS4) {
        s = 0.f;
#pragma unroll
        for (int g = 0; g < NREG; g++)
          s += (pre[g * RSZ + p * NR * 64] + pre[g * RSZ + p * NR * 64 + 16]) +
               (pre[g * RSZ + p * NR * 64 + 32] + pre[g * RSZ + p * NR * 64 + 48]);
      } else {
        s = pre[p * NR * 64];
#pragma unroll
        for (int g = 1; g < NREG; g++) s += pre[g * RSZ + p * NR * 64];
      }
      v[p] = s;
    }
    const int b = ep.b, j = ep.j;
    const TreeLstmCell q_ = treelstm_cell(ep.xw, v, ep.bias, ep.cl, ep.cr);
    const float i = q_.i, o = q_.o, u = q_.u, f_l = q_.f_l, f_r = q_.f_r, c = q_.c, tc = q_.tc, h = q_.h;
    float *g = a.gates + (long)b * 6 * H + j;
    g[0] = i; g[H] = o; g[2 * H] = u; g[3 * H] = f_l; g[4 * H] = f_r; g[5 * H] = tc;
    if (a.msg) {
      float *m = a.msg + b * H2 + j;
      m[0] = h; m[H] = c;
    }
    if (ep.dst >= 0) {
      a.pool_out[ep.dst * H2 + j] = h;
      a.pool_out[ep.dst * H2 + H + j] = c;
    }
    if (ep.out >= 0) a.go[(long)ep.out * H + j] = h;
    float *gl = a.G + (2L * b) * H2 + j, *gr = gl + H2;
    gl[0] = ep.hl; gl[H] = ep.cl; gr[0] = ep.hr; gr[H] = ep.cr;
    a.hlr[(long)b * H + j] = ep.hl + ep.hr;
  }
}

// ------------------------------------------------------------------ forward, a round of leaves
// No children: the gates of x*W + bias only, the message written to the pool row the scatter
// list names and the return value to its output row.
struct RoundLeavesArgs {
  const float *xW;
  long ld_xw;
  const float *bias;
  const int *pair;
  float *gates, *msg, *pool, *go;
  const int *out_rows;
  int n, H;
};

template <int W>
__global__ void treelstm_round_leaves_fwd_kernel(RoundLeavesArgs a) {
  const int H = a.H, hw = H / W;
  const long H2 = 2L * H;
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)a.n * hw) return;
  const int r = (int)(idx / hw), j = (int)(idx % hw) * W;
  const int dst = a.pair[r], out = a.go ? a.out_rows[r] : -1;
  const float *xw = a.xW + r * a.ld_xw + j;
  float gi[W], go[W], gu[W], gf[W], gtc[W], mh[W], mc[W];
#pragma unroll
  for (int k = 0; k < W; k++) {
    // same association as with children: (x*W + 0) + bias
    const float i = sigm_r((xw[k] + 0.f) + a.bias[j + k]);
    const float o = sigm_r((xw[H + k] + 0.f) + a.bias[3 * H + j + k]);
    const float u = tanh_r((xw[2 * H + k] + 0.f) + a.bias[2 * H + j + k]);
    const float f = sigm_r((xw[3 * H + k] + 0.f) + a.bias[H + j + k]);
    const float c = (i * u + f * 0.f) + f * 0.f;
    const float tc = tanh_r(c);
    gi[k] = i; go[k] = o; gu[k] = u; gf[k] = f; gtc[k] = tc; mh[k] = o * tc; mc[k] = c;
  }
  auto st = [](float *p, const float (&v)[W]) {
    if constexpr (W == 4) {
      *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
#pragma unroll
      for (int k = 0; k < W; k++) p[k] = v[k];
    }
  };
  float *g = a.gates + (long)r * 6 * H + j;
  st(g, gi); st(g + H, go); st(g + 2 * H, gu); st(g + 3 * H, gf); st(g + 4 * H, gf); st(g + 5 * H, gtc);
  if (a.msg) {
    float *m = a.msg + r * H2 + j;
    st(m, mh); st(m + H, mc);
  }
  if (dst >= 0) { st(a.pool + dst * H2 + j, mh); st(a.pool + dst * H2 + H + j, mc); }
  if (out >= 0) st(a.go + (long)out * H + j, mh);
}

// ------------------------------------------------------------------ backward, gate part
// Elementwise: reads the message gradient through the scatter list (grad of Scatter is
// Gather), writes the pre-activation gradients and the c half of the children's message
// gradients straight into the children's pool rows (grad of Gather is Scatter).
struct RoundBwdGatesArgs {
  const float *dpool;   // [*, 2H] gradient of the message pool
  const int *pair;      // [n]
  const int *child;     // [2n] or nullptr for a round of leaves
  const float *dret;    // gradient of the pushed return value: row b, or row dret_rows[b] if given
  const int *dret_rows; // [n] or nullptr (grad of FunctionPopRet folded in)
  const float *gates;   // [n, 6H]
  const float *G;       // [2n, 2H] or nullptr for leaves
  float *dxW;           // [n, 4H] (ld_dxw) blocks [i|o|u|f_l+f_r]
  long ld_dxw;
  float *dF;            // [2n, H] rows (2b: f_l, 2b+1: f_r) or nullptr
  float *dpool_out;     // same buffer as dpool
  int n, H;
};

template <int W>
__global__ void treelstm_round_bwd_gates_kernel(RoundBwdGatesArgs a) {
  const int H = a.H, hw = H / W;
  const long H2 = 2L * H;
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)a.n * hw) return;
  const int r = (int)(idx / hw), j = (int)(idx % hw) * W;
  const int src = a.pair[r];
  const int dr_row = a.dret_rows ? a.dret_rows[r] : r;
  const float *g = a.gates + (long)r * 6 * H + j;
  const bool internal = a.child != nullptr;
  int c_l = -1, c_r = -1;
  if (internal) { c_l = a.child[2 * r]; c_r = a.child[2 * r + 1]; }
  float dmh[W], dmc[W], dr[W], gi[W], go[W], gu[W], gfl[W], gfr[W], gtc[W], cl[W], cr[W];
  if constexpr (W == 4) {
    auto ld = [](const float *p, float (&o)[W]) { float4 v = ld4(p); o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w; };
    ld(g, gi); ld(g + H, go); ld(g + 2 * H, gu); ld(g + 3 * H, gfl); ld(g + 4 * H, gfr); ld(g + 5 * H, gtc);
    ld(a.dret + (long)dr_row * H + j, dr);
    if (src >= 0) { ld(a.dpool + src * H2 + j, dmh); ld(a.dpool + src * H2 + H + j, dmc); }
    if (internal) { ld(a.G + (2L * r) * H2 + H + j, cl); ld(a.G + (2L * r + 1) * H2 + H + j, cr); }
  } else {
#pragma unroll
    for (int k = 0; k < W; k++) {
      gi[k] = g[k]; go[k] = g[H + k]; gu[k] = g[2 * H + k]; gfl[k] = g[3 * H + k]; gfr[k] = g[4 * H + k]; gtc[k] = g[5 * H + k];
      dr[k] = a.dret[(long)dr_row * H + j + k];
      if (src >= 0) { dmh[k] = a.dpool[src * H2 + j + k]; dmc[k] = a.dpool[src * H2 + H + j + k]; }
      if (internal) { cl[k] = a.G[(2L * r) * H2 + H + j + k]; cr[k] = a.G[(2L * r + 1) * H2 + H + j + k]; }
    }
  }
  float di[W], dvo[W], du[W], dfs[W], dfl[W], dfr[W], dcl[W], dcr[W];
#pragma unroll
  for (int k = 0; k < W; k++) {
    const float mh = src >= 0 ? dmh[k] : 0.f, mc = src >= 0 ? dmc[k] : 0.f;
    const float c_left = internal ? cl[k] : 0.f, c_right = internal ? cr[k] : 0.f;
    const GateGrad q = gate_grad(gi[k], go[k], gu[k], gfl[k], gfr[k], gtc[k], mh, mc, dr[k], c_left, c_right);
    di[k] = q.di; dvo[k] = q.d_o; du[k] = q.du;
    dfs[k] = q.dfl + q.dfr;
    dfl[k] = q.dfl; dfr[k] = q.dfr;
    dcl[k] = q.dc * gfl[k]; dcr[k] = q.dc * gfr[k];
  }
  auto st = [](float *p, const float (&v)[W]) {
    if constexpr (W == 4) {
      *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
#pragma unroll
      for (int k = 0; k < W; k++) p[k] = v[k];
    }
  };
  float *dx = a.dxW + r * a.ld_dxw + j;
  st(dx, di); st(dx + H, dvo); st(dx + 2 * H, du); st(dx + 3 * H, dfs);
  if (internal) {
    st(a.dF + (2L * r) * H + j, dfl);
    st(a.dF + (2L * r + 1) * H + j, dfr);
    if (c_l >= 0) st(a.dpool_out + c_l * H2 + H + j, dcl);
    if (c_r >= 0) st(a.dpool_out + c_r * H2 + H + j, dcr);
  }
}

// The same for the vertices nobody sends a message gradient to (the roots): BwdGatesRowsArgs and
// treelstm_gates_rows_at (shared with the job form of cavs_run_tasks) are in round_common.h.
template <int W>
__global__ void treelstm_bwd_gates_rows_kernel(BwdGatesRowsArgs a) {
  treelstm_gates_rows_at<W>(a, (long)blockIdx.x * blockDim.x + threadIdx.x);
}

// ------------------------------------------------------------------ backward, children part
// dh_l = [d_i|d_o|d_u] * U_iou^T + d_fl * U_f^T, dh_r likewise with d_fr, written into the h
// half of the children's pool-gradient rows.  UT holds the transposed weights ([3H,H] then
// [H,H]) so that the B operand is TILE consecutive floats per k, as in the forward kernel.
//
// FOLD: the launch also does the gate part of the children.  `child` then names the children
// by slab row over whole-batch slabs; the thread that holds d h of hidden unit j of a child has
// everything the child's gate gradients of that unit need (its saved gates, its d return value,
// d c = d c(parent) * f(parent)), so it writes the child's rows of dxW / dF / dc directly and
// the message gradient never makes the trip through the pool.  What it needs besides the
// products is fetched while they run.
struct RoundBwdChildArgs {
  const float *dxW;   // [n, 4H] (ld_dxw); columns [0, 3H) are read
  long ld_dxw;
  const float *dF;    // [2n, H]
  const float *UT;    // [3H, H] = U_iou^T, then [H, H] = U_f^T
  const int *child;   // [2n]
  float *dpool;       // [*, 2H]
  int n, H;
  // FOLD only; whole-batch slabs, the round starts at slab row row0
  float *dxW_all, *dF_all, *dc_all;
  const float *gates_all, *G_all, *dret;
  const int *dret_rows;
  int row0, leaf_rows;
};

// PACKED (with EXACT, 16x16 tiles): UT is in the tile-major layout of CAVS_TASK_PACK_T.
// ROWS4 (with FOLD, EXACT, PACKED): tiles of four rows on the 4x4x1 shape, as in the forward kernel.
template <int TILE, int WAVES, bool FOLD, bool EXACT, bool PACKED = false, bool ROWS4 = false>
__global__ __launch_bounds__(WAVES * 64, (TILE == 16 && WAVES == 4) ? 4 : 1) void treelstm_round_bwd_children_kernel(RoundBwdChildArgs a) {
  static_assert(!ROWS4 || (FOLD && EXACT && PACKED), "the four-row tiles are for the folded packed launches");
  using M = std::conditional_t<ROWS4, Mma4, Mma<TILE>>;
  constexpr int TR = ROWS4 ? 4 : TILE;  // rows of a tile
  using Acc = typename M::Acc;
  constexpr int RT = 1, kRoundThreads = WAVES * 64;
  constexpr int KS = WAVES / RT, GK = 4 * M::NSLOT, NP = 3, NR = M::NR;
  constexpr int UG = (TILE == 16 && WAVES == 4) ? 1 : 2;
  constexpr int NREG = Regions<TILE, KS>::N, RSZ = RT * NP * NR * 64;
  __shared__ float red[NREG * RSZ];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rt = wave / KS, ks = wave % KS;
  const int x = lane & (TILE - 1), slot = lane / TILE;
  const int H = a.H;
  const long H2 = 2L * H;
  const int j0 = blockIdx.x * TILE;
  const int row = (blockIdx.y * RT + rt) * TR + (x & (TR - 1));
  const bool rin = row < a.n;
  // QUAD: the exact packed loops read A a quad of lanes per row piece (see exact_products)
  constexpr bool QUAD = EXACT && PACKED;
  const int arow_ = QUAD ? (blockIdx.y * RT + rt) * TR + ((lane >> 2) & (TR - 1)) : row, aslot = QUAD ? (lane & 3) : slot;
  const bool ain = arow_ < a.n;
  const float *px = a.dxW + (ain ? arow_ : 0) * a.ld_dxw;
  const float *pfl = a.dF + (ain ? 2L * arow_ : 0) * H, *pfr = pfl + (ain ? H : 0);
  const float *UTio = a.UT + j0 + x, *UTf = a.UT + 3L * H * H + j0 + x;

  // the epilogue's targets, fetched now: child rows of the elements this thread will write
  constexpr int EPT = (RT * NR * 64 + kRoundThreads - 1) / kRoundThreads;
  bool eon[EPT];
  int ecl[EPT], ecr[EPT], ej[EPT], elds[EPT], eb[EPT];
#pragma unroll
  for (int q = 0; q < EPT; q++) {
    const int e = tid + q * kRoundThreads;
    const int l2 = e & 63, r = (e >> 6) % NR, t = e / (64 * NR);
    int b = (blockIdx.y * RT + t) * TILE + M::row(r, l2);
    ej[q] = j0 + (l2 & (TILE - 1));
    elds[q] = (t * NP * NR + r) * 64 + l2;
    eon[q] = e < RT * NR * 64 && b < a.n;
    if constexpr (ROWS4) {  // sixty-four elements: row e / 16, column e % 16, four k slots each
      b = blockIdx.y * TR + (e >> 4);
      ej[q] = j0 + (e & 15);
      elds[q] = (e >> 4) * 64 + (e & 15);
      eon[q] = e < TR * 16 && b < a.n;
    }
    ecl[q] = ecr[q] = -1;
    if (eon[q]) {
      ecl[q] = a.child[2 * b];
      ecr[q] = a.child[2 * b + 1];
    }
    if constexpr (FOLD) eb[q] = b;
  }
  // FOLD: operands of the children's gate gradients ([q][side])
  struct Kid {
    float g[6], dr, cl, cr;
  };
  Kid kid[FOLD ? EPT : 1][2];
  float pdc[FOLD ? EPT : 1], pf[FOLD ? EPT : 1][2];
  int kdr[FOLD ? EPT : 1][2];
  if constexpr (FOLD) {
#pragma unroll
    for (int q = 0; q < EPT; q++) {
      kdr[q][0] = ecl[q] >= 0 ? a.dret_rows[ecl[q]] : 0;
      kdr[q][1] = ecr[q] >= 0 ? a.dret_rows[ecr[q]] : 0;
    }
  }
  auto fetch_kids = [&]() {
    if constexpr (FOLD) {
#pragma unroll
      for (int q = 0; q < EPT; q++) {
        const int j = ej[q];
        const long b = a.row0 + eb[q];
        pdc[q] = pf[q][0] = pf[q][1] = 0.f;
        if (eon[q]) {
          pdc[q] = a.dc_all[b * H + j];
          pf[q][0] = a.gates_all[b * 6 * H + 3 * H + j];
          pf[q][1] = a.gates_all[b * 6 * H + 4 * H + j];
        }
#pragma unroll
        for (int s = 0; s < 2; s++) {
          const long v = s ? ecr[q] : ecl[q];
          Kid &kd = kid[q][s];
#pragma unroll
          for (int t = 0; t < 6; t++) kd.g[t] = 0.f;
          kd.dr = kd.cl = kd.cr = 0.f;
          if (v >= 0) {
            const float *g = a.gates_all + v * 6 * H + j;
#pragma unroll
            for (int t = 0; t < 6; t++) kd.g[t] = g[(long)t * H];
            kd.dr = a.dret[(long)kdr[q][s] * H + j];
            if (v >= a.leaf_rows) {
              kd.cl = a.G_all[(2 * v) * H2 + H + j];
              kd.cr = a.G_all[(2 * v + 1) * H2 + H + j];
            }
          }
        }
      }
    }
  };

  Acc acc[NP];
#pragma unroll
  for (int p = 0; p < NP; p++)
#pragma unroll
    for (int r = 0; r < NR; r++) acc[p][r] = 0.f;

  constexpr int S = GK * UG;
  if constexpr (EXACT) {
    const __amdgpu_buffer_rsrc_t tbuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(a.UT), 0, 4 * H * H * 4, 0x00020000);
    int vb[4];
#pragma unroll
    for (int c = 0; c < 4; c++) vb[c] = ((4 * slot + c) * H + j0 + x) * 4;
    const int ksu = __builtin_amdgcn_readfirstlane(ks);
    // packed: this lane's float4 in the 1 KB block of k-group 0 and this workgroup's column tile,
    // and the distance in bytes between the blocks of consecutive k-groups
    const float4 *lane_pk = reinterpret_cast<const float4 *>(a.UT) + blockIdx.x * 64 + slot * 16 + x;
    const int gstep = (H / 16) * 1024;
    // the operands of the children's gate gradients travel under the longer of the two product
    // groups: with eight wavefronts (a round of a few rows) the second is only two stages
    if constexpr (WAVES == 8) fetch_kids();
    {  // P0: K = 3H
      const int kb = ksu * (3 * H / KS);
      const float *arow[1] = {px + kb + 4 * aslot};
      // one accumulator: a stage of UG k-groups is only 4 * UG MFMAs, too short to cover its own
      // loads, so this product runs with stages three times as long (as many stages as K = H has)
      constexpr int UG0 = 3 * UG;
      if constexpr (PACKED)
        exact_products<TILE, UG0, 1, true, true, ROWS4>(&acc[0], arow, tbuf, vb, 0, gstep, H / KS / S, lane_pk + (kb / 16) * (gstep / 16));
      else
        exact_products<TILE, UG0, 1>(&acc[0], arow, tbuf, vb, kb * H * 4, H * 4, H / KS / S);
    }
    if constexpr (WAVES != 8) fetch_kids();
    {  // P1, P2: K = H, one B operand for both
      const int kb = ksu * (H / KS);
      const float *arow[2] = {pfl + kb + 4 * aslot, pfr + kb + 4 * aslot};
      if constexpr (PACKED)
        exact_products<TILE, UG, 2, true, true, ROWS4>(&acc[1], arow, tbuf, vb, 0, gstep, H / KS / S, lane_pk + 3 * H * H / 4 + (kb / 16) * (gstep / 16));
      else
        exact_products<TILE, UG, 2>(&acc[1], arow, tbuf, vb, (3 * H * H + kb * H) * 4, H * 4, H / KS / S);
    }
  } else {
  {  // P0: K = 3H
    const int K = 3 * H;
    const int kper = ((K + KS - 1) / KS + GK - 1) / GK * GK;
    const int kb = ks * kper, ke = min(K, kb + kper);
    struct Frag {
      float4 a[UG];
      float b[UG][4];
    };
    auto fetch = [&](int k0, Frag &f) {
#pragma unroll
      for (int u = 0; u < UG; u++) {
        const int kk = k0 + GK * u + 4 * slot;
        const bool kin = kk < ke;
        f.a[u] = (kin && rin) ? ld4(px + kk) : zero4();
#pragma unroll
        for (int c = 0; c < 4; c++) f.b[u][c] = kin ? UTio[(long)(kk + c) * H] : 0.f;
      }
    };
    auto multiply = [&](const Frag &f) {
#pragma unroll
      for (int u = 0; u < UG; u++)
#pragma unroll
        for (int c = 0; c < 4; c++) acc[0] = M::mma(elem(f.a[u], c), f.b[u][c], acc[0]);
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
  fetch_kids();
  {  // P1, P2: K = H, one B operand for both
    const int K = H;
    const int kper = ((K + KS - 1) / KS + GK - 1) / GK * GK;
    const int kb = ks * kper, ke = min(K, kb + kper);
    struct Frag {
      float4 l[UG], r[UG];
      float b[UG][4];
    };
    auto fetch = [&](int k0, Frag &f) {
#pragma unroll
      for (int u = 0; u < UG; u++) {
        const int kk = k0 + GK * u + 4 * slot;
        const bool kin = kk < ke;
        f.l[u] = (kin && rin) ? ld4(pfl + kk) : zero4();
        f.r[u] = (kin && rin) ? ld4(pfr + kk) : zero4();
#pragma unroll
        for (int c = 0; c < 4; c++) f.b[u][c] = kin ? UTf[(long)(kk + c) * H] : 0.f;
      }
    };
    auto multiply = [&](const Frag &f) {
#pragma unroll
      for (int u = 0; u < UG; u++)
#pragma unroll
        for (int c = 0; c < 4; c++) {
          acc[1] = M::mma(elem(f.l[u], c), f.b[u][c], acc[1]);
          acc[2] = M::mma(elem(f.r[u], c), f.b[u][c], acc[2]);
        }
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
  }

  park_partials<TILE, NP, KS, NREG, RT>(red, acc, rt, ks, lane);

#pragma unroll
  for (int q = 0; q < EPT; q++) {
    if (!eon[q]) continue;
    const float *pre = red + elds[q];
    float v[NP];
#pragma unroll
    for (int p = 0; p < NP; p++) {
      float s;
      if constexpr (ROWS4) {
        s = 0.f;
#pragma unroll
        for (int g = 0; g < NREG; g++)
          s += (pre[g * RSZ + p * NR * 64] + pre[g * RSZ + p * NR * 64 + 16]) +
               (pre[g * RSZ + p * NR * 64 + 32] + pre[g * RSZ + p * NR * 64 + 48]);
      } else {
        s = pre[p * NR * 64];
#pragma unroll
        for (int g = 1; g < NREG; g++) s += pre[g * RSZ + p * NR * 64];
      }
      v[p] = s;
    }
    if constexpr (FOLD) {
#pragma unroll
      for (int s = 0; s < 2; s++) {
        const long c = s ? ecr[q] : ecl[q];
        if (c < 0) continue;
        const Kid &kd = kid[q][s];
        const int j = ej[q];
        const GateGrad gg = gate_grad(kd.g[0], kd.g[1], kd.g[2], kd.g[3], kd.g[4], kd.g[5], v[0] + v[1 + s], pdc[q] * pf[q][s],
                                      kd.dr, kd.cl, kd.cr);
        float *dx = a.dxW_all + c * a.ld_dxw + j;
        dx[0] = gg.di; dx[H] = gg.d_o; dx[2 * H] = gg.du; dx[3 * H] = gg.dfl + gg.dfr;
        if (c >= a.leaf_rows) {
          a.dF_all[(2 * c) * H + j] = gg.dfl;
          a.dF_all[(2 * c + 1) * H + j] = gg.dfr;
          a.dc_all[c * H + j] = gg.dc;
        }
      }
    } else {
      if (ecl[q] >= 0) a.dpool[ecl[q] * H2 + ej[q]] = v[0] + v[1];
      if (ecr[q] >= 0) a.dpool[ecr[q] * H2 + ej[q]] = v[0] + v[2];
    }
  }
}

// out[c][r] = in[r][c]
__global__ void transpose_kernel(float *__restrict__ out, const float *__restrict__ in, int rows, int cols) {
  __shared__ float tile[32][33];
  const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
  for (int i = ty; i < 32; i += 8)
    if (r0 + i < rows && c0 + tx < cols) tile[i][tx] = in[(long)(r0 + i) * cols + c0 + tx];
  __syncthreads();
  for (int i = ty; i < 32; i += 8)
    if (c0 + i < cols && r0 + tx < rows) out[(long)(c0 + i) * rows + r0 + tx] = tile[tx][i];
}

// the packed variants exist for the shapes cavs_round_packed_ok admits: 16x16 tiles, exact stages
static void launch_bwd_children_packed(const RoundBwdChildArgs &a, hipStream_t st) {
  const RoundPlan p = plan_round(a.n, a.H);
  dim3 grid(a.H / p.tile, (a.n + p.tile - 1) / p.tile);
  if (a.n <= kRows4Max) launch(treelstm_round_bwd_children_kernel<16, 8, true, true, true, true>, dim3(a.H / 16, (a.n + 3) / 4), 512, 0, st, a);
  else if (p.waves == 4) launch(treelstm_round_bwd_children_kernel<16, 4, true, true, true>, grid, 256, 0, st, a);
  else launch(treelstm_round_bwd_children_kernel<16, 8, true, true, true>, grid, 512, 0, st, a);
}

template <bool FOLD>
static void launch_bwd_children(const RoundBwdChildArgs &a, hipStream_t st) {
  const RoundPlan p = plan_round(a.n, a.H);
  dim3 grid(a.H / p.tile, (a.n + p.tile - 1) / p.tile);
  const bool exact = exact_stages(a.H, p);
  if (p.tile == 16 && p.waves == 4) {
    if (exact) launch(treelstm_round_bwd_children_kernel<16, 4, FOLD, true>, grid, 256, 0, st, a);
    else launch(treelstm_round_bwd_children_kernel<16, 4, FOLD, false>, grid, 256, 0, st, a);
  } else if (p.tile == 16) {
    if (exact) launch(treelstm_round_bwd_children_kernel<16, 8, FOLD, true>, grid, 512, 0, st, a);
    else launch(treelstm_round_bwd_children_kernel<16, 8, FOLD, false>, grid, 512, 0, st, a);
  } else if (p.waves == 4) {
    launch(treelstm_round_bwd_children_kernel<32, 4, FOLD, false>, grid, 256, 0, st, a);
  } else {
    launch(treelstm_round_bwd_children_kernel<32, 8, FOLD, false>, grid, 512, 0, st, a);
  }
}

}  // namespace cavs

using namespace cavs;

extern "C" {

int cavs_treelstm_round_fwd(float *pool, const int *child, const int *pair, const float *xW, int ld_xw,
                            const float *U, const float *bias, float *G, float *hlr, float *gates,
                            float *msg, float *graph_out, const int *out_rows, int n, int H, void *stream) {
  CAVS_REQUIRE(n >= 0 && round_shape_ok(H) && ld_xw >= 4 * H && ld_xw % 4 == 0,
               "cavs_treelstm_round_fwd: bad shape n=%d H=%d ld_xw=%d (H must be a multiple of 32)", n, H, ld_xw);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(pool && child && pair && xW && U && bias && G && hlr && gates, "cavs_treelstm_round_fwd: null pointer");
  CAVS_REQUIRE(aligned16(pool) && aligned16(U), "cavs_treelstm_round_fwd: pool and U must be 16-byte aligned");
  CAVS_REQUIRE(!graph_out || out_rows, "cavs_treelstm_round_fwd: graph_out needs out_rows");
  RoundFwdArgs a{pool, child, pair, xW, ld_xw, U, nullptr, bias, G, hlr, gates, msg, pool, graph_out, out_rows, n, H};
  const RoundPlan p = plan_round(n, H);
  dim3 grid(H / p.tile, (n + p.tile - 1) / p.tile);
  hipStream_t st = as_stream(stream);
  const bool exact = exact_stages(H, p);
  if (p.tile == 16 && p.waves == 4) {
    if (exact) launch(treelstm_round_fwd_kernel<16, 4, true>, grid, 256, 0, st, a);
    else launch(treelstm_round_fwd_kernel<16, 4, false>, grid, 256, 0, st, a);
  } else if (p.tile == 16) {
    if (exact) launch(treelstm_round_fwd_kernel<16, 8, true>, grid, 512, 0, st, a);
    else launch(treelstm_round_fwd_kernel<16, 8, false>, grid, 512, 0, st, a);
  } else if (p.waves == 4) {
    launch(treelstm_round_fwd_kernel<32, 4, false>, grid, 256, 0, st, a);
  } else {
    launch(treelstm_round_fwd_kernel<32, 8, false>, grid, 512, 0, st, a);
  }
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_treelstm_round_fwd_packed(float *pool, const int *child, const int *pair, const float *xW, int ld_xw,
                                   const float *U, const float *Upk, const float *bias, float *G, float *hlr, float *gates,
                                   float *msg, float *graph_out, const int *out_rows, int n, int H, void *stream) {
  CAVS_REQUIRE(n >= 0 && ld_xw >= 4 * H && ld_xw % 4 == 0 && cavs_round_packed_ok(n, H),
               "cavs_treelstm_round_fwd_packed: bad shape n=%d H=%d ld_xw=%d (see cavs_round_packed_ok)", n, H, ld_xw);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(pool && child && pair && xW && U && Upk && bias && G && hlr && gates, "cavs_treelstm_round_fwd_packed: null pointer");
  CAVS_REQUIRE(aligned16(pool) && aligned16(U) && aligned16(Upk), "cavs_treelstm_round_fwd_packed: pool, U and Upk must be 16-byte aligned");
  CAVS_REQUIRE(!graph_out || out_rows, "cavs_treelstm_round_fwd_packed: graph_out needs out_rows");
  RoundFwdArgs a{pool, child, pair, xW, ld_xw, U, Upk, bias, G, hlr, gates, msg, pool, graph_out, out_rows, n, H};
  const RoundPlan p = plan_round(n, H);
  dim3 grid(H / 16, (n + 15) / 16);
  hipStream_t st = as_stream(stream);
  if (n <= kRows4Max) launch(treelstm_round_fwd_kernel<16, 8, true, true, true>, dim3(H / 16, (n + 3) / 4), 512, 0, st, a);
  else if (p.waves == 4) launch(treelstm_round_fwd_kernel<16, 4, true, true>, grid, 256, 0, st, a);
  else launch(treelstm_round_fwd_kernel<16, 8, true, true>, grid, 512, 0, st, a);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_treelstm_round_leaves_fwd(float *pool, const int *pair, const float *xW, int ld_xw, const float *bias,
                                   float *gates, float *msg, float *graph_out, const int *out_rows, int n, int H,
                                   void *stream) {
  CAVS_REQUIRE(n >= 0 && H > 0 && ld_xw >= 4 * H, "cavs_treelstm_round_leaves_fwd: bad shape n=%d H=%d ld=%d", n, H, ld_xw);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(pool && pair && xW && bias && gates, "cavs_treelstm_round_leaves_fwd: null pointer");
  CAVS_REQUIRE(!graph_out || out_rows, "cavs_treelstm_round_leaves_fwd: graph_out needs out_rows");
  RoundLeavesArgs a{xW, ld_xw, bias, pair, gates, msg, pool, graph_out, out_rows, n, H};
  hipStream_t st = as_stream(stream);
  const bool vec = H % 4 == 0 && ld_xw % 4 == 0 && aligned16(pool) && aligned16(xW) && aligned16(bias) && aligned16(gates) &&
                   (!msg || aligned16(msg)) && (!graph_out || aligned16(graph_out));
  if (vec) {
    long total = (long)n * (H / 4);
    launch(treelstm_round_leaves_fwd_kernel<4>, (unsigned)((total + 255) / 256), 256, 0, st, a);
  } else {
    long total = (long)n * H;
    launch(treelstm_round_leaves_fwd_kernel<1>, (unsigned)((total + 255) / 256), 256, 0, st, a);
  }
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_treelstm_round_bwd_gates(float *dpool, const int *pair, const int *child, const float *dret,
                                  const int *dret_rows, const float *gates, const float *G, float *dxW,
                                  int ld_dxw, float *dF, int n, int H, void *stream) {
  CAVS_REQUIRE(n >= 0 && H > 0 && ld_dxw >= 4 * H, "cavs_treelstm_round_bwd_gates: bad shape n=%d H=%d ld=%d", n, H, ld_dxw);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(dpool && pair && dret && gates && dxW, "cavs_treelstm_round_bwd_gates: null pointer");
  CAVS_REQUIRE((child && G && dF) || (!child && !G && !dF),
               "cavs_treelstm_round_bwd_gates: child, G and dF must be all set (internal round) or all null (leaves)");
  RoundBwdGatesArgs a{dpool, pair, child, dret, dret_rows, gates, G, dxW, ld_dxw, dF, dpool, n, H};
  hipStream_t st = as_stream(stream);
  const bool vec = H % 4 == 0 && ld_dxw % 4 == 0 && aligned16(dpool) && aligned16(dret) && aligned16(gates) &&
                   aligned16(dxW) && (!G || aligned16(G)) && (!dF || aligned16(dF));
  if (vec) {
    long total = (long)n * (H / 4);
    launch(treelstm_round_bwd_gates_kernel<4>, (unsigned)((total + 255) / 256), 256, 0, st, a);
  } else {
    long total = (long)n * H;
    launch(treelstm_round_bwd_gates_kernel<1>, (unsigned)((total + 255) / 256), 256, 0, st, a);
  }
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_treelstm_round_bwd_children(const float *dxW, int ld_dxw, const float *dF, const float *UT,
                                     const int *child, float *dpool, int n, int H, void *stream) {
  CAVS_REQUIRE(n >= 0 && round_shape_ok(H) && ld_dxw >= 4 * H && ld_dxw % 4 == 0,
               "cavs_treelstm_round_bwd_children: bad shape n=%d H=%d ld=%d (H must be a multiple of 32)", n, H, ld_dxw);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(dxW && dF && UT && child && dpool, "cavs_treelstm_round_bwd_children: null pointer");
  CAVS_REQUIRE(aligned16(dxW) && aligned16(dF), "cavs_treelstm_round_bwd_children: dxW and dF must be 16-byte aligned");
  RoundBwdChildArgs a{dxW, ld_dxw, dF, UT, child, dpool, n, H, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0};
  launch_bwd_children<false>(a, as_stream(stream));
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_treelstm_round_bwd_children_gates(float *dxW, int ld_dxw, float *dF, float *dc, const float *UT,
                                           const int *child_rows, const float *gates, const float *G, const float *dret,
                                           const int *dret_rows, int row0, int n, int leaf_rows, int H, void *stream) {
  CAVS_REQUIRE(n >= 0 && row0 >= 0 && leaf_rows >= 0 && round_shape_ok(H) && ld_dxw >= 4 * H && ld_dxw % 4 == 0,
               "cavs_treelstm_round_bwd_children_gates: bad shape row0=%d n=%d leaf_rows=%d H=%d ld=%d (H must be a multiple of 32)",
               row0, n, leaf_rows, H, ld_dxw);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(dxW && dF && dc && UT && child_rows && gates && G && dret && dret_rows,
               "cavs_treelstm_round_bwd_children_gates: null pointer");
  CAVS_REQUIRE(aligned16(dxW) && aligned16(dF), "cavs_treelstm_round_bwd_children_gates: dxW and dF must be 16-byte aligned");
  RoundBwdChildArgs a{dxW + (long)row0 * ld_dxw, ld_dxw, dF + 2L * row0 * H, UT, child_rows, nullptr, n, H,
                      dxW, dF, dc, gates, G, dret, dret_rows, row0, leaf_rows};
  launch_bwd_children<true>(a, as_stream(stream));
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_round_packed_ok(int n, int H) {
  if (n < 0 || !round_shape_ok(H)) return 0;
  const RoundPlan p = plan_round(n > 0 ? n : 1, H);
  return p.tile == 16 && exact_stages(H, p) ? 1 : 0;
}

int cavs_treelstm_round_bwd_children_gates_packed(float *dxW, int ld_dxw, float *dF, float *dc, const float *UTp,
                                                  const int *child_rows, const float *gates, const float *G,
                                                  const float *dret, const int *dret_rows, int row0, int n, int leaf_rows,
                                                  int H, void *stream) {
  CAVS_REQUIRE(n >= 0 && row0 >= 0 && leaf_rows >= 0 && ld_dxw >= 4 * H && ld_dxw % 4 == 0 && cavs_round_packed_ok(n, H),
               "cavs_treelstm_round_bwd_children_gates_packed: bad shape row0=%d n=%d leaf_rows=%d H=%d ld=%d (see cavs_round_packed_ok)",
               row0, n, leaf_rows, H, ld_dxw);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(dxW && dF && dc && UTp && child_rows && gates && G && dret && dret_rows,
               "cavs_treelstm_round_bwd_children_gates_packed: null pointer");
  CAVS_REQUIRE(aligned16(dxW) && aligned16(dF) && aligned16(UTp),
               "cavs_treelstm_round_bwd_children_gates_packed: dxW, dF and UTp must be 16-byte aligned");
  RoundBwdChildArgs a{dxW + (long)row0 * ld_dxw, ld_dxw, dF + 2L * row0 * H, UTp, child_rows, nullptr, n, H,
                      dxW, dF, dc, gates, G, dret, dret_rows, row0, leaf_rows};
  launch_bwd_children_packed(a, as_stream(stream));
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_treelstm_bwd_gates_rows(const int *rows, int n, const float *dret, const int *dret_rows, const float *gates,
                                 const float *G, float *dxW, int ld_dxw, float *dF, float *dc, int leaf_rows, int H,
                                 void *stream) {
  CAVS_REQUIRE(n >= 0 && H > 0 && leaf_rows >= 0 && ld_dxw >= 4 * H, "cavs_treelstm_bwd_gates_rows: bad shape n=%d H=%d ld=%d", n, H,
               ld_dxw);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(rows && dret && dret_rows && gates && G && dxW && dF && dc, "cavs_treelstm_bwd_gates_rows: null pointer");
  BwdGatesRowsArgs a{rows, dret, dret_rows, gates, G, dxW, ld_dxw, dF, dc, n, H, leaf_rows};
  hipStream_t st = as_stream(stream);
  if (H % 4 == 0) {
    long total = (long)n * (H / 4);
    launch(treelstm_bwd_gates_rows_kernel<4>, (unsigned)((total + 255) / 256), 256, 0, st, a);
  } else {
    long total = (long)n * H;
    launch(treelstm_bwd_gates_rows_kernel<1>, (unsigned)((total + 255) / 256), 256, 0, st, a);
  }
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_transpose(float *out, const float *in, int rows, int cols, void *stream) {
  CAVS_REQUIRE(rows >= 0 && cols >= 0, "cavs_transpose: bad shape %d x %d", rows, cols);
  if (rows == 0 || cols == 0) return CAVS_OK;
  CAVS_REQUIRE(out && in && out != in, "cavs_transpose: null or aliased pointer");
  dim3 grid((cols + 31) / 32, (rows + 31) / 32);
  launch(transpose_kernel, grid, 256, 0, as_stream(stream), out, in, rows, cols);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

}  // extern "C"
