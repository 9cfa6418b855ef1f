// Fused gate kernels of the three vertex functions (Tree-LSTM, chain LSTM,
// Tree-FC), forward and gradient.  One kernel replaces the whole Slice / Add /
// Sigmoid / Tanh / Mul / Concat chain of a round: each lane owns W consecutive
// hidden units of one vertex, reads every operand once with 16-byte accesses and
// writes the message, the saved gates and the pre-activation gradients once.
// HBM-bound; no operand is re-read.
#include "common.h"

namespace cavs {

template <int W>
struct Vec {
  float v[W];
};

template <int W>
__device__ inline Vec<W> vload(const float *p) {
  Vec<W> r;
  if constexpr (W == 4) {
    float4 t = *reinterpret_cast<const float4 *>(p);
    r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w;
  } else {
#pragma unroll
    for (int i = 0; i < W; i++) r.v[i] = p[i];
  }
  return r;
}

template <int W>
__device__ inline void vstore(float *p, const Vec<W> &a) {
  if constexpr (W == 4) {
    *reinterpret_cast<float4 *>(p) = make_float4(a.v[0], a.v[1], a.v[2], a.v[3]);
  } else {
#pragma unroll
    for (int i = 0; i < W; i++) p[i] = a.v[i];
  }
}

template <int W>
__device__ inline Vec<W> vzeros() {
  Vec<W> r;
#pragma unroll
  for (int i = 0; i < W; i++) r.v[i] = 0.f;
  return r;
}

// 1/(1+exp(-x)) and tanh exactly as the reference's generated code spells them
// (cavs/midend/runtime_compiler/expression.h:40-71).
__device__ inline float sigm(float x) { return 1.f / (1.f + expf(-x)); }

// ------------------------------------------------------------------ Tree-LSTM
template <int W>
__global__ void treelstm_fwd_kernel(const float *__restrict__ xW, long ld_xw,
                                    const float *__restrict__ hU, const float *__restrict__ hUf,
                                    const float *__restrict__ G, const float *__restrict__ bias,
                                    float *__restrict__ gates, float *__restrict__ msg, int n,
                                    int H, float *pool = nullptr, const int *__restrict__ pair = nullptr,
                                    float *__restrict__ graph_out = nullptr, const int *__restrict__ out_rows = nullptr) {
  const int hw = H / W;
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)n * hw) return;
  const int r = (int)(idx / hw), j = (int)(idx % hw) * W;
  const float *xw = xW + r * ld_xw + j;
  Vec<W> xi = vload<W>(xw), xo = vload<W>(xw + H), xu = vload<W>(xw + 2 * H), xf = vload<W>(xw + 3 * H);
  Vec<W> hi = vzeros<W>(), ho = hi, hu = hi, fl = hi, fr = hi, cl = hi, cr = hi;
  if (hU) {  // internal round: children exist
    const float *p = hU + (long)r * 3 * H + j;
    hi = vload<W>(p); ho = vload<W>(p + H); hu = vload<W>(p + 2 * H);
    fl = vload<W>(hUf + (long)(2 * r) * H + j);
    fr = vload<W>(hUf + (long)(2 * r + 1) * H + j);
    cl = vload<W>(G + (long)(2 * r) * 2 * H + H + j);
    cr = vload<W>(G + (long)(2 * r + 1) * 2 * H + H + j);
  }
  // bias blocks [i|f|u|o] (apps/paper/tree-lstm-cavs.cc:120-123)
  Vec<W> bi = vload<W>(bias + j), bf = vload<W>(bias + H + j), bu = vload<W>(bias + 2 * H + j),
         bo = vload<W>(bias + 3 * H + j);
  Vec<W> gi, go, gu, gfl, gfr, gtc, mh, mc;
#pragma unroll
  for (int k = 0; k < W; k++) {
    float i = sigm((xi.v[k] + hi.v[k]) + bi.v[k]);
    float o = sigm((xo.v[k] + ho.v[k]) + bo.v[k]);
    float u = tanhf((xu.v[k] + hu.v[k]) + bu.v[k]);
    float f_l = sigm((xf.v[k] + fl.v[k]) + bf.v[k]);
    float f_r = sigm((xf.v[k] + fr.v[k]) + bf.v[k]);
    float c = (i * u + f_l * cl.v[k]) + f_r * cr.v[k];
    float tc = tanhf(c);
    gi.v[k] = i; go.v[k] = o; gu.v[k] = u; gfl.v[k] = f_l; gfr.v[k] = f_r; gtc.v[k] = tc;
    mh.v[k] = o * tc; mc.v[k] = c;
  }
  float *g = gates + (long)r * 6 * H + j;
  vstore<W>(g, gi); vstore<W>(g + H, go); vstore<W>(g + 2 * H, gu);
  vstore<W>(g + 3 * H, gfl); vstore<W>(g + 4 * H, gfr); vstore<W>(g + 5 * H, gtc);
  if (msg) {
    float *m = msg + (long)r * 2 * H + j;
    vstore<W>(m, mh); vstore<W>(m + H, mc);
  }
  // Scatter and Push / FunctionPopRet folded in: the message goes to the pool row the list names,
  // the pushed value to its row of the graph output
  if (pool) {
    const int dst = pair[r];
    if (dst >= 0) { vstore<W>(pool + (long)dst * 2 * H + j, mh); vstore<W>(pool + (long)dst * 2 * H + H + j, mc); }
  }
  if (graph_out) vstore<W>(graph_out + (long)out_rows[r] * H + j, mh);
}

template <int W>
__global__ void treelstm_bwd_kernel(const float *__restrict__ dmsg, const float *__restrict__ dret,
                                    const float *__restrict__ gates, const float *__restrict__ G,
                                    float *__restrict__ dxW, long ld_dxw, float *__restrict__ dF,
                                    float *__restrict__ dG, int n, int H) {
  const int hw = H / W;
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)n * hw) return;
  const int r = (int)(idx / hw), j = (int)(idx % hw) * W;
  const float *g = gates + (long)r * 6 * H + j;
  Vec<W> gi = vload<W>(g), go = vload<W>(g + H), gu = vload<W>(g + 2 * H), gfl = vload<W>(g + 3 * H),
         gfr = vload<W>(g + 4 * H), gtc = vload<W>(g + 5 * H);
  Vec<W> dmh = vload<W>(dmsg + (long)r * 2 * H + j), dmc = vload<W>(dmsg + (long)r * 2 * H + H + j);
  Vec<W> dr = vload<W>(dret + (long)r * H + j);
  Vec<W> cl = vzeros<W>(), cr = cl;
  if (G) {
    cl = vload<W>(G + (long)(2 * r) * 2 * H + H + j);
    cr = vload<W>(G + (long)(2 * r + 1) * 2 * H + H + j);
  }
  Vec<W> di, dvo, du, dfs, dfl, dfr, dcl, dcr;
#pragma unroll
  for (int k = 0; k < W; k++) {
    float i = gi.v[k], o = go.v[k], u = gu.v[k], f_l = gfl.v[k], f_r = gfr.v[k], tc = gtc.v[k];
    float dh = dmh.v[k] + dr.v[k];
    float d_o = dh * tc;
    float dc = dmc.v[k] + (dh * o) * (1.f - tc * tc);
    float del_i = (dc * u) * (i * (1.f - i));
    float del_o = d_o * (o * (1.f - o));
    float del_u = (dc * i) * (1.f - u * u);
    float del_fl = (dc * cl.v[k]) * (f_l * (1.f - f_l));
    float del_fr = (dc * cr.v[k]) * (f_r * (1.f - f_r));
    di.v[k] = del_i; dvo.v[k] = del_o; du.v[k] = del_u; dfs.v[k] = del_fl + del_fr;
    dfl.v[k] = del_fl; dfr.v[k] = del_fr;
    dcl.v[k] = dc * f_l; dcr.v[k] = dc * f_r;
  }
  float *dx = dxW + r * ld_dxw + j;
  vstore<W>(dx, di); vstore<W>(dx + H, dvo); vstore<W>(dx + 2 * H, du); vstore<W>(dx + 3 * H, dfs);
  if (G) {
    vstore<W>(dF + (long)(2 * r) * H + j, dfl);
    vstore<W>(dF + (long)(2 * r + 1) * H + j, dfr);
    vstore<W>(dG + (long)(2 * r) * 2 * H + H + j, dcl);
    vstore<W>(dG + (long)(2 * r + 1) * 2 * H + H + j, dcr);
  }
}

// ------------------------------------------------------------------ chain LSTM
template <int W>
__global__ void lstm_fwd_kernel(const float *__restrict__ a, long ld_a, const float *__restrict__ a2,
                                const float *__restrict__ G, const float *__restrict__ bias,
                                float *__restrict__ gates, float *__restrict__ msg, int n, int H) {
  const int hw = H / W;
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)n * hw) return;
  const int r = (int)(idx / hw), j = (int)(idx % hw) * W;
  const float *p = a + r * ld_a + j;
  Vec<W> ai = vload<W>(p), af = vload<W>(p + H), au = vload<W>(p + 2 * H), ao = vload<W>(p + 3 * H);
  Vec<W> qi = vzeros<W>(), qf = qi, qu = qi, qo = qi, cp = qi;
  if (a2) {
    const float *q = a2 + (long)r * 4 * H + j;
    qi = vload<W>(q); qf = vload<W>(q + H); qu = vload<W>(q + 2 * H); qo = vload<W>(q + 3 * H);
  }
  if (G) cp = vload<W>(G + (long)r * 2 * H + H + j);
  Vec<W> bi = vload<W>(bias + j), bf = vload<W>(bias + H + j), bu = vload<W>(bias + 2 * H + j),
         bo = vload<W>(bias + 3 * H + j);
  Vec<W> gi, gf, gu, go, gtc, mh, mc;
#pragma unroll
  for (int k = 0; k < W; k++) {
    float i = sigm((ai.v[k] + qi.v[k]) + bi.v[k]);
    float f = sigm((af.v[k] + qf.v[k]) + bf.v[k]);
    float u = tanhf((au.v[k] + qu.v[k]) + bu.v[k]);
    float o = sigm((ao.v[k] + qo.v[k]) + bo.v[k]);
    float c = i * u + f * cp.v[k];
    float tc = tanhf(c);
    gi.v[k] = i; gf.v[k] = f; gu.v[k] = u; go.v[k] = o; gtc.v[k] = tc;
    mh.v[k] = o * tc; mc.v[k] = c;
  }
  float *g = gates + (long)r * 5 * H + j;
  vstore<W>(g, gi); vstore<W>(g + H, gf); vstore<W>(g + 2 * H, gu); vstore<W>(g + 3 * H, go);
  vstore<W>(g + 4 * H, gtc);
  float *m = msg + (long)r * 2 * H + j;
  vstore<W>(m, mh); vstore<W>(m + H, mc);
}

template <int W>
__global__ void lstm_bwd_kernel(const float *__restrict__ dmsg, const float *__restrict__ dret,
                                const float *__restrict__ gates, const float *__restrict__ G,
                                float *__restrict__ da, long ld_da, float *__restrict__ dG, int n,
                                int H) {
  const int hw = H / W;
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)n * hw) return;
  const int r = (int)(idx / hw), j = (int)(idx % hw) * W;
  const float *g = gates + (long)r * 5 * H + j;
  Vec<W> gi = vload<W>(g), gf = vload<W>(g + H), gu = vload<W>(g + 2 * H), go = vload<W>(g + 3 * H),
         gtc = vload<W>(g + 4 * H);
  Vec<W> dmh = vload<W>(dmsg + (long)r * 2 * H + j), dmc = vload<W>(dmsg + (long)r * 2 * H + H + j);
  Vec<W> dr = vload<W>(dret + (long)r * H + j);
  Vec<W> cp = vzeros<W>();
  if (G) cp = vload<W>(G + (long)r * 2 * H + H + j);
  Vec<W> di, df, du, dvo, dcp;
#pragma unroll
  for (int k = 0; k < W; k++) {
    float i = gi.v[k], f = gf.v[k], u = gu.v[k], o = go.v[k], tc = gtc.v[k];
    float dh = dmh.v[k] + dr.v[k];
    float d_o = dh * tc;
    float dc = dmc.v[k] + (dh * o) * (1.f - tc * tc);
    di.v[k] = (dc * u) * (i * (1.f - i));
    df.v[k] = (dc * cp.v[k]) * (f * (1.f - f));
    du.v[k] = (dc * i) * (1.f - u * u);
    dvo.v[k] = d_o * (o * (1.f - o));
    dcp.v[k] = dc * f;
  }
  float *d = da + r * ld_da + j;
  vstore<W>(d, di); vstore<W>(d + H, df); vstore<W>(d + 2 * H, du); vstore<W>(d + 3 * H, dvo);
  if (dG) vstore<W>(dG + (long)r * 2 * H + H + j, dcp);
}

// ------------------------------------------------------------------ Tree-FC
template <int W>
__global__ void treefc_fwd_kernel(const float *__restrict__ z, const float *__restrict__ bias,
                                  const float *__restrict__ x, float *__restrict__ h, int n, int H,
                                  int act) {
  const int hw = H / W;
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)n * hw) return;
  const int r = (int)(idx / hw), j = (int)(idx % hw) * W;
  Vec<W> v = z ? vload<W>(z + (long)r * H + j) : vzeros<W>();
  Vec<W> b = bias ? vload<W>(bias + j) : vzeros<W>();
  Vec<W> xi = x ? vload<W>(x + (long)r * H + j) : vzeros<W>();
  Vec<W> o;
#pragma unroll
  for (int k = 0; k < W; k++) {
    float t = v.v[k];
    if (bias) t += b.v[k];
    if (x) t += xi.v[k];
    o.v[k] = act ? tanhf(t) : (t > 0.f ? t : 0.f);
  }
  vstore<W>(h + (long)r * H + j, o);
}

template <int W>
__global__ void treefc_bwd_kernel(const float *__restrict__ dh_m, const float *__restrict__ dret,
                                  const float *__restrict__ h, float *__restrict__ dz, long total,
                                  int act) {
  long idx = ((long)blockIdx.x * blockDim.x + threadIdx.x) * W;
  if (idx >= total) return;
  Vec<W> a = vload<W>(dh_m + idx), b = vload<W>(dret + idx), y = vload<W>(h + idx), o;
#pragma unroll
  for (int k = 0; k < W; k++) {
    float dh = a.v[k] + b.v[k];
    o.v[k] = act ? dh * (1.f - y.v[k] * y.v[k]) : (y.v[k] > 0.f ? dh : 0.f);
  }
  vstore<W>(dz + idx, o);
}

inline bool all_aligned(std::initializer_list<const void *> ps) {
  for (const void *p : ps)
    if (p && !aligned16(p)) return false;
  return true;
}

}  // namespace cavs

using namespace cavs;

#define GATE_GRID(n, H, W) dim3((unsigned)(((long)(n) * ((H) / (W)) + 255) / 256)), dim3(256)

extern "C" {

int cavs_treelstm_gates_fwd(const float *xW, int ld_xw, const float *hU, const float *hUf,
                            const float *G, const float *bias, float *gates, float *msg, int n,
                            int H, void *stream) {
  CAVS_REQUIRE(n >= 0 && H > 0 && ld_xw >= 4 * H, "cavs_treelstm_gates_fwd: bad shape n=%d H=%d ld=%d", n, H, ld_xw);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(xW && bias && gates && msg, "cavs_treelstm_gates_fwd: null pointer");
  CAVS_REQUIRE((hU && hUf && G) || (!hU && !hUf && !G), "cavs_treelstm_gates_fwd: hU, hUf and G must be all set or all null");
  hipStream_t st = as_stream(stream);
  if (H % 4 == 0 && ld_xw % 4 == 0 && all_aligned({xW, hU, hUf, G, bias, gates, msg}))
    launch(treelstm_fwd_kernel<4>, GATE_GRID(n, H, 4), 0, st, xW, ld_xw, hU, hUf, G, bias, gates, msg, n, H, (float *)nullptr,
           (const int *)nullptr, (float *)nullptr, (const int *)nullptr);
  else
    launch(treelstm_fwd_kernel<1>, GATE_GRID(n, H, 1), 0, st, xW, ld_xw, hU, hUf, G, bias, gates, msg, n, H, (float *)nullptr,
           (const int *)nullptr, (float *)nullptr, (const int *)nullptr);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_treelstm_gates_fwd_scatter(const float *xW, int ld_xw, const float *hU, const float *hUf, const float *G, const float *bias,
                                    float *gates, float *msg, float *pool, const int *pair, float *graph_out, const int *out_rows,
                                    int n, int H, void *stream) {
  CAVS_REQUIRE(n >= 0 && H > 0 && ld_xw >= 4 * H, "cavs_treelstm_gates_fwd_scatter: bad shape n=%d H=%d ld=%d", n, H, ld_xw);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(xW && bias && gates && pool && pair, "cavs_treelstm_gates_fwd_scatter: null pointer");
  CAVS_REQUIRE((hU && hUf && G) || (!hU && !hUf && !G), "cavs_treelstm_gates_fwd_scatter: hU, hUf and G must be all set or all null");
  CAVS_REQUIRE(!graph_out || out_rows, "cavs_treelstm_gates_fwd_scatter: graph_out needs out_rows");
  hipStream_t st = as_stream(stream);
  if (H % 4 == 0 && ld_xw % 4 == 0 && all_aligned({xW, hU, hUf, G, bias, gates, msg, pool, graph_out}))
    launch(treelstm_fwd_kernel<4>, GATE_GRID(n, H, 4), 0, st, xW, ld_xw, hU, hUf, G, bias, gates, msg, n, H, pool, pair, graph_out, out_rows);
  else
    launch(treelstm_fwd_kernel<1>, GATE_GRID(n, H, 1), 0, st, xW, ld_xw, hU, hUf, G, bias, gates, msg, n, H, pool, pair, graph_out, out_rows);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_treelstm_gates_bwd(const float *dmsg, const float *dret, const float *gates,
                            const float *G, float *dxW, int ld_dxw, float *dF, float *dG, int n,
                            int H, void *stream) {
  CAVS_REQUIRE(n >= 0 && H > 0 && ld_dxw >= 4 * H, "cavs_treelstm_gates_bwd: bad shape n=%d H=%d ld=%d", n, H, ld_dxw);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(dmsg && dret && gates && dxW, "cavs_treelstm_gates_bwd: null pointer");
  CAVS_REQUIRE((G && dF && dG) || (!G && !dF && !dG), "cavs_treelstm_gates_bwd: G, dF and dG must be all set or all null");
  hipStream_t st = as_stream(stream);
  if (H % 4 == 0 && ld_dxw % 4 == 0 && all_aligned({dmsg, dret, gates, G, dxW, dF, dG}))
    launch(treelstm_bwd_kernel<4>, GATE_GRID(n, H, 4), 0, st, dmsg, dret, gates, G, dxW, ld_dxw, dF, dG, n, H);
  else
    launch(treelstm_bwd_kernel<1>, GATE_GRID(n, H, 1), 0, st, dmsg, dret, gates, G, dxW, ld_dxw, dF, dG, n, H);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_lstm_gates_fwd(const float *a, int ld_a, const float *a2, const float *G,
                        const float *bias, float *gates, float *msg, int n, int H, void *stream) {
  CAVS_REQUIRE(n >= 0 && H > 0 && ld_a >= 4 * H, "cavs_lstm_gates_fwd: bad shape n=%d H=%d ld=%d", n, H, ld_a);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(a && bias && gates && msg, "cavs_lstm_gates_fwd: null pointer");
  hipStream_t st = as_stream(stream);
  if (H % 4 == 0 && ld_a % 4 == 0 && all_aligned({a, a2, G, bias, gates, msg}))
    launch(lstm_fwd_kernel<4>, GATE_GRID(n, H, 4), 0, st, a, ld_a, a2, G, bias, gates, msg, n, H);
  else
    launch(lstm_fwd_kernel<1>, GATE_GRID(n, H, 1), 0, st, a, ld_a, a2, G, bias, gates, msg, n, H);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_lstm_gates_bwd(const float *dmsg, const float *dret, const float *gates, const float *G,
                        float *da, int ld_da, float *dG, int n, int H, void *stream) {
  CAVS_REQUIRE(n >= 0 && H > 0 && ld_da >= 4 * H, "cavs_lstm_gates_bwd: bad shape n=%d H=%d ld=%d", n, H, ld_da);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(dmsg && dret && gates && da, "cavs_lstm_gates_bwd: null pointer");
  CAVS_REQUIRE((G && dG) || (!G && !dG), "cavs_lstm_gates_bwd: G and dG must be both set or both null");
  hipStream_t st = as_stream(stream);
  if (H % 4 == 0 && ld_da % 4 == 0 && all_aligned({dmsg, dret, gates, G, da, dG}))
    launch(lstm_bwd_kernel<4>, GATE_GRID(n, H, 4), 0, st, dmsg, dret, gates, G, da, ld_da, dG, n, H);
  else
    launch(lstm_bwd_kernel<1>, GATE_GRID(n, H, 1), 0, st, dmsg, dret, gates, G, da, ld_da, dG, n, H);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_treefc_fwd(const float *z, const float *bias, const float *x, float *h, int n, int H,
                    int act, void *stream) {
  CAVS_REQUIRE(n >= 0 && H > 0 && (act == 0 || act == 1), "cavs_treefc_fwd: bad argument n=%d H=%d act=%d", n, H, act);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(h, "cavs_treefc_fwd: null output");
  hipStream_t st = as_stream(stream);
  if (H % 4 == 0 && all_aligned({z, bias, x, h}))
    launch(treefc_fwd_kernel<4>, GATE_GRID(n, H, 4), 0, st, z, bias, x, h, n, H, act);
  else
    launch(treefc_fwd_kernel<1>, GATE_GRID(n, H, 1), 0, st, z, bias, x, h, n, H, act);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_treefc_bwd(const float *dh_m, const float *dret, const float *h, float *dz, int n, int H,
                    int act, void *stream) {
  CAVS_REQUIRE(n >= 0 && H > 0 && (act == 0 || act == 1), "cavs_treefc_bwd: bad argument n=%d H=%d act=%d", n, H, act);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(dh_m && dret && h && dz, "cavs_treefc_bwd: null pointer");
  hipStream_t st = as_stream(stream);
  long total = (long)n * H;
  if (total % 4 == 0 && all_aligned({dh_m, dret, h, dz}))
    launch(treefc_bwd_kernel<4>, dim3((unsigned)((total / 4 + 255) / 256)), dim3(256), 0, st, dh_m, dret, h, dz, total, act);
  else
    launch(treefc_bwd_kernel<1>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, dh_m, dret, h, dz, total, act);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

}  // extern "C"
