// Remaining ops of the path: column sums (bias gradients), embedding gather and
// scatter-add, row-broadcast bias add, softmax cross-entropy, SGD and the generic
// elementwise family.  All HBM-bound streaming kernels.
#include "common.h"
#include "embed_common.h"

namespace cavs {

__device__ inline float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ inline float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// ------------------------------------------------------------------ column sums
// Workgroup = 4 waves over a strip of 64 columns; lane = column (256-byte coalesced
// row reads), wave = row phase.  The four partial rows are combined through LDS.
// With more than one row chunk the chunk sums are added with hardware fp32 atomics
// into a pre-zeroed (or accumulating) output.
__global__ __launch_bounds__(256) void colsum_kernel(float *__restrict__ out,
                                                     const float *__restrict__ inp, long ld, int n,
                                                     int w, int rows_per_chunk, int use_atomic,
                                                     int accumulate) {
  __shared__ float part[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = blockIdx.x * 64 + lane;
  const int r0 = blockIdx.y * rows_per_chunk;
  const int r1 = min(n, r0 + rows_per_chunk);
  float acc0 = 0.f, acc1 = 0.f, acc2 = 0.f, acc3 = 0.f;
  if (col < w) {
    int r = r0 + wave;
    for (; r + 12 < r1; r += 16) {
      acc0 += inp[(long)r * ld + col];
      acc1 += inp[(long)(r + 4) * ld + col];
      acc2 += inp[(long)(r + 8) * ld + col];
      acc3 += inp[(long)(r + 12) * ld + col];
    }
    for (; r < r1; r += 4) acc0 += inp[(long)r * ld + col];
  }
  part[wave][lane] = (acc0 + acc1) + (acc2 + acc3);
  __syncthreads();
  if (wave == 0 && col < w) {
    float s = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
    if (use_atomic)
      unsafeAtomicAdd(out + col, s);
    else
      out[col] = accumulate ? out[col] + s : s;
  }
}

// ------------------------------------------------------------------ embedding
// ids are floats; the element offset is int(id * E), as the reference computes it.
__global__ void embed_fwd_kernel(float *__restrict__ out, long ld_out, const float *__restrict__ ids,
                                 const float *__restrict__ table, int n, int E) {
  constexpr int R = 4;
  const int row0 = blockIdx.x * R;
  long off[R];
#pragma unroll
  for (int r = 0; r < R; r++) off[r] = row0 + r < n ? (long)(int)(ids[row0 + r] * (float)E) : -1;
  for (int c = threadIdx.x; c < E; c += blockDim.x) {
    float v[R];
#pragma unroll
    for (int r = 0; r < R; r++) v[r] = off[r] >= 0 ? table[off[r] + c] : 0.f;
#pragma unroll
    for (int r = 0; r < R; r++)
      if (row0 + r < n) out[(long)(row0 + r) * ld_out + c] = v[r];
  }
}

// Pull + lookup in one pass: vertex b of the slab is vertex rows[b] of the feed; its id is
// kept in ids_out[b] for the backward pass.
__global__ void embed_pull_fwd_kernel(float *__restrict__ out, long ld_out, float *__restrict__ ids_out,
                                      const float *__restrict__ x, const int *__restrict__ rows,
                                      const float *__restrict__ table, int n, int E) {
  constexpr int R = 4;
  const int row0 = blockIdx.x * R;
  long off[R];
#pragma unroll
  for (int r = 0; r < R; r++) {
    off[r] = -1;
    if (row0 + r < n) {
      const float id = x[rows[row0 + r]];
      off[r] = (long)(int)(id * (float)E);
      if (threadIdx.x == 0) ids_out[row0 + r] = id;
    }
  }
  for (int c = threadIdx.x; c < E; c += blockDim.x) {
    float v[R];
#pragma unroll
    for (int r = 0; r < R; r++) v[r] = off[r] >= 0 ? table[off[r] + c] : 0.f;
#pragma unroll
    for (int r = 0; r < R; r++)
      if (row0 + r < n) out[(long)(row0 + r) * ld_out + c] = v[r];
  }
}

// Scatter-add of dy rows into the table: embed_bwd_block in embed_common.h, a workgroup per 64
// consecutive rows and 64 columns.
__global__ __launch_bounds__(256) void embed_bwd_kernel(float *__restrict__ dtable, const float *__restrict__ ids,
                                                        const float *__restrict__ dy, long ld_dy, int n, int E) {
  embed_bwd_block(dtable, ids, dy, ld_dy, 1, 0, nullptr, 0, n, E, blockIdx.x, blockIdx.y);
}

// ------------------------------------------------------------------ bias add
__global__ void bias_add_rows_kernel(float *__restrict__ out, const float *__restrict__ inp,
                                     const float *__restrict__ bias, long total, int w) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < total) out[i] = inp[i] + bias[i % w];
}

// ------------------------------------------------------------------ softmax cross-entropy
// One wave per row: max, sum of exp and the gradient in three passes over the row
// (the row stays in cache); reductions are wave-level shuffles, no LDS.
__global__ __launch_bounds__(256) void softmax_xent_kernel(float *__restrict__ loss,
                                                           float *__restrict__ dlogits,
                                                           const float *__restrict__ logits,
                                                           const float *__restrict__ labels, int n,
                                                           int C, float inv_n) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= n) return;
  const float *x = logits + (long)row * C;
  float mx = -INFINITY;
  for (int j = lane; j < C; j += 64) mx = fmaxf(mx, x[j]);
  mx = wave_max(mx);
  float sum = 0.f;
  for (int j = lane; j < C; j += 64) sum += expf(x[j] - mx);
  sum = wave_sum(sum);
  const int lab = (int)labels[row];
  if (loss && lane == 0) loss[row] = -logf(expf(x[lab] - mx) / sum);
  if (dlogits) {
    float *d = dlogits + (long)row * C;
    for (int j = lane; j < C; j += 64) {
      float p = expf(x[j] - mx) / sum;
      d[j] = (j == lab ? p - 1.f : p) * inv_n;
    }
  }
}

// One workgroup per row, the row held in registers between the passes (NV float4 per thread,
// C <= 1024 NV): the logits are read once and the gradient written once, both as float4 -- an
// HBM-bound kernel of 8 bytes per element.  Sums run in a fixed order (lane, wavefront).
template <int NV>
__global__ __launch_bounds__(256) void softmax_xent_rows_kernel(float *__restrict__ loss, float *__restrict__ dlogits,
                                                                const float *__restrict__ logits,
                                                                const float *__restrict__ labels, int C, float inv_n) {
  __shared__ float part[2][4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, row = blockIdx.x, C4 = C / 4;
  const float4 *x = reinterpret_cast<const float4 *>(logits + (long)row * C);
  float4 v[NV];
  float mx = -INFINITY;
#pragma unroll
  for (int k = 0; k < NV; k++) {
    const int j = tid + 256 * k;
    v[k] = j < C4 ? x[j] : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
    mx = fmaxf(fmaxf(mx, fmaxf(v[k].x, v[k].y)), fmaxf(v[k].z, v[k].w));
  }
  mx = wave_max(mx);
  if (lane == 0) part[0][wave] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(part[0][0], part[0][1]), fmaxf(part[0][2], part[0][3]));
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < NV; k++) {  // exp(-inf) = 0 past the end of the row
    v[k].x = expf(v[k].x - mx); v[k].y = expf(v[k].y - mx); v[k].z = expf(v[k].z - mx); v[k].w = expf(v[k].w - mx);
    sum += (v[k].x + v[k].y) + (v[k].z + v[k].w);
  }
  sum = wave_sum(sum);
  if (lane == 0) part[1][wave] = sum;
  __syncthreads();
  sum = (part[1][0] + part[1][1]) + (part[1][2] + part[1][3]);
  const int lab = (int)labels[row];
  if (loss && tid == 0) loss[row] = -logf(expf(logits[(long)row * C + lab] - mx) / sum);
  if (!dlogits) return;
  float4 *d = reinterpret_cast<float4 *>(dlogits + (long)row * C);
#pragma unroll
  for (int k = 0; k < NV; k++) {
    const int j = tid + 256 * k;
    if (j >= C4) continue;
    float4 p = make_float4(v[k].x / sum, v[k].y / sum, v[k].z / sum, v[k].w / sum);
    if (lab >> 2 == j) {
      const int c = lab & 3;
      (c == 0 ? p.x : c == 1 ? p.y : c == 2 ? p.z : p.w) -= 1.f;
    }
    d[j] = make_float4(p.x * inv_n, p.y * inv_n, p.z * inv_n, p.w * inv_n);
  }
}

// ------------------------------------------------------------------ elementwise
__global__ void sgd_kernel(float *__restrict__ w, const float *__restrict__ g, float lr, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) w[i] -= lr * g[i];
}

__global__ void scale_kernel(float *__restrict__ out, const float *__restrict__ a, float s, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) out[i] = s * a[i];
}

__device__ inline float sigm(float x) { return 1.f / (1.f + expf(-x)); }

template <int OP>
__device__ inline float binop(float a, float b) {
  if constexpr (OP == CAVS_EW_ADD) return a + b;
  if constexpr (OP == CAVS_EW_SUB) return a - b;
  if constexpr (OP == CAVS_EW_MUL) return a * b;
  if constexpr (OP == CAVS_EW_DIV) return a / b;
  if constexpr (OP == CAVS_EW_SIGMOID_GRAD) return a * (b * (1.f - b));
  if constexpr (OP == CAVS_EW_TANH_GRAD) return a * (1.f - b * b);
  if constexpr (OP == CAVS_EW_RELU_GRAD) return b > 0.f ? a : 0.f;
  if constexpr (OP == CAVS_EW_EQUAL) return a == b ? 1.f : 0.f;
  return 0.f;
}

template <int OP>
__device__ inline float unop(float a) {
  if constexpr (OP == CAVS_EW_ASSIGN) return a;
  if constexpr (OP == CAVS_EW_NEG) return -a;
  if constexpr (OP == CAVS_EW_ABS) return fabsf(a);
  if constexpr (OP == CAVS_EW_SQUARE) return a * a;
  if constexpr (OP == CAVS_EW_SIGMOID) return sigm(a);
  if constexpr (OP == CAVS_EW_TANH) return tanhf(a);
  if constexpr (OP == CAVS_EW_RELU) return a > 0.f ? a : 0.f;
  return 0.f;
}

template <int OP>
__global__ void ew_binary_kernel(float *__restrict__ out, const float *__restrict__ a, size_t na,
                                 const float *__restrict__ b, size_t nb, size_t n, int accumulate) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    float v = binop<OP>(a[na == n ? i : i % na], b[nb == n ? i : i % nb]);
    out[i] = accumulate ? out[i] + v : v;
  }
}

template <int OP>
__global__ void ew_unary_kernel(float *__restrict__ out, const float *__restrict__ a, size_t n,
                                int accumulate) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    float v = unop<OP>(a[i]);
    out[i] = accumulate ? out[i] + v : v;
  }
}

inline unsigned stream_grid(size_t n) {
  size_t blocks = (n + 255) / 256, cap = (size_t)num_cus() * 16;
  return (unsigned)(blocks < cap ? blocks : cap);
}

}  // namespace cavs

using namespace cavs;

extern "C" {

int cavs_colsum(float *out, const float *inp, int ld, int n, int w, int accumulate, void *stream) {
  CAVS_REQUIRE(n >= 0 && w >= 0 && ld >= w, "cavs_colsum: bad shape n=%d w=%d ld=%d", n, w, ld);
  if (w == 0) return CAVS_OK;
  CAVS_REQUIRE(out, "cavs_colsum: null output");
  hipStream_t st = as_stream(stream);
  if (n == 0) {
    if (!accumulate) return cavs_zero(out, (size_t)w * 4, stream);
    return CAVS_OK;
  }
  CAVS_REQUIRE(inp, "cavs_colsum: null input");
  int strips = (w + 63) / 64;
  int want = (4 * num_cus() + strips - 1) / strips;
  int maxc = (n + 63) / 64;
  int chunks = want < maxc ? want : maxc;
  if (chunks < 1) chunks = 1;
  int rpc = ((n + chunks - 1) / chunks + 3) / 4 * 4;
  chunks = (n + rpc - 1) / rpc;
  if (chunks > 1 && !accumulate) {
    int rc = cavs_zero(out, (size_t)w * 4, stream);
    if (rc) return rc;
  }
  launch(colsum_kernel, dim3(strips, chunks), 256, 0, st, out, inp, ld, n, w, rpc, chunks > 1, accumulate);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_embed_fwd(float *out, int ld_out, const float *ids, const float *table, int n, int E,
                   void *stream) {
  CAVS_REQUIRE(n >= 0 && E > 0 && ld_out >= E, "cavs_embed_fwd: bad shape n=%d E=%d ld=%d", n, E, ld_out);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(out && ids && table, "cavs_embed_fwd: null pointer");
  int block = E >= 256 ? 256 : (E > 64 ? 128 : 64);
  launch(embed_fwd_kernel, (n + 3) / 4, block, 0, as_stream(stream), out, ld_out, ids, table, n, E);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_embed_pull_fwd(float *out, int ld_out, float *ids_out, const float *x, const int *rows,
                        const float *table, int n, int E, void *stream) {
  CAVS_REQUIRE(n >= 0 && E > 0 && ld_out >= E, "cavs_embed_pull_fwd: bad shape n=%d E=%d ld=%d", n, E, ld_out);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(out && ids_out && x && rows && table, "cavs_embed_pull_fwd: null pointer");
  int block = E >= 256 ? 256 : (E > 64 ? 128 : 64);
  launch(embed_pull_fwd_kernel, (n + 3) / 4, block, 0, as_stream(stream), out, ld_out, ids_out, x, rows, table, n, E);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_embed_bwd(float *dtable, const float *ids, const float *dy, int ld_dy, int n, int E,
                   void *stream) {
  CAVS_REQUIRE(n >= 0 && E > 0 && ld_dy >= E, "cavs_embed_bwd: bad shape n=%d E=%d ld=%d", n, E, ld_dy);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(dtable && ids && dy, "cavs_embed_bwd: null pointer");
  launch(embed_bwd_kernel, dim3((n + kEmbedRows - 1) / kEmbedRows, (E + kEmbedCols - 1) / kEmbedCols), 256, 0,
         as_stream(stream), dtable, ids, dy, ld_dy, n, E);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_bias_add_rows(float *out, const float *inp, const float *bias, int n, int w, void *stream) {
  CAVS_REQUIRE(n >= 0 && w >= 0, "cavs_bias_add_rows: bad shape n=%d w=%d", n, w);
  long total = (long)n * w;
  if (total == 0) return CAVS_OK;
  CAVS_REQUIRE(out && inp && bias, "cavs_bias_add_rows: null pointer");
  launch(bias_add_rows_kernel, (unsigned)((total + 255) / 256), 256, 0, as_stream(stream), out, inp, bias, total, w);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_softmax_xent(float *loss, float *dlogits, const float *logits, const float *labels, int n,
                      int C, void *stream) {
  return cavs_softmax_xent_part(loss, dlogits, logits, labels, n, C, n, stream);
}

int cavs_softmax_xent_part(float *loss, float *dlogits, const float *logits, const float *labels, int n,
                           int C, int n_total, void *stream) {
  CAVS_REQUIRE(n >= 0 && C > 0 && n_total >= n, "cavs_softmax_xent: bad shape n=%d of %d C=%d", n, n_total, C);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(logits && labels, "cavs_softmax_xent: null pointer");
  const float inv_n = 1.f / (float)n_total;
  hipStream_t st = as_stream(stream);
  // wide rows: a workgroup per row with the row in registers; narrow ones: a wavefront per row
  if (C >= 512 && C % 4 == 0 && C <= 16384 && aligned16(logits) && (!dlogits || aligned16(dlogits))) {
    if (C <= 2048) launch(softmax_xent_rows_kernel<2>, n, 256, 0, st, loss, dlogits, logits, labels, C, inv_n);
    else if (C <= 4096) launch(softmax_xent_rows_kernel<4>, n, 256, 0, st, loss, dlogits, logits, labels, C, inv_n);
    else if (C <= 10240) launch(softmax_xent_rows_kernel<10>, n, 256, 0, st, loss, dlogits, logits, labels, C, inv_n);
    else launch(softmax_xent_rows_kernel<16>, n, 256, 0, st, loss, dlogits, logits, labels, C, inv_n);
  } else {
    launch(softmax_xent_kernel, (n + 3) / 4, 256, 0, st, loss, dlogits, logits, labels, n, C, inv_n);
  }
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_sgd(float *w, const float *g, float lr, size_t n, void *stream) {
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(w && g, "cavs_sgd: null pointer");
  launch(sgd_kernel, stream_grid(n), 256, 0, as_stream(stream), w, g, lr, n);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_scale(float *out, const float *a, float s, size_t n, void *stream) {
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(out && a, "cavs_scale: null pointer");
  launch(scale_kernel, stream_grid(n), 256, 0, as_stream(stream), out, a, s, n);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_ew_binary(int op, float *out, const float *a, size_t na, const float *b, size_t nb,
                   size_t n, int accumulate, void *stream) {
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(out && a && b && na > 0 && nb > 0 && na <= n && nb <= n, "cavs_ew_binary: bad operands (na=%zu nb=%zu n=%zu)", na, nb, n);
  hipStream_t st = as_stream(stream);
  unsigned grid = stream_grid(n);
#define CAVS_EWB(OP) case OP: launch(ew_binary_kernel<OP>, grid, 256, 0, st, out, a, na, b, nb, n, accumulate); break
  switch (op) {
    CAVS_EWB(CAVS_EW_ADD); CAVS_EWB(CAVS_EW_SUB); CAVS_EWB(CAVS_EW_MUL); CAVS_EWB(CAVS_EW_DIV);
    CAVS_EWB(CAVS_EW_SIGMOID_GRAD); CAVS_EWB(CAVS_EW_TANH_GRAD); CAVS_EWB(CAVS_EW_RELU_GRAD);
    CAVS_EWB(CAVS_EW_EQUAL);
    default: return set_error(CAVS_EINVAL, "cavs_ew_binary: unknown op %d", op);
  }
#undef CAVS_EWB
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_ew_unary(int op, float *out, const float *a, size_t n, int accumulate, void *stream) {
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(out && a, "cavs_ew_unary: null pointer");
  hipStream_t st = as_stream(stream);
  unsigned grid = stream_grid(n);
#define CAVS_EWU(OP) case OP: launch(ew_unary_kernel<OP>, grid, 256, 0, st, out, a, n, accumulate); break
  switch (op) {
    CAVS_EWU(CAVS_EW_ASSIGN); CAVS_EWU(CAVS_EW_NEG); CAVS_EWU(CAVS_EW_ABS); CAVS_EWU(CAVS_EW_SQUARE);
    CAVS_EWU(CAVS_EW_SIGMOID); CAVS_EWU(CAVS_EW_TANH); CAVS_EWU(CAVS_EW_RELU);
    default: return set_error(CAVS_EINVAL, "cavs_ew_unary: unknown op %d", op);
  }
#undef CAVS_EWU
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

}  // extern "C"
