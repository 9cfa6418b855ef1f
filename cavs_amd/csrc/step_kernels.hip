// Per-step work around the rounds, folded into few launches: the classifier head
// (FullyConnected + SoftmaxEntropyLoss and their gradients) for a handful of classes, the
// SGD update of all dense parameters in one launch, a row-sparse update of the embedding
// table, and the bias gradient (column sums of the four gate blocks) in one launch.
// Every one of these is a few microseconds of HBM traffic; as separate library-style
// launches their fixed costs add up to more than a round of the vertex function.
#include <vector>

#include "common.h"
#include "round_common.h"

namespace cavs {

__device__ inline float wsum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// ------------------------------------------------------------------ classifier head
// One wavefront per row, lane l owning columns l, l+64, ... (Q of them) of x and of every row
// of W, all in registers: logits = x * W^T + b by C dot products reduced across the wave,
// softmax / loss / d logits, d x = d logits * W.  The weight and bias gradients accumulate in
// registers over the rows a wavefront owns, are combined per workgroup through LDS and parked
// in `part[workgroup]`; a second kernel sums the workgroups in index order.
template <int C, int Q>
__global__ __launch_bounds__(256) void fc_xent_kernel(const float *__restrict__ X, const float *__restrict__ W,
                                                      const float *__restrict__ b, const float *__restrict__ labels,
                                                      float *__restrict__ loss, float *__restrict__ logits,
                                                      float *__restrict__ dX, float *__restrict__ part, int n, int H,
                                                      float inv_n) {
  extern __shared__ float sm[];  // [4][C*H] weight-gradient partials, then [4][C] bias
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int CH = C * H;
  const bool grad = part != nullptr;
  float w[C][Q], acc[C][Q], dbacc[C], bias[C];
#pragma unroll
  for (int c = 0; c < C; c++) {
    bias[c] = b[c];
    dbacc[c] = 0.f;
#pragma unroll
    for (int q = 0; q < Q; q++) {
      const int col = q * 64 + lane;
      w[c][q] = col < H ? W[c * H + col] : 0.f;
      acc[c][q] = 0.f;
    }
  }
  // the next row of this wavefront is fetched while the current one goes through its chain of
  // wave reductions and exponentials
  const int step = gridDim.x * 4;
  float xn[Q];
  int lab_n = 0;
  auto fetch = [&](int row) {
    if (row >= n) return;
    const float *x = X + (long)row * H;
#pragma unroll
    for (int q = 0; q < Q; q++) {
      const int col = q * 64 + lane;
      xn[q] = col < H ? x[col] : 0.f;
    }
    lab_n = (int)labels[row];
  };
  fetch(blockIdx.x * 4 + wave);
  for (int row = blockIdx.x * 4 + wave; row < n; row += step) {
    float xv[Q], z[C];
#pragma unroll
    for (int q = 0; q < Q; q++) xv[q] = xn[q];
    const int lab = lab_n;
    fetch(row + step);
    float mx = -INFINITY;
#pragma unroll
    for (int c = 0; c < C; c++) {
      float s = 0.f;
#pragma unroll
      for (int q = 0; q < Q; q++) s += xv[q] * w[c][q];
      z[c] = wsum(s) + bias[c];
      mx = fmaxf(mx, z[c]);
    }
    // cavs/backend/op_impl_softmax_entropy_logits_loss.cu:94-140, :212-250
    // every lane repeats this per row: exp through v_exp_f32, one reciprocal for all classes, and
    // -log(e_label / sum) taken as log(sum) - (z_label - max)
    float sum = 0.f, zl = 0.f, e[C];
#pragma unroll
    for (int c = 0; c < C; c++) {
      e[c] = __builtin_amdgcn_exp2f((z[c] - mx) * 1.4426950408889634f);
      sum += e[c];
      if (c == lab) zl = z[c];
    }
    if (lane == 0) loss[row] = __builtin_amdgcn_logf(sum) * 0.6931471805599453f - (zl - mx);
    if (logits) {
#pragma unroll
      for (int c = 0; c < C; c++)
        if (lane == c) logits[(long)row * C + c] = z[c];
    }
    if (!grad) continue;
    float d[C];
    const float inv_sum = __builtin_amdgcn_rcpf(sum);
#pragma unroll
    for (int c = 0; c < C; c++) {
      const float p = e[c] * inv_sum;
      d[c] = (c == lab ? p - 1.f : p) * inv_n;
      dbacc[c] += d[c];
    }
#pragma unroll
    for (int q = 0; q < Q; q++) {
      float dx = 0.f;
#pragma unroll
      for (int c = 0; c < C; c++) {
        dx += d[c] * w[c][q];
        acc[c][q] += d[c] * xv[q];
      }
      const int col = q * 64 + lane;
      if (col < H) dX[(long)row * H + col] = dx;
    }
  }
  if (!grad) return;
  float *mine = sm + wave * CH, *sdb = sm + 4 * CH;
#pragma unroll
  for (int c = 0; c < C; c++) {
#pragma unroll
    for (int q = 0; q < Q; q++) {
      const int col = q * 64 + lane;
      if (col < H) mine[c * H + col] = acc[c][q];
    }
    if (lane == 0) sdb[wave * C + c] = dbacc[c];
  }
  __syncthreads();
  float *out = part + (long)blockIdx.x * (CH + C);
  for (int i = tid; i < CH; i += 256) out[i] = (sm[i] + sm[CH + i]) + (sm[2 * CH + i] + sm[3 * CH + i]);
  if (tid < C) out[CH + tid] = (sdb[tid] + sdb[C + tid]) + (sdb[2 * C + tid] + sdb[3 * C + tid]);
}

// out[i] = sum over the workgroups' partials: four interleaved slices per output, each added
// in index order, combined in a fixed order
__device__ inline void sum_parts_block(const float *__restrict__ part, int nparts, int total, int CH,
                                       float *__restrict__ dW, float *__restrict__ db, int block, float (&s)[4][64]) {
  const int o = threadIdx.x & 63, q = threadIdx.x >> 6;
  const int i = block * 64 + o;
  float a0 = 0.f, a1 = 0.f;
  if (i < total) {
    int p = q;
    // (eight loads in flight; the same additions in the same order as the loops below)
    for (; p + 28 < nparts; p += 32) {
      float v[8];
#pragma unroll
      for (int k = 0; k < 8; k++) v[k] = part[(long)(p + 4 * k) * total + i];
#pragma unroll
      for (int k = 0; k < 8; k += 2) {
        a0 += v[k];
        a1 += v[k + 1];
      }
    }
    for (; p + 4 < nparts; p += 8) {
      a0 += part[(long)p * total + i];
      a1 += part[(long)(p + 4) * total + i];
    }
    for (; p < nparts; p += 4) a0 += part[(long)p * total + i];
  }
  s[q][o] = a0 + a1;
  __syncthreads();
  if (q == 0 && i < total) {
    const float v = (s[0][o] + s[1][o]) + (s[2][o] + s[3][o]);
    if (i < CH) dW[i] = v; else db[i - CH] = v;
  }
}

__global__ __launch_bounds__(256) void fc_xent_reduce_kernel(const float *__restrict__ part, int nparts, int total,
                                                             int CH, float *__restrict__ dW, float *__restrict__ db) {
  __shared__ float s[4][64];
  sum_parts_block(part, nparts, total, CH, dW, db, blockIdx.x, s);
}

static int head_blocks(int n) {
  int want = (n + 7) / 8;  // two rows per wavefront
  int cap = num_cus() * 3 / 2;  // (C3: 0.4086 ms with one workgroup per CU, 0.4076 with one and a half, 0.4081 with two)
  return want < cap ? (want < 1 ? 1 : want) : cap;
}

// columns per lane (Q) for a width; the weights and their gradient live in 2*C*Q registers
static int head_q(int H) { return H <= 256 ? 4 : (H <= 512 ? 8 : 16); }
static bool head_supported(int H, int C) {
  return C >= 1 && C <= 8 && H >= 1 && H <= 1024 && C * head_q(H) <= 64 && (size_t)(4 * C * H + 4 * C) * 4 <= 64 * 1024;
}

// ------------------------------------------------------------------ SGD over several tensors
constexpr int kMaxTensors = 8;
struct SgdBatch {
  float *w[kMaxTensors];
  const float *g[kMaxTensors];
  size_t end[kMaxTensors];  // running element count
  int count;
};

__global__ void sgd_multi_kernel(SgdBatch t, float lr) {
  const size_t total = t.end[t.count - 1];
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    int k = 0;
    while (i >= t.end[k]) k++;
    const size_t j = i - (k ? t.end[k - 1] : 0);
    t.w[k][j] -= lr * t.g[k][j];
  }
}

// ------------------------------------------------------------------ row-sparse embedding update
// A row that was looked up several times in the step is updated once: the first workgroup
// to raise the row's stamp to this step's epoch owns it.  A workgroup takes kSgdChunk lookups
// and asks for a row once however often it occurs among them (parse trees look up one and
// the same row for every internal vertex; one atomic per vertex would serialise on it).
constexpr int kSgdChunk = 16;
struct EmbedSgdLds {
  int row[kSgdChunk];
  long owned[kSgdChunk];
  int n_owned;
};

__device__ inline void embed_sgd_block(float *__restrict__ table, const float *__restrict__ dtable,
                                       const float *__restrict__ ids, int n, int E, float lr, int *__restrict__ stamp,
                                       int epoch, int block, EmbedSgdLds &lds) {
  int (&row)[kSgdChunk] = lds.row;
  long (&owned)[kSgdChunk] = lds.owned;
  int &n_owned = lds.n_owned;
  const int v0 = block * kSgdChunk, tid = threadIdx.x;
  if (tid < kSgdChunk) row[tid] = v0 + tid < n ? (int)ids[v0 + tid] : -1 - tid;
  if (tid == 0) n_owned = 0;
  __syncthreads();
  if (tid < kSgdChunk) {
    bool first = row[tid] >= 0;
    for (int r = 0; r < tid; r++) first = first && row[r] != row[tid];
    if (first && atomicMax(stamp + row[tid], epoch) < epoch)
      owned[atomicAdd(&n_owned, 1)] = (long)(int)(ids[v0 + tid] * (float)E);
  }
  __syncthreads();
  // every owned row of a column is in flight before the first store
  const int cnt = n_owned;
  for (int c = tid; c < E; c += blockDim.x) {
    float t[kSgdChunk], d[kSgdChunk];
#pragma unroll
    for (int r = 0; r < kSgdChunk; r++)
      if (r < cnt) {
        t[r] = table[owned[r] + c];
        d[r] = dtable[owned[r] + c];
      }
#pragma unroll
    for (int r = 0; r < kSgdChunk; r++)
      if (r < cnt) table[owned[r] + c] = t[r] - lr * d[r];
  }
}

__global__ void embed_sgd_kernel(float *__restrict__ table, const float *__restrict__ dtable,
                                 const float *__restrict__ ids, int n, int E, float lr, int *__restrict__ stamp,
                                 int epoch) {
  __shared__ EmbedSgdLds lds;
  embed_sgd_block(table, dtable, ids, n, E, lr, stamp, epoch, blockIdx.x, lds);
}

__global__ void embed_zero_rows_kernel(float *__restrict__ dtable, const float *__restrict__ ids, int E) {
  const long off = (long)(int)(ids[blockIdx.x] * (float)E);
  for (int c = threadIdx.x; c < E; c += blockDim.x) dtable[off + c] = 0.f;
}

// ------------------------------------------------------------------ several small jobs, one launch
// The jobs around the rounds that do not depend on each other (the weight transposes and the
// clearing of the embedding gradient before backward; the updates of the dense parameters and of
// the embedding table after it) are a few microseconds each, most of it launch and drain.  One
// launch runs a list of them: workgroup b belongs to job k with first[k] <= b < first[k+1].
constexpr int kMaxTasks = 12;
struct TaskList {
  cavs_task t[kMaxTasks];
  int first[kMaxTasks + 1];
  int count;
  const int *guard;  // CAVS_TASK_GUARD: when the word it points at is not zero, no job of the launch runs
};

__global__ __launch_bounds__(256) void tasks_kernel(TaskList L) {
  __shared__ union {
    float tile[32][33];
    float pk[16][65];
    EmbedSgdLds sgd;
    float sums[4][64];
  } lds;
  if (L.guard && __hip_atomic_load(L.guard, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) return;
  int k = 0;
  while (k + 1 < L.count && (int)blockIdx.x >= L.first[k + 1]) k++;
  const cavs_task &t = L.t[k];
  const int b = blockIdx.x - L.first[k], nb = L.first[k + 1] - L.first[k], tid = threadIdx.x;
  switch (t.kind) {
    case CAVS_TASK_TRANSPOSE: {  // p0[c][r] = p1[r][c], n0 rows, n1 columns
      const float *__restrict__ in = static_cast<const float *>(t.p1);
      float *__restrict__ out = static_cast<float *>(t.p0);
      const int rows = (int)t.n0, cols = (int)t.n1, gx = (cols + 31) / 32;
      const int c0 = (b % gx) * 32, r0 = (b / gx) * 32, tx = tid & 31, ty = tid >> 5;
      for (int i = ty; i < 32; i += 8)
        if (r0 + i < rows && c0 + tx < cols) lds.tile[i][tx] = in[(long)(r0 + i) * cols + c0 + tx];
      __syncthreads();
      for (int i = ty; i < 32; i += 8)
        if (c0 + i < cols && r0 + tx < rows) out[(long)(c0 + i) * rows + r0 + tx] = lds.tile[tx][i];
      break;
    }
    case CAVS_TASK_SGD_TRANSPOSE: {  // p1 -= f0 * p2 (if p2 is given), then p0[c][r] = p1[r][c]
      float *__restrict__ w = static_cast<float *>(t.p1);
      const float *__restrict__ g = static_cast<const float *>(t.p2);
      float *__restrict__ out = static_cast<float *>(t.p0);
      const int rows = (int)t.n0, cols = (int)t.n1, gx = (cols + 31) / 32;
      const int c0 = (b % gx) * 32, r0 = (b / gx) * 32, tx = tid & 31, ty = tid >> 5;
      for (int i = ty; i < 32; i += 8)
        if (r0 + i < rows && c0 + tx < cols) {
          const long at = (long)(r0 + i) * cols + c0 + tx;
          float v = w[at];
          if (g) {
            v -= t.f0 * g[at];
            w[at] = v;
          }
          lds.tile[i][tx] = v;
        }
      __syncthreads();
      for (int i = ty; i < 32; i += 8)
        if (c0 + i < cols && r0 + tx < rows) out[(long)(c0 + i) * rows + r0 + tx] = lds.tile[tx][i];
      break;
    }
    case CAVS_TASK_PACK_T: {
      // B = p1^T ([K = n1, N = n0]; p1 is [n0, n1] row-major) in the tile-major layout the round
      // kernels' packed product loops read: for k-group g (16 k) and column tile t (16 columns)
      // 256 consecutive floats [slot][x][c] hold B[16g + 4 slot + c][16t + x], so that lane
      // (x, slot) of a wavefront fetches its four k of a k-group as one float4 and the wavefront's
      // sixty-four float4 are one contiguous kilobyte.  A workgroup moves 16 columns x 64 k.
      const float *__restrict__ in = static_cast<const float *>(t.p1);
      float4 *__restrict__ out = static_cast<float4 *>(t.p0);
      const int N = (int)t.n0, K = (int)t.n1, kc = K / 64;
      const int tcol = b / kc, k0 = (b % kc) * 64, r = tid >> 4, q = tid & 15;
      const float4 v = *reinterpret_cast<const float4 *>(in + (long)(16 * tcol + r) * K + k0 + 4 * q);
      const long g = k0 / 16 + q / 4;
      out[((g * (N / 16) + tcol) * 4 + (q & 3)) * 16 + r] = v;
      break;
    }
    case CAVS_TASK_SGD_PACK: {
      // B = p1 ([K = n0, N = n1] row-major) after p1 -= f0 * p2 (if p2 is given), packed tile-major
      // into p0 as above.  A workgroup moves one k-group x 64 columns through LDS.
      float *__restrict__ w = static_cast<float *>(t.p1);
      const float *__restrict__ g = static_cast<const float *>(t.p2);
      float4 *__restrict__ out = static_cast<float4 *>(t.p0);
      const int N = (int)t.n1, nc = N / 64;
      const int kg = b / nc, cb = b % nc, kk = tid >> 4, q = tid & 15;
      const long at = (long)(16 * kg + kk) * N + 64 * cb + 4 * q;
      float4 v = *reinterpret_cast<const float4 *>(w + at);
      if (g) {
        const float4 d = *reinterpret_cast<const float4 *>(g + at);
        v.x -= t.f0 * d.x; v.y -= t.f0 * d.y; v.z -= t.f0 * d.z; v.w -= t.f0 * d.w;
        *reinterpret_cast<float4 *>(w + at) = v;
      }
      lds.pk[kk][4 * q] = v.x; lds.pk[kk][4 * q + 1] = v.y; lds.pk[kk][4 * q + 2] = v.z; lds.pk[kk][4 * q + 3] = v.w;
      __syncthreads();
      const int tt = tid >> 6, slot = (tid >> 4) & 3, x = tid & 15, col = 16 * tt + x;
      out[(((long)kg * (N / 16) + 4 * cb + tt) * 4 + slot) * 16 + x] =
          make_float4(lds.pk[4 * slot][col], lds.pk[4 * slot + 1][col], lds.pk[4 * slot + 2][col], lds.pk[4 * slot + 3][col]);
      break;
    }
    case CAVS_TASK_ZERO_ROWS: {  // p0[int(p1[r] * n1) ...] = 0 for n1 columns, r < n0: one row per workgroup
      float *__restrict__ dtable = static_cast<float *>(t.p0);
      const float *__restrict__ ids = static_cast<const float *>(t.p1);
      const int E = (int)t.n1;
      const long off = (long)(int)(ids[b] * (float)E);
      for (int c = tid; c < E; c += 256) dtable[off + c] = 0.f;
      break;
    }
    case CAVS_TASK_SGD: {  // p0[i] -= f0 * p1[i], i < n0
      float *__restrict__ w = static_cast<float *>(t.p0);
      const float *__restrict__ g = static_cast<const float *>(t.p1);
      const size_t n = (size_t)t.n0, stride = (size_t)nb * 256;
      for (size_t i = (size_t)b * 256 + tid; i < n; i += stride) w[i] -= t.f0 * g[i];
      break;
    }
    case CAVS_TASK_EMBED_SGD:  // cavs_embed_sgd(p0 = table, p1 = dtable, p2 = ids, n0 = n, n1 = E, f0 = lr, p3 = stamp, n2 = epoch)
      embed_sgd_block(static_cast<float *>(t.p0), static_cast<const float *>(t.p1), static_cast<const float *>(t.p2),
                      (int)t.n0, (int)t.n1, t.f0, static_cast<int *>(t.p3), (int)t.n2, b, lds.sgd);
      break;
    case CAVS_TASK_BLOCKS_SGD: {  // block k of p1 ([n1 blocks of n0]) -> block perm(k) of p2 (and p0 -= f0 * it)
      float *__restrict__ w = static_cast<float *>(t.p0);
      const float *__restrict__ src = static_cast<const float *>(t.p1);
      float *__restrict__ gout = static_cast<float *>(t.p2);
      const int bw = (int)t.n0, total = bw * (int)t.n1;
      const int parts = (int)(t.n2 >> 32);  // 0 or 1: p1 is the row itself; more: rows to add up, in index order
      for (int i = b * 256 + tid; i < total; i += nb * 256) {
        const int k = i / bw, d = (int)((t.n2 >> (4 * k)) & 15) * bw + i % bw;
        float g = src[i];
        for (int q = 1; q < parts; q++) g += src[(long)q * total + i];
        if (gout) gout[d] = g;
        if (w) w[d] -= t.f0 * g;
      }
      break;
    }
    case CAVS_TASK_SUM_PARTS:  // p1[i] (i < n2) or p2[i - n2] = sum over p < n0 of p0[p * n1 + i], i < n1
      sum_parts_block(static_cast<const float *>(t.p0), (int)t.n0, (int)t.n1, (int)t.n2, static_cast<float *>(t.p1),
                      static_cast<float *>(t.p2), b, lds.sums);
      break;
    case CAVS_TASK_TREELSTM_GATES_ROWS: {  // cavs_treelstm_bwd_gates_rows as a job
      const BwdGatesRowsArgs a{static_cast<const int *>(t.p0), static_cast<const float *>(t.p1), static_cast<const int *>(t.p2),
                               static_cast<const float *>(t.p3), static_cast<const float *>(t.p4), static_cast<float *>(t.p5),
                               (long)(t.n2 >> 32), static_cast<float *>(t.p6), static_cast<float *>(t.p7), (int)t.n0, (int)t.n1,
                               (int)(t.n2 & 0xffffffffll)};
      treelstm_gates_rows_at<4>(a, (long)b * 256 + tid);
      break;
    }
    default: break;
  }
}

// ------------------------------------------------------------------ column sums of column blocks
// out[dst[k]*bw + c] = sum over rows of inp[r][k*bw + c], for nb blocks of bw columns.
// Workgroup = 4 wavefronts over a strip of 64 columns and a chunk of rows; chunk sums go to
// part[chunk][nb*bw]; the second kernel adds the chunks in index order and permutes.
struct BlockMap {
  int dst[8];
};

__global__ __launch_bounds__(256) void colsum_part_kernel(float *__restrict__ part, const float *__restrict__ inp,
                                                          long ld, int n, int w, int rows_per_chunk) {
  __shared__ float s[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = blockIdx.x * 64 + lane;
  const int r0 = blockIdx.y * rows_per_chunk, r1 = min(n, r0 + rows_per_chunk);
  float a0 = 0.f, a1 = 0.f;
  if (col < w) {
    int r = r0 + wave;
    for (; r + 4 < r1; r += 8) {
      a0 += inp[(long)r * ld + col];
      a1 += inp[(long)(r + 4) * ld + col];
    }
    for (; r < r1; r += 4) a0 += inp[(long)r * ld + col];
  }
  s[wave][lane] = a0 + a1;
  __syncthreads();
  if (wave == 0 && col < w) part[(long)blockIdx.y * w + col] = (s[0][lane] + s[1][lane]) + (s[2][lane] + s[3][lane]);
}

__global__ __launch_bounds__(256) void colsum_blocks_reduce_kernel(float *__restrict__ out, const float *__restrict__ part,
                                                                   int chunks, int w, int bw, BlockMap map) {
  __shared__ float s[4][64];
  const int o = threadIdx.x & 63, q = threadIdx.x >> 6;
  const int col = blockIdx.x * 64 + o;
  float a = 0.f;
  if (col < w)
    for (int c = q; c < chunks; c += 4) a += part[(long)c * w + col];
  s[q][o] = a;
  __syncthreads();
  if (q == 0 && col < w) out[map.dst[col / bw] * bw + col % bw] = (s[0][o] + s[1][o]) + (s[2][o] + s[3][o]);
}

static int colsum_chunks(int n) {
  int c = (n + 127) / 128;
  return c < 1 ? 1 : (c > 32 ? 32 : c);
}

}  // namespace cavs

using namespace cavs;

extern "C" {

size_t cavs_fc_softmax_xent_workspace(int n, int H, int C) {
  if (n <= 0 || !head_supported(H, C)) return 0;
  return (size_t)head_blocks(n) * ((size_t)C * H + C) * sizeof(float);
}

int cavs_fc_softmax_xent_parts(int n) { return n > 0 ? head_blocks(n) : 0; }

int cavs_fc_softmax_xent(const float *X, const float *W, const float *b, const float *labels, float *loss,
                         float *logits, float *dX, float *dW, float *db, void *workspace,
                         size_t workspace_bytes, int n, int H, int C, void *stream) {
  CAVS_REQUIRE(n >= 0 && head_supported(H, C), "cavs_fc_softmax_xent: unsupported shape n=%d H=%d C=%d (C <= 8, H <= 1024, C * columns-per-lane <= 64)", n, H, C);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(X && W && b && labels && loss, "cavs_fc_softmax_xent: null pointer");
  const bool grad = dX || dW || db;
  const bool deferred = dX && !dW && !db;  // the caller sums the partials (CAVS_TASK_SUM_PARTS)
  CAVS_REQUIRE(!grad || deferred || (dX && dW && db), "cavs_fc_softmax_xent: dX alone, or dX, dW and db, or none of them");
  const int blocks = head_blocks(n);
  const size_t need = (size_t)blocks * ((size_t)C * H + C) * sizeof(float);
  CAVS_REQUIRE(!grad || (workspace && workspace_bytes >= need), "cavs_fc_softmax_xent: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  float *part = grad ? static_cast<float *>(workspace) : nullptr;
  const size_t lds = (size_t)(4 * C * H + 4 * C) * sizeof(float);
  hipStream_t st = as_stream(stream);
  const float inv_n = 1.f / (float)n;
  const int q = head_q(H);
#define CAVS_HEAD(CC)                                                                                              \
  case CC:                                                                                                         \
    if (q == 4) launch(fc_xent_kernel<CC, 4>, blocks, 256, lds, st, X, W, b, labels, loss, logits, dX, part, n, H, inv_n);       \
    else if (q == 8) launch(fc_xent_kernel<CC, 8>, blocks, 256, lds, st, X, W, b, labels, loss, logits, dX, part, n, H, inv_n);  \
    else launch(fc_xent_kernel<(CC > 4 ? 1 : CC), 16>, blocks, 256, lds, st, X, W, b, labels, loss, logits, dX, part, n, H, inv_n); \
    break
  switch (C) {
    CAVS_HEAD(1); CAVS_HEAD(2); CAVS_HEAD(3); CAVS_HEAD(4); CAVS_HEAD(5); CAVS_HEAD(6); CAVS_HEAD(7); CAVS_HEAD(8);
  }
#undef CAVS_HEAD
  CAVS_LAUNCH_CHECK();
  if (grad && !deferred) {
    const int total = C * H + C;
    launch(fc_xent_reduce_kernel, (total + 63) / 64, 256, 0, st, part, blocks, total, C * H, dW, db);
    CAVS_LAUNCH_CHECK();
  }
  return CAVS_OK;
}

int cavs_run_tasks(int count, const cavs_task *tasks, void *stream) {
  CAVS_REQUIRE(count >= 0 && count <= kMaxTasks + 1, "cavs_run_tasks: %d jobs, at most %d and a guard", count, kMaxTasks);
  CAVS_REQUIRE(count == 0 || tasks, "cavs_run_tasks: null list");
  TaskList L{};
  int k = 0;
  for (int i = 0; i < count; i++) {
    const cavs_task &t = tasks[i];
    long blocks = 0;
    if (t.kind == CAVS_TASK_GUARD) {
      CAVS_REQUIRE(t.p0 && !L.guard, "cavs_run_tasks: job %d: a guard needs a word to watch, and a launch takes one guard", i);
      L.guard = static_cast<const int *>(t.p0);
      continue;
    }
    switch (t.kind) {
      case CAVS_TASK_TRANSPOSE:
        CAVS_REQUIRE(t.n0 >= 0 && t.n1 >= 0 && t.n0 < (1 << 30) && t.n1 < (1 << 30), "cavs_run_tasks: job %d: bad transpose shape", i);
        if (t.n0 == 0 || t.n1 == 0) continue;
        CAVS_REQUIRE(t.p0 && t.p1 && t.p0 != t.p1, "cavs_run_tasks: job %d: null or aliased pointer", i);
        blocks = ((t.n0 + 31) / 32) * ((t.n1 + 31) / 32);
        break;
      case CAVS_TASK_SGD_TRANSPOSE:
        CAVS_REQUIRE(t.n0 >= 0 && t.n1 >= 0 && t.n0 < (1 << 30) && t.n1 < (1 << 30), "cavs_run_tasks: job %d: bad transpose shape", i);
        if (t.n0 == 0 || t.n1 == 0) continue;
        CAVS_REQUIRE(t.p0 && t.p1 && t.p0 != t.p1 && t.p0 != t.p2, "cavs_run_tasks: job %d: null or aliased pointer", i);
        blocks = ((t.n0 + 31) / 32) * ((t.n1 + 31) / 32);
        break;
      case CAVS_TASK_PACK_T:
        CAVS_REQUIRE(t.n0 >= 0 && t.n1 >= 0 && t.n0 < (1 << 24) && t.n1 < (1 << 24) && t.n0 % 16 == 0 && t.n1 % 64 == 0,
                     "cavs_run_tasks: job %d: bad shape to pack (rows a multiple of 16, columns of 64)", i);
        if (t.n0 == 0 || t.n1 == 0) continue;
        CAVS_REQUIRE(t.p0 && t.p1 && t.p0 != t.p1, "cavs_run_tasks: job %d: null or aliased pointer", i);
        CAVS_REQUIRE(aligned16(t.p0) && aligned16(t.p1), "cavs_run_tasks: job %d: pack needs 16-byte aligned pointers", i);
        blocks = (t.n0 / 16) * (t.n1 / 64);
        break;
      case CAVS_TASK_SGD_PACK:
        CAVS_REQUIRE(t.n0 >= 0 && t.n1 >= 0 && t.n0 < (1 << 24) && t.n1 < (1 << 24) && t.n0 % 16 == 0 && t.n1 % 64 == 0,
                     "cavs_run_tasks: job %d: bad shape to pack (rows a multiple of 16, columns of 64)", i);
        if (t.n0 == 0 || t.n1 == 0) continue;
        CAVS_REQUIRE(t.p0 && t.p1 && t.p0 != t.p1 && t.p0 != t.p2, "cavs_run_tasks: job %d: null or aliased pointer", i);
        CAVS_REQUIRE(aligned16(t.p0) && aligned16(t.p1) && aligned16(t.p2), "cavs_run_tasks: job %d: pack needs 16-byte aligned pointers", i);
        blocks = (t.n0 / 16) * (t.n1 / 64);
        break;
      case CAVS_TASK_ZERO_ROWS:
        CAVS_REQUIRE(t.n0 >= 0 && t.n1 > 0 && t.n1 < (1 << 30), "cavs_run_tasks: job %d: bad shape", i);
        if (t.n0 == 0) continue;
        CAVS_REQUIRE(t.p0 && t.p1, "cavs_run_tasks: job %d: null pointer", i);
        blocks = t.n0;
        break;
      case CAVS_TASK_SGD: {
        CAVS_REQUIRE(t.n0 >= 0, "cavs_run_tasks: job %d: negative size", i);
        if (t.n0 == 0) continue;
        CAVS_REQUIRE(t.p0 && t.p1, "cavs_run_tasks: job %d: null pointer", i);
        const long want = (t.n0 + 1023) / 1024, cap = (long)num_cus() * 4;
        blocks = want < cap ? want : cap;
        break;
      }
      case CAVS_TASK_EMBED_SGD:
        CAVS_REQUIRE(t.n0 >= 0 && t.n1 > 0 && t.n1 < (1 << 30), "cavs_run_tasks: job %d: bad shape", i);
        if (t.n0 == 0) continue;
        CAVS_REQUIRE(t.p0 && t.p1 && t.p2 && t.p3, "cavs_run_tasks: job %d: null pointer", i);
        blocks = (t.n0 + kSgdChunk - 1) / kSgdChunk;
        break;
      case CAVS_TASK_BLOCKS_SGD: {
        CAVS_REQUIRE(t.n0 >= 0 && t.n1 >= 0 && t.n1 <= 8 && t.n0 < (1 << 26) && t.n2 >= 0 && (t.n2 >> 32) <= 4096,
                     "cavs_run_tasks: job %d: bad shape", i);
        if (t.n0 == 0 || t.n1 == 0) continue;
        CAVS_REQUIRE(t.p1 && (t.p0 || t.p2), "cavs_run_tasks: job %d: null pointer", i);
        unsigned seen = 0;
        for (int k = 0; k < (int)t.n1; k++) {
          const int d = (int)((t.n2 >> (4 * k)) & 15);
          CAVS_REQUIRE(d < (int)t.n1 && !(seen >> d & 1u), "cavs_run_tasks: job %d: the block map is not a permutation", i);
          seen |= 1u << d;
        }
        blocks = (t.n0 * t.n1 + 1023) / 1024;
        break;
      }
      case CAVS_TASK_TREELSTM_GATES_ROWS: {
        const long long ld = t.n2 >> 32;
        CAVS_REQUIRE(t.n0 >= 0 && t.n0 < (1 << 24) && t.n1 > 0 && t.n1 < (1 << 20) && t.n1 % 4 == 0 && t.n2 >= 0 && ld >= 4 * t.n1,
                     "cavs_run_tasks: job %d: bad shape of the gate gradients of listed rows", i);
        if (t.n0 == 0) continue;
        CAVS_REQUIRE(t.p0 && t.p1 && t.p2 && t.p3 && t.p4 && t.p5 && t.p6 && t.p7, "cavs_run_tasks: job %d: null pointer", i);
        blocks = (t.n0 * (t.n1 / 4) + 255) / 256;
        break;
      }
      case CAVS_TASK_SUM_PARTS:
        CAVS_REQUIRE(t.n0 >= 0 && t.n1 >= 0 && t.n1 < (1 << 30) && t.n0 < (1 << 30) && t.n2 >= 0 && t.n2 <= t.n1,
                     "cavs_run_tasks: job %d: bad shape", i);
        if (t.n1 == 0) continue;
        CAVS_REQUIRE(t.p0 && (t.n2 == 0 || t.p1) && (t.n2 == t.n1 || t.p2), "cavs_run_tasks: job %d: null pointer", i);
        blocks = (t.n1 + 63) / 64;
        break;
      default:
        CAVS_REQUIRE(false, "cavs_run_tasks: job %d: unknown kind %d", i, t.kind);
    }
    CAVS_REQUIRE(k < kMaxTasks, "cavs_run_tasks: more than %d jobs", kMaxTasks);
    CAVS_REQUIRE(blocks > 0 && L.first[k] + blocks < (1L << 30), "cavs_run_tasks: job %d: too many workgroups", i);
    L.t[k] = t;
    L.first[k + 1] = L.first[k] + (int)blocks;
    k++;
  }
  if (k == 0) return CAVS_OK;
  L.count = k;
  launch(tasks_kernel, (unsigned)L.first[k], 256, 0, as_stream(stream), L);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_sgd_multi(int count, float *const *w, const float *const *g, const size_t *n, float lr, void *stream) {
  CAVS_REQUIRE(count >= 0 && (count == 0 || (w && g && n)), "cavs_sgd_multi: bad arguments");
  hipStream_t st = as_stream(stream);
  for (int i = 0; i < count;) {
    SgdBatch t{};
    size_t run = 0;
    int k = 0;
    for (; i < count && k < kMaxTensors; i++) {
      if (n[i] == 0) continue;
      CAVS_REQUIRE(w[i] && g[i], "cavs_sgd_multi: null tensor %d", i);
      run += n[i];
      t.w[k] = w[i];
      t.g[k] = g[i];
      t.end[k] = run;
      k++;
    }
    if (k == 0) continue;
    t.count = k;
    size_t blocks = (run + 255) / 256, cap = (size_t)num_cus() * 16;
    launch(sgd_multi_kernel, (unsigned)(blocks < cap ? blocks : cap), 256, 0, st, t, lr);
    CAVS_LAUNCH_CHECK();
  }
  return CAVS_OK;
}

int cavs_embed_sgd(float *table, const float *dtable, const float *ids, int n, int E, float lr, int *stamp,
                   int epoch, void *stream) {
  CAVS_REQUIRE(n >= 0 && E > 0, "cavs_embed_sgd: bad shape n=%d E=%d", n, E);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(table && dtable && ids && stamp, "cavs_embed_sgd: null pointer");
  int block = E >= 256 ? 256 : (E > 64 ? 128 : 64);
  launch(embed_sgd_kernel, (n + kSgdChunk - 1) / kSgdChunk, block, 0, as_stream(stream), table, dtable, ids, n, E, lr, stamp, epoch);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_embed_zero_rows(float *dtable, const float *ids, int n, int E, void *stream) {
  CAVS_REQUIRE(n >= 0 && E > 0, "cavs_embed_zero_rows: bad shape n=%d E=%d", n, E);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(dtable && ids, "cavs_embed_zero_rows: null pointer");
  int block = E >= 256 ? 256 : (E > 64 ? 128 : 64);
  launch(embed_zero_rows_kernel, n, block, 0, as_stream(stream), dtable, ids, E);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

size_t cavs_colsum_blocks_workspace(int n, int bw, int nb) {
  if (n <= 0 || bw <= 0 || nb <= 0) return 0;
  return (size_t)colsum_chunks(n) * bw * nb * sizeof(float);
}

int cavs_colsum_parts(int n) { return colsum_chunks(n); }

int cavs_colsum_blocks(float *out, const float *inp, int ld, int n, int bw, int nb, const int *dst_block,
                       void *workspace, size_t workspace_bytes, void *stream) {
  CAVS_REQUIRE(n >= 0 && bw > 0 && nb > 0 && nb <= 8 && ld >= bw * nb, "cavs_colsum_blocks: bad shape n=%d bw=%d nb=%d ld=%d", n, bw, nb, ld);
  CAVS_REQUIRE(!out || dst_block, "cavs_colsum_blocks: null block map");
  BlockMap map{};
  unsigned seen = 0;
  for (int k = 0; out && k < nb; k++) {
    CAVS_REQUIRE(dst_block[k] >= 0 && dst_block[k] < nb && !(seen >> dst_block[k] & 1u), "cavs_colsum_blocks: dst_block is not a permutation");
    seen |= 1u << dst_block[k];
    map.dst[k] = dst_block[k];
  }
  const int w = bw * nb;
  const int chunks = colsum_chunks(n);
  const size_t need = (size_t)chunks * w * sizeof(float);
  if (n == 0) return out ? cavs_zero(out, (size_t)w * 4, stream) : (workspace ? cavs_zero(workspace, need, stream) : CAVS_OK);
  CAVS_REQUIRE(inp, "cavs_colsum_blocks: null input");
  CAVS_REQUIRE(workspace && workspace_bytes >= need, "cavs_colsum_blocks: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  const int rpc = ((n + chunks - 1) / chunks + 3) / 4 * 4;
  hipStream_t st = as_stream(stream);
  float *part = static_cast<float *>(workspace);
  launch(colsum_part_kernel, dim3((w + 63) / 64, chunks), 256, 0, st, part, inp, ld, n, w, rpc);
  CAVS_LAUNCH_CHECK();
  if (!out) return CAVS_OK;  // the chunk sums stay in the workspace
  launch(colsum_blocks_reduce_kernel, (w + 63) / 64, 256, 0, st, out, part, chunks, w, bw, map);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

}  // extern "C"

// ------------------------------------------------------------------ gradient clipping
// ClipOpImpl (cavs/backend/op_impl_clip.cu:26-50): every gradient is scaled by
// clip / max(sum_i ||g_i||_2, clip) -- the SUM of the tensors' norms, as the reference adds
// them.  Three launches, all deterministic: partial sums of squares per tensor in fixed
// chunks, one workgroup that adds them in index order and forms the factor, and the scaling.
namespace cavs {

constexpr int kClipParts = 64;

struct ClipBatch {
  float *g[kMaxTensors];
  size_t n[kMaxTensors];
  int count;
};

__global__ __launch_bounds__(256) void clip_sumsq_kernel(ClipBatch t, float *__restrict__ part) {
  __shared__ float s[256];
  const int k = blockIdx.y, p = blockIdx.x;
  const size_t n = t.n[k], per = (n + kClipParts - 1) / kClipParts;
  const size_t b = (size_t)p * per, e = b + per < n ? b + per : n;
  float a = 0.f;
  for (size_t i = b + threadIdx.x; i < e; i += 256) {
    const float v = t.g[k][i];
    a += v * v;
  }
  s[threadIdx.x] = a;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o) s[threadIdx.x] += s[threadIdx.x + o];
    __syncthreads();
  }
  if (threadIdx.x == 0) part[k * kClipParts + p] = s[0];
}

// factor[0] = clip / max(sum of norms, clip); factor[1] = the sum of norms (for inspection)
__global__ void clip_factor_kernel(const float *__restrict__ part, int count, float clip, float base,
                                   float *__restrict__ factor, int last) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  float total = base;
  for (int k = 0; k < count; k++) {
    float ss = 0.f;
    for (int p = 0; p < kClipParts; p++) ss += part[k * kClipParts + p];
    total += sqrtf(ss);
  }
  factor[1] = total;
  if (last) factor[0] = clip / fmaxf(total, clip);
}

__global__ void clip_scale_kernel(ClipBatch t, const float *__restrict__ factor) {
  const float f = factor[0];
  if (f == 1.f) return;
  const int k = blockIdx.y;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < t.n[k]; i += stride) t.g[k][i] *= f;
}

}  // namespace cavs

extern "C" {

size_t cavs_clip_grads_workspace(int count) {
  return count <= 0 ? 0 : ((size_t)cavs::kMaxTensors * cavs::kClipParts + 2) * sizeof(float);
}

int cavs_clip_grads(int count, float *const *g, const size_t *n, float clip, void *workspace, size_t workspace_bytes,
                    void *stream) {
  CAVS_REQUIRE(count >= 0 && clip > 0.f && (count == 0 || (g && n)), "cavs_clip_grads: bad arguments (count=%d clip=%g)", count, (double)clip);
  if (count == 0) return CAVS_OK;
  CAVS_REQUIRE(workspace && workspace_bytes >= cavs_clip_grads_workspace(count), "cavs_clip_grads: workspace of %zu bytes needed, %zu given",
               cavs_clip_grads_workspace(count), workspace_bytes);
  hipStream_t st = as_stream(stream);
  float *part = static_cast<float *>(workspace), *factor = part + kMaxTensors * kClipParts;
  // norms, eight tensors per pass; the running sum of norms is carried in factor[1]
  std::vector<ClipBatch> batches;
  for (int i = 0; i < count;) {
    ClipBatch t{};
    for (; i < count && t.count < kMaxTensors; i++) {
      if (n[i] == 0) continue;
      CAVS_REQUIRE(g[i], "cavs_clip_grads: null tensor %d", i);
      t.g[t.count] = g[i];
      t.n[t.count] = n[i];
      t.count++;
    }
    if (t.count) batches.push_back(t);
  }
  if (batches.empty()) return CAVS_OK;
  CAVS_REQUIRE(batches.size() == 1, "cavs_clip_grads: at most %d non-empty tensors", kMaxTensors);
  const ClipBatch &t = batches[0];
  launch(clip_sumsq_kernel, dim3(kClipParts, t.count), 256, 0, st, t, part);
  launch(clip_factor_kernel, 1, 64, 0, st, (const float *)part, t.count, clip, 0.f, factor, 1);
  launch(clip_scale_kernel, dim3((unsigned)num_cus() * 4, t.count), 256, 0, st, t, (const float *)factor);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

}  // extern "C"
