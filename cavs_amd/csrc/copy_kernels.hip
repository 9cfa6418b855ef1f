// Level-wise row movement: gather / scatter / zero / copy of [n, w] slabs through
// int32 row lists.  HBM-bound: every payload byte is read once and written once
// with 16-byte lane accesses (a wave moves 1 KiB per instruction), several
// independent rows in flight per lane, and the row id read once per workgroup.
#include "common.h"

namespace cavs {

template <typename V>
__device__ inline V vzero();
template <>
__device__ inline float4 vzero<float4>() { return make_float4(0.f, 0.f, 0.f, 0.f); }
template <>
__device__ inline float vzero<float>() { return 0.f; }

__device__ inline float4 vadd(float4 a, float4 b) {
  return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
}
__device__ inline float vadd(float a, float b) { return a + b; }

// Pins a loaded value in registers at this point of the program, which keeps the
// compiler from sinking the load into the predicated store that consumes it (that
// would leave one load in flight per lane instead of four).
__device__ inline void pin(float4 &v) { asm volatile("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w)); }
__device__ inline void pin(float &v) { asm volatile("" : "+v"(v)); }

constexpr int kRowsPerBlock = 4;

// out[b] = ids[b] >= 0 ? src[ids[b]] : 0.  ids == nullptr copies row b (copy_rows);
// src == nullptr zero-fills (zero_rows).  Strides and widths in units of V.
template <typename V>
__global__ void gather_rows_kernel(V *__restrict__ out, long ld_out, const V *__restrict__ src,
                                   long ld_src, const int *__restrict__ ids, int n, int wv) {
  const int row0 = blockIdx.x * kRowsPerBlock;
  long srow[kRowsPerBlock];
#pragma unroll
  for (int r = 0; r < kRowsPerBlock; r++) {
    int row = row0 + r;
    long id = -1;
    if (row < n && src) id = ids ? ids[row] : row;
    srow[r] = id;
  }
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < wv; c += gridDim.y * blockDim.x) {
    V v[kRowsPerBlock];
#pragma unroll
    for (int r = 0; r < kRowsPerBlock; r++)
      v[r] = srow[r] >= 0 ? src[srow[r] * ld_src + c] : vzero<V>();
#pragma unroll
    for (int r = 0; r < kRowsPerBlock; r++)
      if (row0 + r < n) out[(long)(row0 + r) * ld_out + c] = v[r];
  }
}

// out[b] += inp[b] over a [n, wv] block (PartialAccumulate: a column block of a wider slab)
template <typename V>
__global__ void add_rows_kernel(V *__restrict__ out, long ld_out, const V *__restrict__ inp, long ld_inp,
                                int n, int wv) {
  const int row0 = blockIdx.x * kRowsPerBlock;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < wv; c += gridDim.y * blockDim.x) {
#pragma unroll
    for (int r = 0; r < kRowsPerBlock; r++)
      if (row0 + r < n) {
        V *o = out + (long)(row0 + r) * ld_out + c;
        *o = vadd(*o, inp[(long)(row0 + r) * ld_inp + c]);
      }
  }
}

// dst[ids[b]] = inp[b] for ids[b] >= 0
template <typename V>
__global__ void scatter_rows_kernel(V *__restrict__ dst, long ld_dst, const int *__restrict__ ids,
                                    const V *__restrict__ inp, long ld_inp, int n, int wv) {
  const int row0 = blockIdx.x * kRowsPerBlock;
  long drow[kRowsPerBlock];
#pragma unroll
  for (int r = 0; r < kRowsPerBlock; r++) {
    int row = row0 + r;
    drow[r] = row < n ? (long)ids[row] : -1;
  }
  // loads are unconditional (rows past the end re-read the last row) so that all four are
  // in flight before the first store; only the stores are predicated
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < wv; c += gridDim.y * blockDim.x) {
    V v[kRowsPerBlock];
#pragma unroll
    for (int r = 0; r < kRowsPerBlock; r++) v[r] = inp[(long)min(row0 + r, n - 1) * ld_inp + c];
#pragma unroll
    for (int r = 0; r < kRowsPerBlock; r++) pin(v[r]);
#pragma unroll
    for (int r = 0; r < kRowsPerBlock; r++)
      if (drow[r] >= 0) dst[drow[r] * ld_dst + c] = v[r];
  }
}

// Two vertices per workgroup: G[2b+i] = pool[ids[2b+i]] (or 0), hsum[b] = G[2b] + G[2b+1]
// over the first hv vector columns.
template <typename V>
__global__ void gather_children_kernel(V *__restrict__ G, V *__restrict__ hsum,
                                       const V *__restrict__ pool, const int *__restrict__ ids,
                                       int n, int wv, int hv) {
  constexpr int kNodes = 2;
  const int b0 = blockIdx.x * kNodes;
  long srow[2 * kNodes];
#pragma unroll
  for (int r = 0; r < 2 * kNodes; r++) {
    int row = 2 * b0 + r;
    srow[r] = row < 2 * n ? (long)ids[row] : -1;
  }
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < wv; c += gridDim.y * blockDim.x) {
    V v[2 * kNodes];
#pragma unroll
    for (int r = 0; r < 2 * kNodes; r++)
      v[r] = srow[r] >= 0 ? pool[srow[r] * wv + c] : vzero<V>();
#pragma unroll
    for (int r = 0; r < 2 * kNodes; r++)
      if (2 * b0 + r < 2 * n) G[(long)(2 * b0 + r) * wv + c] = v[r];
    if (hsum && c < hv) {
#pragma unroll
      for (int k = 0; k < kNodes; k++)
        if (b0 + k < n) hsum[(long)(b0 + k) * hv + c] = vadd(v[2 * k], v[2 * k + 1]);
    }
  }
}

inline int block_for(int wv) { return wv >= 256 ? 256 : (wv > 128 ? 256 : (wv > 64 ? 128 : 64)); }

// grid for `row_blocks` workgroups' worth of rows, wv vector columns each: few but wide rows (a
// flat parameter viewed as one row) are split along the columns as well, so that the launch still
// covers the chip
inline dim3 grid_for(int row_blocks, int wv, int block) {
  int gy = 1;
  if (row_blocks < 1024) {
    const int by_width = (wv + 4 * block - 1) / (4 * block);  // at least four columns per lane
    const int wanted = (1024 + row_blocks - 1) / row_blocks;
    gy = by_width < wanted ? by_width : wanted;
    if (gy < 1) gy = 1;
  }
  return dim3(row_blocks, gy);
}

inline bool vec_ok(const void *a, long lda, const void *b, long ldb, int w) {
  return (w % 4 == 0) && (lda % 4 == 0) && (ldb % 4 == 0) && (!a || aligned16(a)) &&
         (!b || aligned16(b));
}

static int launch_gather(float *out, int ld_out, const float *src, int ld_src, const int *ids,
                         int n, int w, hipStream_t st) {
  if (n == 0 || w == 0) return CAVS_OK;
  int grid = (n + kRowsPerBlock - 1) / kRowsPerBlock;
  if (vec_ok(out, ld_out, src, ld_src, w)) {
    int wv = w / 4;
    launch(gather_rows_kernel<float4>, grid_for(grid, wv, block_for(wv)), block_for(wv), 0, st,
        reinterpret_cast<float4 *>(out), ld_out / 4, reinterpret_cast<const float4 *>(src),
        ld_src / 4, ids, n, wv);
  } else {
    launch(gather_rows_kernel<float>, grid_for(grid, w, block_for(w)), block_for(w), 0, st, out, ld_out, src, ld_src, ids, n, w);
  }
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

}  // namespace cavs

using namespace cavs;

extern "C" {

int cavs_gather_rows(float *out, int ld_out, const float *src, int ld_src, const int *ids, int n,
                     int w, void *stream) {
  CAVS_REQUIRE(n >= 0 && w >= 0 && ld_out >= w && ld_src >= w, "cavs_gather_rows: bad shape n=%d w=%d ld_out=%d ld_src=%d", n, w, ld_out, ld_src);
  if (n == 0 || w == 0) return CAVS_OK;
  CAVS_REQUIRE(out && src && ids, "cavs_gather_rows: null pointer");
  return launch_gather(out, ld_out, src, ld_src, ids, n, w, as_stream(stream));
}

int cavs_copy_rows(float *out, int ld_out, const float *inp, int ld_inp, int n, int w,
                   void *stream) {
  CAVS_REQUIRE(n >= 0 && w >= 0 && ld_out >= w && ld_inp >= w, "cavs_copy_rows: bad shape n=%d w=%d", n, w);
  if (n == 0 || w == 0) return CAVS_OK;
  CAVS_REQUIRE(out && inp, "cavs_copy_rows: null pointer");
  return launch_gather(out, ld_out, inp, ld_inp, nullptr, n, w, as_stream(stream));
}

int cavs_add_rows(float *out, int ld_out, const float *inp, int ld_inp, int n, int w, void *stream) {
  CAVS_REQUIRE(n >= 0 && w >= 0 && ld_out >= w && ld_inp >= w, "cavs_add_rows: bad shape n=%d w=%d", n, w);
  if (n == 0 || w == 0) return CAVS_OK;
  CAVS_REQUIRE(out && inp, "cavs_add_rows: null pointer");
  hipStream_t st = as_stream(stream);
  int grid = (n + kRowsPerBlock - 1) / kRowsPerBlock;
  if (vec_ok(out, ld_out, inp, ld_inp, w))
    launch(add_rows_kernel<float4>, grid_for(grid, w / 4, block_for(w / 4)), block_for(w / 4), 0, st,
           reinterpret_cast<float4 *>(out), ld_out / 4, reinterpret_cast<const float4 *>(inp), ld_inp / 4, n, w / 4);
  else
    launch(add_rows_kernel<float>, grid_for(grid, w, block_for(w)), block_for(w), 0, st, out, ld_out, inp, ld_inp, n, w);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_zero_rows(float *out, int ld_out, int n, int w, void *stream) {
  CAVS_REQUIRE(n >= 0 && w >= 0 && ld_out >= w, "cavs_zero_rows: bad shape n=%d w=%d", n, w);
  if (n == 0 || w == 0) return CAVS_OK;
  CAVS_REQUIRE(out, "cavs_zero_rows: null pointer");
  return launch_gather(out, ld_out, nullptr, ld_out, nullptr, n, w, as_stream(stream));
}

int cavs_scatter_rows(float *dst, int ld_dst, const int *ids, const float *inp, int ld_inp, int n,
                      int w, void *stream) {
  CAVS_REQUIRE(n >= 0 && w >= 0 && ld_dst >= w && ld_inp >= w, "cavs_scatter_rows: bad shape n=%d w=%d", n, w);
  if (n == 0 || w == 0) return CAVS_OK;
  CAVS_REQUIRE(dst && ids && inp, "cavs_scatter_rows: null pointer");
  hipStream_t st = as_stream(stream);
  int grid = (n + kRowsPerBlock - 1) / kRowsPerBlock;
  if (vec_ok(dst, ld_dst, inp, ld_inp, w)) {
    int wv = w / 4;
    launch(scatter_rows_kernel<float4>, grid_for(grid, wv, block_for(wv)), block_for(wv), 0, st,
        reinterpret_cast<float4 *>(dst), ld_dst / 4, ids, reinterpret_cast<const float4 *>(inp),
        ld_inp / 4, n, wv);
  } else {
    launch(scatter_rows_kernel<float>, grid_for(grid, w, block_for(w)), block_for(w), 0, st, dst, ld_dst, ids, inp, ld_inp, n, w);
  }
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_gather_children(float *G, float *hsum, const float *pool, const int *ids, int n, int w,
                         int hw, void *stream) {
  CAVS_REQUIRE(n >= 0 && w > 0 && hw >= 0 && hw <= w, "cavs_gather_children: bad shape n=%d w=%d hw=%d", n, w, hw);
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(G && pool && ids, "cavs_gather_children: null pointer");
  hipStream_t st = as_stream(stream);
  int grid = (n + 1) / 2;
  if (w % 4 == 0 && hw % 4 == 0 && aligned16(G) && aligned16(pool) && (!hsum || aligned16(hsum))) {
    launch(gather_children_kernel<float4>, grid, block_for(w / 4), 0, st, 
        reinterpret_cast<float4 *>(G), reinterpret_cast<float4 *>(hsum),
        reinterpret_cast<const float4 *>(pool), ids, n, w / 4, hw / 4);
  } else {
    launch(gather_children_kernel<float>, grid, block_for(w), 0, st, G, hsum, pool, ids, n, w, hw);
  }
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

}  // extern "C"
