// The embedding gradient's scatter-add, shared by cavs_embed_bwd and by the grouped products'
// launch that reduces K-split partials (which feeds it the product's partials directly).
#ifndef CAVS_CSRC_EMBED_COMMON_H_
#define CAVS_CSRC_EMBED_COMMON_H_

#include "common.h"

namespace cavs {

// Scatter-add of dy rows into the table.  A workgroup takes 64 consecutive rows and 64 columns
// (row chunk bx, column chunk by).
// Parse trees look up one and the same table row for every internal vertex, and atomic adds to
// one address serialise, so the workgroup first finds the id that occurs most often among its
// rows (its "hot" id), adds those rows up (each wavefront its 16 rows in registers, then the
// four partial sums in wavefront order) and issues one atomic add per column for them; every
// other row goes to the table with an atomic add of its own.
// dy is the sum of `parts` arrays `part_stride` floats apart, added in index order (one array:
// the plain case); when `copy` is given the summed value is also stored there (row stride ld_copy).
constexpr int kEmbedRows = 64, kEmbedCols = 64;
__device__ inline void embed_bwd_block(float *__restrict__ dtable, const float *__restrict__ ids, const float *__restrict__ dy,
                                       long ld_dy, int parts, long part_stride, float *__restrict__ copy, long ld_copy, int n, int E,
                                       int bx, int by) {
  __shared__ long off[kEmbedRows];
  __shared__ int count[kEmbedRows];
  __shared__ int hot_row;
  __shared__ float part[4][kEmbedCols];
  const int row0 = bx * kEmbedRows, tid = threadIdx.x;
  const int rows = min(kEmbedRows, n - row0);
  if (tid < kEmbedRows) off[tid] = tid < rows ? (long)(int)(ids[row0 + tid] * (float)E) : -1 - tid;
  __syncthreads();
  if (tid < kEmbedRows) {  // occurrences of this row's id, counted at its first occurrence only
    int c = 0;
    bool first = tid < rows;
    for (int r = 0; r < rows; r++) {
      if (off[r] == off[tid]) {
        c++;
        if (r < tid) first = false;
      }
    }
    count[tid] = first ? c : 0;
  }
  __syncthreads();
  if (tid == 0) {
    int best = 0;
    for (int r = 1; r < rows; r++)
      if (count[r] > count[best]) best = r;  // ties: the earliest row
    hot_row = best;
  }
  __syncthreads();
  const long hot = off[hot_row];
  const bool combine = count[hot_row] > 1;
  const int q = tid >> 6, lane = tid & 63, c = by * kEmbedCols + lane;
  constexpr int U = kEmbedRows / 4;  // rows per wavefront, all in flight
  const int r0 = q * U;
  float sum = 0.f;
  if (c < E) {
    float v[U];
#pragma unroll
    for (int u = 0; u < U; u++) v[u] = r0 + u < rows ? dy[(long)(row0 + r0 + u) * ld_dy + c] : 0.f;
    if (parts == 2) {  // the usual split: both parts' loads in flight together
      float w[U];
      const float *dz = dy + part_stride;
#pragma unroll
      for (int u = 0; u < U; u++) w[u] = r0 + u < rows ? dz[(long)(row0 + r0 + u) * ld_dy + c] : 0.f;
#pragma unroll
      for (int u = 0; u < U; u++) v[u] += w[u];
    } else {
      for (int z = 1; z < parts; z++) {
        const float *dz = dy + z * part_stride;
#pragma unroll
        for (int u = 0; u < U; u++)
          if (r0 + u < rows) v[u] += dz[(long)(row0 + r0 + u) * ld_dy + c];
      }
    }
    if (copy) {
#pragma unroll
      for (int u = 0; u < U; u++)
        if (r0 + u < rows) copy[(long)(row0 + r0 + u) * ld_copy + c] = v[u];
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      if (r0 + u >= rows) continue;
      const long o = off[r0 + u];
      if (combine && o == hot) sum += v[u];  // in row order
      else unsafeAtomicAdd(dtable + o + c, v[u]);
    }
  }
  if (!combine) return;  // the same for the whole workgroup
  part[q][lane] = sum;
  __syncthreads();
  if (q == 0 && c < E) unsafeAtomicAdd(dtable + hot + c, ((part[0][lane] + part[1][lane]) + part[2][lane]) + part[3][lane]);
}

}  // namespace cavs
#endif
