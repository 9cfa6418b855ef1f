// FP32 GEMM on the CDNA4 matrix cores (v_mfma_f32_32x32x2_f32), row-major, for the
// gate products of the vertex functions: NN (X*W), NT (dY*W^T) and TN (X^T*dY).
//
// Workgroup = 4 wavefronts (2x2) over a BM x BN tile of C, BK deep (128x128x16 for
// problems that fill the chip, 64x64x32 otherwise).  A and B
// tiles are staged through LDS as [k][m] / [k][n] panels (double buffered, one
// barrier per k-tile), so each MFMA operand read is a conflict-free ds_read_b32 of
// 32 consecutive floats per half-wave.  Global loads are 16-byte per lane; the
// k-contiguous operand (A of NN/NT, B of NT) is transposed on its way into LDS.
// Workgroup ids are remapped so that consecutive tiles (which share an A row panel)
// run on the same XCD and hit the same L2.  Products with too few tiles to fill the
// chip take one of two other routes: skinny ones (the tail rounds of a batch) a
// kernel whose wavefronts split K inside the workgroup, tall-K ones (the deferred
// weight gradients) split K over workgroups with the partials reduced in a fixed
// order by a second kernel.
#include <algorithm>
#include <type_traits>

#include <atomic>

#include "bench_probes.h"
#include "common.h"
#include "embed_common.h"

namespace cavs {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int PAD = 4;
constexpr int kThreads = 256;

struct GemmArgs {
  int M, N, K;
  const float *A;
  long lda;
  const float *B;
  long ldb;
  float *C;
  long ldc;
  float alpha, beta;
  const float *D;  // optional addend rows D[r >> dshift, :]
  long ldd;
  int dshift;
  int kchunk;      // K range per blockIdx.y (multiple of BK); == K when not split
  float *ws;       // split-K workspace (counters + partial tiles) or nullptr
  // cavs_embed_pull_sgemm (NN form only): row r of A is row int(pull_x[pull_rows[r]] * K) / K of the
  // table A points at (a negative id: a zero row); the workgroups of a row tile also leave the
  // rows they read in pull_copy (row stride ld_copy; each takes every tilesN-th k-tile) and those
  // of the first column tile the ids in pull_ids
  const int *pull_rows = nullptr;
  const float *pull_x = nullptr;
  float *pull_copy = nullptr;
  long ld_copy = 0;
  float *pull_ids = nullptr;
  // A block the caller knows about (cavs_gemm_desc::zero_kind and friends): the tiles it covers
  // run a shorter k range, or none
  int zkind = 0, zrows = 0, zcol = 0;
  // > 0: the launch is two launches back to back, the first zseg tiles (the row tiles inside the
  // block, whose workgroups do less) and the rest, each padded to a multiple of 8 workgroups and
  // dealt to the XCDs by itself: with one deal over all tiles the XCDs that hold the first
  // tiles would finish early and the others set the time as before
  int zseg = 0;
};

// Loader of one BX x BK operand tile.  KC: the operand's k index is the contiguous
// one in memory (element (x,k) at P[x*ld + k]); otherwise element at P[k*ld + x].
template <int BX, int BK, bool KC, bool VEC, bool FASTK = false>
struct TileLoader {
  static constexpr int NV = BX * BK / 4 / kThreads;  // float4 per thread
  static constexpr int KQ = BK / 4;                  // float4 per row of a k-contiguous tile
  static constexpr int PER = BX / 4;                 // float4 per k row otherwise
  float4 reg[NV];
  // Fixed per thread before the k loop (prepare): where float4 i of this thread sits in the
  // operand at k = 0, which of its x are inside, and its k relative to the tile's first.  In
  // the loop only the tile's k advances -- a pointer bump, or a wave-uniform k * ld -- instead
  // of a 64-bit row * stride product on the vector ALU per load and k-tile.
  long base[NV];
  int krel[NV];
  bool xin[NV][4];
  // Fast path (VEC): when every x of the tile is inside the operand and the offsets fit 32 bits,
  // a k-tile that lies wholly inside the k range is fetched with unconditional loads at a
  // wave-uniform pointer plus this byte offset -- no predicate, no 64-bit address arithmetic on
  // the vector ALU (8192^3: 126.6 -> 133.9 TFLOP/s).  The k loop runs in two parts, the k-tiles
  // that take it and the rest, so that neither carries the other's code.
  unsigned boff[NV];
  bool fast = false;
  // gathered rows (prepare_pull): where the float4 goes as well, or nullptr; the workgroup copies
  // the k-tiles whose number is copy_rem modulo copy_mod (the column tiles of a row tile share the
  // copying of the panel they all read)
  float *copy[NV];
  int copy_mod = 1, copy_rem = 0;

  __device__ inline void prepare(long ld, int x0, int X, int tid) {
#pragma unroll
    for (int i = 0; i < NV; i++) {
      copy[i] = nullptr;
      if constexpr (KC) {
        const int gx = x0 + tid / KQ + (kThreads / KQ) * i;
        krel[i] = 4 * (tid % KQ);
        base[i] = (long)gx * ld + krel[i];
#pragma unroll
        for (int c = 0; c < 4; c++) xin[i][c] = gx < X;
      } else {
        const int gx = x0 + 4 * (tid % PER);
        krel[i] = tid / PER + (kThreads / PER) * i;
        base[i] = (long)krel[i] * ld + gx;
#pragma unroll
        for (int c = 0; c < 4; c++) xin[i][c] = gx + c < X;
      }
      if constexpr (FASTK) boff[i] = (unsigned)(base[i] * 4);
    }
    if constexpr (FASTK) fast = VEC && x0 + BX <= X && (KC ? (long)X * ld : (long)BK * ld) < (1L << 30);
  }

  // k-contiguous operand whose rows are looked up: row x0 + r of the operand is the table row that
  // starts at float int(ids(x0 + r) * K) of P (EmbeddingLookup's offset), ids(b) = px[rows[b]]
  __device__ inline void prepare_pull(const int *__restrict__ rows, const float *__restrict__ px, int K, int x0, int X, int tid,
                                      float *__restrict__ copy_to, long ld_copy, float *__restrict__ ids_out, int mod, int rem) {
    static_assert(KC, "looked-up rows are k-contiguous");
    copy_mod = mod;
    copy_rem = rem;
    fast = false;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      const int gx = x0 + tid / KQ + (kThreads / KQ) * i;
      krel[i] = 4 * (tid % KQ);
      long off = -1;
      if (gx < X) {
        const float id = px[rows[gx]];
        off = (long)(int)(id * (float)K);
        if (ids_out && krel[i] == 0) ids_out[gx] = id;
      }
      base[i] = (off >= 0 ? off : 0) + krel[i];
#pragma unroll
      for (int c = 0; c < 4; c++) xin[i][c] = off >= 0;
      copy[i] = (copy_to && gx < X) ? copy_to + (long)gx * ld_copy + krel[i] : nullptr;
    }
  }

  // the tile whose first k is k0, wholly inside the k range, of an operand with `fast` set
  __device__ inline void load_fast(const float *__restrict__ P, long ld, int k0) {
    const char *Pk = reinterpret_cast<const char *>(KC ? P + k0 : P + (long)k0 * ld);
#pragma unroll
    for (int i = 0; i < NV; i++) reg[i] = *reinterpret_cast<const float4 *>(Pk + boff[i]);
  }

  // the tile whose first k is k0 (wave-uniform)
  __device__ inline void load(const float *__restrict__ P, long ld, int k0, int Kend) {
    const float *Pk = KC ? P + k0 : P + (long)k0 * ld;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      bool kin[4];
#pragma unroll
      for (int c = 0; c < 4; c++) kin[c] = KC ? (k0 + krel[i] + c < Kend) : (k0 + krel[i] < Kend);
      const float *q = Pk + base[i];
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if constexpr (VEC) {
        // whole float4 in or out (X, K multiples of 4 along the contiguous index)
        if (xin[i][0] && kin[0]) v = *reinterpret_cast<const float4 *>(q);
      } else {
        if (xin[i][0] && kin[0]) v.x = q[0];
        if (xin[i][1] && kin[1]) v.y = q[1];
        if (xin[i][2] && kin[2]) v.z = q[2];
        if (xin[i][3] && kin[3]) v.w = q[3];
      }
      reg[i] = v;
      if constexpr (KC) {
        if (copy[i] && (k0 / BK) % copy_mod == copy_rem) {  // (a row without an id leaves zeros)
          if constexpr (VEC) {
            if (kin[0]) *reinterpret_cast<float4 *>(copy[i] + k0) = v;
          } else {
            if (kin[0]) copy[i][k0] = v.x;
            if (kin[1]) copy[i][k0 + 1] = v.y;
            if (kin[2]) copy[i][k0 + 2] = v.z;
            if (kin[3]) copy[i][k0 + 3] = v.w;
          }
        }
      }
    }
  }

  __device__ inline void store(float *__restrict__ S, int tid) const {
    constexpr int LD = BX + PAD;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      if constexpr (KC) {
        int x = tid / KQ + (kThreads / KQ) * i, k = 4 * (tid % KQ);
        S[(k + 0) * LD + x] = reg[i].x;
        S[(k + 1) * LD + x] = reg[i].y;
        S[(k + 2) * LD + x] = reg[i].z;
        S[(k + 3) * LD + x] = reg[i].w;
      } else {
        int k = tid / PER + (kThreads / PER) * i, x = 4 * (tid % PER);
        *reinterpret_cast<float4 *>(S + k * LD + x) = reg[i];
      }
    }
  }
};

// Remap the linear workgroup id so that ids that are consecutive after the remap
// were dispatched to the same XCD (hardware deals workgroups round-robin over 8 XCDs).
__device__ inline int xcd_remap(int l, int total) {
  constexpr int X = 8;
  int per = total / X, rem = total % X;
  int xcd = l % X, local = l / X;
  return xcd * per + (xcd < rem ? xcd : rem) + local;
}

// One BM x BN tile of C (or of split `z` of its K range) by the calling workgroup.  `t` is the
// tile's index, row-major over the tiles of C; As / Bs are the workgroup's two LDS panels of
// 2 * BK * (BM + PAD) and 2 * BK * (BN + PAD) floats.
// FASTK: the k loop has a first part for k-tiles that take the loaders' fast path.
template <int BM, int BN, int BK, bool TA, bool TB, bool VEC, bool FASTK = true>
__device__ __forceinline__ void gemm_tile(const GemmArgs &g, int t, int z, float *__restrict__ As_, float *__restrict__ Bs_) {
  constexpr int WM = BM / 2, WN = BN / 2, TM = WM / 32, TN = WN / 32;
  constexpr int LDA = BM + PAD, LDB = BN + PAD;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tilesN = (g.N + BN - 1) / BN;
  const int m0 = (t / tilesN) * BM, n0 = (t % tilesN) * BN;
  int kbeg = z * g.kchunk;
  int kend = min(g.K, kbeg + g.kchunk);
  if (g.zkind == CAVS_GEMM_C_UNUSED) {  // rows below zrows of C are not wanted from column zcol on: left zero
    if (m0 + BM <= g.zrows && n0 >= g.zcol) kend = kbeg;
  } else if (g.zkind == CAVS_GEMM_A_ZERO) {  // rows below zrows of A (row-major M x K) are zero from k = zcol on
    if (!TA && m0 + BM <= g.zrows) kend = max(kbeg, min(kend, g.zcol));
  } else if (g.zkind == CAVS_GEMM_B_ZERO) {  // rows k < zrows of B (row-major K x N) are zero from column zcol on
    if (!TB && n0 >= g.zcol) kbeg = min(kend, max(kbeg, g.zrows / 32 * 32));
  }

  TileLoader<BM, BK, !TA, VEC, FASTK> la;
  TileLoader<BN, BK, TB, VEC, FASTK> lb;
  if constexpr (!TA) {
    if (g.pull_rows) {
      // the column tiles of this row tile that do run share the copying
      const int active = (g.zkind == CAVS_GEMM_C_UNUSED && m0 + BM <= g.zrows) ? min(tilesN, (g.zcol + BN - 1) / BN) : tilesN;
      la.prepare_pull(g.pull_rows, g.pull_x, g.K, m0, g.M, tid, g.pull_copy, g.ld_copy, n0 == 0 ? g.pull_ids : nullptr, active,
                      t % tilesN);
    }
    else la.prepare(g.lda, m0, g.M, tid);
  } else {
    la.prepare(g.lda, m0, g.M, tid);
  }
  lb.prepare(g.ldb, n0, g.N, tid);

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  const int nk = (kend - kbeg + BK - 1) / BK;
  // k-tiles 0 .. nfast - 1 lie wholly inside the k range of operands that take the fast loads
  const int nfast = (FASTK && la.fast && lb.fast) ? (kend - kbeg) / BK : 0;
  if (nk > 0) {
    if (FASTK && nfast > 0) {
      la.load_fast(g.A, g.lda, kbeg);
      lb.load_fast(g.B, g.ldb, kbeg);
    } else {
      la.load(g.A, g.lda, kbeg, kend);
      lb.load(g.B, g.ldb, kbeg, kend);
    }
    la.store(As_, tid);
    lb.store(Bs_, tid);
  }
  __syncthreads();
  const int arow = wm * WM + (lane & 31), brow = wn * WN + (lane & 31), khalf = lane >> 5;
  // The MFMAs of the k-tile in LDS buffer `cur` (spelled out in each loop through a macro: as a
  // lambda the compiler scheduled the 64 x 64 kernels 2 % slower).  Operand fragments: the reads of
  // AHEAD steps are in flight while a step's MFMAs issue, so a wavefront does not stall on LDS
  // latency between them; the scheduler barriers keep that order (the compiler's scheduler would
  // sink each read to its use).
  constexpr int STEPS = BK / 2, AHEAD = (TM * TN == 1) ? 4 : 2;
#define CAVS_TILE_PRODUCTS(cur)                                                                            \
  do {                                                                                                     \
    const float *as = As_ + (cur) * (BK * LDA), *bs = Bs_ + (cur) * (BK * LDB);                            \
    float a[STEPS][TM], b[STEPS][TN];                                                                      \
    auto read = [&](int st) {                                                                              \
      _Pragma("unroll") for (int i = 0; i < TM; i++) a[st][i] = as[(2 * st + khalf) * LDA + arow + 32 * i]; \
      _Pragma("unroll") for (int j = 0; j < TN; j++) b[st][j] = bs[(2 * st + khalf) * LDB + brow + 32 * j]; \
    };                                                                                                     \
    _Pragma("unroll") for (int st = 0; st < AHEAD && st < STEPS; st++) read(st);                           \
    __builtin_amdgcn_sched_barrier(0);                                                                     \
    _Pragma("unroll") for (int st = 0; st < STEPS; st++) {                                                 \
      if (st + AHEAD < STEPS) read(st + AHEAD);                                                            \
      __builtin_amdgcn_sched_barrier(0);                                                                   \
      _Pragma("unroll") for (int i = 0; i < TM; i++)                                                       \
        _Pragma("unroll") for (int j = 0; j < TN; j++)                                                     \
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[st][i], b[st][j], acc[i][j], 0, 0, 0);        \
      __builtin_amdgcn_sched_barrier(0);                                                                   \
    }                                                                                                      \
  } while (0)
  // iteration kt fetches tile kt + 1 while it multiplies tile kt
  if constexpr (FASTK) {
    // first the iterations whose next tile takes the fast loads, then the rest
    const int split = nfast > 1 ? nfast - 1 : 0;
    for (int kt = 0; kt < split; kt++) {
      const int cur = kt & 1;
      la.load_fast(g.A, g.lda, kbeg + (kt + 1) * BK);
      lb.load_fast(g.B, g.ldb, kbeg + (kt + 1) * BK);
      CAVS_TILE_PRODUCTS(cur);
      la.store(As_ + (cur ^ 1) * (BK * LDA), tid);
      lb.store(Bs_ + (cur ^ 1) * (BK * LDB), tid);
      __syncthreads();
    }
    for (int kt = split; kt < nk; kt++) {
      const int cur = kt & 1;
      if (kt + 1 < nk) {
        la.load(g.A, g.lda, kbeg + (kt + 1) * BK, kend);
        lb.load(g.B, g.ldb, kbeg + (kt + 1) * BK, kend);
      }
      CAVS_TILE_PRODUCTS(cur);
      if (kt + 1 < nk) {
        la.store(As_ + (cur ^ 1) * (BK * LDA), tid);
        lb.store(Bs_ + (cur ^ 1) * (BK * LDB), tid);
      }
      __syncthreads();
    }
  } else {
    for (int kt = 0; kt < nk; kt++) {
      const int cur = kt & 1;
      if (kt + 1 < nk) {
        la.load(g.A, g.lda, kbeg + (kt + 1) * BK, kend);
        lb.load(g.B, g.ldb, kbeg + (kt + 1) * BK, kend);
      }
      CAVS_TILE_PRODUCTS(cur);
      if (kt + 1 < nk) {
        la.store(As_ + (cur ^ 1) * (BK * LDA), tid);
        lb.store(Bs_ + (cur ^ 1) * (BK * LDB), tid);
      }
      __syncthreads();
    }
  }

#undef CAVS_TILE_PRODUCTS
  // C layout of the 32x32 accumulator: element r of lane l is row 8*(r/4) + 4*(l/32) + r%4,
  // column l%32.
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++) {
      const int col = n0 + wn * WN + 32 * j + (lane & 31);
      if (col >= g.N) continue;
      const int rbase = m0 + wm * WM + 32 * i + 4 * khalf;
      // the three forms of the store are chosen once per tile (the conditions are the same
      // for every lane), not once per element
      if (g.ws) {  // split K: park the partial sum, the reduce kernel finishes the job
        float *w = g.ws + (long)z * g.M * g.N + col;
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int row = rbase + 8 * (r / 4) + (r % 4);
          if (row < g.M) w[(long)row * g.N] = acc[i][j][r];
        }
      } else if (g.beta == 0.f && !g.D) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int row = rbase + 8 * (r / 4) + (r % 4);
          if (row < g.M) g.C[row * g.ldc + col] = g.alpha * acc[i][j][r];
        }
      } else {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int row = rbase + 8 * (r / 4) + (r % 4);
          if (row >= g.M) continue;
          float v = g.alpha * acc[i][j][r];
          if (g.beta != 0.f) v += g.beta * g.C[row * g.ldc + col];
          if (g.D) v += g.D[(long)(row >> g.dshift) * g.ldd + col];
          g.C[row * g.ldc + col] = v;
        }
      }
    }
}

template <int BM, int BN, int BK, bool TA, bool TB, bool VEC>
__global__ __launch_bounds__(kThreads) void sgemm_mfma_kernel(GemmArgs g) {
  __shared__ __attribute__((aligned(16))) float As[2 * BK * (BM + PAD)];
  __shared__ __attribute__((aligned(16))) float Bs[2 * BK * (BN + PAD)];
  const int tiles = ((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN);
  int t;
  if (g.zseg > 0) {
    const int first = (g.zseg + 7) & ~7, b = blockIdx.x;
    if (b < first) {
      t = xcd_remap(b, first);
      if (t >= g.zseg) return;
    } else {
      const int rest = tiles - g.zseg;
      t = xcd_remap(b - first, (rest + 7) & ~7);
      if (t >= rest) return;
      t += g.zseg;
    }
  } else {
    t = xcd_remap(blockIdx.x, tiles);
  }
  // (the fast part of the k loop pays on the large tile; the 64 x 64 launches are products with
  // short K or ragged edges, which it only made larger)
  gemm_tile<BM, BN, BK, TA, TB, VEC, BM == 128>(g, t, blockIdx.y, As, Bs);
}

// Several independent products in one launch (the deferred weight gradients of a step and the
// embedding gradient's product): alone, each of them is a single round of workgroups that all
// load, multiply and store at the same time; together their phases overlap and the chip sees
// one long launch.  Workgroup b belongs to product p with first[p] <= b < first[p+1] (each
// product's share is padded to a multiple of 8, so that b % 8 is the XCD within the share as
// well); within the share, tile = local % tiles[p] and K split = local / tiles[p].
constexpr int kGroupMax = 8;
struct GemmGroup {
  GemmArgs g[kGroupMax];
  int first[kGroupMax + 1];
  int tiles[kGroupMax];
  int splits[kGroupMax];
  int form[kGroupMax];  // transA * 2 + transB
  int count;
};

template <bool VEC>
__global__ __launch_bounds__(kThreads) void sgemm_group_kernel(GemmGroup G) {
  constexpr int BM = 64, BN = 64, BK = 32;
  __shared__ __attribute__((aligned(16))) float As[2 * BK * (BM + PAD)];
  __shared__ __attribute__((aligned(16))) float Bs[2 * BK * (BN + PAD)];
  int p = 0;
  while (p + 1 < G.count && (int)blockIdx.x >= G.first[p + 1]) p++;
  const int local = blockIdx.x - G.first[p];
  const int share = G.tiles[p] * G.splits[p];
  const int padded = G.first[p + 1] - G.first[p];
  const int w = xcd_remap(local, padded);
  if (w >= share) return;
  const int t = w % G.tiles[p], z = w / G.tiles[p];
  const GemmArgs &g = G.g[p];
  switch (G.form[p]) {
    case 0: gemm_tile<BM, BN, BK, false, false, VEC, true>(g, t, z, As, Bs); break;
    case 1: gemm_tile<BM, BN, BK, false, true, VEC, true>(g, t, z, As, Bs); break;
    case 2: gemm_tile<BM, BN, BK, true, false, VEC, true>(g, t, z, As, Bs); break;
    default: gemm_tile<BM, BN, BK, true, true, VEC, true>(g, t, z, As, Bs); break;
  }
}

// the split products of a group, reduced in one launch (same fixed order as splitk_reduce_kernel)
__global__ void splitk_reduce_group_kernel(GemmGroup R) {
  // first[] counts 256-thread workgroups per product here
  int p = 0;
  while (p + 1 < R.count && (int)blockIdx.x >= R.first[p + 1]) p++;
  const GemmArgs &g = R.g[p];
  const int splits = R.splits[p];
  long idx = (long)(blockIdx.x - R.first[p]) * blockDim.x + threadIdx.x;
  long total = (long)g.M * g.N;
  if (idx >= total) return;
  float acc = 0.f;
  for (int z = 0; z < splits; z++) acc += g.ws[(long)z * total + idx];
  int r = (int)(idx / g.N), c = (int)(idx % g.N);
  float v = g.alpha * acc;
  if (g.beta != 0.f) v += g.beta * g.C[r * g.ldc + c];
  if (g.D) v += g.D[(long)(r >> g.dshift) * g.ldd + c];
  g.C[r * g.ldc + c] = v;
}

// What the matrix pipes sustain with nothing else in the way (cavs_mfma_probe): every wavefront
// issues `iters` rounds of eight independent 32x32x2 MFMAs on operands it keeps in registers.
__global__ __launch_bounds__(256) void mfma_probe_kernel(float *__restrict__ out, int iters) {
  floatx16 acc[8];
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[i][r] = 0.f;
  const float a = 1.f + (threadIdx.x & 7) * 0.125f, b = 0.5f - (threadIdx.x & 3) * 0.0625f;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[i], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) s += acc[i][r];
  out[(long)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// The embedding gradient behind one product of a group (cavs_sgemm_group_embed_bwd): the rows of
// that product's result are scatter-added into the table by extra workgroups of the launch that
// reduces the other products' K splits, reading the product's own partials directly.
struct EmbedTail {
  float *dtable;
  const float *ids;
  const float *dy;   // the result, or the first of `parts` partial results `part_stride` floats apart
  long ld_dy, part_stride;
  int parts;
  float *copy;       // where the summed result goes as well (the product's C) when parts > 1
  long ld_copy;
  int n, E, gx;      // gx row chunks of 64
};

__global__ __launch_bounds__(256) void splitk_reduce_group_embed_kernel(GemmGroup R, EmbedTail e) {
  const int nred = R.first[R.count];
  if ((int)blockIdx.x >= nred) {
    const int vb = blockIdx.x - nred;
    embed_bwd_block(e.dtable, e.ids, e.dy, e.ld_dy, e.parts, e.part_stride, e.copy, e.ld_copy, e.n, e.E, vb % e.gx, vb / e.gx);
    return;
  }
  int p = 0;
  while (p + 1 < R.count && (int)blockIdx.x >= R.first[p + 1]) p++;
  const GemmArgs &g = R.g[p];
  const int splits = R.splits[p];
  long idx = (long)(blockIdx.x - R.first[p]) * blockDim.x + threadIdx.x;
  long total = (long)g.M * g.N;
  if (idx >= total) return;
  float acc = 0.f;
  for (int z = 0; z < splits; z++) acc += g.ws[(long)z * total + idx];
  int r = (int)(idx / g.N), c = (int)(idx % g.N);
  float v = g.alpha * acc;
  if (g.beta != 0.f) v += g.beta * g.C[r * g.ldc + c];
  g.C[r * g.ldc + c] = v;
}

// C = alpha * sum_z ws[z] + beta * C (+ D rows), z ascending: a fixed order, so the
// result does not depend on how the workgroups were scheduled.
__global__ void splitk_reduce_kernel(GemmArgs g, int splits) {
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  long total = (long)g.M * g.N;
  if (idx >= total) return;
  float acc = 0.f;
  for (int z = 0; z < splits; z++) acc += g.ws[(long)z * total + idx];
  int r = (int)(idx / g.N), c = (int)(idx % g.N);
  float v = g.alpha * acc;
  if (g.beta != 0.f) v += g.beta * g.C[r * g.ldc + c];
  if (g.D) v += g.D[(long)(r >> g.dshift) * g.ldd + c];
  g.C[r * g.ldc + c] = v;
}

// Skinny products (few rows: the tail rounds of a batch).  Such a product is a
// latency chain, not a throughput problem: the weights must stream past a handful of
// rows.  One workgroup owns a (32*TM) x 32 tile of C and its W wavefronts split K
// between them; every wavefront feeds the MFMA straight from global memory (the B
// operand of a 32x32x2 step is 32 consecutive floats per half-wave, so no LDS staging
// is needed) with several k-groups in flight, and the W partial tiles are summed
// through LDS in wavefront order (deterministic).  A is [M,K] row-major; B is [K,N]
// (TB = false) or [N,K] (TB = true).  Needs K, lda (and ldb when TB) multiples of 4.
template <int TM, bool TB, int W>
__global__ __launch_bounds__(W * 64) void sgemm_skinny_kernel(GemmArgs g) {
  constexpr int U = 4;  // k-groups of 8 in flight
  __shared__ float red[TM * 16 * 64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int j = lane & 31, h = lane >> 5;
  const int n0 = blockIdx.x * 32, m0 = blockIdx.y * 32 * TM;
  const int kper = ((g.K + W - 1) / W + 7) / 8 * 8;
  const int kb = wave * kper, ke = min(g.K, kb + kper);
  const bool col_ok = n0 + j < g.N;

  floatx16 acc[TM];
#pragma unroll
  for (int t = 0; t < TM; t++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[t][r] = 0.f;

  // one stage = U groups of 8 k values; the next stage's operands are fetched before
  // the MFMAs of the current one are issued, so memory latency overlaps the matrix pipe
  auto fetch = [&](int k0, float4 (&a)[U][TM], float (&b)[U][4]) {
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int kk = k0 + 8 * u + 4 * h;
      const bool kin = kk < ke;
#pragma unroll
      for (int t = 0; t < TM; t++) {
        const int row = m0 + 32 * t + j;
        a[u][t] = (kin && row < g.M) ? *reinterpret_cast<const float4 *>(g.A + (long)row * g.lda + kk)
                                     : make_float4(0.f, 0.f, 0.f, 0.f);
      }
      if constexpr (TB) {
        float4 q = (kin && col_ok) ? *reinterpret_cast<const float4 *>(g.B + (long)(n0 + j) * g.ldb + kk)
                                   : make_float4(0.f, 0.f, 0.f, 0.f);
        b[u][0] = q.x; b[u][1] = q.y; b[u][2] = q.z; b[u][3] = q.w;
      } else {
#pragma unroll
        for (int c = 0; c < 4; c++)
          b[u][c] = (col_ok && kk + c < ke) ? g.B[(long)(kk + c) * g.ldb + n0 + j] : 0.f;
      }
    }
  };
  auto multiply = [&](const float4 (&a)[U][TM], const float (&b)[U][4]) {
#pragma unroll
    for (int u = 0; u < U; u++)
#pragma unroll
      for (int t = 0; t < TM; t++) {
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u][t].x, b[u][0], acc[t], 0, 0, 0);
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u][t].y, b[u][1], acc[t], 0, 0, 0);
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u][t].z, b[u][2], acc[t], 0, 0, 0);
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u][t].w, b[u][3], acc[t], 0, 0, 0);
      }
  };
  float4 a0[U][TM], a1[U][TM];
  float b0[U][4], b1[U][4];
  constexpr int S = 8 * U;
  if (kb < ke) fetch(kb, a0, b0);
  for (int k0 = kb; k0 < ke; k0 += 2 * S) {
    if (k0 + S < ke) fetch(k0 + S, a1, b1);
    multiply(a0, b0);
    if (k0 + S < ke) {
      if (k0 + 2 * S < ke) fetch(k0 + 2 * S, a0, b0);
      multiply(a1, b1);
    }
  }

  // sum the W partial tiles in wavefront order
  for (int w = 0; w < W; w++) {
    if (wave == w) {
#pragma unroll
      for (int t = 0; t < TM; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          float *p = red + (t * 16 + r) * 64 + lane;
          *p = (w == 0) ? acc[t][r] : *p + acc[t][r];
        }
    }
    __syncthreads();
  }
  // epilogue: the W*64 threads share the TM*1024 outputs; element (t, r, lane') sits at
  // row 32t + 8(r/4) + 4(lane'/32) + r%4, column lane'%32
  for (int e = tid; e < TM * 1024; e += W * 64) {
    const int l2 = e & 63, r = (e >> 6) & 15, t = e >> 10;
    const int row = m0 + 32 * t + 8 * (r / 4) + 4 * (l2 >> 5) + (r % 4), col = n0 + (l2 & 31);
    if (row >= g.M || col >= g.N) continue;
    float v = g.alpha * red[e];
    if (g.beta != 0.f) v += g.beta * g.C[row * g.ldc + col];
    if (g.D) v += g.D[(long)(row >> g.dshift) * g.ldd + col];
    g.C[row * g.ldc + col] = v;
  }
}

struct GemmPlan {
  enum Kind { TILE128, TILE64, SKINNY } kind;
  int splits;   // > 1: partial tiles to the workspace + reduce kernel (TILE64 only)
  int kchunk;
  long tiles;
};

static bool skinny_ok(int tA, int tB, int K, const float *A, int lda, const float *B, int ldb) {
  if (tA || K % 4 || lda % 4 || !aligned16(A)) return false;
  if (tB && (ldb % 4 || !aligned16(B))) return false;
  return true;
}

static GemmPlan plan_gemm(int tA, int tB, int M, int N, int K, bool skinny_allowed, bool allow_split) {
  GemmPlan p;
  const long cus = num_cus();
  const long t128 = (long)((M + 127) / 128) * ((N + 127) / 128);
  const long t64 = (long)((M + 63) / 64) * ((N + 63) / 64);
  p.splits = 1;
  p.kchunk = K > 0 ? K : 1;
  // the large tile needs at least two rounds of workgroups to hide its ragged last round
  if (t128 >= 2 * cus) {
    p.kind = GemmPlan::TILE128;
    p.tiles = t128;
    return p;
  }
  // Tall-K products whose large tiles give each CU one workgroup or less (the deferred weight
  // gradients of big batches: 8x32 tiles, K = all rows): one workgroup per CU cannot hide the
  // latency of its own global loads, so K is split until about three share a CU.
  if (allow_split && 4 * t128 >= cus && K >= 4096) {
    long s = (3 * cus + t128 - 1) / t128;
    // one or two more splits when they even out the workgroups per CU (316 tiles: three splits are
    // 3.7 per CU, a fourth round at 70 %; four splits are 4.94: 90.8 -> 95.5 TFLOP/s at 512 x 10000
    // x 7331); ties keep the fewer splits (less partial traffic)
    auto fill = [&](long sp) {
      const long w = t128 * sp, rounds = (w + cus - 1) / cus;
      return (double)w / (double)(rounds * cus);
    };
    for (long c = s + 1; c <= s + 2; c++)
      if (fill(c) > fill(s) + 0.02) s = c;
    if (s > K / 1024) s = K / 1024;
    if (s > 1) {
      int kchunk = (int)(((K + s - 1) / s + 31) / 32 * 32);
      int splits = (K + kchunk - 1) / kchunk;
      if (splits > 1) {
        p.kind = GemmPlan::TILE128;
        p.tiles = t128;
        p.splits = splits;
        p.kchunk = kchunk;
        return p;
      }
    }
  }
  p.kind = GemmPlan::TILE64;
  p.tiles = t64;
  if (t64 >= 2 * cus || K < 64) return p;
  // the skinny kernel reads a k-contiguous B (NT) sixteen bytes per lane and row, which only
  // pays for a handful of rows; with B row-major (NN) it holds up to about a thousand
  if (skinny_allowed && M <= (tB ? 128 : 1024)) {
    p.kind = GemmPlan::SKINNY;
    return p;
  }
  if (allow_split && K >= 256) {
    long want = (3 * cus + t64 - 1) / t64;
    long maxs = K / 128;  // at least four k-tiles per split
    long s = want < maxs ? want : maxs;
    if (s > 32) s = 32;
    if (s > 1) {
      int kchunk = (int)(((K + s - 1) / s + 31) / 32 * 32);
      int splits = (K + kchunk - 1) / kchunk;
      if (splits > 1) {
        p.splits = splits;
        p.kchunk = kchunk;
      }
    }
  }
  return p;
}

static size_t plan_workspace(const GemmPlan &p, int M, int N) {
  return p.splits > 1 ? sizeof(float) * (size_t)p.splits * M * N : 0;
}

static bool vec_path_ok(const GemmArgs &g, int tA, int tB) {
  if (!aligned16(g.A) || !aligned16(g.B) || g.lda % 4 || g.ldb % 4) return false;
  // the contiguous index of each operand must come in whole float4s
  if (!tA ? (g.K % 4) : (g.M % 4)) return false;
  if (tB ? (g.K % 4) : (g.N % 4)) return false;
  return true;
}

// LDS a tile launch of the calling thread asks for on top of its panels (cavs_sgemm_group_beside): the
// workgroups then take more of a CU than they use, and fewer of them share one
static thread_local unsigned t_lds_pad = 0;

template <int BM, int BN, int BK>
static void launch_tile(const GemmArgs &args, int tA, int tB, bool vec, const GemmPlan &p, hipStream_t st) {
  GemmArgs g = args;
  dim3 grid((unsigned)p.tiles, p.splits), block(kThreads);
  if (g.zkind == CAVS_GEMM_A_ZERO || g.zkind == CAVS_GEMM_C_UNUSED) {
    const long inside = (long)(std::min(g.zrows, g.M) / BM) * ((g.N + BN - 1) / BN);
    if (inside > 0 && inside < p.tiles) {
      g.zseg = (int)inside;
      grid.x = (unsigned)((inside + 7) / 8 * 8 + (p.tiles - inside + 7) / 8 * 8);
    }
  }
#define CAVS_GEMM_CASE(TA, TB)                                                  \
  if (vec)                                                                      \
    launch(sgemm_mfma_kernel<BM, BN, BK, TA, TB, true>, grid, block, t_lds_pad, st, g);      \
  else                                                                          \
    launch(sgemm_mfma_kernel<BM, BN, BK, TA, TB, false>, grid, block, t_lds_pad, st, g)
  if (!tA && !tB) { CAVS_GEMM_CASE(false, false); }
  else if (!tA && tB) { CAVS_GEMM_CASE(false, true); }
  else if (tA && !tB) { CAVS_GEMM_CASE(true, false); }
  else { CAVS_GEMM_CASE(true, true); }
#undef CAVS_GEMM_CASE
}

static int check_gemm(const char *who, int tA, int tB, int M, int N, int K, const float *A, int lda,
                      const float *B, int ldb, const float *C, int ldc) {
  CAVS_REQUIRE(M >= 0 && N >= 0 && K >= 0, "%s: negative dimension M=%d N=%d K=%d", who, M, N, K);
  if (M == 0 || N == 0) return CAVS_OK;
  CAVS_REQUIRE(C && ldc >= N, "%s: bad C (ldc=%d, N=%d)", who, ldc, N);
  if (K > 0) {
    CAVS_REQUIRE(A && B, "%s: null operand", who);
    CAVS_REQUIRE(lda >= (tA ? M : K), "%s: lda=%d too small", who, lda);
    CAVS_REQUIRE(ldb >= (tB ? K : N), "%s: ldb=%d too small", who, ldb);
  }
  return CAVS_OK;
}

template <bool TB>
static void launch_skinny(const GemmArgs &g, hipStream_t st) {
  constexpr int W = 8;
  if (g.M <= 32) {
    dim3 grid((g.N + 31) / 32, 1);
    launch(sgemm_skinny_kernel<1, TB, W>, grid, W * 64, 0, st, g);
  } else {
    dim3 grid((g.N + 31) / 32, (g.M + 63) / 64);
    launch(sgemm_skinny_kernel<2, TB, W>, grid, W * 64, 0, st, g);
  }
}

// the looked-up rows of cavs_embed_pull_sgemm (GemmArgs::pull_*)
struct PullRows {
  const int *rows;
  const float *x;
  float *copy;
  long ld_copy;
  float *ids;
};

// What the caller knows about a block of an operand or of the result (cavs_gemm_desc::zero_kind,
// zero_rows, zero_col).  It is a licence, not an order: set() keeps it only in the forms the tile
// routine acts on and the kernels that never look at it give the plain product.
struct BlockHint {
  int kind = 0, rows = 0, col = 0;
  void set(GemmArgs *g, int tA, int tB, bool plain_store) const {
    if (rows <= 0 || col < 0) return;
    const bool ok = (kind == CAVS_GEMM_C_UNUSED && plain_store && col > 0) || (kind == CAVS_GEMM_A_ZERO && !tA && col % 4 == 0) ||
                    (kind == CAVS_GEMM_B_ZERO && !tB);
    if (!ok) return;
    g->zkind = kind;
    g->zrows = rows;
    g->zcol = col;
  }
};

static int run_gemm(const char *who, int tA, int tB, int M, int N, int K, float alpha, const float *A,
                    int lda, const float *B, int ldb, float beta, float *C, int ldc, const float *D,
                    int ldd, int dshift, void *ws, size_t ws_bytes, void *stream, const PullRows *pull = nullptr,
                    const BlockHint *hint = nullptr) {
  int rc = check_gemm(who, tA, tB, M, N, K, A, lda, B, ldb, C, ldc);
  if (rc || M == 0 || N == 0) return rc;
  GemmPlan p = plan_gemm(tA, tB, M, N, K, !pull && skinny_ok(tA, tB, K, A, lda, B, ldb), ws != nullptr);
  hipStream_t st = as_stream(stream);
  GemmArgs g{M, N, K, A, lda, B, ldb, C, ldc, alpha, beta, D, ldd, dshift, p.kchunk, nullptr};
  if (hint) hint->set(&g, tA, tB, beta == 0.f && !D);
  if (pull) {
    g.pull_rows = pull->rows;
    g.pull_x = pull->x;
    g.pull_copy = pull->copy;
    g.ld_copy = pull->ld_copy;
    g.pull_ids = pull->ids;
  }
  if (p.kind == GemmPlan::SKINNY) {
    if (tB) launch_skinny<true>(g, st); else launch_skinny<false>(g, st);
    CAVS_LAUNCH_CHECK();
    return CAVS_OK;
  }
  if (p.splits > 1) {
    size_t need = plan_workspace(p, M, N);
    CAVS_REQUIRE(ws_bytes >= need && aligned16(ws), "%s: workspace of %zu bytes needed, %zu given", who, need, ws_bytes);
    g.ws = static_cast<float *>(ws);
  }
  bool vec = vec_path_ok(g, tA, tB);
  // The chip holds four 64x64 workgroups per CU with K panels of 32 (their LDS) and eight with
  // panels of 16.  A launch of a few more than four per CU runs them as a second round behind
  // the first (2048 x 2048 x 300: 29.0 us; 2112 rows: 36.7), so launches between one and two
  // rounds take the narrow panels and stay resident at once (2482 rows: 40.2 -> 33.1 us);
  // everywhere else the wide panels are faster.
  const long wgs = p.tiles * p.splits, slots = 4L * num_cus();
  if (p.kind == GemmPlan::TILE128)
    launch_tile<128, 128, 16>(g, tA, tB, vec, p, st);
  else if (wgs > slots && wgs <= 2 * slots)
    launch_tile<64, 64, 16>(g, tA, tB, vec, p, st);
  else
    launch_tile<64, 64, 32>(g, tA, tB, vec, p, st);
  CAVS_LAUNCH_CHECK();
  if (p.splits > 1) {
    long total = (long)M * N;
    launch(splitk_reduce_kernel, (unsigned)((total + 255) / 256), 256, 0, st, g, p.splits);
    CAVS_LAUNCH_CHECK();
  }
  return CAVS_OK;
}

// Plans a group: every product on the 64x64 tile, K split so that all workgroups of the group
// together are about four per CU (what a CU holds at once; inside a training step eight per CU
// measured no better, though it is in a back-to-back loop), each with at least 256 of K.
// `tail_product` >= 0: that product's result is handed on to the embedding scatter-add (dtable, ids)
static int run_group(int count, const cavs_gemm_desc *d, void *ws, size_t ws_bytes, size_t *need_out, void *stream,
                     int tail_product = -1, float *dtable = nullptr, const float *ids = nullptr) {
  CAVS_REQUIRE(count >= 0 && count <= kGroupMax, "cavs_sgemm_group: %d products, at most %d", count, kGroupMax);
  CAVS_REQUIRE(count == 0 || d, "cavs_sgemm_group: null descriptors");
  EmbedTail tail{};
  if (tail_product >= 0 && !need_out) {
    CAVS_REQUIRE(tail_product < count, "cavs_sgemm_group_embed_bwd: product %d of %d", tail_product, count);
    const cavs_gemm_desc &q = d[tail_product];
    CAVS_REQUIRE(q.alpha == 1.f && q.beta == 0.f, "cavs_sgemm_group_embed_bwd: the product that feeds the table takes alpha = 1, beta = 0");
    CAVS_REQUIRE((q.M == 0 || q.N == 0) || (dtable && ids), "cavs_sgemm_group_embed_bwd: null pointer");
    // unsplit (or run alone): the scatter-add reads C
    tail = EmbedTail{dtable, ids, q.C, q.ldc, 0, 1, nullptr, 0, q.M, q.N, (q.M + kEmbedRows - 1) / kEmbedRows};
  }
  GemmGroup G{}, R{};
  double work = 0;
  long tiles[kGroupMax];
  bool alone[kGroupMax];
  int grouped = 0;
  size_t most = 0;
  for (int p = 0; p < count; p++) {
    const cavs_gemm_desc &q = d[p];
    if (!need_out) {
      int rc = check_gemm("cavs_sgemm_group", q.transA, q.transB, q.M, q.N, q.K, q.A, q.lda, q.B, q.ldb, q.C, q.ldc);
      if (rc) return rc;
    }
    CAVS_REQUIRE(q.M >= 0 && q.N >= 0 && q.K >= 0, "cavs_sgemm_group: negative dimension in product %d", p);
    CAVS_REQUIRE(q.zero_kind >= 0 && q.zero_kind <= CAVS_GEMM_B_ZERO && q.zero_rows >= 0 && q.zero_col >= 0,
                 "cavs_sgemm_group: bad block hint in product %d (kind %d, rows %d, col %d)", p, q.zero_kind, q.zero_rows, q.zero_col);
    tiles[p] = (long)((q.M + 63) / 64) * ((q.N + 63) / 64);
    // a product that fills the chip with large tiles by itself is better off on them, alone
    alone[p] = q.M > 0 && q.N > 0 && plan_gemm(q.transA, q.transB, q.M, q.N, q.K, false, true).kind == GemmPlan::TILE128;
    if (!alone[p] && q.M > 0 && q.N > 0) grouped++;
  }
  for (int p = 0; p < count; p++) {
    const cavs_gemm_desc &q = d[p];
    if (q.M == 0 || q.N == 0) continue;
    if (!alone[p] && grouped >= 2) {
      work += (double)tiles[p] * q.K;
      continue;
    }
    alone[p] = true;
    most = std::max(most, plan_workspace(plan_gemm(q.transA, q.transB, q.M, q.N, q.K, false, true), q.M, q.N));
  }
  const long slots = 4 * num_cus();
  long kc = (long)(work / (double)slots);
  kc = (kc + 31) / 32 * 32;
  if (kc < 256) kc = 256;
  // The chip holds `slots` of these workgroups at once.  A launch of a few more runs them as a
  // second round behind the first -- a whole workgroup's time for a handful of tiles (measured:
  // 1024 workgroups 95 us, 1032 workgroups 122 us) -- so the k chunk grows until the launch fits,
  // unless the tiles alone overflow it.
  auto launch_size = [&](long chunk) {
    long total = 0;
    for (int p = 0; p < count; p++) {
      const cavs_gemm_desc &q = d[p];
      if (q.M == 0 || q.N == 0 || alone[p]) continue;
      long s = q.K > 0 ? (q.K + chunk / 2) / chunk : 1;
      if (s < 1) s = 1;
      const long kchunk = q.K > 0 ? ((q.K + s - 1) / s + 31) / 32 * 32 : 1;
      const long splits = q.K > 0 ? (q.K + kchunk - 1) / kchunk : 1;
      total += (tiles[p] * splits + 7) / 8 * 8;
    }
    return total;
  };
  if (launch_size(1L << 30) <= slots)
    while (launch_size(kc) > slots) kc += 32;
  size_t need = 0;
  bool vec = true;
  int n = 0, nr = 0;
  for (int p = 0; p < count; p++) {
    const cavs_gemm_desc &q = d[p];
    if (q.M == 0 || q.N == 0 || alone[p]) continue;
    long s = q.K > 0 ? (q.K + kc / 2) / kc : 1;
    if (s < 1) s = 1;
    int kchunk = q.K > 0 ? (int)(((q.K + s - 1) / s + 31) / 32 * 32) : 1;
    int splits = q.K > 0 ? (q.K + kchunk - 1) / kchunk : 1;
    GemmArgs g{q.M, q.N, q.K, q.A, q.lda, q.B, q.ldb, q.C, q.ldc, q.alpha, q.beta, nullptr, 0, 0, kchunk, nullptr};
    BlockHint{q.zero_kind, q.zero_rows, q.zero_col}.set(&g, q.transA, q.transB, q.beta == 0.f);
    if (splits > 1) {
      if (ws) g.ws = reinterpret_cast<float *>(static_cast<char *>(ws) + need);
      need += ((size_t)splits * q.M * q.N * sizeof(float) + 255) / 256 * 256;
    }
    if (!need_out && !vec_path_ok(g, q.transA, q.transB)) vec = false;
    G.g[n] = g;
    G.tiles[n] = (int)tiles[p];
    G.splits[n] = splits;
    G.form[n] = (q.transA ? 2 : 0) + (q.transB ? 1 : 0);
    G.first[n + 1] = G.first[n] + (int)((tiles[p] * splits + 7) / 8 * 8);
    n++;
    if (splits > 1 && p == tail_product && !need_out) {
      // the scatter-add sums this product's partials itself (and leaves the sum in C as well)
      tail.dy = g.ws;
      tail.ld_dy = q.N;
      tail.part_stride = (long)q.M * q.N;
      tail.parts = splits;
      tail.copy = q.C;
      tail.ld_copy = q.ldc;
    } else if (splits > 1) {
      R.g[nr] = g;
      R.splits[nr] = splits;
      R.first[nr + 1] = R.first[nr] + (int)(((long)q.M * q.N + 255) / 256);
      nr++;
    }
  }
  G.count = n;
  R.count = nr;
  need = std::max(need, most);
  if (need_out) {
    *need_out = need;
    return CAVS_OK;
  }
  CAVS_REQUIRE(need == 0 || (ws && ws_bytes >= need && aligned16(ws)), "cavs_sgemm_group: workspace of %zu bytes needed, %zu given", need, ws_bytes);
  // the products that run alone share the workspace with the group: the stream orders them
  for (int p = 0; p < count; p++) {
    const cavs_gemm_desc &q = d[p];
    if (q.M == 0 || q.N == 0 || !alone[p]) continue;
    const BlockHint hint{q.zero_kind, q.zero_rows, q.zero_col};
    int rc = run_gemm("cavs_sgemm_group", q.transA, q.transB, q.M, q.N, q.K, q.alpha, q.A, q.lda, q.B, q.ldb, q.beta,
                      q.C, q.ldc, nullptr, 0, 0, ws, ws_bytes, stream, nullptr, &hint);
    if (rc) return rc;
  }
  hipStream_t st = as_stream(stream);
  if (n > 0) {
    if (vec) launch(sgemm_group_kernel<true>, (unsigned)G.first[n], kThreads, 0, st, G);
    else launch(sgemm_group_kernel<false>, (unsigned)G.first[n], kThreads, 0, st, G);
    CAVS_LAUNCH_CHECK();
  }
  const bool with_tail = tail_product >= 0 && tail.n > 0 && tail.E > 0;
  if (with_tail) {
    const int gy = (tail.E + kEmbedCols - 1) / kEmbedCols;
    launch(splitk_reduce_group_embed_kernel, (unsigned)(R.first[nr] + tail.gx * gy), 256, 0, st, R, tail);
    CAVS_LAUNCH_CHECK();
  } else if (nr > 0) {
    launch(splitk_reduce_group_kernel, (unsigned)R.first[nr], 256, 0, st, R);
    CAVS_LAUNCH_CHECK();
  }
  return CAVS_OK;
}

// Split-K partials of cavs_sgemm_splitk_static: device memory that exists from the moment the
// code object is loaded, so that entry point never has to ask the allocator for any.  Every GPU
// the library runs on holds its own copy until the process ends.
constexpr size_t kStaticScratchBytes = size_t(32) << 20;
constexpr int kStaticScratchDevices = 64;
static __device__ __align__(256) float scratch[kStaticScratchBytes / sizeof(float)];
// Device address of `scratch` on each GPU (the array's name is only a host-side stand-in for the
// symbol; kernels, fills and copies take the address looked up here).
static std::atomic<float *> g_scratch_ptr[kStaticScratchDevices];

// Looks the address up for the current device, once (two threads that both find it missing look
// it up twice and store the same value).
int static_scratch_setup(float **out) {
  int dev = 0;
  CAVS_HIP_TRY(hipGetDevice(&dev));
  CAVS_REQUIRE(dev >= 0 && dev < kStaticScratchDevices, "static scratch: device %d out of range", dev);
  float *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ptr) {
    CAVS_HIP_TRY(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)));
    CAVS_REQUIRE(ptr && aligned16(ptr), "static scratch: no usable address on device %d", dev);
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);
  }
  if (out) *out = ptr;
  return CAVS_OK;
}

}  // namespace cavs

using namespace cavs;

extern "C" {

int cavs_mfma_probe(float *out, size_t out_floats, int iters, double *flops, void *stream) {
  const int blocks = 4 * num_cus();
  CAVS_REQUIRE(out && iters > 0 && out_floats >= (size_t)blocks * 256, "cavs_mfma_probe: output of %d floats needed", blocks * 256);
  launch(mfma_probe_kernel, blocks, 256, 0, as_stream(stream), out, iters);
  CAVS_LAUNCH_CHECK();
  if (flops) *flops = (double)blocks * 4 * iters * 8 * 2.0 * 32 * 32 * 2;
  return CAVS_OK;
}

size_t cavs_sgemm_splitk_static_max_bytes(void) { return kStaticScratchBytes; }

int cavs_sgemm_splitk_static(int transA, int transB, int M, int N, int K, float alpha, const float *A,
                             int lda, const float *B, int ldb, float beta, float *C, int ldc, void *stream) {
  float *ptr = nullptr;
  int rc = static_scratch_setup(&ptr);
  if (rc) return rc;
  if (M > 0 && N > 0 && K > 0) {
    // the same plan run_gemm makes when it is handed a workspace
    GemmPlan p = plan_gemm(transA, transB, M, N, K, skinny_ok(transA, transB, K, A, lda, B, ldb), true);
    size_t need = p.kind == GemmPlan::SKINNY ? 0 : plan_workspace(p, M, N);
    if (need > kStaticScratchBytes)
      return set_error(CAVS_EINVAL,
                       "cavs_sgemm_splitk_static: M=%d N=%d K=%d needs %zu bytes of split-K partials, the built-in "
                       "scratch holds %zu; use cavs_sgemm_splitk with a workspace of the caller's",
                       M, N, K, need, kStaticScratchBytes);
  }
  // partials are written before they are read, every element of them: nothing of the previous
  // call's contents has to be cleared
  return run_gemm("cavs_sgemm_splitk_static", transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc,
                  nullptr, 0, 0, ptr, kStaticScratchBytes, stream);
}

size_t cavs_sgemm_group_workspace(int count, const cavs_gemm_desc *products) {
  size_t need = 0;
  if (run_group(count, products, nullptr, 0, &need, nullptr) != CAVS_OK) return 0;
  return need;
}

int cavs_sgemm_group(int count, const cavs_gemm_desc *products, void *workspace, size_t workspace_bytes,
                     void *stream) {
  return run_group(count, products, workspace, workspace_bytes, nullptr, stream);
}

int cavs_sgemm_group_beside(int count, const cavs_gemm_desc *products, void *workspace, size_t workspace_bytes,
                            void *stream) {
  t_lds_pad = 22u << 10;  // with the 33 KB of a tile's panels: two workgroups per CU
  const int rc = run_group(count, products, workspace, workspace_bytes, nullptr, stream);
  t_lds_pad = 0;
  return rc;
}

int cavs_sgemm_group_embed_bwd(int count, const cavs_gemm_desc *products, int embed_product, float *dtable, const float *ids,
                               void *workspace, size_t workspace_bytes, void *stream) {
  CAVS_REQUIRE(embed_product >= 0, "cavs_sgemm_group_embed_bwd: product %d", embed_product);
  return run_group(count, products, workspace, workspace_bytes, nullptr, stream, embed_product, dtable, ids);
}

int cavs_embed_pull_sgemm(float *C, int ldc, float *e_out, int ld_e, float *ids_out, const float *x, const int *rows,
                          const float *table, int n, int E, const float *B, int ldb, int N, int unused_rows, int unused_col,
                          void *stream) {
  CAVS_REQUIRE(n >= 0 && E > 0 && N >= 0 && ld_e >= E, "cavs_embed_pull_sgemm: bad shape n=%d E=%d N=%d ld_e=%d", n, E, N, ld_e);
  CAVS_REQUIRE(unused_rows >= 0 && unused_col >= 0, "cavs_embed_pull_sgemm: bad unused block (rows %d, col %d)", unused_rows, unused_col);
  const BlockHint hint{CAVS_GEMM_C_UNUSED, unused_rows, unused_col};
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(e_out && ids_out && x && rows && table, "cavs_embed_pull_sgemm: null pointer");
  // the copy goes out in whole float4s on the vector path
  CAVS_REQUIRE(E % 4 != 0 || (aligned16(e_out) && ld_e % 4 == 0), "cavs_embed_pull_sgemm: e_out must be 16-byte aligned with ld_e a multiple of 4");
  // A product large enough for the 128 x 128 tiles gains nothing from the saved launch and its
  // workgroups are slowed by the lookups (7331 x 2048 x 512: 157 -> 180 us): the two calls then.
  if (N == 0 || plan_gemm(0, 0, n, N, E, false, false).kind == GemmPlan::TILE128) {
    int rc = cavs_embed_pull_fwd(e_out, ld_e, ids_out, x, rows, table, n, E, stream);
    if (rc || N == 0) return rc;
    return run_gemm("cavs_embed_pull_sgemm", 0, 0, n, N, E, 1.f, e_out, ld_e, B, ldb, 0.f, C, ldc, nullptr, 0, 0, nullptr, 0, stream,
                    nullptr, &hint);
  }
  const PullRows pull{rows, x, e_out, ld_e, ids_out};
  return run_gemm("cavs_embed_pull_sgemm", 0, 0, n, N, E, 1.f, table, E, B, ldb, 0.f, C, ldc, nullptr, 0, 0, nullptr, 0, stream, &pull,
                  &hint);
}

int cavs_sgemm(int transA, int transB, int M, int N, int K, float alpha, const float *A, int lda,
               const float *B, int ldb, float beta, float *C, int ldc, void *stream) {
  return run_gemm("cavs_sgemm", transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, nullptr, 0,
                  0, nullptr, 0, stream);
}

int cavs_sgemm_addrows(int transA, int transB, int M, int N, int K, const float *A, int lda,
                       const float *B, int ldb, const float *D, int ldd, int d_shift, float *C,
                       int ldc, void *workspace, size_t workspace_bytes, void *stream) {
  if (M > 0 && N > 0)
    CAVS_REQUIRE(D && ldd >= N && d_shift >= 0 && d_shift < 31, "cavs_sgemm_addrows: bad addend (ldd=%d shift=%d)", ldd, d_shift);
  return run_gemm("cavs_sgemm_addrows", transA, transB, M, N, K, 1.f, A, lda, B, ldb, 0.f, C, ldc, D, ldd,
                  d_shift, workspace, workspace_bytes, stream);
}

size_t cavs_sgemm_splitk_workspace(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  // sized for the split plan whether or not a given call ends up taking the skinny path
  return plan_workspace(plan_gemm(0, 0, M, N, K, false, true), M, N);
}

int cavs_sgemm_splitk(int transA, int transB, int M, int N, int K, float alpha, const float *A,
                      int lda, const float *B, int ldb, float beta, float *C, int ldc,
                      void *workspace, size_t workspace_bytes, void *stream) {
  return run_gemm("cavs_sgemm_splitk", transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc,
                  nullptr, 0, 0, workspace, workspace_bytes, stream);
}

}  // extern "C"
