// FP32 GEMM on the CDNA4 matrix cores (v_mfma_f32_32x32x2_f32), row-major, for the
// gate products of the vertex functions: NN (X*W), NT (dY*W^T) and TN (X^T*dY).
//
// Workgroup = 4 wavefronts (2x2) over a BM x BN tile of C, BK = 16 deep.  A and B
// tiles are staged through LDS as [k][m] / [k][n] panels (double buffered, one
// barrier per k-tile), so each MFMA operand read is a conflict-free ds_read_b32 of
// 32 consecutive floats per half-wave.  Global loads are 16-byte per lane; the
// k-contiguous operand (A of NN/NT, B of NT) is transposed on its way into LDS.
// Workgroup ids are remapped so that consecutive tiles (which share an A row panel)
// run on the same XCD and hit the same L2.
#include "common.h"

namespace cavs {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int BK = 16;
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
  float *ws;       // split-K partials [splits][M][N] or nullptr
};

// Loader of one BX x BK operand tile.  KC: the operand's k index is the contiguous
// one in memory (element (x,k) at P[x*ld + k]); otherwise element at P[k*ld + x].
template <int BX, bool KC, bool VEC>
struct TileLoader {
  static constexpr int NV = BX * BK / 4 / kThreads;  // float4 per thread
  float4 reg[NV];

  __device__ inline void load(const float *__restrict__ P, long ld, int x0, int k0, int X,
                              int Kend, int tid) {
#pragma unroll
    for (int i = 0; i < NV; i++) {
      int gx, gk;
      long off, step;
      bool xin[4], kin[4];
      if constexpr (KC) {
        gx = x0 + tid / 4 + 64 * i;
        gk = k0 + 4 * (tid % 4);
        off = (long)gx * ld + gk;
        step = 1;
#pragma unroll
        for (int c = 0; c < 4; c++) { xin[c] = gx < X; kin[c] = gk + c < Kend; }
      } else {
        constexpr int PER = BX / 4;  // float4 per k row
        gk = k0 + tid / PER + (kThreads / PER) * i;
        gx = x0 + 4 * (tid % PER);
        off = (long)gk * ld + gx;
        step = 1;
#pragma unroll
        for (int c = 0; c < 4; c++) { xin[c] = gx + c < X; kin[c] = gk < Kend; }
      }
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if constexpr (VEC) {
        // whole float4 in or out (X, K multiples of 4 along the contiguous index)
        if (xin[0] && kin[0]) v = *reinterpret_cast<const float4 *>(P + off);
      } else {
        if (xin[0] && kin[0]) v.x = P[off];
        if (xin[1] && kin[1]) v.y = P[off + step];
        if (xin[2] && kin[2]) v.z = P[off + 2 * step];
        if (xin[3] && kin[3]) v.w = P[off + 3 * step];
      }
      reg[i] = v;
    }
  }

  __device__ inline void store(float *__restrict__ S, int tid) const {
    constexpr int LD = BX + PAD;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      if constexpr (KC) {
        int x = tid / 4 + 64 * i, k = 4 * (tid % 4);
        S[(k + 0) * LD + x] = reg[i].x;
        S[(k + 1) * LD + x] = reg[i].y;
        S[(k + 2) * LD + x] = reg[i].z;
        S[(k + 3) * LD + x] = reg[i].w;
      } else {
        constexpr int PER = BX / 4;
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

template <int BM, int BN, bool TA, bool TB, bool VEC>
__global__ __launch_bounds__(kThreads) void sgemm_mfma_kernel(GemmArgs g) {
  constexpr int WM = BM / 2, WN = BN / 2, TM = WM / 32, TN = WN / 32;
  constexpr int LDA = BM + PAD, LDB = BN + PAD;
  __shared__ __attribute__((aligned(16))) float As[2][BK * LDA];
  __shared__ __attribute__((aligned(16))) float Bs[2][BK * LDB];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tilesN = (g.N + BN - 1) / BN, tilesM = (g.M + BM - 1) / BM;
  const int t = xcd_remap(blockIdx.x, tilesM * tilesN);
  const int m0 = (t / tilesN) * BM, n0 = (t % tilesN) * BN;
  const int kbeg = blockIdx.y * g.kchunk;
  const int kend = min(g.K, kbeg + g.kchunk);

  TileLoader<BM, !TA, VEC> la;
  TileLoader<BN, TB, VEC> lb;

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  const int nk = (kend - kbeg + BK - 1) / BK;
  if (nk > 0) {
    la.load(g.A, g.lda, m0, kbeg, g.M, kend, tid);
    lb.load(g.B, g.ldb, n0, kbeg, g.N, kend, tid);
    la.store(As[0], tid);
    lb.store(Bs[0], tid);
  }
  __syncthreads();
  const int arow = wm * WM + (lane & 31), brow = wn * WN + (lane & 31), khalf = lane >> 5;
  for (int kt = 0; kt < nk; kt++) {
    const int cur = kt & 1;
    if (kt + 1 < nk) {
      la.load(g.A, g.lda, m0, kbeg + (kt + 1) * BK, g.M, kend, tid);
      lb.load(g.B, g.ldb, n0, kbeg + (kt + 1) * BK, g.N, kend, tid);
    }
    const float *as = As[cur], *bs = Bs[cur];
#pragma unroll
    for (int kk = 0; kk < BK; kk += 2) {
      float a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; i++) a[i] = as[(kk + khalf) * LDA + arow + 32 * i];
#pragma unroll
      for (int j = 0; j < TN; j++) b[j] = bs[(kk + khalf) * LDB + brow + 32 * j];
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < nk) {
      la.store(As[cur ^ 1], tid);
      lb.store(Bs[cur ^ 1], tid);
    }
    __syncthreads();
  }

  // C layout of the 32x32 accumulator: element r of lane l is row 8*(r/4) + 4*(l/32) + r%4,
  // column l%32.
  float *out = g.ws ? g.ws + (long)blockIdx.y * g.M * g.N : g.C;
  const long ldo = g.ws ? g.N : g.ldc;
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++) {
      const int col = n0 + wn * WN + 32 * j + (lane & 31);
      if (col >= g.N) continue;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int row = m0 + wm * WM + 32 * i + 8 * (r / 4) + 4 * khalf + (r % 4);
        if (row >= g.M) continue;
        float v = acc[i][j][r];
        if (!g.ws) {
          v *= g.alpha;
          if (g.beta != 0.f) v += g.beta * out[row * ldo + col];
          if (g.D) v += g.D[(long)(row >> g.dshift) * g.ldd + col];
        }
        out[row * ldo + col] = v;
      }
    }
}

// C = alpha * sum_z ws[z] + beta * C, z ascending (fixed order: deterministic)
__global__ void splitk_reduce_kernel(const float *__restrict__ ws, int splits, int M, int N,
                                     float alpha, float beta, float *__restrict__ C, long ldc) {
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  long total = (long)M * N;
  if (idx >= total) return;
  float acc = 0.f;
  for (int z = 0; z < splits; z++) acc += ws[(long)z * total + idx];
  int r = (int)(idx / N), c = (int)(idx % N);
  float v = alpha * acc;
  if (beta != 0.f) v += beta * C[r * ldc + c];
  C[r * ldc + c] = v;
}

template <int BM, int BN>
static void launch_tile(const GemmArgs &g, int tA, int tB, bool vec, int splits, hipStream_t st) {
  int tiles = ((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN);
  dim3 grid(tiles, splits), block(kThreads);
#define CAVS_GEMM_CASE(TA, TB)                                                                   \
  if (vec)                                                                                       \
    sgemm_mfma_kernel<BM, BN, TA, TB, true><<<grid, block, 0, st>>>(g);                           \
  else                                                                                           \
    sgemm_mfma_kernel<BM, BN, TA, TB, false><<<grid, block, 0, st>>>(g)
  if (!tA && !tB) { CAVS_GEMM_CASE(false, false); }
  else if (!tA && tB) { CAVS_GEMM_CASE(false, true); }
  else if (tA && !tB) { CAVS_GEMM_CASE(true, false); }
  else { CAVS_GEMM_CASE(true, true); }
#undef CAVS_GEMM_CASE
}

static bool vec_path_ok(const GemmArgs &g, int tA, int tB) {
  if (!aligned16(g.A) || !aligned16(g.B) || g.lda % 4 || g.ldb % 4) return false;
  // the contiguous index of each operand must come in whole float4s
  if (!tA ? (g.K % 4) : (g.M % 4)) return false;
  if (tB ? (g.K % 4) : (g.N % 4)) return false;
  return true;
}

static void launch_gemm(const GemmArgs &g, int tA, int tB, int splits, hipStream_t st) {
  bool vec = vec_path_ok(g, tA, tB);
  long big_tiles = (long)((g.M + 127) / 128) * ((g.N + 127) / 128) * splits;
  if (big_tiles >= num_cus())
    launch_tile<128, 128>(g, tA, tB, vec, splits, st);
  else
    launch_tile<64, 64>(g, tA, tB, vec, splits, st);
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

static int choose_splits(int M, int N, int K) {
  long tiles = (long)((M + 127) / 128) * ((N + 127) / 128);
  int cus = num_cus();
  if (tiles >= cus || K < 4 * BK) return 1;
  long want = (2L * cus + tiles - 1) / tiles;
  long maxs = K / (2 * BK);
  long s = want < maxs ? want : maxs;
  if (s > 64) s = 64;
  return s < 1 ? 1 : (int)s;
}

}  // namespace cavs

using namespace cavs;

extern "C" {

int cavs_sgemm(int transA, int transB, int M, int N, int K, float alpha, const float *A, int lda,
               const float *B, int ldb, float beta, float *C, int ldc, void *stream) {
  int rc = check_gemm("cavs_sgemm", transA, transB, M, N, K, A, lda, B, ldb, C, ldc);
  if (rc || M == 0 || N == 0) return rc;
  GemmArgs g{M, N, K, A, lda, B, ldb, C, ldc, alpha, beta, nullptr, 0, 0, K > 0 ? K : 1, nullptr};
  launch_gemm(g, transA, transB, 1, as_stream(stream));
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

int cavs_sgemm_addrows(int transA, int transB, int M, int N, int K, const float *A, int lda,
                       const float *B, int ldb, const float *D, int ldd, int d_shift, float *C,
                       int ldc, void *stream) {
  int rc = check_gemm("cavs_sgemm_addrows", transA, transB, M, N, K, A, lda, B, ldb, C, ldc);
  if (rc || M == 0 || N == 0) return rc;
  CAVS_REQUIRE(D && ldd >= N && d_shift >= 0 && d_shift < 31, "cavs_sgemm_addrows: bad addend (ldd=%d shift=%d)", ldd, d_shift);
  GemmArgs g{M, N, K, A, lda, B, ldb, C, ldc, 1.f, 0.f, D, ldd, d_shift, K > 0 ? K : 1, nullptr};
  launch_gemm(g, transA, transB, 1, as_stream(stream));
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

size_t cavs_sgemm_splitk_workspace(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  int s = choose_splits(M, N, K);
  return s > 1 ? (size_t)s * M * N * sizeof(float) : 0;
}

int cavs_sgemm_splitk(int transA, int transB, int M, int N, int K, float alpha, const float *A,
                      int lda, const float *B, int ldb, float beta, float *C, int ldc,
                      void *workspace, size_t workspace_bytes, void *stream) {
  int rc = check_gemm("cavs_sgemm_splitk", transA, transB, M, N, K, A, lda, B, ldb, C, ldc);
  if (rc || M == 0 || N == 0) return rc;
  int splits = K > 0 ? choose_splits(M, N, K) : 1;
  hipStream_t st = as_stream(stream);
  if (splits <= 1) {
    GemmArgs g{M, N, K, A, lda, B, ldb, C, ldc, alpha, beta, nullptr, 0, 0, K > 0 ? K : 1, nullptr};
    launch_gemm(g, transA, transB, 1, st);
    CAVS_LAUNCH_CHECK();
    return CAVS_OK;
  }
  size_t need = (size_t)splits * M * N * sizeof(float);
  CAVS_REQUIRE(workspace && workspace_bytes >= need && aligned16(workspace),
               "cavs_sgemm_splitk: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  int kchunk = ((K + splits - 1) / splits + BK - 1) / BK * BK;
  splits = (K + kchunk - 1) / kchunk;
  GemmArgs g{M, N, K, A, lda, B, ldb, C, ldc, alpha, beta, nullptr, 0, 0, kchunk,
             static_cast<float *>(workspace)};
  launch_gemm(g, transA, transB, splits, st);
  CAVS_LAUNCH_CHECK();
  long total = (long)M * N;
  splitk_reduce_kernel<<<(unsigned)((total + 255) / 256), 256, 0, st>>>(
      static_cast<const float *>(workspace), splits, M, N, alpha, beta, C, ldc);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

}  // extern "C"
