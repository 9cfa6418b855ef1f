// Shared pieces of the fused round kernels: the two MFMA tile shapes, operand helpers, the
// per-wavefront partial-tile reduction through LDS, and the tile / wavefront plan.
#ifndef CAVS_CSRC_ROUND_COMMON_H_
#define CAVS_CSRC_ROUND_COMMON_H_

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

__device__ inline float4 ld4(const float *p) { return *reinterpret_cast<const float4 *>(p); }
__device__ inline float4 zero4() { return make_float4(0.f, 0.f, 0.f, 0.f); }
__device__ inline float elem(const float4 &v, int c) { return c == 0 ? v.x : c == 1 ? v.y : c == 2 ? v.z : v.w; }
__device__ inline float sigm_r(float x) { return 1.f / (1.f + expf(-x)); }


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
// CU several 32x32 tiles (600 rows: 32 us against 40).  Eight wavefronts per workgroup up to
// 64 rows (shortest latency chain); four beyond, compiled for four workgroups per CU so that
// their latency chains overlap; 32x32 tiles above a thousand rows, where operand reuse counts.
inline RoundPlan plan_round(int n) {
  if (n <= 64) return {16, 8};
  if (n <= 1024) return {16, 4};
  return {32, 8};
}

}  // namespace cavs
#endif
