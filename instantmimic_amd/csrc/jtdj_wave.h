// H = M + J' diag(D [state == quad]) J of one world on one wavefront, for up to four 16-column
// blocks (the first Hessian of a dense Newton solve below 64 dofs), and the store of a lane's share
// of a 16 x 16 accumulator tile into H and its mirror image.
// Reference: upstream's solver._update_gradient as src/instantmimic/utils/mjw_kernels/newton_fusion.py:470
// calls it (the dense Newton's full assembly ahead of the first factor).
// An element's sum is the chain fma(J[r][i] * Dc[r], J[r][j], .) over the rows in order, from M:
// what the workgroup-per-world kernel of blocked_kernels.hip forms (a row with weight zero leaves
// every chain as it is).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace im {

typedef float float4v __attribute__((ext_vector_type(4)));

// Stores what one lane holds of a tile into H and its mirror image: rows i0 .. i0 + 3 of column j
// (the elements with i <= j < nv count).  Right of the diagonal blocks (`off`) the mirror image of a
// lane's four values is four consecutive words of row j: one 16-byte store where H allows it (`vec`).
__device__ __forceinline__ void store_h_mirrored(float *__restrict__ Hw, int nv, int nv_pad, bool vec, int i0, int j,
                                                 float4v h, bool off) {
  if (j >= nv) return;
#pragma unroll
  for (int v = 0; v < 4; ++v)
    if (i0 + v < nv && i0 + v <= j) Hw[(int64_t)(i0 + v) * nv_pad + j] = h[v];
  if (off && vec && i0 + 3 < nv) {
    *(float4v *)(Hw + (int64_t)j * nv_pad + i0) = h;
  } else {
#pragma unroll
    for (int v = 0; v < 4; ++v)
      if (i0 + v < nv && i0 + v < j) Hw[(int64_t)j * nv_pad + i0 + v] = h[v];
  }
}

// NB blocks of 16 columns (nv <= 16 NB).  elemid (nv, nv): the element of the world's row Mw that
// lies at (i, j), negative outside M's pattern.  Operands come straight from memory in the layout
// of v_mfma_f32_16x16x4_f32 (lane l supplies row 4 q + l / 16, column 16 b + l % 16 of step q: four
// rows of 64 bytes per load), the next sixteen rows' loads in flight behind the current ones'
// products; nothing is staged.
template <int NB>
__device__ __forceinline__ void jtdj_wave(const float *__restrict__ Mw, const int32_t *__restrict__ elemid,
                                          const float *__restrict__ Jw, const float *__restrict__ Dw,
                                          const int32_t *__restrict__ sw, int nefc, int quad, int nv,
                                          float *__restrict__ Hw, int pad, bool vec, int lane) {
  constexpr int NT = NB * (NB + 1) / 2;
  const int c = lane & 15, kq = lane >> 4;
  const int nstep = (nefc + 3) >> 2;
  float u[4][NB], dk[4], un[4][NB], dn[4];
  // the operands of four steps (sixteen rows): asked for a group ahead of the products that use them
  auto fetch = [&](int q0, float (&uu)[4][NB], float (&dd)[4]) __attribute__((always_inline)) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int row = 4 * (q0 + s) + kq;
      const bool in = row < nefc;
      const int rowc = in ? row : nefc - 1;
      const float dv = Dw[rowc];
      const int st = sw[rowc];
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        const int col = 16 * b + c;
        const float jv = Jw[(int64_t)rowc * nv + (col < nv ? col : nv - 1)];
        uu[s][b] = (in && col < nv) ? jv : 0.0f;
      }
      dd[s] = (in && st == quad) ? dv : 0.0f;
    }
  };
  if (nstep > 0) fetch(0, u, dk);  // on their way while M is gathered
  float4v acc[NT];
  {  // the accumulators start from M (a lane holds column j = l % 16 and rows 4 (l / 16) + v of a tile)
    int m = 0;
#pragma unroll
    for (int bi = 0; bi < NB; ++bi)
#pragma unroll
      for (int bj = bi; bj < NB; ++bj, ++m) {
        const int j = 16 * bj + c, jc = j < nv ? j : nv - 1;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int i = 16 * bi + 4 * kq + v, ic = i < nv ? i : nv - 1;
          const int id = elemid[ic * nv + jc];
          const float mv = Mw[id < 0 ? 0 : id];
          acc[m][v] = (i < nv && j < nv && id >= 0) ? mv : 0.0f;
        }
      }
  }
  for (int q0 = 0; q0 < nstep; q0 += 4) {
    if (q0 + 4 < nstep) fetch(q0 + 4, un, dn);
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      float wt[NB];
#pragma unroll
      for (int b = 0; b < NB; ++b) wt[b] = u[s][b] * dk[s];
      int m = 0;
#pragma unroll
      for (int bi = 0; bi < NB; ++bi)
#pragma unroll
        for (int bj = bi; bj < NB; ++bj, ++m)
          acc[m] = __builtin_amdgcn_mfma_f32_16x16x4f32(wt[bi], u[s][bj], acc[m], 0, 0, 0);
    }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      dk[s] = dn[s];
#pragma unroll
      for (int b = 0; b < NB; ++b) u[s][b] = un[s][b];
    }
  }
  int m = 0;
#pragma unroll
  for (int bi = 0; bi < NB; ++bi)
#pragma unroll
    for (int bj = bi; bj < NB; ++bj, ++m) store_h_mirrored(Hw, nv, pad, vec, 16 * bi + 4 * kq, 16 * bj + c, acc[m], bi != bj);
}

}  // namespace im
