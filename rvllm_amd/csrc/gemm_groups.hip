// Many small products in one launch, C_g = A_g * W_g^T, with 32-bit multiply-adds: the products of a group of
// attention heads (one matrix a head, the heads' inputs and outputs side by side in a row) and of a set of experts
// (one matrix an expert, rows sorted by expert).
//
//   heads    group g = blockIdx.z;  A_g = a + g * a_group_stride (its columns inside a row of lda),
//            W_g = w + g * w_group_stride, C_g = c + g * c_group_stride
//   experts  tile_group[blockIdx.y] names the group of a tile of 64 rows (-1: the tile holds no rows and the block
//            does nothing); a_group_stride and c_group_stride are 0; with `row_index` row r of A is row
//            row_index[r] of a (-1: a row of zeros), so the sorted rows need not be copied together first
//
// With `gate`, C = (A W^T) * sigmoid(gate), gate laid out like C (ldg).  Every output is one chain of fused
// multiply-adds over k in order, as in gemm_plain: it does not depend on where its row lies or on the other rows.
#include "common.h"

#define GG_BM 64
#define GG_BN 64
#define GG_BK 16

template <typename TA, typename TW, typename TC>
__global__ void __launch_bounds__(256)
gemm_groups_plain_kernel(const TA* __restrict__ a, const TW* __restrict__ w, TC* __restrict__ c,
                         const int* __restrict__ row_index, const int* __restrict__ tile_group, int M, int N, int K,
                         long long lda, long long ldw, long long ldc, long long a_group_stride,
                         long long w_group_stride, long long c_group_stride, const TC* __restrict__ gate,
                         long long ldg) {
  __shared__ float a_s[GG_BK][GG_BM + 4];
  __shared__ float w_s[GG_BK][GG_BN + 4];
  const int group = tile_group ? tile_group[blockIdx.y] : (int)blockIdx.z;
  if (group < 0) return;  // the whole block alike
  a += (size_t)group * a_group_stride;
  w += (size_t)group * w_group_stride;
  c += (size_t)group * c_group_stride;
  if (gate) gate += (size_t)group * c_group_stride;
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * GG_BM, n0 = blockIdx.x * GG_BN;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  const int lr = tid / 4, lk = (tid % 4) * 4;
  const int am = m0 + lr;
  long long a_row = -1;
  if (am < M) a_row = row_index ? row_index[am] : am;
  const int wn = n0 + lr;
  for (int k0 = 0; k0 < K; k0 += GG_BK) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int k = k0 + lk + e;
      a_s[lk + e][lr] = (a_row >= 0 && k < K) ? rv_to_float(a[(size_t)a_row * lda + k]) : 0.f;
      w_s[lk + e][lr] = (wn < N && k < K) ? rv_to_float(w[(size_t)wn * ldw + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GG_BK; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = a_s[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = w_s[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (gate) v *= 1.0f / (1.0f + expf(-rv_to_float(gate[(size_t)m * ldg + n])));
      c[(size_t)m * ldc + n] = rv_from_float<TC>(v);
    }
  }
}

// groups > 0: the heads' form (tile_group and row_index null).  groups == 0: the experts' form; tile_group holds
// ceil(M / 64) entries, row_index (or null) M.
extern "C" int rv_gemm_groups_plain(hipStream_t stream, const void* a, int a_dtype, const void* w, int w_dtype, void* c,
                                    int c_dtype, const int* row_index, const int* tile_group, int groups, int M, int N,
                                    int K, long long lda, long long ldw, long long ldc, long long a_group_stride,
                                    long long w_group_stride, long long c_group_stride, const void* gate,
                                    long long ldg) {
  RV_CHECK(M >= 0 && N > 0 && K > 0 && groups >= 0, "gemm_groups: bad sizes M=%d N=%d K=%d groups=%d", M, N, K, groups);
  RV_CHECK((groups > 0) == (tile_group == nullptr), "gemm_groups: either a number of groups or the groups of the row tiles");
  RV_CHECK(ldw >= K && ldc >= N && lda >= K, "gemm_groups: leading dimensions too small");
  RV_CHECK(gate == nullptr || ldg >= N, "gemm_groups: the gate's rows are too short");
  if (M == 0) return 0;
  dim3 grid(rv_div_up(N, GG_BN), rv_div_up(M, GG_BM), groups > 0 ? groups : 1), block(256);
  RV_CHECK(grid.y < 65536 && grid.z < 65536, "gemm_groups: too many row tiles or groups for one launch");
#define RV_GG(TA, TW, TC)                                                                                          \
  gemm_groups_plain_kernel<TA, TW, TC><<<grid, block, 0, stream>>>(                                                \
      (const TA*)a, (const TW*)w, (TC*)c, row_index, tile_group, M, N, K, lda, ldw, ldc, a_group_stride,           \
      w_group_stride, c_group_stride, (const TC*)gate, ldg)
  if (a_dtype == RV_F32 && w_dtype == RV_F32 && c_dtype == RV_F32) RV_GG(float, float, float);
  else if (a_dtype == RV_BF16 && w_dtype == RV_BF16 && c_dtype == RV_BF16) RV_GG(bf16_t, bf16_t, bf16_t);
  else return rv_fail("gemm_groups: unsupported dtypes a=%d w=%d c=%d", a_dtype, w_dtype, c_dtype);
#undef RV_GG
  RV_LAUNCH_CHECK("gemm_groups_plain");
  return 0;
}
