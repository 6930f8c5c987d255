// The cache write of latent attention: a token's compressed key/value vector, RMS-normed, into its page.
//
//   c = raw * rsqrt(mean(raw^2) + eps) * (offset + w)        32-bit, as the row norms
//
// raw are `rank` columns (from col0 on) of a projection's rows [tokens, ld].  The cache holds one key/value head
// of `rank` dimensions: c goes to the key pages (one row a slot) and to the value pages (transposed inside groups
// of 16 slots, kv_layout.h), so that the attention kernels, which score the queries against c and sum c itself
// under the probabilities, read both operands in the order they sum them.  One wave a token.
#include "common.h"
#include "kv_layout.h"

#define LAT_MAX_RANK 512
#define LAT_PER_LANE (LAT_MAX_RANK / RV_WAVE)

template <typename T>
__global__ void __launch_bounds__(256)
latent_norm_write_kernel(const T* __restrict__ raw, long long ld, int col0, const void* __restrict__ w, int w_f32,
                         float eps, float offset, const int* __restrict__ positions,
                         const int* __restrict__ token_req, const int* __restrict__ block_table, int table_width,
                         T* __restrict__ k_pages, T* __restrict__ v_pages, int page_size, int num_pages, int rank,
                         int num_tokens) {
  const int lane = threadIdx.x & (RV_WAVE - 1);
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= num_tokens) return;  // the whole wave
  const T* r = raw + (size_t)t * ld + col0;
  float val[LAT_PER_LANE];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < LAT_PER_LANE; ++e) {
    const int i = e * RV_WAVE + lane;
    val[e] = i < rank ? rv_to_float(r[i]) : 0.f;
    ss = fmaf(val[e], val[e], ss);
  }
  ss = rv_wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)rank + eps);
  const int p = positions[t];
  const int logical = p / page_size;
  const int page = (p >= 0 && logical < table_width) ? block_table[(size_t)token_req[t] * table_width + logical] : -1;
  if (page < 0 || page >= num_pages) return;  // no page: nothing is written, and attention makes the fault show
  const int slot = p % page_size;
#pragma unroll
  for (int e = 0; e < LAT_PER_LANE; ++e) {
    const int i = e * RV_WAVE + lane;
    if (i < rank) {
      const T c = rv_from_float<T>(val[e] * inv * (offset + rv_load_w(w, w_f32, i)));
      k_pages[rv_k_index(page, 0, slot, i, 1, page_size, rank)] = c;
      v_pages[rv_v_index(page, 0, slot, i, 1, page_size, rank)] = c;
    }
  }
}

extern "C" int rv_latent_norm_write(hipStream_t stream, const void* raw, long long ld, int col0, const void* w,
                                    int w_f32, float eps, float offset, const int* positions, const int* token_req,
                                    const int* block_table, int table_width, void* k_pages, void* v_pages,
                                    int page_size, int num_pages, int rank, int num_tokens, int dtype) {
  RV_CHECK(num_tokens >= 0 && rank > 0 && rank <= LAT_MAX_RANK, "latent_norm_write: rank %d must be in 1..%d", rank,
           LAT_MAX_RANK);
  RV_CHECK(col0 >= 0 && ld >= (long long)col0 + rank, "latent_norm_write: the columns lie outside the rows");
  RV_CHECK(page_size > 0 && page_size % RV_V_GROUP == 0 && num_pages > 0 && table_width > 0,
           "latent_norm_write: bad cache geometry");
  if (num_tokens == 0) return 0;
  dim3 grid(rv_div_up(num_tokens, 4)), block(256);
#define RV_LW(T)                                                                                                  \
  latent_norm_write_kernel<T><<<grid, block, 0, stream>>>((const T*)raw, ld, col0, w, w_f32, eps, offset, positions, \
                                                          token_req, block_table, table_width, (T*)k_pages,       \
                                                          (T*)v_pages, page_size, num_pages, rank, num_tokens)
  if (dtype == RV_F32) RV_LW(float);
  else if (dtype == RV_BF16) RV_LW(bf16_t);
  else return rv_fail("latent_norm_write: unsupported dtype %d", dtype);
#undef RV_LW
  RV_LAUNCH_CHECK("latent_norm_write");
  return 0;
}
