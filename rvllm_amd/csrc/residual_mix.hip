// The residual stream kept in 32 bits, for layers whose branches run in parallel and whose outputs are averaged
// over depth:
//
//   scalar_rmsnorm   y = x * rsqrt(mean(x^2) + eps) * g          g one number for the whole row
//   residual_mix     X = x + mult * (a + f)                       a, f: the mixer's and the feed-forward's branch
//                    x <- sum_j w[j] * X_j, j = 0 .. terms-1      X_0 the embedding's output, X_(terms-1) = X;
//                    next = scalar_rmsnorm(x)                     optionally, for the layer after
//
// x is float whatever the activations' type (TO: float or bf16); all arithmetic is 32-bit.  A block takes a row;
// the order of a row's additions depends on the width alone, so a row's result does not depend on what else
// is in the batch.  Without depth weights the second line is left out (x <- X).
#include "common.h"

#define RM_THREADS 256

template <typename TI, typename TO>
__global__ void __launch_bounds__(RM_THREADS)
scalar_rmsnorm_kernel(const TI* __restrict__ x, const int* __restrict__ row_index, const void* __restrict__ g,
                      int g_f32, TO* __restrict__ y, int width, float eps) {
  __shared__ float scratch[16];
  const int in_row = row_index ? row_index[blockIdx.x] : (int)blockIdx.x;
  const TI* xr = x + (size_t)in_row * width;
  TO* yr = y + (size_t)blockIdx.x * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += RM_THREADS) {
    const float v = rv_to_float(xr[i]);
    ss = fmaf(v, v, ss);
  }
  ss = rv_block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  const float gain = rv_load_w(g, g_f32, 0);
  for (int i = threadIdx.x; i < width; i += RM_THREADS) yr[i] = rv_from_float<TO>(rv_to_float(xr[i]) * inv * gain);
}

extern "C" int rv_scalar_rmsnorm(hipStream_t stream, const void* x, int x_dtype, const int* row_index, const void* g,
                                 int g_f32, void* y, int y_dtype, int rows, int width, float eps) {
  RV_CHECK(rows >= 0 && width > 0 && g != nullptr, "scalar_rmsnorm: bad arguments rows=%d width=%d", rows, width);
  if (rows == 0) return 0;
  dim3 grid(rows), block(RM_THREADS);
#define RV_SN(TI, TO) \
  scalar_rmsnorm_kernel<TI, TO><<<grid, block, 0, stream>>>((const TI*)x, row_index, g, g_f32, (TO*)y, width, eps)
  if (x_dtype == RV_F32 && y_dtype == RV_F32) RV_SN(float, float);
  else if (x_dtype == RV_F32 && y_dtype == RV_BF16) RV_SN(float, bf16_t);
  else if (x_dtype == RV_BF16 && y_dtype == RV_BF16) RV_SN(bf16_t, bf16_t);
  else return rv_fail("scalar_rmsnorm: unsupported dtypes %d -> %d", x_dtype, y_dtype);
#undef RV_SN
  RV_LAUNCH_CHECK("scalar_rmsnorm");
  return 0;
}

// V consecutive values of a branch (V is 1 or 4): stored as T, or the sum of `slices` 32-bit partial sums.
template <typename T, int V>
__device__ __forceinline__ void rm_branch_vec(const void* p, int slices, long long stride, size_t at, float* out) {
#pragma unroll
  for (int v = 0; v < V; ++v) out[v] = 0.f;
  if (p == nullptr) return;
  if (slices == 0) {
    if constexpr (V == 4 && sizeof(T) == 2) {
      const uint2 q = *(const uint2*)((const uint16_t*)p + at);
      out[0] = __uint_as_float(q.x << 16), out[1] = __uint_as_float(q.x & 0xffff0000u);
      out[2] = __uint_as_float(q.y << 16), out[3] = __uint_as_float(q.y & 0xffff0000u);
    } else if constexpr (V == 4) {
      const float4 q = *(const float4*)((const float*)p + at);
      out[0] = q.x, out[1] = q.y, out[2] = q.z, out[3] = q.w;
    } else {
      out[0] = rv_to_float(((const T*)p)[at]);
    }
    return;
  }
  for (int s = 0; s < slices; ++s) {
    const float* q = (const float*)p + (size_t)s * stride + at;
    if constexpr (V == 4) {
      const float4 r = *(const float4*)q;
      out[0] += r.x, out[1] += r.y, out[2] += r.z, out[3] += r.w;
    } else {
      out[0] += q[0];
    }
  }
}

template <int V>
__device__ __forceinline__ void rm_load(const float* p, float* out) {
  if constexpr (V == 4) {
    const float4 q = *(const float4*)p;
    out[0] = q.x, out[1] = q.y, out[2] = q.z, out[3] = q.w;
  } else {
    out[0] = p[0];
  }
}
template <int V>
__device__ __forceinline__ void rm_store(float* p, const float* in) {
  if constexpr (V == 4) *(float4*)p = make_float4(in[0], in[1], in[2], in[3]);
  else p[0] = in[0];
}

// V values a thread and turn: 4 where the width is a multiple of 4 (16-byte reads of the streams), else 1.  Every
// stream of the history is read before anything is written, so that the reads are on their way together.
#define RM_MAX_TERMS_AT_ONCE 8
template <typename T, int V>
__global__ void __launch_bounds__(RM_THREADS)
residual_mix_kernel(float* __restrict__ x, const void* __restrict__ a, int a_slices, long long a_stride,
                    const void* __restrict__ f, int f_slices, long long f_stride, float mult,
                    float* __restrict__ history, long long history_stride, int terms, int seed_history,
                    const void* __restrict__ depth_w, int depth_w_f32, const void* __restrict__ g_next,
                    int g_next_f32, T* __restrict__ next, float eps_next, int width) {
  __shared__ float scratch[16];
  const size_t row0 = (size_t)blockIdx.x * width;
  float ss = 0.f;
  for (int i = threadIdx.x * V; i < width; i += RM_THREADS * V) {
    const size_t at = row0 + i;
    float x_in[V], br_a[V], br_f[V], x_new[V], out[V];
    rm_load<V>(x + at, x_in);
    rm_branch_vec<T, V>(a, a_slices, a_stride, at, br_a);
    rm_branch_vec<T, V>(f, f_slices, f_stride, at, br_f);
#pragma unroll
    for (int v = 0; v < V; ++v) out[v] = x_new[v] = fmaf(mult, br_a[v] + br_f[v], x_in[v]);
    if (history != nullptr) {
#pragma unroll
      for (int v = 0; v < V; ++v) out[v] = 0.f;
      for (int j0 = 0; j0 + 1 < terms; j0 += RM_MAX_TERMS_AT_ONCE) {
        float xj[RM_MAX_TERMS_AT_ONCE][V];
#pragma unroll
        for (int jj = 0; jj < RM_MAX_TERMS_AT_ONCE; ++jj) {  // a stream past the last repeats it and weighs nothing
          const int j = j0 + jj + 1 < terms ? j0 + jj : terms - 2;
          rm_load<V>(((j == 0 && seed_history) ? x : history + (size_t)j * history_stride) + at, xj[jj]);
        }
#pragma unroll
        for (int jj = 0; jj < RM_MAX_TERMS_AT_ONCE; ++jj) {
          if (j0 + jj + 1 < terms) {
            const float wj = rv_load_w(depth_w, depth_w_f32, j0 + jj);
#pragma unroll
            for (int v = 0; v < V; ++v) out[v] = fmaf(wj, xj[jj][v], out[v]);
          }
        }
      }
      const float w_last = rv_load_w(depth_w, depth_w_f32, terms - 1);
#pragma unroll
      for (int v = 0; v < V; ++v) out[v] = fmaf(w_last, x_new[v], out[v]);
      if (seed_history) rm_store<V>(history + at, x_in);  // the first layer's input is the embedding's output, X_0
      rm_store<V>(history + (size_t)(terms - 1) * history_stride + at, x_new);
    }
    rm_store<V>(x + at, out);
#pragma unroll
    for (int v = 0; v < V; ++v) ss = fmaf(out[v], out[v], ss);
  }
  if (next == nullptr) return;
  ss = rv_block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps_next);
  const float gain = rv_load_w(g_next, g_next_f32, 0);
  // every thread reads back what it wrote itself
  for (int i = threadIdx.x * V; i < width; i += RM_THREADS * V) {
    float o[V];
    rm_load<V>(x + row0 + i, o);
#pragma unroll
    for (int v = 0; v < V; ++v) next[row0 + i + v] = rv_from_float<T>(o[v] * inv * gain);
  }
}

// x [rows, width] float, in place.  a, f: branches of type `dtype` [rows, width] (slices 0) or 32-bit partial sums
// [slices][rows][width]; f may be null.  history: float [>= terms][history_stride] or null; entries 1 .. terms-2 were
// written by earlier calls, entry 0 too unless `seed_history`.  depth_w: `terms` weights.  next / g_next: null, or
// the output of the following norm (type `dtype`) and its gain.
extern "C" int rv_residual_mix(hipStream_t stream, float* x, const void* a, int a_slices, long long a_stride,
                               const void* f, int f_slices, long long f_stride, float mult, float* history,
                               long long history_stride, int terms, int seed_history, const void* depth_w,
                               int depth_w_f32, const void* g_next, int g_next_f32, void* next, float eps_next,
                               int dtype, int rows, int width) {
  RV_CHECK(rows >= 0 && width > 0 && x != nullptr && a != nullptr, "residual_mix: bad arguments rows=%d width=%d", rows, width);
  RV_CHECK(a_slices >= 0 && f_slices >= 0 && (a_slices == 0 || a_stride >= (long long)rows * width) &&
               (f_slices == 0 || f_stride >= (long long)rows * width), "residual_mix: bad partial sums");
  RV_CHECK((history == nullptr) || (depth_w != nullptr && terms >= 2 && history_stride >= (long long)rows * width),
           "residual_mix: a depth average needs its weights, two terms at least and room for a layer's rows");
  RV_CHECK((g_next == nullptr) == (next == nullptr), "residual_mix: the next norm needs both gain and output");
  if (rows == 0) return 0;
  dim3 grid(rows), block(RM_THREADS);
  // four values a thread where rows, streams and partial sums all start on 16-byte boundaries
  const bool vec = width % 4 == 0 && history_stride % 4 == 0 && a_stride % 4 == 0 && f_stride % 4 == 0 &&
                   (((uintptr_t)x | (uintptr_t)a | (uintptr_t)f | (uintptr_t)history) & 15) == 0;
#define RV_RM(T, V)                                                                                                    \
  residual_mix_kernel<T, V><<<grid, block, 0, stream>>>(x, a, a_slices, a_stride, f, f_slices, f_stride, mult, history, \
                                                        history_stride, terms, seed_history, depth_w, depth_w_f32,     \
                                                        g_next, g_next_f32, (T*)next, eps_next, width)
  if (dtype == RV_F32) { if (vec) RV_RM(float, 4); else RV_RM(float, 1); }
  else if (dtype == RV_BF16) { if (vec) RV_RM(bf16_t, 4); else RV_RM(bf16_t, 1); }
  else return rv_fail("residual_mix: unsupported dtype %d", dtype);
#undef RV_RM
  RV_LAUNCH_CHECK("residual_mix");
  return 0;
}
