// The sandwich of norms around a branch with the residual stream kept in 32 bits and a learned scale a channel:
//
//   rmsnorm_cast         y = x / sqrt(mean(x^2) + eps) * (offset + w)          x of one type, y of another
//   add_rmsnorm_scaled   x <- x + branch / sqrt(mean(branch^2) + eps) * (offset + w_post) * scale
//                        (branch may be wa * branch + wb * branch2: two mixers side by side, each with its weight)
//                        next = x / sqrt(mean(x^2) + eps_next) * (offset_next + w_next)   optionally
//
// x is float whatever the activations' type T; the branch is stored as T or given as unreduced 32-bit partial sums
// of a product; `scale` (one number a channel) may be null.  All arithmetic is 32-bit.  A block takes a row, and
// the order of a row's additions depends on the width alone.
#include "common.h"

#define RS_THREADS 256

template <typename TI, typename TO>
__global__ void __launch_bounds__(RS_THREADS)
rmsnorm_cast_kernel(const TI* __restrict__ x, const int* __restrict__ row_index, const void* __restrict__ w, int w_f32,
                    TO* __restrict__ y, int width, float eps, float offset) {
  __shared__ float scratch[16];
  const int in_row = row_index ? row_index[blockIdx.x] : (int)blockIdx.x;
  const TI* xr = x + (size_t)in_row * width;
  TO* yr = y + (size_t)blockIdx.x * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += RS_THREADS) {
    const float v = rv_to_float(xr[i]);
    ss = fmaf(v, v, ss);
  }
  ss = rv_block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += RS_THREADS)
    yr[i] = rv_from_float<TO>(rv_to_float(xr[i]) * inv * (offset + rv_load_w(w, w_f32, i)));
}

extern "C" int rv_rmsnorm_cast(hipStream_t stream, const void* x, int x_dtype, const int* row_index, const void* w,
                               int w_f32, void* y, int y_dtype, int rows, int width, float eps, float offset) {
  RV_CHECK(rows >= 0 && width > 0 && x && w && y, "rmsnorm_cast: bad arguments rows=%d width=%d", rows, width);
  if (rows == 0) return 0;
  dim3 grid(rows), block(RS_THREADS);
#define RV_NC(TI, TO) \
  rmsnorm_cast_kernel<TI, TO><<<grid, block, 0, stream>>>((const TI*)x, row_index, w, w_f32, (TO*)y, width, eps, offset)
  if (x_dtype == RV_F32 && y_dtype == RV_F32) RV_NC(float, float);
  else if (x_dtype == RV_F32 && y_dtype == RV_BF16) RV_NC(float, bf16_t);
  else if (x_dtype == RV_BF16 && y_dtype == RV_BF16) RV_NC(bf16_t, bf16_t);
  else return rv_fail("rmsnorm_cast: unsupported dtypes %d -> %d", x_dtype, y_dtype);
#undef RV_NC
  RV_LAUNCH_CHECK("rmsnorm_cast");
  return 0;
}

template <typename T>
__device__ __forceinline__ float rs_branch(const void* p, int slices, long long stride, size_t at) {
  if (slices == 0) return rv_to_float(((const T*)p)[at]);
  const float* q = (const float*)p + at;
  float v = 0.f;
  int s = 0;
  for (; s + 4 <= slices; s += 4) {  // four reads on their way at a time, added in the slices' order
    const float a = q[(size_t)s * stride], b = q[(size_t)(s + 1) * stride], c = q[(size_t)(s + 2) * stride],
                d = q[(size_t)(s + 3) * stride];
    v = (((v + a) + b) + c) + d;
  }
  for (; s < slices; ++s) v += q[(size_t)s * stride];
  return v;
}

// V values side by side (1, or 4 where rows and slices start on 16-byte boundaries) of a branch.
template <typename T, int V>
__device__ __forceinline__ void rs_load_branch(const void* p, bool sliced, size_t at, float* out) {
  if (sliced || sizeof(T) == 4) {
    if constexpr (V == 4) {
      const float4 q = *(const float4*)((const float*)p + at);
      out[0] = q.x, out[1] = q.y, out[2] = q.z, out[3] = q.w;
    } else {
      out[0] = ((const float*)p)[at];
    }
  } else if constexpr (V == 4) {
    const uint2 q = *(const uint2*)((const uint16_t*)p + at);
    out[0] = __uint_as_float(q.x << 16), out[1] = __uint_as_float(q.x & 0xffff0000u);
    out[2] = __uint_as_float(q.y << 16), out[3] = __uint_as_float(q.y & 0xffff0000u);
  } else {
    out[0] = rv_to_float(((const T*)p)[at]);
  }
}

// E: groups of V values a thread keeps in registers (its share of a row of up to E * V * RS_THREADS numbers); 0: any
// width, the branch is read twice.  The reads of all a thread's groups are on their way together, slice after slice.
template <typename T, int E, int V>
__global__ void __launch_bounds__(RS_THREADS)
add_rmsnorm_scaled_kernel(const void* __restrict__ branch, int slices, long long slice_stride,
                          const void* __restrict__ branch2, int slices2, long long slice_stride2, float wa, float wb,
                          const void* __restrict__ w_post, int w_post_f32, const void* __restrict__ scale,
                          int scale_f32, float* __restrict__ x, const void* __restrict__ w_next, int w_next_f32,
                          T* __restrict__ next, int width, float eps, float offset, float eps_next,
                          float offset_next) {
  __shared__ float scratch[16];
  const size_t row0 = (size_t)blockIdx.x * width;
  constexpr int N = E > 0 ? E : 1;
  float val[N][V], res[N][V], gain[N][V];
  float ss = 0.f;
  if constexpr (E > 0) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int i = (e * RS_THREADS + threadIdx.x) * V;
#pragma unroll
      for (int v = 0; v < V; ++v) val[e][v] = res[e][v] = gain[e][v] = 0.f;
      if (i < width) {
        rs_load_branch<float, V>(x, false, row0 + i, res[e]);
#pragma unroll
        for (int v = 0; v < V; ++v)
          gain[e][v] = (offset + rv_load_w(w_post, w_post_f32, i + v)) * (scale ? rv_load_w(scale, scale_f32, i + v) : 1.0f);
      }
    }
    const int rounds = slices > 0 ? slices : 1;
    for (int s = 0; s < rounds; ++s) {
      float part[E][V];
#pragma unroll
      for (int e = 0; e < E; ++e) {
        const int i = (e * RS_THREADS + threadIdx.x) * V;
#pragma unroll
        for (int v = 0; v < V; ++v) part[e][v] = 0.f;
        if (i < width) rs_load_branch<T, V>(branch, slices > 0, (size_t)s * slice_stride + row0 + i, part[e]);
      }
#pragma unroll
      for (int e = 0; e < E; ++e)
#pragma unroll
        for (int v = 0; v < V; ++v) val[e][v] += part[e][v];
    }
    if (branch2 != nullptr) {
      float other[E][V];
#pragma unroll
      for (int e = 0; e < E; ++e)
#pragma unroll
        for (int v = 0; v < V; ++v) other[e][v] = 0.f;
      const int rounds2 = slices2 > 0 ? slices2 : 1;
      for (int s = 0; s < rounds2; ++s) {
        float part[E][V];
#pragma unroll
        for (int e = 0; e < E; ++e) {
          const int i = (e * RS_THREADS + threadIdx.x) * V;
#pragma unroll
          for (int v = 0; v < V; ++v) part[e][v] = 0.f;
          if (i < width) rs_load_branch<T, V>(branch2, slices2 > 0, (size_t)s * slice_stride2 + row0 + i, part[e]);
        }
#pragma unroll
        for (int e = 0; e < E; ++e)
#pragma unroll
          for (int v = 0; v < V; ++v) other[e][v] += part[e][v];
      }
#pragma unroll
      for (int e = 0; e < E; ++e)
#pragma unroll
        for (int v = 0; v < V; ++v) val[e][v] = wa * val[e][v] + wb * other[e][v];
    }
#pragma unroll
    for (int e = 0; e < E; ++e)
#pragma unroll
      for (int v = 0; v < V; ++v) ss = fmaf(val[e][v], val[e][v], ss);
  } else {
    for (int i = threadIdx.x; i < width; i += RS_THREADS) {
      float v = rs_branch<T>(branch, slices, slice_stride, row0 + i);
      if (branch2 != nullptr) v = wa * v + wb * rs_branch<T>(branch2, slices2, slice_stride2, row0 + i);
      ss = fmaf(v, v, ss);
    }
  }
  ss = rv_block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  float ss2 = 0.f;
  if constexpr (E > 0) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int i = (e * RS_THREADS + threadIdx.x) * V;
      if (i < width) {
#pragma unroll
        for (int v = 0; v < V; ++v) {
          res[e][v] = res[e][v] + val[e][v] * inv * gain[e][v];
          ss2 = fmaf(res[e][v], res[e][v], ss2);
        }
        if constexpr (V == 4) *(float4*)(x + row0 + i) = make_float4(res[e][0], res[e][1], res[e][2], res[e][3]);
        else x[row0 + i] = res[e][0];
      }
    }
  } else {
    for (int i = threadIdx.x; i < width; i += RS_THREADS) {
      const float g = (offset + rv_load_w(w_post, w_post_f32, i)) * (scale ? rv_load_w(scale, scale_f32, i) : 1.0f);
      float v = rs_branch<T>(branch, slices, slice_stride, row0 + i);
      if (branch2 != nullptr) v = wa * v + wb * rs_branch<T>(branch2, slices2, slice_stride2, row0 + i);
      const float r = x[row0 + i] + v * inv * g;
      x[row0 + i] = r;
      ss2 = fmaf(r, r, ss2);
    }
  }
  if (next == nullptr) return;
  ss2 = rv_block_sum(ss2, scratch);
  const float inv2 = 1.0f / sqrtf(ss2 / (float)width + eps_next);
  if constexpr (E > 0) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int i = (e * RS_THREADS + threadIdx.x) * V;
      if (i < width) {
#pragma unroll
        for (int v = 0; v < V; ++v)
          next[row0 + i + v] = rv_from_float<T>(res[e][v] * inv2 * (offset_next + rv_load_w(w_next, w_next_f32, i + v)));
      }
    }
  } else {
    // every thread reads back what it wrote itself
    for (int i = threadIdx.x; i < width; i += RS_THREADS)
      next[row0 + i] = rv_from_float<T>(x[row0 + i] * inv2 * (offset_next + rv_load_w(w_next, w_next_f32, i)));
  }
}

// branch: `dtype` values [rows, width] (slices 0) or 32-bit partial sums [slices][rows][width]; branch2: the same or
// null; x: float, in place; next: `dtype`, with w_next, or both null.
extern "C" int rv_add_rmsnorm_scaled(hipStream_t stream, const void* branch, int slices, long long slice_stride,
                                     const void* branch2, int slices2, long long slice_stride2, float wa, float wb,
                                     const void* w_post, int w_post_f32, const void* scale, int scale_f32, float* x,
                                     const void* w_next, int w_next_f32, void* next, int dtype, int rows, int width,
                                     float eps, float offset, float eps_next, float offset_next) {
  RV_CHECK(rows >= 0 && width > 0 && branch && w_post && x, "add_rmsnorm_scaled: bad arguments rows=%d width=%d", rows,
           width);
  RV_CHECK((w_next == nullptr) == (next == nullptr), "add_rmsnorm_scaled: the next norm needs both weight and output");
  RV_CHECK(slices >= 0 && (slices == 0 || slice_stride >= (long long)rows * width), "add_rmsnorm_scaled: bad partial sums");
  RV_CHECK(slices2 >= 0 && (slices2 == 0 || slice_stride2 >= (long long)rows * width),
           "add_rmsnorm_scaled: bad partial sums of the second branch");
  if (rows == 0) return 0;
  dim3 grid(rows), block(RS_THREADS);
  // four values a thread and turn where rows, slices and streams all start on 16-byte boundaries
  const bool vec = width % 4 == 0 && slice_stride % 4 == 0 && slice_stride2 % 4 == 0 &&
                   (((uintptr_t)x | (uintptr_t)branch | (uintptr_t)branch2) & 15) == 0;
#define RV_AS(T, E, V)                                                                                                  \
  add_rmsnorm_scaled_kernel<T, E, V><<<grid, block, 0, stream>>>(branch, slices, slice_stride, branch2, slices2,        \
                                                                 slice_stride2, wa, wb, w_post, w_post_f32,             \
                                                                 scale, scale_f32, x, w_next, w_next_f32, (T*)next,     \
                                                                 width, eps, offset, eps_next, offset_next)
#define RV_AS_T(T)                                                 \
  do {                                                             \
    const int e_ = rv_div_up(width, RS_THREADS * (vec ? 4 : 1));   \
    if (vec && e_ <= 1) RV_AS(T, 1, 4);                            \
    else if (vec && e_ <= 2) RV_AS(T, 2, 4);                       \
    else if (vec && e_ <= 4) RV_AS(T, 4, 4);                       \
    else if (vec && e_ <= 8) RV_AS(T, 8, 4);                       \
    else if (!vec && e_ <= 2) RV_AS(T, 2, 1);                      \
    else if (!vec && e_ <= 8) RV_AS(T, 8, 1);                      \
    else RV_AS(T, 0, 1);                                           \
  } while (0)
  if (dtype == RV_F32) RV_AS_T(float);
  else if (dtype == RV_BF16) RV_AS_T(bf16_t);
  else return rv_fail("add_rmsnorm_scaled: unsupported dtype %d", dtype);
#undef RV_AS_T
#undef RV_AS
  RV_LAUNCH_CHECK("add_rmsnorm_scaled");
  return 0;
}

// x[i] = x[i] * a over `total` 32-bit numbers (the logits' multiplier).
__global__ void scale_f32_kernel(float* __restrict__ x, long long total, float a) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx < total) x[idx] *= a;
}

extern "C" int rv_scale_f32(hipStream_t stream, float* x, long long total, float a) {
  RV_CHECK(total >= 0 && x, "scale_f32: bad arguments");
  if (total == 0) return 0;
  scale_f32_kernel<<<dim3(rv_div_up(total, 256)), dim3(256), 0, stream>>>(x, total, a);
  RV_LAUNCH_CHECK("scale_f32");
  return 0;
}

// out[t][c] = a * x[t][c] + b * y[t][c]: two mixers side by side, each with its weight; x and y of type `dtype` or
// unreduced 32-bit partial sums of a product; the sum is 32-bit and stays 32-bit (the consumer takes it as the one
// slice of a product's partial sums).
template <typename T>
__global__ void weighted_sum_kernel(const void* __restrict__ x, int x_slices, long long x_stride,
                                    const void* __restrict__ y, int y_slices, long long y_stride, float a, float b,
                                    float* __restrict__ out, long long total) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  out[idx] = a * rs_branch<T>(x, x_slices, x_stride, (size_t)idx) + b * rs_branch<T>(y, y_slices, y_stride, (size_t)idx);
}

extern "C" int rv_weighted_sum(hipStream_t stream, const void* x, int x_slices, long long x_stride, const void* y,
                               int y_slices, long long y_stride, float a, float b, float* out, int dtype, int rows,
                               int width) {
  RV_CHECK(x && y && out && rows >= 0 && width > 0, "weighted_sum: bad arguments");
  if (rows == 0) return 0;
  const long long total = (long long)rows * width;
  dim3 grid(rv_div_up(total, 256)), block(256);
  if (dtype == RV_F32)
    weighted_sum_kernel<float><<<grid, block, 0, stream>>>(x, x_slices, x_stride, y, y_slices, y_stride, a, b, out, total);
  else if (dtype == RV_BF16)
    weighted_sum_kernel<bf16_t><<<grid, block, 0, stream>>>(x, x_slices, x_stride, y, y_slices, y_stride, a, b, out, total);
  else
    return rv_fail("weighted_sum: unsupported dtype %d", dtype);
  RV_LAUNCH_CHECK("weighted_sum");
  return 0;
}
