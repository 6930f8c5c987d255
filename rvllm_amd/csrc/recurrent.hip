// Mixers that carry a state of fixed size from token to token instead of keys and values:
//
//   causal_conv        a short convolution over time for every channel, its activation, and optionally the
//                      scaling of groups of channels to unit length
//   conv_state_update  the last taps - 1 inputs of every channel, kept for the request's next step
//   delta_rule         the gated delta rule, a matrix S [dk, dv] a head:
//                        S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//   selective_scan     a diagonal state S [channel, n]:
//                        S <- exp(dt A) S + dt x B;  y = S . C + D x;  y <- y silu(z)
//   head_norm_gate     o / rms(o) * w * silu(gate), a head at a time
//   gate_mul           a * sigmoid(gate) or a * silu(gate), element by element
//
// The states, the decays, their exponentials and logarithms, the step sizes and the unit norms are 32-bit whatever
// the activations' type T; the convolution's sum is 32-bit and its activated output is rounded to T once.  A
// request's tokens are walked in their order by the waves that own a part of its state, so what a token's output
// is does not depend on how the request's tokens were cut into steps or on what else the step holds.  The state of
// a request lies in its slot, `slot_stride` floats apart from the next; a slot is all zeros when a request gets it.
#include "common.h"

#define REC_MAX_TAPS 16

__device__ __forceinline__ float rec_softplus(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }
__device__ __forceinline__ float rec_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float rec_silu(float x) { return x / (1.0f + expf(-x)); }

// Sum over the `lanes` (a power of two) neighbouring lanes that share a column or channel.
__device__ __forceinline__ float rec_group_sum(float v, int lanes) {
  for (int off = lanes >> 1; off > 0; off >>= 1) v += __shfl_xor(v, off, RV_WAVE);
  return v;
}

// ---------------------------------------------------------------------------
// Short causal convolution.  Channel c of token t at position p:
//   y = act(bias[c] + sum_j w[c][j] * in[p - (taps - 1) + j][c]),   j = 0 .. taps - 1 (the last tap is the token's own)
// Inputs from before the step's first token of the request come from the state (its row s holds the input at
// position first - (taps - 1) + s); a fresh slot's zeros are the zeros before the start of a sequence.
// A wave takes a group of `group` channels of one token; with unit_eps >= 0 the group's outputs are divided by
// sqrt(sum y^2 + unit_eps) and the first `scaled_groups` groups multiplied by `group_scale`.
// ---------------------------------------------------------------------------
template <typename T, typename TO>
__global__ void __launch_bounds__(256)
causal_conv_kernel(const T* __restrict__ in, long long ld_in, const float* __restrict__ w, const float* __restrict__ bias,
                   int taps, const float* __restrict__ state, long long slot_stride, long long state_off,
                   int state_ld, const int* __restrict__ positions, const int* __restrict__ token_req,
                   const int* __restrict__ q_start, const int* __restrict__ chunk_start,
                   const int* __restrict__ state_slot, TO* __restrict__ out, long long ld_out, int channels, int group,
                   int groups, int num_tokens, float unit_eps, int scaled_groups, float group_scale) {
  const int lane = threadIdx.x & (RV_WAVE - 1);
  const long long unit = (long long)blockIdx.x * (blockDim.x / RV_WAVE) + threadIdx.x / RV_WAVE;
  if (unit >= (long long)num_tokens * groups) return;  // the whole wave
  const int t = (int)(unit / groups);
  const int grp = (int)(unit - (long long)t * groups);
  const int req = token_req[t];
  const int first_pos = chunk_start[req];
  const int first_tok = q_start[req];
  const int rel = positions[t] - first_pos;  // place of the token in its portion
  const float* st = state + (long long)state_slot[req] * slot_stride + state_off;
  float ss = 0.f;
  for (int c0 = 0; c0 < group; c0 += RV_WAVE) {  // (two passes when the group is normed: the sum, then the store)
    const int c = grp * group + c0 + lane;
    if (c0 + lane < group && c < channels) {
      float acc = bias ? bias[c] : 0.f;
      for (int j = 0; j < taps; ++j) {
        const int r = rel - (taps - 1) + j;
        const float x = r >= 0 ? rv_to_float(in[(long long)(first_tok + r) * ld_in + c])
                               : st[(long long)(taps - 1 + r) * state_ld + c];
        acc = fmaf(w[(long long)c * taps + j], x, acc);
      }
      const float y = rv_round_to<T>(rec_silu(acc));
      if (unit_eps < 0.f) out[(long long)t * ld_out + c] = rv_from_float<TO>(y);
      ss = fmaf(y, y, ss);
    }
  }
  if (unit_eps < 0.f) return;
  ss = rv_wave_sum(ss);
  const float mult = (grp < scaled_groups ? group_scale : 1.0f) / sqrtf(ss + unit_eps);
  for (int c0 = 0; c0 < group; c0 += RV_WAVE) {
    const int c = grp * group + c0 + lane;
    if (c0 + lane < group && c < channels) {
      float acc = bias ? bias[c] : 0.f;
      for (int j = 0; j < taps; ++j) {
        const int r = rel - (taps - 1) + j;
        const float x = r >= 0 ? rv_to_float(in[(long long)(first_tok + r) * ld_in + c])
                               : st[(long long)(taps - 1 + r) * state_ld + c];
        acc = fmaf(w[(long long)c * taps + j], x, acc);
      }
      out[(long long)t * ld_out + c] = rv_from_float<TO>(rv_round_to<T>(rec_silu(acc)) * mult);
    }
  }
}

// in: [tokens, ld_in] of type `dtype`, the channels from the given address on.  w: float [channels, taps]; bias:
// float [channels] or null.  state: float, row s of a slot's block at state_off + s * state_ld.  out: float
// (out_f32) or `dtype`.  unit_eps < 0: no unit length.
extern "C" int rv_causal_conv(hipStream_t stream, const void* in, int dtype, long long ld_in, const float* w,
                              const float* bias, int taps, const float* state, long long slot_stride,
                              long long state_off, int state_ld, const int* positions, const int* token_req,
                              const int* q_start, const int* chunk_start, const int* state_slot, void* out,
                              int out_f32, long long ld_out, int channels, int group, int num_tokens, float unit_eps,
                              int scaled_groups, float group_scale) {
  RV_CHECK(in && w && state && positions && token_req && q_start && chunk_start && state_slot && out,
           "causal_conv: null argument");
  RV_CHECK(taps >= 1 && taps <= REC_MAX_TAPS && channels > 0 && group > 0 && num_tokens >= 0 && state_ld >= channels,
           "causal_conv: bad sizes taps=%d channels=%d group=%d", taps, channels, group);
  if (num_tokens == 0) return 0;
  const int groups = rv_div_up(channels, group);
  const long long units = (long long)num_tokens * groups;
  dim3 grid(rv_div_up(units, 4)), block(256);
#define RV_CC(T, TO)                                                                                                 \
  causal_conv_kernel<T, TO><<<grid, block, 0, stream>>>((const T*)in, ld_in, w, bias, taps, state, slot_stride,      \
                                                        state_off, state_ld, positions, token_req, q_start,          \
                                                        chunk_start, state_slot, (TO*)out, ld_out, channels, group,  \
                                                        groups, num_tokens, unit_eps, scaled_groups, group_scale)
  if (dtype == RV_F32) RV_CC(float, float);
  else if (dtype == RV_BF16 && out_f32) RV_CC(bf16_t, float);
  else if (dtype == RV_BF16) RV_CC(bf16_t, bf16_t);
  else return rv_fail("causal_conv: unsupported dtype %d", dtype);
#undef RV_CC
  RV_LAUNCH_CHECK("causal_conv");
  return 0;
}

// After the step: row s of the state becomes the input at position end - (taps - 1) + s, taken from the step's
// tokens or, where the portion is shorter than taps - 1, from the rows the state held.  A thread owns a channel of
// a request and reads all it needs before it writes.
template <typename T>
__global__ void conv_state_update_kernel(const T* __restrict__ in, long long ld_in, int taps, float* __restrict__ state,
                                         long long slot_stride, long long state_off, int state_ld,
                                         const int* __restrict__ q_start, const int* __restrict__ state_slot,
                                         int channels) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int req = blockIdx.y;
  if (c >= channels) return;
  const int first_tok = q_start[req];
  const int n = q_start[req + 1] - first_tok;
  float* st = state + (long long)state_slot[req] * slot_stride + state_off;
  float keep[REC_MAX_TAPS];
#pragma unroll
  for (int s = 0; s < REC_MAX_TAPS - 1; ++s) {
    if (s < taps - 1) {
      const int r = n - (taps - 1) + s;
      keep[s] = r >= 0 ? rv_to_float(in[(long long)(first_tok + r) * ld_in + c]) : st[(long long)(s + n) * state_ld + c];
    }
  }
#pragma unroll
  for (int s = 0; s < REC_MAX_TAPS - 1; ++s)
    if (s < taps - 1) st[(long long)s * state_ld + c] = keep[s];
}

extern "C" int rv_conv_state_update(hipStream_t stream, const void* in, int dtype, long long ld_in, int taps,
                                    float* state, long long slot_stride, long long state_off, int state_ld,
                                    const int* q_start, const int* state_slot, int channels, int num_requests) {
  RV_CHECK(in && state && q_start && state_slot, "conv_state_update: null argument");
  RV_CHECK(taps >= 1 && taps <= REC_MAX_TAPS && channels > 0 && state_ld >= channels && num_requests >= 0,
           "conv_state_update: bad sizes");
  if (num_requests == 0 || taps == 1) return 0;
  dim3 grid(rv_div_up(channels, 256), num_requests), block(256);
  if (dtype == RV_F32)
    conv_state_update_kernel<float><<<grid, block, 0, stream>>>((const float*)in, ld_in, taps, state, slot_stride,
                                                                state_off, state_ld, q_start, state_slot, channels);
  else if (dtype == RV_BF16)
    conv_state_update_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)in, ld_in, taps, state, slot_stride,
                                                                 state_off, state_ld, q_start, state_slot, channels);
  else
    return rv_fail("conv_state_update: unsupported dtype %d", dtype);
  RV_LAUNCH_CHECK("conv_state_update");
  return 0;
}

// ---------------------------------------------------------------------------
// Gated delta rule.  A column j of a head's S (its dk numbers) never meets another column, so `lanes` neighbouring
// lanes own one: lane `sub` of them holds rows sub, sub + lanes, ... (PER at most).  A wave holds 64 / lanes
// columns of one head of one request and walks the request's tokens of this step in order; the next token's
// operands are asked for before this token's are used.
//   qkv  float [tokens, ld]: q of key head g at q_off + g dk, k at k_off + g dk, v of head h at v_off + h dv
//   ab   T [tokens, ld_ab]: the decay's input a at a_col + h, beta's input at b_col + h
//   g = exp(-exp(A_log[h]) softplus(a + dt_bias[h])),  beta = sigmoid(b)
//   S    float [heads, dk, dv] at s_off of the request's slot
//   out  float [tokens, heads dv]
// ---------------------------------------------------------------------------
template <typename T, int PER>
__global__ void __launch_bounds__(RV_WAVE)
delta_rule_kernel(const float* __restrict__ qkv, long long ld, int q_off, int k_off, int v_off,
                  const T* __restrict__ ab, long long ld_ab, int a_col, int b_col, const float* __restrict__ A_log,
                  const float* __restrict__ dt_bias, float* __restrict__ state, long long slot_stride,
                  long long s_off, const int* __restrict__ q_start, const int* __restrict__ state_slot,
                  float* __restrict__ out, int heads, int kv_heads, int dk, int dv, int lanes) {
  const int lane = threadIdx.x;
  const int cols = RV_WAVE / lanes;
  const int sub = lane % lanes;
  const int j = blockIdx.x * cols + lane / lanes;
  const int h = blockIdx.y;
  const int req = blockIdx.z;
  const int g = h / (heads / kv_heads);
  const bool col = j < dv;
  const int jj = col ? j : dv - 1;  // a lane past the last column works on a copy and writes nothing
  float* S_mem = state + (long long)state_slot[req] * slot_stride + s_off + (long long)h * dk * dv + jj;
  float S[PER];
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int i = e * lanes + sub;
    S[e] = i < dk ? S_mem[(long long)i * dv] : 0.f;
  }
  const float rate = -expf(A_log[h]);
  const float bias = dt_bias[h];
  const int t0 = q_start[req], t1 = q_start[req + 1];
  float kk[PER], qq[PER], vv, a_in, b_in;
  auto fetch = [&](int t, float (&k_)[PER], float (&q_)[PER], float& v_, float& a_, float& b_) {
    const float* row = qkv + (long long)t * ld;
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      const int i = e * lanes + sub;
      k_[e] = i < dk ? row[k_off + g * dk + i] : 0.f;
      q_[e] = i < dk ? row[q_off + g * dk + i] : 0.f;
    }
    v_ = row[v_off + h * dv + jj];
    a_ = rv_to_float(ab[(long long)t * ld_ab + a_col + h]);
    b_ = rv_to_float(ab[(long long)t * ld_ab + b_col + h]);
  };
  if (t0 < t1) fetch(t0, kk, qq, vv, a_in, b_in);
  for (int t = t0; t < t1; ++t) {
    float nk[PER], nq[PER], nv = 0.f, na = 0.f, nb = 0.f;
    if (t + 1 < t1) fetch(t + 1, nk, nq, nv, na, nb);
    const float decay = expf(rate * rec_softplus(a_in + bias));
    const float beta = rec_sigmoid(b_in);
    float dot = 0.f;
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      S[e] *= decay;
      dot = fmaf(S[e], kk[e], dot);
    }
    dot = rec_group_sum(dot, lanes);
    const float u = beta * (vv - dot);
    float o = 0.f;
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      S[e] = fmaf(kk[e], u, S[e]);
      o = fmaf(S[e], qq[e], o);
    }
    o = rec_group_sum(o, lanes);
    if (col && sub == 0) out[(long long)t * heads * dv + h * dv + j] = o;
    if (t + 1 < t1) {
#pragma unroll
      for (int e = 0; e < PER; ++e) kk[e] = nk[e], qq[e] = nq[e];
      vv = nv, a_in = na, b_in = nb;
    }
  }
  if (col) {
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      const int i = e * lanes + sub;
      if (i < dk) S_mem[(long long)i * dv] = S[e];
    }
  }
}

#define REC_DELTA_PER_MAX 16

// How many lanes share a column of S for this key size: the fewest (a power of two) that leave a lane at most
// REC_DELTA_PER_MAX rows.  A function of dk alone, so that a token's sums are added in one order always.
extern "C" int rv_delta_rule_lanes(int dk) {
  int lanes = 1;
  while (lanes < RV_WAVE && rv_div_up(dk, lanes) > REC_DELTA_PER_MAX) lanes *= 2;
  return lanes;
}

extern "C" int rv_delta_rule(hipStream_t stream, const float* qkv, long long ld, int q_off, int k_off, int v_off,
                             const void* ab, int dtype, long long ld_ab, int a_col, int b_col, const float* A_log,
                             const float* dt_bias, float* state, long long slot_stride, long long s_off,
                             const int* q_start, const int* state_slot, float* out, int num_requests, int heads,
                             int kv_heads, int dk, int dv) {
  RV_CHECK(qkv && ab && A_log && dt_bias && state && q_start && state_slot && out, "delta_rule: null argument");
  RV_CHECK(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dk > 0 && dv > 0 && num_requests >= 0,
           "delta_rule: bad sizes heads=%d kv_heads=%d dk=%d dv=%d", heads, kv_heads, dk, dv);
  const int lanes = rv_delta_rule_lanes(dk);
  const int per = rv_div_up(dk, lanes);
  RV_CHECK(per <= REC_DELTA_PER_MAX, "delta_rule: a key size of %d is more than %d", dk, REC_DELTA_PER_MAX * RV_WAVE);
  if (num_requests == 0) return 0;
  dim3 grid(rv_div_up(dv, RV_WAVE / lanes), heads, num_requests), block(RV_WAVE);
#define RV_DR(T, PER)                                                                                                \
  delta_rule_kernel<T, PER><<<grid, block, 0, stream>>>(qkv, ld, q_off, k_off, v_off, (const T*)ab, ld_ab, a_col,    \
                                                        b_col, A_log, dt_bias, state, slot_stride, s_off, q_start,   \
                                                        state_slot, out, heads, kv_heads, dk, dv, lanes)
#define RV_DR_T(T)                \
  do {                            \
    if (per <= 4) RV_DR(T, 4);    \
    else if (per <= 8) RV_DR(T, 8); \
    else RV_DR(T, 16);            \
  } while (0)
  if (dtype == RV_F32) RV_DR_T(float);
  else if (dtype == RV_BF16) RV_DR_T(bf16_t);
  else return rv_fail("delta_rule: unsupported dtype %d", dtype);
#undef RV_DR_T
#undef RV_DR
  RV_LAUNCH_CHECK("delta_rule");
  return 0;
}

// ---------------------------------------------------------------------------
// Selective scan.  `lanes` neighbouring lanes own a channel: lane `sub` holds the states sub, sub + lanes, ...
//   x    T [tokens, ld_x]    the convolved, activated input      z   T [tokens, ld_z]   the gate's input
//   dt   T [tokens, ld_dt]   the step's projection; step = softplus(dt + dt_bias[c])
//   bc   T [tokens, ld_bc]   B at b_col, C at c_col, `n_state` each
//   A = -exp(A_log [channels, n_state]);  D [channels]
//   S    float [channels, n_state] at s_off of the request's slot
//   out  T [tokens, channels] = (S . C + D x) silu(z)
// ---------------------------------------------------------------------------
template <typename T, int PER>
__global__ void __launch_bounds__(RV_WAVE)
selective_scan_kernel(const T* __restrict__ x, long long ld_x, const T* __restrict__ z, long long ld_z,
                      const T* __restrict__ dt, long long ld_dt, const float* __restrict__ dt_bias,
                      const T* __restrict__ bc, long long ld_bc, int b_col, int c_col,
                      const float* __restrict__ A_log, const float* __restrict__ D, float* __restrict__ state,
                      long long slot_stride, long long s_off, const int* __restrict__ q_start,
                      const int* __restrict__ state_slot, T* __restrict__ out, int channels, int n_state, int lanes) {
  const int lane = threadIdx.x;
  const int per_wave = RV_WAVE / lanes;
  const int sub = lane % lanes;
  const int ch = blockIdx.x * per_wave + lane / lanes;
  const int req = blockIdx.y;
  const bool live = ch < channels;
  const int c = live ? ch : channels - 1;
  float* S_mem = state + (long long)state_slot[req] * slot_stride + s_off + (long long)c * n_state;
  float S[PER], A[PER];
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int n = e * lanes + sub;
    S[e] = n < n_state ? S_mem[n] : 0.f;
    A[e] = n < n_state ? -expf(A_log[(long long)c * n_state + n]) : 0.f;
  }
  const float bias = dt_bias[c];
  const float skip = D[c];
  const int t0 = q_start[req], t1 = q_start[req + 1];
  float Bn[PER], Cn[PER], xv, zv, dv;
  auto fetch = [&](int t, float (&B_)[PER], float (&C_)[PER], float& x_, float& z_, float& d_) {
    const T* row = bc + (long long)t * ld_bc;
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      const int n = e * lanes + sub;
      B_[e] = n < n_state ? rv_to_float(row[b_col + n]) : 0.f;
      C_[e] = n < n_state ? rv_to_float(row[c_col + n]) : 0.f;
    }
    x_ = rv_to_float(x[(long long)t * ld_x + c]);
    z_ = rv_to_float(z[(long long)t * ld_z + c]);
    d_ = rv_to_float(dt[(long long)t * ld_dt + c]);
  };
  if (t0 < t1) fetch(t0, Bn, Cn, xv, zv, dv);
  for (int t = t0; t < t1; ++t) {
    float nB[PER], nC[PER], nx = 0.f, nz = 0.f, nd = 0.f;
    if (t + 1 < t1) fetch(t + 1, nB, nC, nx, nz, nd);
    const float step = rec_softplus(dv + bias);
    const float sx = step * xv;
    float y = 0.f;
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      S[e] = fmaf(expf(step * A[e]), S[e], sx * Bn[e]);
      y = fmaf(S[e], Cn[e], y);
    }
    y = rec_group_sum(y, lanes);
    y = fmaf(skip, xv, y);
    if (live && sub == 0) out[(long long)t * channels + ch] = rv_from_float<T>(y * rec_silu(zv));
    if (t + 1 < t1) {
#pragma unroll
      for (int e = 0; e < PER; ++e) Bn[e] = nB[e], Cn[e] = nC[e];
      xv = nx, zv = nz, dv = nd;
    }
  }
  if (live) {
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      const int n = e * lanes + sub;
      if (n < n_state) S_mem[n] = S[e];
    }
  }
}

#define REC_SCAN_PER 4

// Lanes that share a channel: the fewest (a power of two) that leave a lane at most REC_SCAN_PER states.
extern "C" int rv_selective_scan_lanes(int n_state) {
  int lanes = 1;
  while (lanes < RV_WAVE && rv_div_up(n_state, lanes) > REC_SCAN_PER) lanes *= 2;
  return lanes;
}

extern "C" int rv_selective_scan(hipStream_t stream, const void* x, long long ld_x, const void* z, long long ld_z,
                                 const void* dt, long long ld_dt, const float* dt_bias, const void* bc,
                                 long long ld_bc, int b_col, int c_col, const float* A_log, const float* D,
                                 float* state, long long slot_stride, long long s_off, const int* q_start,
                                 const int* state_slot, void* out, int dtype, int num_requests, int channels,
                                 int n_state) {
  RV_CHECK(x && z && dt && dt_bias && bc && A_log && D && state && q_start && state_slot && out,
           "selective_scan: null argument");
  RV_CHECK(channels > 0 && n_state > 0 && num_requests >= 0, "selective_scan: bad sizes");
  const int lanes = rv_selective_scan_lanes(n_state);
  RV_CHECK(rv_div_up(n_state, lanes) <= REC_SCAN_PER, "selective_scan: %d states a channel are more than %d", n_state,
           REC_SCAN_PER * RV_WAVE);
  if (num_requests == 0) return 0;
  dim3 grid(rv_div_up(channels, RV_WAVE / lanes), num_requests), block(RV_WAVE);
#define RV_SS(T)                                                                                                   \
  selective_scan_kernel<T, REC_SCAN_PER><<<grid, block, 0, stream>>>(                                              \
      (const T*)x, ld_x, (const T*)z, ld_z, (const T*)dt, ld_dt, dt_bias, (const T*)bc, ld_bc, b_col, c_col, A_log, \
      D, state, slot_stride, s_off, q_start, state_slot, (T*)out, channels, n_state, lanes)
  if (dtype == RV_F32) RV_SS(float);
  else if (dtype == RV_BF16) RV_SS(bf16_t);
  else return rv_fail("selective_scan: unsupported dtype %d", dtype);
#undef RV_SS
  RV_LAUNCH_CHECK("selective_scan");
  return 0;
}

// ---------------------------------------------------------------------------
// out[t][h][:] = o[t][h][:] / sqrt(mean(o[t][h][:]^2) + eps) * w[:] * silu(gate[t][h][:]); a wave a (token, head).
// o: float [tokens, heads dv]; gate: T, rows ld_gate apart; w: float [dv], shared by the heads; out: T.
// ---------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
head_norm_gate_kernel(const float* __restrict__ o, const T* __restrict__ gate, long long ld_gate,
                      const float* __restrict__ w, T* __restrict__ out, int heads, int dv, float eps, long long units) {
  const int lane = threadIdx.x & (RV_WAVE - 1);
  const long long unit = (long long)blockIdx.x * (blockDim.x / RV_WAVE) + threadIdx.x / RV_WAVE;
  if (unit >= units) return;
  const long long t = unit / heads;
  const int h = (int)(unit - t * heads);
  const float* row = o + unit * dv;
  float ss = 0.f;
  for (int d = lane; d < dv; d += RV_WAVE) ss = fmaf(row[d], row[d], ss);
  ss = rv_wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)dv + eps);
  for (int d = lane; d < dv; d += RV_WAVE) {
    const float gv = rv_to_float(gate[t * ld_gate + (long long)h * dv + d]);
    out[unit * dv + d] = rv_from_float<T>(row[d] * inv * w[d] * rec_silu(gv));
  }
}

extern "C" int rv_head_norm_gate(hipStream_t stream, const float* o, const void* gate, long long ld_gate,
                                 const float* w, void* out, int dtype, int num_tokens, int heads, int dv, float eps) {
  RV_CHECK(o && gate && w && out && heads > 0 && dv > 0 && num_tokens >= 0, "head_norm_gate: bad arguments");
  if (num_tokens == 0) return 0;
  const long long units = (long long)num_tokens * heads;
  dim3 grid(rv_div_up(units, 4)), block(256);
  if (dtype == RV_F32)
    head_norm_gate_kernel<float><<<grid, block, 0, stream>>>(o, (const float*)gate, ld_gate, w, (float*)out, heads, dv,
                                                             eps, units);
  else if (dtype == RV_BF16)
    head_norm_gate_kernel<bf16_t><<<grid, block, 0, stream>>>(o, (const bf16_t*)gate, ld_gate, w, (bf16_t*)out, heads,
                                                              dv, eps, units);
  else
    return rv_fail("head_norm_gate: unsupported dtype %d", dtype);
  RV_LAUNCH_CHECK("head_norm_gate");
  return 0;
}

// ---------------------------------------------------------------------------
// a[t][c] *= act(gate[t][c]), in place; act 0: sigmoid, 1: silu.  gate's rows are ld_gate apart.
// ---------------------------------------------------------------------------
template <typename T>
__global__ void gate_mul_kernel(T* __restrict__ a, const T* __restrict__ gate, long long ld_gate, int width,
                                long long total, int act) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const long long t = idx / width;
  const float gv = rv_to_float(gate[t * ld_gate + (idx - t * width)]);
  const float m = act == 0 ? rec_sigmoid(gv) : rec_silu(gv);
  a[idx] = rv_from_float<T>(rv_to_float(a[idx]) * m);
}

extern "C" int rv_gate_mul(hipStream_t stream, void* a, const void* gate, long long ld_gate, int dtype, int rows,
                           int width, int act) {
  RV_CHECK(a && gate && rows >= 0 && width > 0 && ld_gate >= width && (act == 0 || act == 1), "gate_mul: bad arguments");
  if (rows == 0) return 0;
  const long long total = (long long)rows * width;
  dim3 grid(rv_div_up(total, 256)), block(256);
  if (dtype == RV_F32)
    gate_mul_kernel<float><<<grid, block, 0, stream>>>((float*)a, (const float*)gate, ld_gate, width, total, act);
  else if (dtype == RV_BF16)
    gate_mul_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t*)a, (const bf16_t*)gate, ld_gate, width, total, act);
  else
    return rv_fail("gate_mul: unsupported dtype %d", dtype);
  RV_LAUNCH_CHECK("gate_mul");
  return 0;
}
