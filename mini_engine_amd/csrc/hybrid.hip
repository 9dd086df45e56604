// Kernels of mixers that run two token mixers side by side, one of them a recurrence whose state rows decay each at
// a rate of their own: the mix of a token's input with the previous token's, the recurrence itself under two update
// rules, the weighted sum of the two mixers' outputs, and the small elementwise steps around them (a bias on a
// projection's rows, an elementwise sigmoid gate, a clamped gated activation). Everything that the recurrence reads
// besides the projections is formed here in float32: decays and their exponentials, softplus, write strengths, unit
// lengths.
#include "common.h"

__device__ __forceinline__ float hy_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }
__device__ __forceinline__ float hy_softplus(float v) { return v > 20.f ? v : log1pf(expf(v)); }

// ------------------------------------------------------------------ rows + bias
// out[t, c] = (sum_p x[p, t, c]) + bias[c] for c < nb, without a bias beyond; x: `parts` stacked slices.
template <typename TX, typename TY>
__global__ void add_bias_kernel(const TX* __restrict__ x, int parts, int64_t part_stride, int64_t x_stride,
                                const float* __restrict__ bias, int nb, TY* __restrict__ out, int64_t T, int n) {
  const int64_t total = T * n;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / n;
    const int c = (int)(i - t * n);
    float v = 0.f;
    for (int p = 0; p < parts; ++p) v += to_f32<TX>(x[p * part_stride + t * x_stride + c]);
    if (c < nb) v += bias[c];
    out[i] = from_f32<TY>(v);
  }
}

extern "C" int me_add_bias(const void* x, int x_dtype, int parts, int64_t part_stride, int64_t x_stride, const float* bias, int nb,
                           void* out, int out_dtype, int64_t T, int n, hipStream_t stream) {
  if (T == 0 || n == 0) return 0;
  ME_CHECK(parts >= 1 && nb >= 0 && nb <= n, "add_bias: bad slice count or bias length");
  const int64_t total = T * n;
  const dim3 grid((unsigned)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535)), block(256);
#define AB(TX, TY) add_bias_kernel<TX, TY><<<grid, block, 0, stream>>>((const TX*)x, parts, part_stride, x_stride, bias, nb, (TY*)out, T, n)
  if (x_dtype == ME_F32 && out_dtype == ME_F32) AB(float, float);
  else if (x_dtype == ME_F32) AB(float, bf16_t);
  else if (out_dtype == ME_F32) AB(bf16_t, float);
  else AB(bf16_t, bf16_t);
#undef AB
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ o *= sigmoid(g), element by element
template <typename TX>
__global__ void sigmoid_gate_kernel(TX* __restrict__ o, int64_t o_stride, const TX* __restrict__ g, int64_t g_stride, int64_t T, int n) {
  const int64_t total = T * n;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / n;
    const int c = (int)(i - t * n);
    TX* at = o + t * o_stride + c;
    *at = from_f32<TX>(to_f32<TX>(*at) * hy_sigmoid(to_f32<TX>(g[t * g_stride + c])));
  }
}

extern "C" int me_sigmoid_gate(void* o, int64_t o_stride, const void* g, int64_t g_stride, int dtype, int64_t T, int n, hipStream_t stream) {
  if (T == 0 || n == 0) return 0;
  const int64_t total = T * n;
  const dim3 grid((unsigned)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535)), block(256);
  if (dtype == ME_F32) sigmoid_gate_kernel<float><<<grid, block, 0, stream>>>((float*)o, o_stride, (const float*)g, g_stride, T, n);
  else sigmoid_gate_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t*)o, o_stride, (const bf16_t*)g, g_stride, T, n);
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ clamped gated activation
// g = min(gu[t, i], limit), u = clamp(gu[t, I + i], -limit, limit); out = g * sigmoid(alpha * g) * (u + 1).
template <typename TX>
__global__ void glu_clamped_kernel(const TX* __restrict__ gu, int64_t gu_stride, TX* __restrict__ out, int64_t T, int I, float limit, float alpha) {
  const int64_t total = T * I;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / I;
    const int c = (int)(i - t * I);
    const float g = fminf(to_f32<TX>(gu[t * gu_stride + c]), limit);
    const float u = fminf(fmaxf(to_f32<TX>(gu[t * gu_stride + I + c]), -limit), limit);
    out[i] = from_f32<TX>(g * hy_sigmoid(alpha * g) * (u + 1.0f));
  }
}

extern "C" int me_glu_clamped(const void* gu, int64_t gu_stride, void* out, int dtype, int64_t T, int I, float limit, float alpha, hipStream_t stream) {
  if (T == 0 || I == 0) return 0;
  ME_CHECK(limit > 0.f, "glu_clamped: the limit must be positive");
  const int64_t total = T * I;
  const dim3 grid((unsigned)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535)), block(256);
  if (dtype == ME_F32) glu_clamped_kernel<float><<<grid, block, 0, stream>>>((const float*)gu, gu_stride, (float*)out, T, I, limit, alpha);
  else glu_clamped_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)gu, gu_stride, (bf16_t*)out, T, I, limit, alpha);
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ weighted sum of sublayer outputs
// out[t, c] = sum_i scale_i * gate_i[t] * ((sum_p term_i[p, t, c]) + bias_i[c]), float32. Terms are rows in the compute dtype or
// stacked float32 partial sums. gate_i[t] = sigmoid(g_i[t * gate_stride_i]) for a term that has gate rows g_i (in the compute
// dtype or float32), else 1. With w: the norm on the sum as well, stream' = stream + w * out / rms(out), one
// workgroup per row (the sum is held in LDS between the two passes), the new stream also rounded to TY.
#define WS_MAX_TERMS 4
struct WsArgs {
  const void* term[WS_MAX_TERMS]; int dtype[WS_MAX_TERMS]; int parts[WS_MAX_TERMS]; int64_t part_stride[WS_MAX_TERMS];
  float scale[WS_MAX_TERMS]; const float* bias[WS_MAX_TERMS];
  const void* gate[WS_MAX_TERMS]; int gate_dtype[WS_MAX_TERMS]; int64_t gate_stride[WS_MAX_TERMS];
  int count, n;
};

__device__ __forceinline__ float ws_value(const WsArgs& a, int64_t t, int c) {
  float total = 0.f;
  for (int i = 0; i < a.count; ++i) {
    float v = 0.f;
    if (a.dtype[i] == ME_F32) {
      const float* x = (const float*)a.term[i];
      for (int p = 0; p < a.parts[i]; ++p) v += x[p * a.part_stride[i] + t * a.n + c];
    } else {
      v = to_f32<bf16_t>(((const bf16_t*)a.term[i])[t * a.n + c]);
    }
    if (a.bias[i] != nullptr) v += a.bias[i][c];
    if (a.gate[i] != nullptr) {
      const float g = a.gate_dtype[i] == ME_F32 ? ((const float*)a.gate[i])[t * a.gate_stride[i]]
                                                : to_f32<bf16_t>(((const bf16_t*)a.gate[i])[t * a.gate_stride[i]]);
      v *= 1.0f / (1.0f + expf(-g));
    }
    total += a.scale[i] * v;
  }
  return total;
}

__global__ void weighted_sum_kernel(WsArgs a, float* __restrict__ out, int64_t T) {
  const int64_t total = T * a.n;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / a.n;
    out[i] = ws_value(a, t, (int)(i - t * a.n));
  }
}

template <typename TY>
__global__ void weighted_sum_norm_kernel(WsArgs a, const float* __restrict__ w, float eps, const float* __restrict__ stream_in,
                                         float* __restrict__ stream_out, TY* __restrict__ rounded) {
  __shared__ float scratch[16];
  extern __shared__ float row[];
  const int64_t t = blockIdx.x;
  float ss = 0.f;
  for (int c = threadIdx.x; c < a.n; c += blockDim.x) {
    const float v = ws_value(a, t, c);
    row[c] = v;
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)a.n + eps);
  for (int c = threadIdx.x; c < a.n; c += blockDim.x) {
    const float v = stream_in[t * a.n + c] + w[c] * (row[c] * inv);
    stream_out[t * a.n + c] = v;
    if (rounded != nullptr) rounded[t * a.n + c] = from_f32<TY>(v);
  }
}

extern "C" int me_weighted_sum(int count, const void** terms, const int* dtypes, const int* parts, const int64_t* part_strides,
                               const float* scales, const float** biases, float* out, const float* w, float eps,
                               const float* stream_in, float* stream_out, void* rounded, int rounded_dtype, int64_t T, int n,
                               const void** gates, const int* gate_dtypes, const int64_t* gate_strides, hipStream_t stream) {
  if (T == 0 || n == 0) return 0;
  ME_CHECK(count >= 1 && count <= WS_MAX_TERMS, "weighted_sum: 1..%d terms", WS_MAX_TERMS);
  WsArgs a;
  a.count = count; a.n = n;
  for (int i = 0; i < count; ++i) {
    ME_CHECK(parts[i] >= 1 && (dtypes[i] == ME_F32 || parts[i] == 1), "weighted_sum: partial sums are float32");
    a.term[i] = terms[i]; a.dtype[i] = dtypes[i]; a.parts[i] = parts[i]; a.part_stride[i] = part_strides[i];
    a.scale[i] = scales[i]; a.bias[i] = biases[i];
    a.gate[i] = gates ? gates[i] : nullptr; a.gate_dtype[i] = gates ? gate_dtypes[i] : ME_F32; a.gate_stride[i] = gates ? gate_strides[i] : 0;
  }
  if (w == nullptr) {
    const int64_t total = T * n;
    const dim3 grid((unsigned)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535)), block(256);
    weighted_sum_kernel<<<grid, block, 0, stream>>>(a, out, T);
  } else {
    ME_CHECK(n <= 15360 && stream_in != nullptr && stream_out != nullptr, "weighted_sum: rows of up to 15360 with a stream");
    const dim3 grid((unsigned)T), block(n >= 1024 ? 256 : (n > 256 ? 128 : 64));
    const size_t lds = (size_t)n * sizeof(float);
    if (rounded == nullptr || rounded_dtype == ME_F32)
      weighted_sum_norm_kernel<float><<<grid, block, lds, stream>>>(a, w, eps, stream_in, stream_out, (float*)rounded);
    else
      weighted_sum_norm_kernel<bf16_t><<<grid, block, lds, stream>>>(a, w, eps, stream_in, stream_out, (bf16_t*)rounded);
  }
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ a token's input mixed with the previous token's
// out[s, t, c] = x[t, c] + (before[t, c] - x[t, c]) * mu[s, c], s < S. before: the row of the request's previous token;
// for the first token of the request's tokens in this step it comes from the request's state row (zeros at position 0,
// which the step function has written there), which then takes the step's last row. The thread of a request's first
// token reads the state before it writes it, so a step needs no second launch.
template <typename TX>
__global__ void token_shift_kernel(const TX* __restrict__ x, int64_t x_stride, const float* __restrict__ mu, int S,
                                   float* __restrict__ state, int64_t state_stride, const int32_t* __restrict__ slots,
                                   const int32_t* __restrict__ cu, const int32_t* __restrict__ seq_of_token,
                                   TX* __restrict__ out, int64_t T, int n) {
  const int64_t t = blockIdx.x;
  const int b = seq_of_token[t];
  const int64_t first = cu[b], last = (int64_t)cu[b + 1] - 1;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < n; c += gridDim.y * blockDim.x) {
    const float now = to_f32<TX>(x[t * x_stride + c]);
    float before;
    if (t == first) {
      float* held = state + (int64_t)slots[b] * state_stride + c;
      before = *held;
      *held = to_f32<TX>(x[last * x_stride + c]);
    } else {
      before = to_f32<TX>(x[(t - 1) * x_stride + c]);
    }
    const float d = before - now;
    for (int s = 0; s < S; ++s) out[((int64_t)s * T + t) * n + c] = from_f32<TX>(now + d * mu[(int64_t)s * n + c]);
  }
}

extern "C" int me_token_shift(const void* x, int64_t x_stride, int dtype, const float* mu, int S, float* state, int64_t state_stride,
                              const int32_t* slots, const int32_t* cu, const int32_t* seq_of_token, void* out, int64_t T, int n,
                              hipStream_t stream) {
  if (T == 0 || n == 0) return 0;
  ME_CHECK(S >= 1 && T <= 2147483647ll, "token_shift: bad sizes");
  const dim3 block(n >= 256 ? 256 : 64);
  const unsigned gy = (unsigned)((n + block.x - 1) / block.x < 64 ? (n + block.x - 1) / block.x : 64);
  const dim3 grid((unsigned)T, gy);
  if (dtype == ME_F32)
    token_shift_kernel<float><<<grid, block, 0, stream>>>((const float*)x, x_stride, mu, S, state, state_stride, slots, cu, seq_of_token, (float*)out, T, n);
  else
    token_shift_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)x, x_stride, mu, S, state, state_stride, slots, cu, seq_of_token, (bf16_t*)out, T, n);
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ the recurrence with a decay per state row
// Per request and head a state S [N, P] in float32, walked over the request's tokens of this step in order.
//   RULE 0 (bonus):  d_n = exp(-exp(raw[t, h, n] + base[h, n]));
//                    y_p = sum_n q_n (S[n, p] + bonus[h, n] k_n v_p);   S[n, p] <- d_n S[n, p] + k_n v_p
//   RULE 1 (delta):  d_n = exp(-rate[h] softplus(raw[t, h, n] + base[h, n])),  beta = sigmoid(beta_raw[t, h]);
//                    S[n, p] <- d_n S[n, p];  u_p = beta (v_p - sum_n S[n, p] k_n);  S[n, p] <- S[n, p] + k_n u_p;
//                    y_p = sum_n S[n, p] q_n
//   RULE 2 (gated):  d_n = sigmoid(raw[t, h, n] + base[h, n]) ^ rate[h] = exp(-rate[h] softplus(-(raw + base)));
//                    S[n, p] <- d_n S[n, p] + k_n v_p;   y_p = sum_n S[n, p] q_n
// With `unit`: q and k are first divided by sqrt(sum of their squares + unit_eps) per head; q is multiplied by q_scale.
// Every sum runs over n only, so a column p of the state never meets another: a wave takes 64 / RG columns of one head
// and a lane NR / RG of a column's rows, kept in registers for the whole walk; with RG > 1 the RG lanes of a column,
// neighbours in the wave, add their partial sums by exchanges inside a row of 16 lanes. q, k and the decays of a token, which all columns share, are
// formed once per wave in LDS, eight tokens at a time into one of two buffers; the next eight tokens' raw values are on
// their way while the current eight are worked on, so a wave waits for memory once per eight tokens. The products
// and sums of the walk are written as explicit fused multiply-adds: a token's result then does not depend on its place
// among the eight (the compiler is free to fuse each unrolled copy otherwise).
struct DrArgs {
  const void* q; const void* k; const void* v; const void* raw; const void* beta;
  int64_t q_stride, k_stride, v_stride, raw_stride, beta_stride;
  const float* base; const float* rate; const float* bonus;
  float* state; int64_t state_stride;
  const int32_t* slots; const int32_t* cu;
  float* y;
  int H, G, N, P;
  int unit; float unit_eps, q_scale;
};

#define DR_TB 8          // tokens whose shared values are formed at once and wait in LDS

// Sum over the RG neighbouring lanes that share a state column (RG 1, 4 or 16, aligned groups), left in all of them: lane
// exchanges inside a row of 16 lanes (quad permutations, then rotations of the row), no trip through LDS.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int RG>
__device__ __forceinline__ float group_sum(float v) {
  if (RG >= 2) v += dpp_f<0xB1>(v);      // quad_perm [1, 0, 3, 2]
  if (RG >= 4) v += dpp_f<0x4E>(v);      // quad_perm [2, 3, 0, 1]
  if (RG >= 8) v += dpp_f<0x124>(v);     // row_ror 4
  if (RG >= 16) v += dpp_f<0x128>(v);    // row_ror 8
  return v;
}

// What a token's q, k, raw decay and write strength become before the recurrence reads them, for one wave that holds
// rows lane, lane + 64, ... of one head: q and k at unit length and scaled, the decay, and the token's own number
// (sigmoid(beta), or sum_n q_n bonus_n k_n under the bonus rule), which every lane gets.
template <int PER, int RULE>
__device__ __forceinline__ float shape_token(const DrArgs& a, int lane, int nr_rows, float (&q)[PER], float (&k)[PER], float (&d)[PER],
                                             const float (&base)[PER], const float (&bonus)[PER], float rate, float beta) {
  float qs = a.q_scale, ks = 1.0f;
  if (a.unit) {
    float q2 = 0.f, k2 = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i) { q2 += q[i] * q[i]; k2 += k[i] * k[i]; }
    qs = a.q_scale / sqrtf(wave_sum(q2) + a.unit_eps);
    ks = 1.0f / sqrtf(wave_sum(k2) + a.unit_eps);
  }
  float own = 0.f;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int n = lane + 64 * i;
    q[i] *= qs;
    k[i] *= ks;
    float dv;
    if (RULE == 0) dv = expf(-expf(d[i] + base[i]));
    else if (RULE == 2) dv = expf(-rate * hy_softplus(-(d[i] + base[i])));
    else dv = expf(-rate * hy_softplus(d[i] + base[i]));
    d[i] = (n < a.N && n < nr_rows) ? dv : 1.0f;
    own += q[i] * bonus[i] * k[i];
  }
  if (RULE == 2) return 0.f;
  return RULE == 1 ? hy_sigmoid(beta) : wave_sum(own);
}

// One wave per (token, head): the shaped values of every token at once, for a recurrence kernel that then only streams
// them (PRE): pre_q, pre_k, pre_d [T, H, NR] and pre_x [T, H], float32.
template <typename TX, int NR, int RULE>
__global__ void __launch_bounds__(64) decay_prepare_kernel(DrArgs a, float* __restrict__ pre_q, float* __restrict__ pre_k,
                                                           float* __restrict__ pre_d, float* __restrict__ pre_x) {
  constexpr int PER = (NR + 63) / 64;
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const int g = h / (a.H / a.G);
  const TX* qp = (const TX*)a.q; const TX* kp = (const TX*)a.k; const TX* rp = (const TX*)a.raw; const TX* bp = (const TX*)a.beta;
  float q[PER], k[PER], d[PER], base[PER], bonus[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int n = lane + 64 * i;
    const bool in = n < a.N && n < NR;
    base[i] = in ? a.base[h * a.N + n] : 0.f;
    bonus[i] = (RULE == 0 && in) ? a.bonus[h * a.N + n] : 0.f;
    q[i] = in ? to_f32<TX>(qp[t * a.q_stride + g * a.N + n]) : 0.f;
    k[i] = in ? to_f32<TX>(kp[t * a.k_stride + g * a.N + n]) : 0.f;
    d[i] = in ? to_f32<TX>(rp[t * a.raw_stride + h * a.N + n]) : 0.f;
  }
  const float beta = RULE == 1 ? to_f32<TX>(bp[t * a.beta_stride + h]) : 0.f;
  const float x = shape_token<PER, RULE>(a, lane, NR, q, k, d, base, bonus, RULE != 0 ? a.rate[h] : 0.f, beta);
  const int64_t at = (t * a.H + h) * NR;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int n = lane + 64 * i;
    if (n < NR) { pre_q[at + n] = q[i]; pre_k[at + n] = k[i]; pre_d[at + n] = d[i]; }
  }
  if (lane == 0) pre_x[t * a.H + h] = x;
}

template <typename TX, int NR, int RG, int RULE, bool PRE>
__global__ void __launch_bounds__(64) decay_rows_kernel(DrArgs a, const float* __restrict__ pre_q, const float* __restrict__ pre_k,
                                                        const float* __restrict__ pre_d, const float* __restrict__ pre_x) {
  constexpr int PC = 64 / RG;            // columns per wave
  constexpr int RL = NR / RG;            // rows per lane
  constexpr int PER = (NR + 63) / 64;    // rows of q, k and the decay that a lane brings to LDS for the wave
  __shared__ float sq[2][DR_TB][NR], sk[2][DR_TB][NR], sd[2][DR_TB][NR];
  const int lane = threadIdx.x;
  const int col_blocks = (a.P + PC - 1) / PC;
  const int cb = blockIdx.x % col_blocks;
  const int h = (blockIdx.x / col_blocks) % a.H;
  const int b = blockIdx.x / (col_blocks * a.H);
  const int g = h / (a.H / a.G);
  const int64_t first = a.cu[b];
  const int n_tok = (int)(a.cu[b + 1] - first);
  if (n_tok <= 0) return;
  // the RG lanes of a column are neighbours; lane rg of them keeps rows rg, rg + RG, ... (neighbours read neighbouring
  // words of LDS, the lanes of the wave's other columns the same words)
  const int p = cb * PC + lane / RG;
  const int rg = lane % RG;
  const bool live = p < a.P;
  const int pc = live ? p : a.P - 1;
  float* srow = a.state + (int64_t)a.slots[b] * a.state_stride + (int64_t)h * a.N * a.P;
  float S[RL];
#pragma unroll
  for (int i = 0; i < RL; ++i) S[i] = (i * RG + rg < a.N) ? srow[(int64_t)(i * RG + rg) * a.P + pc] : 0.f;

  const TX* qp = (const TX*)a.q; const TX* kp = (const TX*)a.k; const TX* vp = (const TX*)a.v;
  const TX* rp = (const TX*)a.raw; const TX* bp = (const TX*)a.beta;
  float base[PER], bonus[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int n = lane + 64 * i;
    const bool in = !PRE && n < a.N && n < NR;
    base[i] = in ? a.base[h * a.N + n] : 0.f;
    bonus[i] = (RULE == 0 && in) ? a.bonus[h * a.N + n] : 0.f;
  }
  const float rate = (RULE != 0 && !PRE) ? a.rate[h] : 0.f;
  // a batch of tokens on its way (n*) and the batch being worked on (c*): a lane's own column's v and the token's own
  // number (the write strength, or under the bonus rule sum_n q_n bonus_n k_n)
  float nq[DR_TB][PER], nk[DR_TB][PER], nr[DR_TB][PER], nv[DR_TB], nb[DR_TB];
  float cv[DR_TB], cx[DR_TB];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int j = 0; j < DR_TB; ++j) {
      if (t0 + j < n_tok) {
        const int64_t row = first + t0 + j;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
          const int n = lane + 64 * i;
          if (PRE) {
            const int64_t at = (row * a.H + h) * NR + (n < NR ? n : 0);
            nq[j][i] = pre_q[at]; nk[j][i] = pre_k[at]; nr[j][i] = pre_d[at];
          } else {
            const bool in = n < a.N && n < NR;
            nq[j][i] = in ? to_f32<TX>(qp[row * a.q_stride + g * a.N + n]) : 0.f;
            nk[j][i] = in ? to_f32<TX>(kp[row * a.k_stride + g * a.N + n]) : 0.f;
            nr[j][i] = in ? to_f32<TX>(rp[row * a.raw_stride + h * a.N + n]) : 0.f;
          }
        }
        nv[j] = to_f32<TX>(vp[row * a.v_stride + h * a.P + pc]);
        if (PRE) nb[j] = pre_x[row * a.H + h];
        else nb[j] = RULE == 1 ? to_f32<TX>(bp[row * a.beta_stride + h]) : 0.f;
      }
    }
  };
  // the fetched batch's shared values into LDS buffer `buf`, its per-lane values into c*
  auto settle = [&](int t0, int buf) {
#pragma unroll
    for (int j = 0; j < DR_TB; ++j) {
      if (t0 + j < n_tok) {
        float x = nb[j];
        if (!PRE) x = shape_token<PER, RULE>(a, lane, NR, nq[j], nk[j], nr[j], base, bonus, rate, nb[j]);
#pragma unroll
        for (int i = 0; i < PER; ++i) {
          const int n = lane + 64 * i;
          // row n belongs to lane n % RG of a column as its row n / RG: a lane's rows lie side by side in LDS, so that it
          // reads them four at a time
          const int at = (n % RG) * RL + n / RG;
          if (n < NR) { sq[buf][j][at] = nq[j][i]; sk[buf][j][at] = nk[j][i]; sd[buf][j][at] = nr[j][i]; }
        }
        cv[j] = nv[j];
        cx[j] = x;
      }
    }
  };
  fetch(0);
  for (int t0 = 0, buf = 0; t0 < n_tok; t0 += DR_TB, buf ^= 1) {
    settle(t0, buf);
    __syncthreads();      // the batch is in LDS; the other buffer, which the next batch will take, has been read by all
    if (t0 + DR_TB < n_tok) fetch(t0 + DR_TB);
#pragma unroll
    for (int j = 0; j < DR_TB; ++j) {
      if (t0 + j < n_tok) {
        const float v = cv[j];
        float y = 0.f;
        if (RULE == 0) {
#pragma unroll
          for (int i = 0; i < RL; ++i) {
            const int n = rg * RL + i;
            y = fmaf(sq[buf][j][n], S[i], y);
            S[i] = fmaf(sd[buf][j][n], S[i], sk[buf][j][n] * v);
          }
        } else if (RULE == 2) {
#pragma unroll
          for (int i = 0; i < RL; ++i) {
            const int n = rg * RL + i;
            S[i] = fmaf(sd[buf][j][n], S[i], sk[buf][j][n] * v);
            y = fmaf(sq[buf][j][n], S[i], y);
          }
        } else {
          float dot = 0.f;
#pragma unroll
          for (int i = 0; i < RL; ++i) {
            const int n = rg * RL + i;
            S[i] *= sd[buf][j][n];
            dot = fmaf(S[i], sk[buf][j][n], dot);
          }
          dot = group_sum<RG>(dot);
          const float u = cx[j] * (v - dot);
#pragma unroll
          for (int i = 0; i < RL; ++i) {
            const int n = rg * RL + i;
            S[i] = fmaf(sk[buf][j][n], u, S[i]);
            y = fmaf(S[i], sq[buf][j][n], y);
          }
        }
        y = group_sum<RG>(y);
        if (RULE == 0) y = fmaf(cx[j], v, y);       // the current token's own term: v_p * sum_n q_n bonus_n k_n
        if (live && rg == 0) a.y[(first + t0 + j) * (int64_t)(a.H * a.P) + h * a.P + p] = y;
      }
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < RL; ++i)
      if (i * RG + rg < a.N) srow[(int64_t)(i * RG + rg) * a.P + p] = S[i];
  }
}

template <typename TX, int NR, int RG, bool PRE>
static void launch_decay_rows(const DrArgs& a, int rule, int num_seqs, int64_t T, float* pre, hipStream_t stream) {
  constexpr int PC = 64 / RG;
  const dim3 grid((unsigned)(num_seqs * a.H * ((a.P + PC - 1) / PC))), block(64);
  float* pq = pre; float* pk = pre; float* pd = pre; float* px = pre;
  if (PRE) {
    const int64_t each = T * a.H * NR;
    pk = pre + each; pd = pre + 2 * each; px = pre + 3 * each;
    const dim3 pgrid((unsigned)T, a.H);
    if (rule == 0) decay_prepare_kernel<TX, NR, 0><<<pgrid, block, 0, stream>>>(a, pq, pk, pd, px);
    else if (rule == 2) decay_prepare_kernel<TX, NR, 2><<<pgrid, block, 0, stream>>>(a, pq, pk, pd, px);
    else decay_prepare_kernel<TX, NR, 1><<<pgrid, block, 0, stream>>>(a, pq, pk, pd, px);
  }
  if (rule == 0) decay_rows_kernel<TX, NR, RG, 0, PRE><<<grid, block, 0, stream>>>(a, pq, pk, pd, px);
  else if (rule == 2) decay_rows_kernel<TX, NR, RG, 2, PRE><<<grid, block, 0, stream>>>(a, pq, pk, pd, px);
  else decay_rows_kernel<TX, NR, RG, 1, PRE><<<grid, block, 0, stream>>>(a, pq, pk, pd, px);
}

// row_groups: lanes that share a column: 1 or 4 (4 gives four times the waves with a quarter of the rows each) with the
// tokens' values shaped inside the kernel; 4 or 16 with `pre`, scratch of 3 T H NR + T H floats (NR: N rounded up to 32, 64,
// 128 or 256) that a first kernel fills with the shaped values of all tokens at once, so that the walk only streams them.
extern "C" int me_decay_rows_recurrence(const void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v, int64_t v_stride,
                                        const void* raw, int64_t raw_stride, const void* beta, int64_t beta_stride, int dtype,
                                        const float* base, const float* rate, const float* bonus, float* state, int64_t state_stride,
                                        const int32_t* slots, const int32_t* cu, float* y, int num_seqs, int H, int G, int N, int P,
                                        int rule, int unit, float unit_eps, float q_scale, int row_groups, int64_t T, float* pre, hipStream_t stream) {
  if (num_seqs == 0) return 0;
  ME_CHECK(H >= 1 && G >= 1 && H % G == 0 && N >= 1 && N <= 256 && P >= 1, "decay_rows_recurrence: %d heads over %d groups, state %d x %d "
           "(up to 256 rows)", H, G, N, P);
  ME_CHECK(rule >= 0 && rule <= 2, "decay_rows_recurrence: unknown rule %d", rule);
  ME_CHECK(rule == 0 ? bonus != nullptr : (rate != nullptr && (rule == 2 || beta != nullptr)), "decay_rows_recurrence: the rule's constants are missing");
  ME_CHECK(pre == nullptr ? (row_groups == 1 || row_groups == 4) : (row_groups == 4 || row_groups == 16),
           "decay_rows_recurrence: 1 or 4 lanes to a column, 4 or 16 over prepared values");
  ME_CHECK(T >= 0 && T <= 2147483647ll && H <= 65535, "decay_rows_recurrence: too many tokens or heads");
  ME_CHECK((int64_t)num_seqs * H * ((P + 3) / 4) <= 2147483647ll, "decay_rows_recurrence: too many workgroups");
  DrArgs a;
  a.q = q; a.k = k; a.v = v; a.raw = raw; a.beta = beta;
  a.q_stride = q_stride; a.k_stride = k_stride; a.v_stride = v_stride; a.raw_stride = raw_stride; a.beta_stride = beta_stride;
  a.base = base; a.rate = rate; a.bonus = bonus; a.state = state; a.state_stride = state_stride; a.slots = slots; a.cu = cu; a.y = y;
  a.H = H; a.G = G; a.N = N; a.P = P; a.unit = unit; a.unit_eps = unit_eps; a.q_scale = q_scale;
#define DR_NR(TX, NR)                                                           \
  do {                                                                          \
    if (pre != nullptr && row_groups == 16) launch_decay_rows<TX, NR, 16, true>(a, rule, num_seqs, T, pre, stream); \
    else if (pre != nullptr) launch_decay_rows<TX, NR, 4, true>(a, rule, num_seqs, T, pre, stream);                 \
    else if (row_groups == 4) launch_decay_rows<TX, NR, 4, false>(a, rule, num_seqs, T, pre, stream);               \
    else launch_decay_rows<TX, NR, 1, false>(a, rule, num_seqs, T, pre, stream);                                    \
  } while (0)
#define DR(TX)                            \
  do {                                    \
    if (N <= 32) DR_NR(TX, 32);           \
    else if (N <= 64) DR_NR(TX, 64);      \
    else if (N <= 128) DR_NR(TX, 128);    \
    else DR_NR(TX, 256);                  \
  } while (0)
  if (dtype == ME_F32) DR(float); else DR(bf16_t);
#undef DR
#undef DR_NR
  ME_LAUNCH_CHECK();
  return 0;
}
