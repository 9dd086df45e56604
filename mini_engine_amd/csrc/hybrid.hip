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
// out[t, c] = sum_i scale_i * ((sum_p term_i[p, t, c]) + bias_i[c]), float32. Terms are rows in the compute dtype or
// stacked float32 partial sums. With w: the norm on the sum as well, stream' = stream + w * out / rms(out), one
// workgroup per row (the sum is held in LDS between the two passes), the new stream also rounded to TY.
#define WS_MAX_TERMS 4
struct WsArgs {
  const void* term[WS_MAX_TERMS]; int dtype[WS_MAX_TERMS]; int parts[WS_MAX_TERMS]; int64_t part_stride[WS_MAX_TERMS];
  float scale[WS_MAX_TERMS]; const float* bias[WS_MAX_TERMS];
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
                               hipStream_t stream) {
  if (T == 0 || n == 0) return 0;
  ME_CHECK(count >= 1 && count <= WS_MAX_TERMS, "weighted_sum: 1..%d terms", WS_MAX_TERMS);
  WsArgs a;
  a.count = count; a.n = n;
  for (int i = 0; i < count; ++i) {
    ME_CHECK(parts[i] >= 1 && (dtypes[i] == ME_F32 || parts[i] == 1), "weighted_sum: partial sums are float32");
    a.term[i] = terms[i]; a.dtype[i] = dtypes[i]; a.parts[i] = parts[i]; a.part_stride[i] = part_strides[i];
    a.scale[i] = scales[i]; a.bias[i] = biases[i];
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
// With `unit`: q and k are first divided by sqrt(sum of their squares + unit_eps) per head; q is multiplied by q_scale.
// Every sum runs over n only, so a column p of the state never meets another: a wave takes 64 / RG columns of one head
// and a lane NR / RG of a column's rows, kept in registers for the whole walk; with RG > 1 the RG lanes of a column
// add their partial sums through the lanes' exchange. q, k and the decays of a token, which all columns share, are
// formed once per wave in LDS; the next token's raw values are on their way while the current token is worked on.
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

template <typename TX, int NR, int RG, int RULE>
__global__ void __launch_bounds__(64) decay_rows_kernel(DrArgs a) {
  constexpr int PC = 64 / RG;            // columns per wave
  constexpr int RL = NR / RG;            // rows per lane
  constexpr int PER = (NR + 63) / 64;    // rows of q, k and the decay that a lane forms for the wave
  __shared__ float sq[NR], sk[NR], sd[NR];
  const int lane = threadIdx.x;
  const int col_blocks = (a.P + PC - 1) / PC;
  const int cb = blockIdx.x % col_blocks;
  const int h = (blockIdx.x / col_blocks) % a.H;
  const int b = blockIdx.x / (col_blocks * a.H);
  const int g = h / (a.H / a.G);
  const int64_t first = a.cu[b];
  const int n_tok = (int)(a.cu[b + 1] - first);
  if (n_tok <= 0) return;
  const int p = cb * PC + lane % PC;
  const int r0 = (lane / PC) * RL;
  const bool live = p < a.P;
  const int pc = live ? p : a.P - 1;
  float* srow = a.state + (int64_t)a.slots[b] * a.state_stride + (int64_t)h * a.N * a.P;
  float S[RL];
#pragma unroll
  for (int i = 0; i < RL; ++i) S[i] = (r0 + i < a.N) ? srow[(int64_t)(r0 + i) * a.P + pc] : 0.f;

  const TX* qp = (const TX*)a.q; const TX* kp = (const TX*)a.k; const TX* vp = (const TX*)a.v;
  const TX* rp = (const TX*)a.raw; const TX* bp = (const TX*)a.beta;
  float base[PER], bonus[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int n = lane + 64 * i;
    const bool in = n < a.N && n < NR;
    base[i] = in ? a.base[h * a.N + n] : 0.f;
    bonus[i] = (RULE == 0 && in) ? a.bonus[h * a.N + n] : 0.f;
  }
  const float rate = RULE == 1 ? a.rate[h] : 0.f;
  float nq[PER], nk[PER], nr[PER], nv, nb = 0.f;
  auto fetch = [&](int t) {
    const int64_t row = first + t;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int n = lane + 64 * i;
      const bool in = n < a.N && n < NR;
      nq[i] = in ? to_f32<TX>(qp[row * a.q_stride + g * a.N + n]) : 0.f;
      nk[i] = in ? to_f32<TX>(kp[row * a.k_stride + g * a.N + n]) : 0.f;
      nr[i] = in ? to_f32<TX>(rp[row * a.raw_stride + h * a.N + n]) : 0.f;
    }
    nv = to_f32<TX>(vp[row * a.v_stride + h * a.P + pc]);
    if (RULE == 1) nb = to_f32<TX>(bp[row * a.beta_stride + h]);
  };
  fetch(0);
  for (int t = 0; t < n_tok; ++t) {
    // this token's shared values into LDS
    float qs = 0.f, ks = 0.f;
    if (a.unit) {
#pragma unroll
      for (int i = 0; i < PER; ++i) { qs += nq[i] * nq[i]; ks += nk[i] * nk[i]; }
      qs = wave_sum(qs); ks = wave_sum(ks);
      qs = a.q_scale / sqrtf(qs + a.unit_eps);
      ks = 1.0f / sqrtf(ks + a.unit_eps);
    } else {
      qs = a.q_scale; ks = 1.0f;
    }
    __syncthreads();                     // the token before has been read by every lane
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int n = lane + 64 * i;
      if (n < NR) {
        const bool in = n < a.N;
        sq[n] = nq[i] * qs;
        sk[n] = nk[i] * ks;
        float d;
        if (RULE == 0) d = expf(-expf(nr[i] + base[i]));
        else d = expf(-rate * hy_softplus(nr[i] + base[i]));
        sd[n] = in ? d : 1.0f;
      }
    }
    const float v = nv;
    const float beta = RULE == 1 ? hy_sigmoid(nb) : 0.f;
    float bon[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) bon[i] = bonus[i];
    __syncthreads();
    if (t + 1 < n_tok) fetch(t + 1);
    float y = 0.f;
    if (RULE == 0) {
#pragma unroll
      for (int i = 0; i < RL; ++i) {
        const int n = r0 + i;
        const float kv = sk[n] * v;
        // the bonus of row n: kept by lane n % 64 of the wave; every lane needs the rows of its own slice
        y += sq[n] * S[i];
        S[i] = sd[n] * S[i] + kv;
      }
    } else {
      float dot = 0.f;
#pragma unroll
      for (int i = 0; i < RL; ++i) {
        const int n = r0 + i;
        S[i] *= sd[n];
        dot += S[i] * sk[n];
      }
#pragma unroll
      for (int off = PC; off < 64; off <<= 1) dot += __shfl_xor(dot, off, ME_WAVE);
      const float u = beta * (v - dot);
#pragma unroll
      for (int i = 0; i < RL; ++i) {
        const int n = r0 + i;
        S[i] += sk[n] * u;
        y += S[i] * sq[n];
      }
    }
#pragma unroll
    for (int off = PC; off < 64; off <<= 1) y += __shfl_xor(y, off, ME_WAVE);
    if (RULE == 0) {
      // the current token's own term: v_p * sum_n q_n bonus_n k_n, one number per wave
      float own = 0.f;
#pragma unroll
      for (int i = 0; i < PER; ++i) { const int n = lane + 64 * i; if (n < NR) own += sq[n] * bon[i] * sk[n]; }
      own = wave_sum(own);
      y += own * v;
    }
    if (live && lane < PC) a.y[(first + t) * (int64_t)(a.H * a.P) + h * a.P + p] = y;
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < RL; ++i)
      if (r0 + i < a.N) srow[(int64_t)(r0 + i) * a.P + p] = S[i];
  }
}

template <typename TX, int NR, int RG>
static void launch_decay_rows(const DrArgs& a, int rule, int num_seqs, hipStream_t stream) {
  constexpr int PC = 64 / RG;
  const dim3 grid((unsigned)(num_seqs * a.H * ((a.P + PC - 1) / PC))), block(64);
  if (rule == 0) decay_rows_kernel<TX, NR, RG, 0><<<grid, block, 0, stream>>>(a);
  else decay_rows_kernel<TX, NR, RG, 1><<<grid, block, 0, stream>>>(a);
}

// row_groups: lanes that share a column (1 or 4); 4 gives four times the waves with a quarter of the rows each.
extern "C" int me_decay_rows_recurrence(const void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v, int64_t v_stride,
                                        const void* raw, int64_t raw_stride, const void* beta, int64_t beta_stride, int dtype,
                                        const float* base, const float* rate, const float* bonus, float* state, int64_t state_stride,
                                        const int32_t* slots, const int32_t* cu, float* y, int num_seqs, int H, int G, int N, int P,
                                        int rule, int unit, float unit_eps, float q_scale, int row_groups, hipStream_t stream) {
  if (num_seqs == 0) return 0;
  ME_CHECK(H >= 1 && G >= 1 && H % G == 0 && N >= 1 && N <= 256 && P >= 1, "decay_rows_recurrence: %d heads over %d groups, state %d x %d "
           "(up to 256 rows)", H, G, N, P);
  ME_CHECK(rule == 0 || rule == 1, "decay_rows_recurrence: unknown rule %d", rule);
  ME_CHECK(rule == 0 ? bonus != nullptr : (rate != nullptr && beta != nullptr), "decay_rows_recurrence: the rule's constants are missing");
  ME_CHECK(row_groups == 1 || row_groups == 4, "decay_rows_recurrence: 1 or 4 lanes to a column");
  ME_CHECK((int64_t)num_seqs * H * ((P + 15) / 16) <= 2147483647ll, "decay_rows_recurrence: too many workgroups");
  DrArgs a;
  a.q = q; a.k = k; a.v = v; a.raw = raw; a.beta = beta;
  a.q_stride = q_stride; a.k_stride = k_stride; a.v_stride = v_stride; a.raw_stride = raw_stride; a.beta_stride = beta_stride;
  a.base = base; a.rate = rate; a.bonus = bonus; a.state = state; a.state_stride = state_stride; a.slots = slots; a.cu = cu; a.y = y;
  a.H = H; a.G = G; a.N = N; a.P = P; a.unit = unit; a.unit_eps = unit_eps; a.q_scale = q_scale;
#define DR_NR(TX, NR)                                                           \
  do {                                                                          \
    if (row_groups == 4) launch_decay_rows<TX, NR, 4>(a, rule, num_seqs, stream); \
    else launch_decay_rows<TX, NR, 1>(a, rule, num_seqs, stream);               \
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
