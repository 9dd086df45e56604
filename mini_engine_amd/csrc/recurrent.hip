// Kernels of the mixers that keep a fixed-size state per request (linear attention with a decay, selective
// state-space layers), of blocks whose norms sit on the sublayers' outputs, and a few elementwise helpers.
//
//   add_rms_norm      stream += w * y / rms(y)                      (float32 stream, rounded copy for the next product)
//   activation        silu / squared relu of a row view
//   head_gate         o[t, h, :] *= sigmoid(g[t, h])
//   causal_conv       short causal convolution per channel over a request's tokens, continued from its state, + silu
//   recurrence        S_t = a_t S_(t-1) + b_t k_t v_t^T,  y_t = S_t^T q_t (+ skip v_t): float32 state per head
//   gated_rms_norm    unit root mean square per group with a gate in front of or behind it
//
// Everything that enters a recurrence is float32: step sizes, decays, their exponentials, the state, the sums.
#include "common.h"
#include <type_traits>

#define RC_MAX_PARTIALS 8

// ------------------------------------------------------------------ stream += w * y / rms(y)
// One workgroup per row. y may be `parts` stacked float32 partial sums, added here in a fixed order.
template <typename TX, typename TY>
__global__ void add_rms_norm_kernel(const TX* __restrict__ y, int parts, int64_t part_stride, const float* __restrict__ w,
                                    const float* __restrict__ stream_in, float* __restrict__ stream_out,
                                    TY* __restrict__ rounded, int n, float eps) {
  __shared__ float scratch[16];
  extern __shared__ float row[];
  const int64_t t = blockIdx.x;
  const TX* yr = y + t * n;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = 0.f;
    for (int p = 0; p < parts; ++p) v += to_f32<TX>(yr[p * part_stride + i]);
    row[i] = v;
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float s = stream_in[t * n + i] + row[i] * inv * w[i];
    stream_out[t * n + i] = s;
    if (rounded) rounded[t * n + i] = from_f32<TY>(s);
  }
}

// The same for rows of up to 4,096 elements in whole groups of 4: a thread owns one group, asks for every operand of it
// at once (each partial sum, the stream, the weight) and keeps it in registers: one trip to memory before the
// workgroup's sum and none behind it, which is what a step of a few rows waits for.
template <typename T> struct Group4;
template <> struct Group4<float> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <> struct Group4<bf16_t> {
  static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[4]) {
    const bf16x4 t = *reinterpret_cast<const bf16x4*>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = static_cast<float>(t[i]);
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[4]) {
    bf16x4 t;
#pragma unroll
    for (int i = 0; i < 4; ++i) t[i] = static_cast<bf16_t>(v[i]);
    *reinterpret_cast<bf16x4*>(p) = t;
  }
};

template <typename TX, typename TY>
__global__ void add_rms_norm_regs_kernel(const TX* __restrict__ y, int parts, int64_t part_stride, const float* __restrict__ w,
                                         const float* __restrict__ stream_in, float* __restrict__ stream_out,
                                         TY* __restrict__ rounded, int n, float eps) {
  __shared__ float scratch[16];
  const int64_t t = blockIdx.x;
  const int i = threadIdx.x * 4;
  const bool on = i < n;
  float part[RC_MAX_PARTIALS][4], sv[4] = {0.f, 0.f, 0.f, 0.f}, wv[4] = {0.f, 0.f, 0.f, 0.f}, yv[4] = {0.f, 0.f, 0.f, 0.f};
  if (on) {
#pragma unroll
    for (int p = 0; p < RC_MAX_PARTIALS; ++p)
      if (p < parts) Group4<TX>::load(y + p * part_stride + t * n + i, part[p]);
    Group4<float>::load(stream_in + t * n + i, sv);
    Group4<float>::load(w + i, wv);
#pragma unroll
    for (int p = 0; p < RC_MAX_PARTIALS; ++p)
      if (p < parts) {
#pragma unroll
        for (int e = 0; e < 4; ++e) yv[e] += part[p][e];
      }
  }
  float ss = yv[0] * yv[0] + yv[1] * yv[1] + yv[2] * yv[2] + yv[3] * yv[3];
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
  if (on) {
    float r[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) r[e] = sv[e] + yv[e] * inv * wv[e];
    Group4<float>::store(stream_out + t * n + i, r);
    if (rounded) Group4<TY>::store(rounded + t * n + i, r);
  }
}

template <typename TX, typename TY>
static void launch_add_rms_norm(const TX* y, int parts, int64_t part_stride, const float* w, const float* stream_in,
                                float* stream_out, TY* rounded, int64_t T, int n, float eps, hipStream_t stream) {
  const bool aligned = ((reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(stream_in) |
                         reinterpret_cast<uintptr_t>(stream_out) | reinterpret_cast<uintptr_t>(rounded)) % 16) == 0;
  if (n <= 4096 && n % 4 == 0 && aligned && (parts == 1 || part_stride % 4 == 0)) {
    const int threads = ((n / 4) + 63) / 64 * 64;
    add_rms_norm_regs_kernel<TX, TY><<<dim3((unsigned)T), dim3(threads), 0, stream>>>(y, parts, part_stride, w, stream_in,
                                                                                     stream_out, rounded, n, eps);
    return;
  }
  add_rms_norm_kernel<TX, TY><<<dim3((unsigned)T), dim3(n >= 1024 ? 256 : (n > 256 ? 128 : 64)), (size_t)n * sizeof(float), stream>>>(
      y, parts, part_stride, w, stream_in, stream_out, rounded, n, eps);
}

extern "C" int me_add_rms_norm(const void* y, int y_dtype, int parts, int64_t part_stride, const float* w,
                               const float* stream_in, float* stream_out, void* rounded, int64_t T, int n, float eps,
                               hipStream_t stream) {
  if (T == 0) return 0;
  ME_CHECK(n >= 1 && n <= 15360, "add_rms_norm: width %d outside 1..15360", n);
  ME_CHECK(parts >= 1 && parts <= RC_MAX_PARTIALS && (parts == 1 || y_dtype == ME_F32), "add_rms_norm: up to %d float32 partial sums", RC_MAX_PARTIALS);
  if (y_dtype == ME_F32)
    launch_add_rms_norm<float, float>((const float*)y, parts, part_stride, w, stream_in, stream_out, (float*)nullptr, T, n, eps, stream);
  else
    launch_add_rms_norm<bf16_t, bf16_t>((const bf16_t*)y, parts, part_stride, w, stream_in, stream_out, (bf16_t*)rounded, T, n, eps, stream);
  ME_LAUNCH_CHECK();
  return 0;
}

// float32 partial sums with a bfloat16 rounded copy (products split over K on the bfloat16 path)
extern "C" int me_add_rms_norm_partials(const float* y, int parts, int64_t part_stride, const float* w, const float* stream_in,
                                        float* stream_out, void* rounded, int64_t T, int n, float eps, hipStream_t stream) {
  if (T == 0) return 0;
  ME_CHECK(n >= 1 && n <= 15360, "add_rms_norm: width %d outside 1..15360", n);
  ME_CHECK(parts >= 1 && parts <= RC_MAX_PARTIALS, "add_rms_norm: up to %d partial sums", RC_MAX_PARTIALS);
  launch_add_rms_norm<float, bf16_t>(y, parts, part_stride, w, stream_in, stream_out, (bf16_t*)rounded, T, n, eps, stream);
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ activations
__device__ __forceinline__ float sigmoid_f(float v) { return 1.0f / (1.0f + expf(-v)); }
__device__ __forceinline__ float silu_f(float v) { return v * sigmoid_f(v); }

template <typename TX, int KIND>
__global__ void activation_kernel(const TX* __restrict__ x, int64_t x_stride, TX* __restrict__ out, int64_t T, int n) {
  const int64_t total = T * n;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / n;
    const float v = to_f32<TX>(x[t * x_stride + (i - t * n)]);
    float r;
    if (KIND == 0) r = silu_f(v);
    else if (KIND == 2) r = tanhf(v);
    else if (KIND == 3) r = 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));     // gelu, tanh form
    else { const float p = fmaxf(v, 0.f); r = p * p; }
    out[i] = from_f32<TX>(r);
  }
}

extern "C" int me_activation(const void* x, int64_t x_stride, void* out, int dtype, int kind, int64_t T, int n, hipStream_t stream) {
  if (T == 0 || n == 0) return 0;
  ME_CHECK(kind >= 0 && kind <= 3, "activation: unknown kind %d", kind);
  const int64_t total = T * n;
  const dim3 grid((unsigned)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535)), block(256);
#define ACT(TX, K) activation_kernel<TX, K><<<grid, block, 0, stream>>>((const TX*)x, x_stride, (TX*)out, T, n)
  if (dtype == ME_F32) { if (kind == 0) ACT(float, 0); else if (kind == 1) ACT(float, 1); else if (kind == 2) ACT(float, 2); else ACT(float, 3); }
  else { if (kind == 0) ACT(bf16_t, 0); else if (kind == 1) ACT(bf16_t, 1); else if (kind == 2) ACT(bf16_t, 2); else ACT(bf16_t, 3); }
#undef ACT
  ME_LAUNCH_CHECK();
  return 0;
}

// o[t, h, :] *= sigmoid(g[t, h]); o contiguous [T, H * D], g a view with token stride g_stride.
template <typename TX>
__global__ void head_gate_kernel(TX* __restrict__ o, const TX* __restrict__ g, int64_t g_stride, int64_t T, int H, int D) {
  const int64_t total = T * H * D;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t th = i / D;
    const int64_t t = th / H;
    const int h = (int)(th - t * H);
    o[i] = from_f32<TX>(to_f32<TX>(o[i]) * sigmoid_f(to_f32<TX>(g[t * g_stride + h])));
  }
}

extern "C" int me_head_gate(void* o, const void* g, int64_t g_stride, int dtype, int64_t T, int H, int D, hipStream_t stream) {
  if (T == 0) return 0;
  const int64_t total = T * H * D;
  const dim3 grid((unsigned)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535)), block(256);
  if (dtype == ME_F32) head_gate_kernel<float><<<grid, block, 0, stream>>>((float*)o, (const float*)g, g_stride, T, H, D);
  else head_gate_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t*)o, (const bf16_t*)g, g_stride, T, H, D);
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ short causal convolution + silu
// out[t, c] = silu(bias[c] + sum_j w[c, j] * in(t - (taps - 1) + j)); the inputs before the step's first token of a
// request come from its state row: per channel taps - 1 values, oldest first. One thread per (token, channel).
#define CONV_MAX_TAPS 16

#define CONV_TOKENS 32       // tokens of one request that a thread walks

// One thread per (request, block of CONV_TOKENS tokens, channel): it walks its tokens in order with the last taps - 1
// inputs in registers, so every input is read once and the step's metadata once per workgroup.
template <typename TX>
__global__ void causal_conv_kernel(const TX* __restrict__ x, int64_t x_stride, const float* __restrict__ w,
                                   const float* __restrict__ bias, const float* __restrict__ state, int64_t state_stride,
                                   const int32_t* __restrict__ slots, const int32_t* __restrict__ cu,
                                   TX* __restrict__ out, int C, int taps, int blocks_per_seq) {
  const int b = blockIdx.x / blocks_per_seq, blk = blockIdx.x - b * blocks_per_seq;
  const int64_t first = cu[b];
  const int n = (int)(cu[b + 1] - first);
  const int l0 = blk * CONV_TOKENS;
  if (l0 >= n) return;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int l1 = l0 + CONV_TOKENS < n ? l0 + CONV_TOKENS : n;
  const float* held = state + (int64_t)slots[b] * state_stride + (int64_t)c * (taps - 1);
  float wv[CONV_MAX_TAPS], seen[CONV_MAX_TAPS];
  for (int j = 0; j < taps; ++j) wv[j] = w[(int64_t)c * taps + j];
  // seen[j], j < taps - 1: the inputs at local positions l0 - (taps - 1) + j
  for (int j = 0; j < taps - 1; ++j) {
    const int src = l0 - (taps - 1) + j;
    seen[j] = src >= 0 ? to_f32<TX>(x[(first + src) * x_stride + c]) : held[src + taps - 1];
  }
  const float bc = bias != nullptr ? bias[c] : 0.f;
  for (int l = l0; l < l1; ++l) {
    const float now = to_f32<TX>(x[(first + l) * x_stride + c]);
    float acc = bc + wv[taps - 1] * now;
    for (int j = 0; j < taps - 1; ++j) acc += wv[j] * seen[j];
    out[(first + l) * C + c] = from_f32<TX>(silu_f(acc));
    for (int j = 0; j + 1 < taps - 1; ++j) seen[j] = seen[j + 1];
    if (taps > 1) seen[taps - 2] = now;
  }
}

// The state moves on: per (request, channel) the last taps - 1 inputs of (held inputs, this step's inputs).
template <typename TX>
__global__ void causal_conv_state_kernel(const TX* __restrict__ x, int64_t x_stride, float* __restrict__ state,
                                         int64_t state_stride, const int32_t* __restrict__ slots,
                                         const int32_t* __restrict__ cu, int C, int taps) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int64_t first = cu[b];
  const int n = (int)(cu[b + 1] - first);
  if (n <= 0) return;
  float* held = state + (int64_t)slots[b] * state_stride + (int64_t)c * (taps - 1);
  float next[CONV_MAX_TAPS];
  for (int s = 0; s < taps - 1; ++s) {
    const int src = n - (taps - 1) + s;
    next[s] = src >= 0 ? to_f32<TX>(x[(first + src) * x_stride + c]) : held[src + taps - 1];
  }
  for (int s = 0; s < taps - 1; ++s) held[s] = next[s];
}

// A step of single tokens (token b is request b's): output and state in one pass, one thread per (request, channel).
template <typename TX>
__global__ void causal_conv_step_kernel(const TX* __restrict__ x, int64_t x_stride, const float* __restrict__ w,
                                        const float* __restrict__ bias, float* __restrict__ state, int64_t state_stride,
                                        const int32_t* __restrict__ slots, TX* __restrict__ out, int C, int taps) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  float* held = state + (int64_t)slots[b] * state_stride + (int64_t)c * (taps - 1);
  const float now = to_f32<TX>(x[(int64_t)b * x_stride + c]);
  float seen[CONV_MAX_TAPS];
  for (int s = 0; s < taps - 1; ++s) seen[s] = held[s];
  float acc = (bias != nullptr ? bias[c] : 0.f) + w[(int64_t)c * taps + taps - 1] * now;
  for (int s = 0; s < taps - 1; ++s) acc += w[(int64_t)c * taps + s] * seen[s];
  out[(int64_t)b * C + c] = from_f32<TX>(silu_f(acc));
  for (int s = 0; s + 1 < taps - 1; ++s) held[s] = seen[s + 1];
  if (taps > 1) held[taps - 2] = now;
}

// max_tokens: no request brings more tokens than this.
extern "C" int me_causal_conv(const void* x, int64_t x_stride, int dtype, const float* w, const float* bias, float* state,
                              int64_t state_stride, const int32_t* slots, const int32_t* cu, int max_tokens,
                              void* out, int64_t T, int num_seqs, int C, int taps, hipStream_t stream) {
  if (T == 0 || C == 0) return 0;
  ME_CHECK(taps >= 1 && taps <= CONV_MAX_TAPS, "causal_conv: %d taps outside 1..%d", taps, CONV_MAX_TAPS);
  const dim3 block(C >= 256 ? 256 : 64);
  ME_CHECK(T <= 2147483647ll && num_seqs <= 65535 && (C + block.x - 1) / block.x <= 65535,
           "causal_conv: too many tokens, requests or channels for one launch");
  const dim3 grid((unsigned)T, (C + block.x - 1) / block.x);
  if (T == num_seqs) {                     // every request brings one token
    if (dtype == ME_F32)
      causal_conv_step_kernel<float><<<grid, block, 0, stream>>>((const float*)x, x_stride, w, bias, state, state_stride, slots,
                                                                 (float*)out, C, taps);
    else
      causal_conv_step_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)x, x_stride, w, bias, state, state_stride, slots,
                                                                  (bf16_t*)out, C, taps);
    ME_LAUNCH_CHECK();
    return 0;
  }
  const int blocks_per_seq = (max_tokens + CONV_TOKENS - 1) / CONV_TOKENS;
  ME_CHECK(max_tokens >= 1 && (int64_t)num_seqs * blocks_per_seq <= 2147483647ll, "causal_conv: bad token bound %d", max_tokens);
  const dim3 wgrid((unsigned)(num_seqs * blocks_per_seq), (C + block.x - 1) / block.x);
  if (dtype == ME_F32)
    causal_conv_kernel<float><<<wgrid, block, 0, stream>>>((const float*)x, x_stride, w, bias, state, state_stride, slots, cu,
                                                           (float*)out, C, taps, blocks_per_seq);
  else
    causal_conv_kernel<bf16_t><<<wgrid, block, 0, stream>>>((const bf16_t*)x, x_stride, w, bias, state, state_stride, slots, cu,
                                                            (bf16_t*)out, C, taps, blocks_per_seq);
  ME_LAUNCH_CHECK();
  if (taps > 1) {
    const dim3 sgrid((C + block.x - 1) / block.x, num_seqs);
    if (dtype == ME_F32)
      causal_conv_state_kernel<float><<<sgrid, block, 0, stream>>>((const float*)x, x_stride, state, state_stride, slots, cu, C, taps);
    else
      causal_conv_state_kernel<bf16_t><<<sgrid, block, 0, stream>>>((const bf16_t*)x, x_stride, state, state_stride, slots, cu, C, taps);
    ME_LAUNCH_CHECK();
  }
  return 0;
}

// ------------------------------------------------------------------ the recurrence
// One wave per (request, one or two heads, 64 or 128 columns of P, NT rows of N, span of tokens). A lane keeps CL
// columns of its NT state rows in registers (CL = 1, or 2: two blocks of 64 columns of one head, or the same 64
// columns of two heads that share k and q); the tokens' k and q slices, decays and input scales pass through LDS 8
// tokens at a time and are read from there by all lanes at once, while the next 8 tokens' values are already on
// their way into registers. Products and sums are float32 in the order of the tokens.
//
// A launch is one of three passes (PASS):
//   0  whole: a request's tokens from its state row, y written, the state row written back
//   1  spans, first pass: every span of `span` tokens from zero; its end state and the product of its decays go to
//      scratch (no y)
//   2  spans, last pass: every span from the state that precedes it (the carry kernel has put it into scratch), y
//      written; the span that ends the request's tokens writes the state row
// Between 1 and 2 the carry kernel walks a request's spans in order: in[0] = state row, in[c + 1] = decay[c] * in[c]
// + end[c].
struct RecArgs {
  const void* q; const void* k; const void* v;      // [T, G * N], [T, G * N], [T, H * P] views, token strides below
  int64_t q_stride, k_stride, v_stride;
  const void* dt; int64_t dt_stride;                // [T, H] view, or null: fixed decays
  const float* decay;                               // [H] fixed decays (dt null)
  const float* dt_bias; const float* rate; const float* skip;   // [H] each (skip may be null)
  float* state; int64_t state_stride;               // [slots, H * N * P] view
  const int32_t* slots; const int32_t* cu;
  float* y; int64_t y_slice_stride;                 // [slices of N, T, H * P] float32
  float* span_state; float* span_decay;             // scratch: [requests, spans, H, N, P], [requests, spans, H]
  int H, G, N, P, span, max_spans;
  int silu;                                         // q, k and v pass silu on their way in
};

#define REC_TB 8

// HPB heads and PPB blocks of 64 columns per wave; CL = HPB * PPB columns per lane.
template <typename TX, int NT, int PASS, int HPB, int PPB>
__global__ void __launch_bounds__(64) recurrence_kernel(RecArgs a) {
  constexpr int CL = HPB * PPB;
  constexpr int KR = REC_TB * NT / 64;               // k (and q) values a lane carries to LDS per batch of tokens
  using Cell = std::conditional_t<PASS == 1, float, float2>;       // the first pass of spans reads no q
  __shared__ Cell skq[REC_TB][NT];
  __shared__ float sa[HPB][REC_TB], sb[HPB][REC_TB];
  const int lane = threadIdx.x;
  const int heads_blocks = a.H / HPB;
  const int b = blockIdx.x / heads_blocks, h0 = (blockIdx.x - b * heads_blocks) * HPB;
  const int g = h0 / (a.H / a.G);
  const int slices = (a.N + NT - 1) / NT;
  const int slice = blockIdx.z % slices;
  const int c = blockIdx.z / slices;                  // span index (0 in pass 0)
  const int n0 = slice * NT;
  const int64_t first = a.cu[b], end_all = a.cu[b + 1];
  int64_t t0 = first, t1 = end_all;
  if (PASS != 0) {
    t0 = first + (int64_t)c * a.span;
    t1 = t0 + a.span < end_all ? t0 + a.span : end_all;
  }
  if (t0 >= t1) return;
  int head[CL], p[CL];
  bool on[CL];
#pragma unroll
  for (int j = 0; j < CL; ++j) {
    head[j] = h0 + (HPB == 2 ? j : 0);
    p[j] = (blockIdx.y * PPB + (PPB == 2 ? j : 0)) * 64 + lane;
    on[j] = p[j] < a.P;
    if (!on[j]) p[j] = 0;
  }
  const TX* qp = (const TX*)a.q + (int64_t)g * a.N + n0;
  const TX* kp = (const TX*)a.k + (int64_t)g * a.N + n0;
  const bool silu = a.silu != 0;

  // what a lane fetches for a batch of tokens
  float kreg[KR], qreg[KR], vreg[CL][REC_TB], areg = 1.f, breg = 0.f;
  // every load is unconditional, from an address clamped into the span and the slice; what lies outside becomes zero
  // afterwards (a load behind a branch would make the wave wait for each one before it asks for the next)
  const int n_last = a.N - 1 - n0;
  auto fetch = [&](int64_t tb) {
    const int nt = (int)(t1 - tb < REC_TB ? t1 - tb : REC_TB);
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      const int i = lane + r * 64, tt = i / NT, nn = i - tt * NT;
      const bool have = tt < nt && nn <= n_last;
      const int64_t at = tb + (tt < nt ? tt : nt - 1);
      const int col = nn <= n_last ? nn : n_last;
      const float kk = to_f32<TX>(kp[at * a.k_stride + col]);
      kreg[r] = have ? kk : 0.f;
      if (PASS != 1) {
        const float qq = to_f32<TX>(qp[at * a.q_stride + col]);
        qreg[r] = have ? qq : 0.f;
      }
    }
#pragma unroll
    for (int j = 0; j < CL; ++j)
#pragma unroll
      for (int tt = 0; tt < REC_TB; ++tt) {
        const float x = to_f32<TX>(((const TX*)a.v)[(tb + (tt < nt ? tt : nt - 1)) * a.v_stride + (int64_t)head[j] * a.P + p[j]]);
        vreg[j][tt] = (tt < nt && on[j]) ? x : 0.f;
      }
    {
      const int sub = lane < HPB * REC_TB ? lane : 0;
      const int hh = h0 + sub / REC_TB, tt = sub % REC_TB;
      const int64_t at = tb + (tt < nt ? tt : nt - 1);
      if (a.dt) {
        const float z = to_f32<TX>(((const TX*)a.dt)[at * a.dt_stride + hh]) + a.dt_bias[hh];
        const float step = z > 20.f ? z : log1pf(expf(z));
        areg = expf(-a.rate[hh] * step);
        breg = step;
      } else {
        areg = a.decay[hh];
        breg = 1.f;
      }
      if (tt >= nt) { areg = 1.f; breg = 0.f; }
    }
  };

  fetch(t0);
  float S[CL][NT];
  float* row[CL];
  float* span_row[CL];
#pragma unroll
  for (int j = 0; j < CL; ++j) {
    row[j] = a.state + (int64_t)a.slots[b] * a.state_stride + (int64_t)head[j] * a.N * a.P;
    span_row[j] = PASS == 0 ? nullptr : a.span_state + (((int64_t)b * a.max_spans + c) * a.H + head[j]) * (int64_t)a.N * a.P;
    if (PASS == 1) {
#pragma unroll
      for (int i = 0; i < NT; ++i) S[j][i] = 0.f;
    } else {
      const float* from = PASS == 0 ? row[j] : span_row[j];
#pragma unroll
      for (int i = 0; i < NT; ++i) {
        const float held = from[(int64_t)(n0 + (i <= n_last ? i : n_last)) * a.P + p[j]];
        S[j][i] = (on[j] && i <= n_last) ? held : 0.f;
      }
    }
  }
  float skip[CL];
#pragma unroll
  for (int j = 0; j < CL; ++j) skip[j] = a.skip ? a.skip[head[j]] : 0.f;
  float total_decay[HPB];
#pragma unroll
  for (int j = 0; j < HPB; ++j) total_decay[j] = 1.f;

  for (int64_t tb = t0; tb < t1; tb += REC_TB) {
    const int nt = (int)(t1 - tb < REC_TB ? t1 - tb : REC_TB);
    __syncthreads();                                  // the batch before has been read
    float vv[CL][REC_TB];
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      const int i = lane + r * 64, tt = i / NT, nn = i - tt * NT;
      float kk = kreg[r], qq = PASS != 1 ? qreg[r] : 0.f;
      if (silu) { kk = silu_f(kk); qq = silu_f(qq); }
      if constexpr (PASS == 1) skq[tt][nn] = kk;
      else skq[tt][nn] = make_float2(kk, qq);
    }
    if (lane < HPB * REC_TB) { sa[lane / REC_TB][lane % REC_TB] = areg; sb[lane / REC_TB][lane % REC_TB] = breg; }
#pragma unroll
    for (int j = 0; j < CL; ++j)
#pragma unroll
      for (int tt = 0; tt < REC_TB; ++tt) vv[j][tt] = silu ? silu_f(vreg[j][tt]) : vreg[j][tt];
    if (tb + REC_TB < t1) fetch(tb + REC_TB);         // the next batch travels while this one is computed
    __syncthreads();
#pragma unroll
    for (int tt = 0; tt < REC_TB; ++tt) {
      if (tt >= nt) break;
      float da[CL], bv[CL], acc[CL];
#pragma unroll
      for (int j = 0; j < CL; ++j) {
        const int hj = HPB == 2 ? j : 0;
        da[j] = sa[hj][tt];
        bv[j] = sb[hj][tt] * vv[j][tt];
        acc[j] = 0.f;
      }
#pragma unroll
      for (int i = 0; i < NT; ++i) {
        if constexpr (PASS == 1) {
          const float kk = skq[tt][i];
#pragma unroll
          for (int j = 0; j < CL; ++j) S[j][i] = da[j] * S[j][i] + kk * bv[j];
        } else {
          const float2 kq = skq[tt][i];
#pragma unroll
          for (int j = 0; j < CL; ++j) {
            S[j][i] = da[j] * S[j][i] + kq.x * bv[j];
            acc[j] += S[j][i] * kq.y;
          }
        }
      }
      if (PASS == 1) {
#pragma unroll
        for (int j = 0; j < HPB; ++j) total_decay[j] *= sa[j][tt];
      } else {
#pragma unroll
        for (int j = 0; j < CL; ++j)
          if (on[j]) {
            if (slice == 0) acc[j] += skip[j] * vv[j][tt];
            a.y[slice * a.y_slice_stride + (tb + tt) * ((int64_t)a.H * a.P) + (int64_t)head[j] * a.P + p[j]] = acc[j];
          }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < CL; ++j) {
    if (PASS == 1) {
      if (on[j])
#pragma unroll
        for (int i = 0; i < NT; ++i)
          if (n0 + i < a.N) span_row[j][(int64_t)(n0 + i) * a.P + p[j]] = S[j][i];
    } else if (on[j] && t1 == end_all) {
#pragma unroll
      for (int i = 0; i < NT; ++i)
        if (n0 + i < a.N) row[j][(int64_t)(n0 + i) * a.P + p[j]] = S[j][i];
    }
  }
  if (PASS == 1 && lane == 0 && blockIdx.y == 0 && slice == 0)
#pragma unroll
    for (int j = 0; j < HPB; ++j) a.span_decay[((int64_t)b * a.max_spans + c) * a.H + h0 + j] = total_decay[j];
}

// in[0] = the request's state row; in[c + 1] = decay[c] * in[c] + end[c]. scratch[c] holds end[c] on entry and in[c] on
// exit. One thread per state element, the spans in order.
__global__ void recurrence_carry_kernel(RecArgs a) {
  const int b = blockIdx.y;
  const int64_t per_head = (int64_t)a.N * a.P, per_req = per_head * a.H;
  const int64_t e = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (e >= per_req) return;
  const int h = (int)(e / per_head);
  const int64_t len = a.cu[b + 1] - a.cu[b];
  const int spans = (int)((len + a.span - 1) / a.span);
  if (spans <= 0) return;
  float carry = a.state[(int64_t)a.slots[b] * a.state_stride + e];
  for (int c = 0; c < spans; ++c) {
    float* at = a.span_state + ((int64_t)b * a.max_spans + c) * per_req + e;
    const float ended = *at;
    *at = carry;
    carry = a.span_decay[((int64_t)b * a.max_spans + c) * a.H + h] * carry + ended;
  }
}

// A step of single tokens (token b is request b's): the state streams through once. One workgroup of four waves per
// (request, head, 64 columns); each wave takes a quarter of the N rows, eight rows' loads in flight at a time, and
// the four partial outputs meet in LDS. Nothing of the state stays in registers, so many waves fit a SIMD, which is
// what a kernel that only waits for memory needs.
template <typename TX>
__global__ void __launch_bounds__(256) recurrence_step_kernel(RecArgs a) {
  extern __shared__ float kq[];                       // k[N], q[N], then 4 x 64 partial outputs
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int b = blockIdx.x / a.H, h = blockIdx.x - b * a.H;
  const int g = h / (a.H / a.G);
  const int p = blockIdx.y * 64 + lane;
  const bool on = p < a.P;
  const int pc = on ? p : 0;
  float* sk = kq;
  float* sq = kq + a.N;
  float* part = kq + 2 * a.N;
  const bool silu = a.silu != 0;
  for (int i = threadIdx.x; i < a.N; i += 256) {
    float kk = to_f32<TX>(((const TX*)a.k)[(int64_t)b * a.k_stride + (int64_t)g * a.N + i]);
    float qq = to_f32<TX>(((const TX*)a.q)[(int64_t)b * a.q_stride + (int64_t)g * a.N + i]);
    if (silu) { kk = silu_f(kk); qq = silu_f(qq); }
    sk[i] = kk; sq[i] = qq;
  }
  float vv = to_f32<TX>(((const TX*)a.v)[(int64_t)b * a.v_stride + (int64_t)h * a.P + pc]);
  if (silu) vv = silu_f(vv);
  float da, db;
  if (a.dt) {
    const float z = to_f32<TX>(((const TX*)a.dt)[(int64_t)b * a.dt_stride + h]) + a.dt_bias[h];
    const float step = z > 20.f ? z : log1pf(expf(z));
    da = expf(-a.rate[h] * step);
    db = step;
  } else {
    da = a.decay[h];
    db = 1.f;
  }
  const float bv = db * vv;
  float* row = a.state + (int64_t)a.slots[b] * a.state_stride + (int64_t)h * a.N * a.P + pc;
  const int per = (a.N + 3) / 4;
  const int r0 = wave * per, r1 = r0 + per < a.N ? r0 + per : a.N;
  __syncthreads();
  float acc = 0.f;
  for (int r = r0; r < r1; r += 8) {
    float held[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) held[i] = row[(int64_t)(r + i < r1 ? r + i : r1 - 1) * a.P];
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (r + i < r1) {
        const float next = da * held[i] + sk[r + i] * bv;
        acc += next * sq[r + i];
        if (on) row[(int64_t)(r + i) * a.P] = next;
      }
  }
  part[wave * 64 + lane] = acc;
  __syncthreads();
  if (wave == 0 && on) {
    float y = part[lane] + part[64 + lane] + part[128 + lane] + part[192 + lane];
    if (a.skip) y += a.skip[h] * vv;
    a.y[(int64_t)b * a.H * a.P + (int64_t)h * a.P + p] = y;
  }
}

template <typename TX, int NT, int HPB, int PPB>
static int launch_recurrence(RecArgs& a, int num_seqs, int spans, hipStream_t stream) {
  const int slices = (a.N + NT - 1) / NT;
  const dim3 block(64);
  const unsigned pblocks = (a.P + 64 * PPB - 1) / (64 * PPB);
  if (spans <= 1) {
    recurrence_kernel<TX, NT, 0, HPB, PPB><<<dim3(num_seqs * (a.H / HPB), pblocks, slices), block, 0, stream>>>(a);
    ME_LAUNCH_CHECK();
    return 0;
  }
  const dim3 grid(num_seqs * (a.H / HPB), pblocks, slices * spans);
  recurrence_kernel<TX, NT, 1, HPB, PPB><<<grid, block, 0, stream>>>(a);
  ME_LAUNCH_CHECK();
  const int64_t per_req = (int64_t)a.H * a.N * a.P;
  recurrence_carry_kernel<<<dim3((unsigned)((per_req + 255) / 256), num_seqs), dim3(256), 0, stream>>>(a);
  ME_LAUNCH_CHECK();
  recurrence_kernel<TX, NT, 2, HPB, PPB><<<grid, block, 0, stream>>>(a);
  ME_LAUNCH_CHECK();
  return 0;
}

// spans <= 1: every request's tokens in one pass. Otherwise the tokens are cut into spans of `span` tokens that run
// side by side (at most `spans` per request), and scratch holds spans * H * N * P + spans * H floats per request.
// columns: 1, or 2: a lane keeps two columns of the state (two blocks of 64 columns of one head where P > 64, else
// the same columns of two neighbouring heads of one group, which needs an even number of heads per group).
extern "C" int me_linear_recurrence(const void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v,
                                    int64_t v_stride, int dtype, const void* dt, int64_t dt_stride, const float* decay,
                                    const float* dt_bias, const float* rate, const float* skip, float* state,
                                    int64_t state_stride, const int32_t* slots, const int32_t* cu, float* y,
                                    int64_t y_slice_stride, int num_seqs, int H, int G, int N, int P, int rows_per_wave,
                                    int columns, int silu, int span, int spans, float* scratch, hipStream_t stream) {
  if (num_seqs == 0) return 0;
  ME_CHECK(H >= 1 && G >= 1 && H % G == 0 && N >= 1 && P >= 1, "recurrence: bad sizes H=%d G=%d N=%d P=%d", H, G, N, P);
  ME_CHECK((dt != nullptr) != (decay != nullptr), "recurrence: give fixed decays or step sizes, not both");
  ME_CHECK(dt == nullptr || (dt_bias && rate), "recurrence: step sizes need their bias and rates");
  ME_CHECK((int64_t)num_seqs * H <= 2147483647ll, "recurrence: too many (request, head) pairs");
  ME_CHECK(spans <= 1 || (span >= 1 && scratch != nullptr), "recurrence: spans need a length and scratch");
  const bool two_heads = columns == 2 && P <= 64;
  ME_CHECK(columns == 1 || columns == 2, "recurrence: 1 or 2 columns per lane");
  ME_CHECK(!two_heads || (H / G) % 2 == 0, "recurrence: two heads per wave need an even number of heads per group");
  RecArgs a;
  a.q = q; a.k = k; a.v = v; a.q_stride = q_stride; a.k_stride = k_stride; a.v_stride = v_stride;
  a.dt = dt; a.dt_stride = dt_stride; a.decay = decay; a.dt_bias = dt_bias; a.rate = rate; a.skip = skip;
  a.state = state; a.state_stride = state_stride; a.slots = slots; a.cu = cu; a.y = y; a.y_slice_stride = y_slice_stride;
  a.H = H; a.G = G; a.N = N; a.P = P; a.span = span > 0 ? span : 1; a.max_spans = spans > 1 ? spans : 1;
  a.silu = silu;
  a.span_state = scratch;
  a.span_decay = scratch ? scratch + (int64_t)num_seqs * a.max_spans * H * N * P : nullptr;
  if (rows_per_wave == 0) {                // a step of single tokens: one pass over the state, one output
    ME_CHECK((int64_t)(2 * N + 256) * 4 <= 64 * 1024 && (P + 63) / 64 <= 65535, "recurrence: a state of %d rows does not fit the step kernel", N);
    const dim3 grid(num_seqs * H, (P + 63) / 64);
    const size_t lds = (size_t)(2 * N + 256) * sizeof(float);
    if (dtype == ME_F32) recurrence_step_kernel<float><<<grid, dim3(256), lds, stream>>>(a);
    else recurrence_step_kernel<bf16_t><<<grid, dim3(256), lds, stream>>>(a);
    ME_LAUNCH_CHECK();
    return 0;
  }
  const int slices = (N + rows_per_wave - 1) / rows_per_wave;
  ME_CHECK((int64_t)slices * a.max_spans <= 65535, "recurrence: too many slices and spans for one launch");
#define REC_NT(TX, NT)                                                                               \
  do {                                                                                               \
    if (columns == 1) return launch_recurrence<TX, NT, 1, 1>(a, num_seqs, spans, stream);            \
    if (two_heads) return launch_recurrence<TX, NT, 2, 1>(a, num_seqs, spans, stream);               \
    return launch_recurrence<TX, NT, 1, 2>(a, num_seqs, spans, stream);                              \
  } while (0)
#define REC(TX)                                                                              \
  switch (rows_per_wave) {                                                                   \
    case 16: REC_NT(TX, 16);                                                                 \
    case 32: REC_NT(TX, 32);                                                                 \
    case 48: REC_NT(TX, 48);                                                                 \
    case 64: REC_NT(TX, 64);                                                                 \
    default: ME_CHECK(false, "recurrence: %d state rows per wave is not one of 16, 32, 48, 64", rows_per_wave); \
  }
  if (dtype == ME_F32) { REC(float) } else { REC(bf16_t) }
#undef REC
#undef REC_NT
  return 0;
}

// ------------------------------------------------------------------ unit rms per group, with a gate
// KIND 0: u = y * silu(gate); out = u / rms_group(u) * w.    KIND 1: out = y / rms_group(y) * w * sigmoid(gate).
// KIND 2: out = y / rms_group(y) * w * silu(gate).
// y: `parts` stacked float32 slices [parts, T, n], added here. One workgroup per row.
template <typename TX, int KIND>
__global__ void gated_rms_norm_kernel(const float* __restrict__ y, int parts, int64_t part_stride, const TX* __restrict__ gate,
                                      int64_t gate_stride, const float* __restrict__ w, TX* __restrict__ out, int n,
                                      int groups, float eps) {
  __shared__ float scratch[16];
  extern __shared__ float row[];
  const int64_t t = blockIdx.x;
  const int per = n / groups;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = 0.f;
    for (int p = 0; p < parts; ++p) v += y[p * part_stride + t * n + i];
    if (KIND == 0) v *= silu_f(to_f32<TX>(gate[t * gate_stride + i]));
    row[i] = v;
  }
  __syncthreads();
  for (int g = 0; g < groups; ++g) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < per; i += blockDim.x) { const float v = row[g * per + i]; ss += v * v; }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)per + eps);
    for (int i = threadIdx.x; i < per; i += blockDim.x) {
      const int j = g * per + i;
      float r = row[j] * inv * w[j];
      if (KIND == 1) r *= sigmoid_f(to_f32<TX>(gate[t * gate_stride + j]));
      if (KIND == 2) r *= silu_f(to_f32<TX>(gate[t * gate_stride + j]));
      out[t * n + j] = from_f32<TX>(r);
    }
  }
}

extern "C" int me_gated_rms_norm(const float* y, int parts, int64_t part_stride, const void* gate, int64_t gate_stride,
                                 int dtype, const float* w, void* out, int64_t T, int n, int groups, int kind, float eps,
                                 hipStream_t stream) {
  if (T == 0) return 0;
  ME_CHECK(n >= 1 && n <= 15360 && groups >= 1 && n % groups == 0, "gated_rms_norm: width %d, %d groups", n, groups);
  ME_CHECK(parts >= 1 && parts <= 64 && kind >= 0 && kind <= 2, "gated_rms_norm: bad slice count or kind");
  const dim3 grid((unsigned)T), block(n >= 1024 ? 256 : (n > 256 ? 128 : 64));
  const size_t lds = (size_t)n * sizeof(float);
#define GN(TX, K) gated_rms_norm_kernel<TX, K><<<grid, block, lds, stream>>>(y, parts, part_stride, (const TX*)gate, gate_stride, w, (TX*)out, n, groups, eps)
  if (dtype == ME_F32) { if (kind == 0) GN(float, 0); else if (kind == 1) GN(float, 1); else GN(float, 2); }
  else { if (kind == 0) GN(bf16_t, 0); else if (kind == 1) GN(bf16_t, 1); else GN(bf16_t, 2); }
#undef GN
  ME_LAUNCH_CHECK();
  return 0;
}
