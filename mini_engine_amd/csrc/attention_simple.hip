// Paged causal attention, the exact and slow form: one workgroup per (query token, head),
// scalar float32 arithmetic throughout. It is the float32 path of the engine and takes any
// head size, page size and head grouping.
//
// Formulas as in the reference's pure-torch paged path (layers/attention.py:21-40): key j of
// the request is kept iff j <= position of the query (and j < context length); scores are
// scale * q.k; softmax over kept keys; output = sum p_j v_j. A window w additionally keeps
// only j > position - w (not in the reference). Three further options: `keep_first` n keeps the keys j < n visible
// behind a window; `softcap` c > 0 bends every score to c * tanh(score / c) before the softmax; `sinks` (one float per
// query head) adds exp(sink) to the softmax's denominator, a term without key or value.
//
// Keys are processed in chunks whose boundaries are multiples of the chunk size counted from
// position 0 of the request, so the order of every sum for a given token is the same however
// the request was cut into steps or batched.
#include "common.h"

#define AS_THREADS 256

template <typename T>
__global__ void __launch_bounds__(AS_THREADS)
attn_simple_kernel(const T* __restrict__ q, int64_t q_stride, T* __restrict__ out, int64_t out_stride,
                   const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                   const int32_t* __restrict__ block_tables, int bt_stride,
                   const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ positions,
                   const int32_t* __restrict__ context_lens, int Hq, int Hkv, int D, int page, float scale,
                   int window, int keep_first, float softcap, const float* __restrict__ sinks) {
  extern __shared__ float lds[];
  float* qs = lds;                 // D
  float* sc = lds + D;             // AS_THREADS scores / probabilities
  __shared__ float red[16];

  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  const int kvh = h / (Hq / Hkv);
  const int b = seq_of_token[t];
  const int pos = positions[t];
  const int32_t* bt = block_tables + (int64_t)b * bt_stride;
  const int tid = threadIdx.x;

  for (int d = tid; d < D; d += AS_THREADS) qs[d] = to_f32<T>(q[t * q_stride + (int64_t)h * D + d]);
  __syncthreads();

  // keys [lo, hi): up to the query's own position, never past the request's context (a padding
  // row has context 0 and sees nothing)
  const int hi = min(pos + 1, context_lens[b]);
  // window > 0: the last `window` keys; window < 0: a block mask, only the keys of the query's own block of -window positions
  const int lo = window > 0 ? max(0, pos - window + 1) : (window < 0 ? pos - pos % (-window) : 0);
  // behind a window the first keep_first keys stay visible: the chunks walk [0, kept) and then [lo, hi)
  const int kept = (window > 0 && keep_first > 0) ? min(min(keep_first, lo), hi) : 0;
  float m = -INFINITY, l = 0.f;
  // thread d < D owns output channel d (two channels per thread when D > AS_THREADS)
  float acc0 = 0.f, acc1 = 0.f;

  const int first_c0 = (lo / AS_THREADS) * AS_THREADS;
  for (int c0 = kept > 0 ? 0 : first_c0; c0 < hi; c0 += AS_THREADS) {
    if (c0 >= kept && c0 < first_c0) { c0 = first_c0 - AS_THREADS; continue; }   // nothing visible between the kept keys and the window
    const int j = c0 + tid;
    float s = -INFINITY;
    bool keep = (j >= lo || j < kept) && j < hi;
    if (keep) {
      const int64_t pg = bt[j / page];
      keep = pg >= 0;                        // a page that is not held is never dereferenced
      if (keep) {
        const int off = j % page;
        const T* kr = k_cache + ((pg * Hkv + kvh) * (int64_t)page + off) * D;
        float dot = 0.f;
        for (int d = 0; d < D; ++d) dot += qs[d] * to_f32<T>(kr[d]);
        s = dot * scale;
        if (softcap > 0.f) s = softcap * tanhf(s / softcap);
      }
    }
    // chunk max
    float cm = wave_max(s);
    __syncthreads();
    if ((tid & 63) == 0) red[tid >> 6] = cm;
    __syncthreads();
    cm = red[0];
    for (int w = 1; w < AS_THREADS / 64; ++w) cm = fmaxf(cm, red[w]);
    const float m_new = fmaxf(m, cm);
    const float p = (keep && m_new > -INFINITY) ? expf(s - m_new) : 0.f;
    sc[tid] = p;
    float ps = wave_sum(p);
    __syncthreads();
    if ((tid & 63) == 0) red[8 + (tid >> 6)] = ps;
    __syncthreads();
    ps = 0.f;
    for (int w = 0; w < AS_THREADS / 64; ++w) ps += red[8 + w];
    const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);   // m finite implies m_new finite
    l = l * alpha + ps;
    m = m_new;
    acc0 *= alpha;
    acc1 *= alpha;
    const int jb = kept > 0 ? c0 : max(c0, lo), je = min(c0 + AS_THREADS, hi);
    for (int dd = 0; dd < 2; ++dd) {
      const int d = tid + dd * AS_THREADS;
      if (d < D) {
        float a = 0.f;
        for (int jj = jb; jj < je; ++jj) {
          if (jj < lo && jj >= kept) continue;   // its probability is 0 and its page may have been given back
          const int64_t pg = bt[jj / page];
          if (pg < 0) continue;                // its probability is 0
          const int off = jj % page;
          a += sc[jj - c0] * to_f32<T>(v_cache[((pg * Hkv + kvh) * (int64_t)D + d) * page + off]);
        }
        if (dd == 0) acc0 += a; else acc1 += a;
      }
    }
    __syncthreads();
  }
  if (sinks != nullptr) {
    // the sink joins the denominator under the same running maximum; alone (no visible key) it leaves an output of zero
    const float sk = sinks[h];
    const float m_new = fmaxf(m, sk);
    const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
    l = l * alpha + expf(sk - m_new);
    acc0 *= alpha;
    acc1 *= alpha;
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
  if (tid < D) out[t * out_stride + (int64_t)h * D + tid] = from_f32<T>(acc0 * inv);
  if (tid + AS_THREADS < D) out[t * out_stride + (int64_t)h * D + tid + AS_THREADS] = from_f32<T>(acc1 * inv);
}

extern "C" int me_attn_simple(const void* q, int64_t q_stride, void* out, int64_t out_stride, int dtype,
                              const void* k_cache, const void* v_cache, const int32_t* block_tables,
                              int bt_stride, const int32_t* seq_of_token, const int32_t* positions,
                              const int32_t* context_lens, int64_t num_tokens, int Hq, int Hkv, int D, int page, float scale, int window,
                              int keep_first, float softcap, const float* sinks, hipStream_t stream) {
  if (num_tokens == 0) return 0;
  ME_CHECK(Hq >= 1 && Hkv >= 1 && Hq % Hkv == 0, "attention: %d query heads are not a multiple of %d key heads", Hq, Hkv);
  ME_CHECK(D >= 1 && D <= 2 * AS_THREADS, "attention (float32 path): head_dim %d outside 1..%d", D, 2 * AS_THREADS);
  ME_CHECK(page >= 1, "attention: bad page size");
  ME_CHECK(keep_first >= 0 && softcap >= 0.f, "attention: keep_first and softcap must not be negative");
  dim3 grid(num_tokens, Hq), block(AS_THREADS);
  size_t lds = (size_t)(D + AS_THREADS) * sizeof(float);
  if (dtype == ME_F32)
    attn_simple_kernel<float><<<grid, block, lds, stream>>>(
        (const float*)q, q_stride, (float*)out, out_stride, (const float*)k_cache, (const float*)v_cache,
        block_tables, bt_stride, seq_of_token, positions, context_lens, Hq, Hkv, D, page, scale, window, keep_first, softcap, sinks);
  else if (dtype == ME_BF16)
    attn_simple_kernel<bf16_t><<<grid, block, lds, stream>>>(
        (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache,
        block_tables, bt_stride, seq_of_token, positions, context_lens, Hq, Hkv, D, page, scale, window, keep_first, softcap, sinks);
  else
    ME_CHECK(false, "attention: bad dtype code %d", dtype);
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ further terms of a softmax that another kernel has formed
// The matrix-core kernels attend over one contiguous range of keys. What a mask or a softmax has beyond that joins here:
// the keys at positions below keep_first that a window has left behind, and a sink per head. out holds the other
// kernel's normalised result and lse the natural logarithm of its denominator (-inf: it saw no key). With
// (m2, l2, acc2) the kept keys' maximum, sum and weighted values, sk the sink and M the largest of lse, m2, sk:
//   out <- (out e^(lse - M) + acc2 e^(m2 - M)) / (e^(lse - M) + l2 e^(m2 - M) + e^(sk - M)).
// One wave per (token, head); for the scores four neighbouring lanes share a key, sixteen keys at a time; for the values a
// lane takes the channels lane, lane + 64, ...
#define AT_MAX_D 512
template <typename T>
__global__ void __launch_bounds__(64)
attn_tail_kernel(const T* __restrict__ q, int64_t q_stride, T* __restrict__ out, int64_t out_stride, const float* __restrict__ lse,
                 const T* __restrict__ k_cache, const T* __restrict__ v_cache, const int32_t* __restrict__ block_tables, int bt_stride,
                 const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ positions,
                 const int32_t* __restrict__ context_lens, int Hq, int Hkv, int D, int page, float scale, int window,
                 int keep_first, float softcap, const float* __restrict__ sinks) {
  __shared__ float qs[AT_MAX_D];
  __shared__ float sc[64];
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const int kvh = h / (Hq / Hkv);
  const int b = seq_of_token[t];
  const int pos = positions[t];
  const int32_t* bt = block_tables + (int64_t)b * bt_stride;
  const int hi = min(pos + 1, context_lens[b]);
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int kept = (window > 0 && keep_first > 0) ? min(min(keep_first, lo), hi) : 0;
  float m2 = -INFINITY, l2 = 0.f;
  float acc[AT_MAX_D / 64];
#pragma unroll
  for (int i = 0; i < AT_MAX_D / 64; ++i) acc[i] = 0.f;
  if (kept > 0) {
    for (int d = lane; d < D; d += 64) qs[d] = to_f32<T>(q[t * q_stride + (int64_t)h * D + d]);
    __syncthreads();
    // sixteen keys at a time: four neighbouring lanes share a key, each with every fourth of the head's dimensions
    const int part = lane & 3;
    for (int c0 = 0; c0 < kept; c0 += 16) {
      const int j = c0 + (lane >> 2);
      float s = -INFINITY;
      int64_t pg = -1;
      if (j < kept) pg = bt[j / page];
      float dot = 0.f;
      if (pg >= 0) {
        const T* kr = k_cache + ((pg * Hkv + kvh) * (int64_t)page + j % page) * D;
        for (int d = part; d < D; d += 4) dot += qs[d] * to_f32<T>(kr[d]);      // neighbours read neighbouring words
      }
      dot += __shfl_xor(dot, 1, ME_WAVE);
      dot += __shfl_xor(dot, 2, ME_WAVE);
      if (pg >= 0) {
        s = dot * scale;
        if (softcap > 0.f) s = softcap * tanhf(s / softcap);
      }
      const float m_new = fmaxf(m2, wave_max(s));
      const float p = (s > -INFINITY) ? expf(s - m_new) : 0.f;
      const float alpha = (m2 == -INFINITY) ? 0.f : expf(m2 - m_new);
      l2 = l2 * alpha + wave_sum(part == 0 ? p : 0.f);
      m2 = m_new;
      __syncthreads();
      if (part == 0) sc[lane >> 2] = p;
      __syncthreads();
      const int je = min(16, kept - c0);
#pragma unroll
      for (int i = 0; i < AT_MAX_D / 64; ++i) {
        const int d = lane + 64 * i;
        if (d < D) {
          float a = 0.f;
          for (int jj = 0; jj < je; ++jj) {
            const int64_t vp = bt[(c0 + jj) / page];
            if (vp < 0) continue;
            a += sc[jj] * to_f32<T>(v_cache[((vp * Hkv + kvh) * (int64_t)D + d) * page + (c0 + jj) % page]);
          }
          acc[i] = acc[i] * alpha + a;
        }
      }
    }
  }
  const float l1 = lse[t * Hq + h];
  const float sk = sinks != nullptr ? sinks[h] : -INFINITY;
  const float M = fmaxf(fmaxf(l1, m2), sk);
  float w1 = 0.f, w2 = 0.f, ws = 0.f;
  if (M > -INFINITY) {
    w1 = l1 > -INFINITY ? expf(l1 - M) : 0.f;
    w2 = m2 > -INFINITY ? expf(m2 - M) : 0.f;
    ws = sk > -INFINITY ? expf(sk - M) : 0.f;
  }
  const float denom = w1 + w2 * l2 + ws;
  const float inv = denom > 0.f ? 1.f / denom : 0.f;
#pragma unroll
  for (int i = 0; i < AT_MAX_D / 64; ++i) {
    const int d = lane + 64 * i;
    if (d < D) {
      T* at = out + t * out_stride + (int64_t)h * D + d;
      *at = from_f32<T>((to_f32<T>(*at) * w1 + acc[i] * w2) * inv);
    }
  }
}

extern "C" int me_attn_tail(const void* q, int64_t q_stride, void* out, int64_t out_stride, const float* lse, int dtype,
                            const void* k_cache, const void* v_cache, const int32_t* block_tables, int bt_stride,
                            const int32_t* seq_of_token, const int32_t* positions, const int32_t* context_lens,
                            int64_t num_tokens, int Hq, int Hkv, int D, int page, float scale, int window, int keep_first,
                            float softcap, const float* sinks, hipStream_t stream) {
  if (num_tokens == 0) return 0;
  ME_CHECK(Hq >= 1 && Hkv >= 1 && Hq % Hkv == 0 && Hq <= 65535, "attention tail: %d query heads over %d key heads", Hq, Hkv);
  ME_CHECK(D >= 1 && D <= AT_MAX_D && page >= 1 && keep_first >= 0 && softcap >= 0.f, "attention tail: head size 1..%d", AT_MAX_D);
  ME_CHECK(lse != nullptr && num_tokens <= 2147483647ll, "attention tail: the other kernel's denominators are missing");
  dim3 grid((unsigned)num_tokens, Hq), block(64);
  if (dtype == ME_F32)
    attn_tail_kernel<float><<<grid, block, 0, stream>>>((const float*)q, q_stride, (float*)out, out_stride, lse, (const float*)k_cache,
        (const float*)v_cache, block_tables, bt_stride, seq_of_token, positions, context_lens, Hq, Hkv, D, page, scale, window,
        keep_first, softcap, sinks);
  else
    attn_tail_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, lse, (const bf16_t*)k_cache,
        (const bf16_t*)v_cache, block_tables, bt_stride, seq_of_token, positions, context_lens, Hq, Hkv, D, page, scale, window,
        keep_first, softcap, sinks);
  ME_LAUNCH_CHECK();
  return 0;
}
