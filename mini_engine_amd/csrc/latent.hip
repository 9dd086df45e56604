// Attention over a latent that all heads share (one normed vector and one rotated key part per token in the cache).
//
//   latent_prepare   per token, from the rows of the layer's packed product: the latent's RMS norm with its weight, the
//                    rotation of the shared key part and of every query head's rotating part (adjacent pairs), and
//                    the write into the pages: the key page takes [latent | rotated part | zeros], the value page
//                    (transposed inside a page) the latent. One pass, norm and angles in float32.
//   heads_linear     y[t, h, :] = W[h] x[t, h, :]: a product per head (queries into the latent's space, attention
//                    results out of it). bfloat16, v_mfma_f32_16x16x32_bf16: for few tokens a wave per 16 x 16 tile with
//                    operands straight from memory; from 256 tokens on a workgroup keeps its head's matrix in LDS and
//                    every token row is read once; float32, and sizes whose rows are no whole 16-byte pieces: one
//                    thread per output, a sequential sum over K.
//
// Attention itself is the paged kernels' business: with the queries carried into the latent's space, every head
// reads the same keys ([latent | rotated part]) and values (the latent), a single key/value head of size
// rank + rotating dimensions.
#include "common.h"

struct LatentArgs {
  const void* rows; int64_t row_stride;       // the packed product's rows
  int q_off, kv_off;                          // where the query heads and the latent's rows begin in a row
  int H, dn, dr, R, D;                        // heads, unrotated and rotating query dimensions, rank, the kernels' head size
  const float* norm_w; float eps;             // the latent's norm
  const float* table; int64_t table_rows;     // [positions, dr / 2, 2] cos, sin
  const int32_t* positions; const int32_t* slots;
  void* qa; int64_t qa_stride;                // [T, H * D]: the rotated part goes to slots R .. R + dr of every head
  void* k_cache; void* v_cache; int page;     // [pages, 1, page, D], [pages, 1, D, page]; null: this layer writes none
};

template <typename TX>
__global__ void __launch_bounds__(128) latent_prepare_kernel(LatentArgs a) {
  __shared__ float scratch[16];
  const int64_t t = blockIdx.x;
  const TX* row = (const TX*)a.rows + t * a.row_stride;
  int pos = a.positions[t];
  if (pos < 0 || pos >= a.table_rows) pos = 0;              // the host bounds positions; never read outside the table
  const float* cs = a.table + (int64_t)pos * a.dr;          // dr / 2 pairs of (cos, sin)
  const int half = a.dr / 2;
  // the queries' rotating parts, and zeros behind them
  TX* qa = (TX*)a.qa + t * a.qa_stride;
  for (int i = threadIdx.x; i < a.H * half; i += blockDim.x) {
    const int h = i / half, j = i - h * half;
    const TX* q = row + a.q_off + (int64_t)h * (a.dn + a.dr) + a.dn + 2 * j;
    const float u = to_f32<TX>(q[0]), v = to_f32<TX>(q[1]);
    const float c = cs[2 * j], s = cs[2 * j + 1];
    TX* o = qa + (int64_t)h * a.D + a.R + 2 * j;
    o[0] = from_f32<TX>(u * c - v * s);
    o[1] = from_f32<TX>(v * c + u * s);
  }
  const int pad = a.D - a.R - a.dr;
  for (int i = threadIdx.x; i < a.H * pad; i += blockDim.x) {
    const int h = i / pad, j = i - h * pad;
    qa[(int64_t)h * a.D + a.R + a.dr + j] = from_f32<TX>(0.f);
  }
  if (a.k_cache == nullptr) return;
  const int slot = a.slots[t];
  const TX* kv = row + a.kv_off;
  float ss = 0.f;
  for (int i = threadIdx.x; i < a.R; i += blockDim.x) { const float v = to_f32<TX>(kv[i]); ss += v * v; }
  ss = block_sum(ss, scratch);
  if (slot < 0) return;
  const float inv = 1.0f / sqrtf(ss / (float)a.R + a.eps);
  const int64_t pg = slot / a.page, off = slot - pg * a.page;
  TX* kp = (TX*)a.k_cache + (pg * a.page + off) * a.D;
  TX* vp = (TX*)a.v_cache + pg * a.D * a.page + off;
  for (int i = threadIdx.x; i < a.R; i += blockDim.x) {
    const TX c = from_f32<TX>(to_f32<TX>(kv[i]) * inv * a.norm_w[i]);
    kp[i] = c;
    vp[(int64_t)i * a.page] = c;
  }
  for (int j = threadIdx.x; j < half; j += blockDim.x) {
    const float u = to_f32<TX>(kv[a.R + 2 * j]), v = to_f32<TX>(kv[a.R + 2 * j + 1]);
    const float c = cs[2 * j], s = cs[2 * j + 1];
    kp[a.R + 2 * j] = from_f32<TX>(u * c - v * s);
    kp[a.R + 2 * j + 1] = from_f32<TX>(v * c + u * s);
  }
  for (int i = a.R + a.dr + threadIdx.x; i < a.D; i += blockDim.x) kp[i] = from_f32<TX>(0.f);
  for (int i = a.R + threadIdx.x; i < a.D; i += blockDim.x) vp[(int64_t)i * a.page] = from_f32<TX>(0.f);
}

extern "C" int me_latent_prepare(const void* rows, int64_t row_stride, int dtype, int q_off, int kv_off, int H, int dn, int dr, int R,
                                 int D, const float* norm_w, float eps, const float* table, int64_t table_rows,
                                 const int32_t* positions, const int32_t* slots, void* qa, int64_t qa_stride, void* k_cache,
                                 void* v_cache, int page, int64_t T, hipStream_t stream) {
  if (T == 0) return 0;
  ME_CHECK(H >= 1 && dn >= 0 && dr >= 0 && dr % 2 == 0 && R >= 1 && D >= R + dr, "latent_prepare: %d heads of %d + %d, rank %d, head size %d",
           H, dn, dr, R, D);
  ME_CHECK(T <= 2147483647ll && (k_cache == nullptr || (v_cache && slots && norm_w && page >= 1)), "latent_prepare: missing operand");
  ME_CHECK(dr == 0 || (table != nullptr && table_rows >= 1), "latent_prepare: the rotation needs its table");
  LatentArgs a;
  a.rows = rows; a.row_stride = row_stride; a.q_off = q_off; a.kv_off = kv_off; a.H = H; a.dn = dn; a.dr = dr; a.R = R; a.D = D;
  a.norm_w = norm_w; a.eps = eps; a.table = table; a.table_rows = table_rows; a.positions = positions; a.slots = slots;
  a.qa = qa; a.qa_stride = qa_stride; a.k_cache = k_cache; a.v_cache = v_cache; a.page = page;
  if (dtype == ME_F32) latent_prepare_kernel<float><<<dim3((unsigned)T), dim3(128), 0, stream>>>(a);
  else latent_prepare_kernel<bf16_t><<<dim3((unsigned)T), dim3(128), 0, stream>>>(a);
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ a product per head
struct HeadsArgs {
  const void* x; int64_t x_stride, x_head;     // x[t, h, k] at t * x_stride + h * x_head + k
  const void* w;                               // [H, N, K]
  void* y; int64_t y_stride, y_head;           // y[t, h, n] at t * y_stride + h * y_head + n
  int64_t T; int H, N, K;
};

// A wave per tile of 16 tokens x 16 features of one head; a workgroup's 4 waves take 64 tokens. Lane (n, g) brings 8
// neighbours of K from weight row n and from token row n, from 8 g on, 32 of K a step.
__global__ void __launch_bounds__(256) heads_linear_mfma_kernel(HeadsArgs a) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = lane & 15, g = lane >> 4;
  const int h = blockIdx.z;
  const int n0 = blockIdx.x * 16;
  const int64_t t0 = (int64_t)blockIdx.y * 64 + wave * 16;
  if (t0 >= a.T) return;
  const int64_t t = min(t0 + n, a.T - 1);
  const int f = min(n0 + n, a.N - 1);
  const bf16_t* xr = (const bf16_t*)a.x + t * a.x_stride + (int64_t)h * a.x_head + 8 * g;
  const bf16_t* wr = (const bf16_t*)a.w + ((int64_t)h * a.N + f) * a.K + 8 * g;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < a.K; k0 += 128) {
    bf16x8 wa[4], xb[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + 32 * i;
      const bool in = k + 8 * g < a.K;
      wa[i] = in ? *reinterpret_cast<const bf16x8*>(wr + k) : zero;
      xb[i] = in ? *reinterpret_cast<const bf16x8*>(xr + k) : zero;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[i], xb[i], acc, 0, 0, 0);
  }
  // lane (n, g): features n0 + 4 g .. + 3 of token t0 + n
  if (t0 + n >= a.T) return;
  bf16_t* o = (bf16_t*)a.y + (t0 + n) * a.y_stride + (int64_t)h * a.y_head;
#pragma unroll
  for (int q = 0; q < 4; ++q)
    if (n0 + 4 * g + q < a.N) o[n0 + 4 * g + q] = from_f32<bf16_t>(acc[q]);
}

// Many tokens: a workgroup stages its head's whole matrix in LDS once (rows 16 bytes apart from a multiple of 128 bytes, so
// that the 16 lanes of an operand read touch all banks) and its 4 waves walk tiles of 16 tokens: a wave holds its tile's
// rows in registers (K32 steps of 32) and runs down the matrix's rows 16 at a time. Tokens are read once and results written
// once, 8 bytes a lane where the output's strides allow.
template <int K32>
__global__ void __launch_bounds__(256) heads_linear_lds_kernel(HeadsArgs a, int tiles_per_wave, int wide_stores) {
  extern __shared__ __align__(16) unsigned char hl_lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = lane & 15, g = lane >> 4;
  const int h = blockIdx.y;
  const int KP = (a.K + 31) / 32 * 32, ld = KP + 8, NP = (a.N + 15) / 16 * 16, pieces = KP / 8;
  const bf16_t* w = (const bf16_t*)a.w + (int64_t)h * a.N * a.K;
  for (int i = threadIdx.x; i < NP * pieces; i += 256) {
    const int r = i / pieces, c = i - r * pieces;
    const uint4 v = (r < a.N && 8 * c < a.K) ? *reinterpret_cast<const uint4*>(w + (int64_t)r * a.K + 8 * c) : make_uint4(0u, 0u, 0u, 0u);
    *reinterpret_cast<uint4*>(hl_lds + ((size_t)r * ld + 8 * c) * 2) = v;
  }
  __syncthreads();
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  const int64_t first = ((int64_t)blockIdx.x * 4 + wave) * 16 * tiles_per_wave;
  for (int tile = 0; tile < tiles_per_wave; ++tile) {
    const int64_t t0 = first + 16 * tile;
    if (t0 >= a.T) break;
    const int64_t t = min(t0 + n, a.T - 1);
    const bf16_t* xr = (const bf16_t*)a.x + t * a.x_stride + (int64_t)h * a.x_head + 8 * g;
    bf16x8 xb[K32];
#pragma unroll
    for (int i = 0; i < K32; ++i) xb[i] = 32 * i + 8 * g < a.K ? *reinterpret_cast<const bf16x8*>(xr + 32 * i) : zero;
    bf16_t* o = (bf16_t*)a.y + (t0 + n) * a.y_stride + (int64_t)h * a.y_head;
    for (int n0 = 0; n0 < a.N; n0 += 16) {
      const unsigned char* wr = hl_lds + ((size_t)(n0 + n) * ld + 8 * g) * 2;
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < K32; ++i)
        if (32 * i < KP) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(wr + 64 * i), xb[i], acc, 0, 0, 0);
      if (t0 + n >= a.T) continue;
      const int f = n0 + 4 * g;
      if (wide_stores && f + 3 < a.N) {
        bf16x4 r;
#pragma unroll
        for (int q = 0; q < 4; ++q) r[q] = from_f32<bf16_t>(acc[q]);
        *reinterpret_cast<bf16x4*>(o + f) = r;
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (f + q < a.N) o[f + q] = from_f32<bf16_t>(acc[q]);
      }
    }
  }
}

template <int K32>
static int launch_heads_lds(const HeadsArgs& a, size_t lds, int tiles, int wide, hipStream_t stream) {
  static bool allowed = false;
  if (!allowed && lds > 48 * 1024) {
    hipError_t err = hipFuncSetAttribute((const void*)heads_linear_lds_kernel<K32>, hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
    ME_CHECK(err == hipSuccess, "heads_linear: cannot get %zu bytes of LDS: %s", lds, hipGetErrorString(err));
    allowed = true;
  }
  const int64_t per_group = 64ll * tiles;
  heads_linear_lds_kernel<K32><<<dim3((unsigned)((a.T + per_group - 1) / per_group), (unsigned)a.H), dim3(256), lds, stream>>>(a, tiles, wide);
  ME_LAUNCH_CHECK();
  return 0;
}

template <typename TX>
__global__ void __launch_bounds__(256) heads_linear_simple_kernel(HeadsArgs a) {
  const int64_t total = a.T * a.H * a.N;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t th = i / a.N;
    const int n = (int)(i - th * a.N);
    const int64_t t = th / a.H;
    const int h = (int)(th - t * a.H);
    const TX* xr = (const TX*)a.x + t * a.x_stride + (int64_t)h * a.x_head;
    const TX* wr = (const TX*)a.w + ((int64_t)h * a.N + n) * a.K;
    float s = 0.f;
    for (int k = 0; k < a.K; ++k) s = fmaf(to_f32<TX>(xr[k]), to_f32<TX>(wr[k]), s);
    ((TX*)a.y)[t * a.y_stride + (int64_t)h * a.y_head + n] = from_f32<TX>(s);
  }
}

extern "C" int me_heads_linear(const void* x, int64_t x_stride, int64_t x_head, const void* w, void* y, int64_t y_stride, int64_t y_head,
                               int dtype, int64_t T, int H, int N, int K, hipStream_t stream) {
  if (T == 0) return 0;
  ME_CHECK(H >= 1 && H <= 65535 && N >= 1 && K >= 1 && T <= 2147483647ll, "heads_linear: %d heads of %d x %d", H, N, K);
  HeadsArgs a;
  a.x = x; a.x_stride = x_stride; a.x_head = x_head; a.w = w; a.y = y; a.y_stride = y_stride; a.y_head = y_head;
  a.T = T; a.H = H; a.N = N; a.K = K;
  const bool pieces = K % 8 == 0 && x_stride % 8 == 0 && x_head % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(w) % 16 == 0;
  const size_t lds = (size_t)((N + 15) / 16 * 16) * ((K + 31) / 32 * 32 + 8) * 2;
  if (dtype == ME_BF16 && pieces && T >= 256 && K <= 512 && lds <= 128 * 1024) {
    // as many tokens to a workgroup as still leave about a thousand workgroups
    const int tiles = T * H <= 65536 ? 1 : (T * H <= 131072 ? 2 : 4);
    const int wide = y_stride % 4 == 0 && y_head % 4 == 0 && reinterpret_cast<uintptr_t>(y) % 8 == 0;
    if (K <= 128) return launch_heads_lds<4>(a, lds, tiles, wide, stream);
    if (K <= 256) return launch_heads_lds<8>(a, lds, tiles, wide, stream);
    return launch_heads_lds<16>(a, lds, tiles, wide, stream);
  }
  if (dtype == ME_BF16 && pieces && (T + 63) / 64 <= 65535) {
    heads_linear_mfma_kernel<<<dim3((unsigned)((N + 15) / 16), (unsigned)((T + 63) / 64), (unsigned)H), dim3(256), 0, stream>>>(a);
  } else {
    const int64_t total = T * H * N;
    const dim3 grid((unsigned)((total + 255) / 256 < 1048576 ? (total + 255) / 256 : 1048576));
    if (dtype == ME_F32) heads_linear_simple_kernel<float><<<grid, dim3(256), 0, stream>>>(a);
    else heads_linear_simple_kernel<bf16_t><<<grid, dim3(256), 0, stream>>>(a);
  }
  ME_LAUNCH_CHECK();
  return 0;
}
