// A feed-forward made of many small gated experts of which every token uses a few.
//
//   moe_route      float32 router: logits = W x; scores = their softmax over all experts or their sigmoids; the choice
//                  goes by the scores plus an optional correction per expert; optionally only the experts of the best
//                  groups of neighbours stay eligible (a group scores as the sum of its `group_top` largest choice
//                  scores); the `top` largest are chosen; their weights are the scores without the correction, times
//                  a constant, divided by their sum or not (`RouteRule`)
//   moe_sort       (token, choice) pairs ordered by expert, cut into tiles of 16, 64 or 128 rows that never span two experts
//   moe_gate_up    per tile: silu(x W_gate^T) * (x W_up^T) of the tile's expert, token rows gathered through the order;
//                  or, for experts without a gate, relu(x W_up^T)^2
//   moe_down       per tile: the expert's down product, times the pair's weight, into float32 [top, T, hidden]: one
//                  partial sum per choice, for a consumer that adds them (no atomics: the result does not depend on
//                  what else is in the batch)
//   moe_*_simple   the same two products with one wave per output element: the float32 path, and sizes whose rows
//                  are not whole 16-byte pieces
//
// The tiled kernels: a workgroup owns 64 pair rows x 64 weight rows (or 128 x 128), its 4 waves 2 x 2 sub-tiles
// (v_mfma_f32_16x16x32_bf16, weight rows as the A operand, so that a lane holds 4 consecutive features of one
// row); K is walked 64 at a time through two LDS buffers, the next step's 16-byte pieces on their way in registers
// while the current one is multiplied; piece c of row R lies at c ^ (R >> 1 & 7), so that the 16 lanes of an operand
// read touch 16 different bank groups. Pieces beyond K are zeros, so K needs to be a multiple of 8 only.
#include "common.h"

#define MOE_MAX_EXPERTS 1024
#define MOE_TM 64

// ------------------------------------------------------------------ router
// Orders a wave's LDS writes before its later reads of them by other lanes.
__device__ __forceinline__ void wave_settle() {
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

__device__ __forceinline__ void wave_argmax(float& v, int& i) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(v, off, ME_WAVE);
    const int oi = __shfl_xor(i, off, ME_WAVE);
    if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
  }
}

// Four neighbours of a row as float32 (one 8- or 16-byte read).
__device__ __forceinline__ void load4(const float* p, float (&v)[4]) {
  const float4 t = *reinterpret_cast<const float4*>(p);
  v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void load4(const bf16_t* p, float (&v)[4]) {
  const bf16x4 t = *reinterpret_cast<const bf16x4*>(p);
#pragma unroll
  for (int j = 0; j < 4; ++j) v[j] = static_cast<float>(t[j]);
}

// Router logits: a workgroup of 4 waves takes `tokens_per_group` tokens (their rows wait in LDS) and `experts_per_group`
// experts, a wave every fourth of them; a lane walks K in steps of 64 and the wave adds up. float32 [T, E] out.
template <typename TX>
__global__ void __launch_bounds__(256)
moe_logits_kernel(const TX* __restrict__ x, int64_t ldx, const float* __restrict__ w, int64_t T, int n, int E,
                  int tokens_per_group, int experts_per_group, float* __restrict__ logits) {
  extern __shared__ __align__(16) unsigned char route_lds[];
  const int TT = tokens_per_group;
  TX* xs = reinterpret_cast<TX*>(route_lds);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t t0 = (int64_t)blockIdx.x * TT;
  const int live = (int)min((int64_t)TT, T - t0);
  constexpr int EPV = 16 / sizeof(TX);       // elements of a 16-byte piece
  if (n % EPV == 0 && ldx % EPV == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0) {
    const int pieces = n / EPV;
    for (int i = threadIdx.x; i < TT * pieces; i += blockDim.x) {
      const int tt = i / pieces, c = i - tt * pieces;
      const uint4 v = tt < live ? *reinterpret_cast<const uint4*>(x + (t0 + tt) * ldx + c * EPV) : make_uint4(0u, 0u, 0u, 0u);
      *reinterpret_cast<uint4*>(xs + tt * n + c * EPV) = v;
    }
  } else {
    for (int i = threadIdx.x; i < TT * n; i += blockDim.x) {
      const int tt = i / n, k = i - tt * n;
      xs[i] = tt < live ? x[(t0 + tt) * ldx + k] : from_f32<TX>(0.f);
    }
  }
  __syncthreads();
  const int e0 = blockIdx.y * experts_per_group, e1 = min(E, e0 + experts_per_group);
  const bool vec = (n & 3) == 0;           // rows in whole groups of 4: a lane takes 4 neighbours at a time
  for (int e = e0 + wave; e < e1; e += 4) {
    float acc[8];
#pragma unroll
    for (int tt = 0; tt < 8; ++tt) acc[tt] = 0.f;
    const float* we = w + (int64_t)e * n;
    if (vec) {
#pragma unroll 4
      for (int k = lane * 4; k < n; k += 256) {
        const float4 wv = *reinterpret_cast<const float4*>(we + k);
#pragma unroll
        for (int tt = 0; tt < 8; ++tt)
          if (tt < TT) {
            float xv[4];
            load4(xs + tt * n + k, xv);
            acc[tt] += wv.x * xv[0] + wv.y * xv[1] + wv.z * xv[2] + wv.w * xv[3];
          }
      }
    } else {
      for (int k = lane; k < n; k += 64) {
        const float wv = we[k];
#pragma unroll
        for (int tt = 0; tt < 8; ++tt)
          if (tt < TT) acc[tt] += wv * to_f32<TX>(xs[tt * n + k]);
      }
    }
#pragma unroll
    for (int tt = 0; tt < 8; ++tt)
      if (tt < TT) {
        const float s = wave_sum(acc[tt]);
        if (lane == 0 && tt < live) logits[(t0 + tt) * E + e] = s;
      }
  }
}

// How scores become a choice. sigmoid 0: softmax over all experts, 1: a sigmoid per expert. correction: float32 [E]
// added to the scores for the choice only (null: none). A group's score is the sum of its group_top largest choice
// scores. normalise: the chosen scores are divided by their sum. The weights are multiplied by scale.
struct RouteRule {
  int top, group_count, group_keep, group_top, sigmoid, normalise;
  float scale;
  const float* correction;
};

// The choice for one token by one wave. s, m: E floats of LDS each, gs: group_count floats. Choice scores may be
// negative: an expert out of the race is at -inf, a group that is kept at +inf.
__device__ __forceinline__ void select_token(const float* __restrict__ logits, int64_t t, int E, const RouteRule& r, float* s, float* m,
                                             float* gs, int32_t* __restrict__ ids, float* __restrict__ weights) {
  const int lane = threadIdx.x & 63;
  const int top = r.top, group_count = r.group_count, group_keep = r.group_keep;
  const int per = E / group_count;
  if (r.sigmoid) {
    for (int e = lane; e < E; e += 64) s[e] = 1.0f / (1.0f + expf(-logits[t * E + e]));
  } else {
    float hi = -INFINITY;
    for (int e = lane; e < E; e += 64) { s[e] = logits[t * E + e]; hi = fmaxf(hi, s[e]); }
    hi = wave_max(hi);
    float sum = 0.f;
    for (int e = lane; e < E; e += 64) { const float p = expf(s[e] - hi); s[e] = p; sum += p; }
    sum = wave_sum(sum);
    for (int e = lane; e < E; e += 64) s[e] = s[e] / sum;
  }
  for (int e = lane; e < E; e += 64) m[e] = r.correction ? s[e] + r.correction[e] : s[e];
  wave_settle();
  if (group_count > 1 && group_keep < group_count) {
    const int count = r.group_top < per ? r.group_top : per;
    for (int g = lane; g < group_count; g += 64) {
      // the group's largest choice scores one after the other: each time the largest that comes behind the one before
      // (by value, then by index)
      float total = 0.f, pv = INFINITY;
      int pi = -1;
      for (int c = 0; c < count; ++c) {
        float bv = -INFINITY;
        int bi = -1;
        for (int j = 0; j < per; ++j) {
          const float v = m[g * per + j];
          const bool behind = v < pv || (v == pv && j > pi);
          if (behind && (bi < 0 || v > bv)) { bv = v; bi = j; }
        }
        if (bi < 0) break;
        total += bv; pv = bv; pi = bi;
      }
      gs[g] = total;
    }
    wave_settle();
    // the best groups one after the other; a kept group's score becomes +inf, the others' experts leave the race
    for (int kept = 0; kept < group_keep; ++kept) {
      float bv = -INFINITY; int bi = 0x7fffffff;
      for (int g = lane; g < group_count; g += 64)
        if (gs[g] != INFINITY && (bi == 0x7fffffff || gs[g] > bv)) { bv = gs[g]; bi = g; }
      wave_argmax(bv, bi);
      if (bi >= group_count) bi = 0;          // scores that are no numbers: still a valid index
      if (lane == 0) gs[bi] = INFINITY;
      wave_settle();
    }
    for (int e = lane; e < E; e += 64)
      if (gs[e / per] != INFINITY) m[e] = -INFINITY;
    wave_settle();
  }
  float total = 0.f;
  int mine = 0;              // lane j keeps the j-th choice (top <= 64)
  for (int j = 0; j < top; ++j) {
    float bv = -INFINITY; int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64)
      if (m[e] > bv) { bv = m[e]; bi = e; }
    wave_argmax(bv, bi);
    if (bi >= E) bi = 0;
    if (lane == 0) m[bi] = -INFINITY;
    wave_settle();
    if (lane == j) mine = bi;
    total += s[bi];
  }
  if (lane < top) {
    ids[t * top + lane] = mine;
    weights[t * top + lane] = r.scale * (r.normalise ? s[mine] / (total + 1e-20f) : s[mine]);
  }
}

// The choice: a wave per token (4 tokens a workgroup). LDS per token: E scores, E working copies, the group scores.
__global__ void __launch_bounds__(256)
moe_select_kernel(const float* __restrict__ logits, int64_t T, int E, RouteRule rule,
                  int32_t* __restrict__ ids, float* __restrict__ weights) {
  extern __shared__ __align__(16) unsigned char route_lds[];
  const int wave = threadIdx.x >> 6;
  const int64_t t = (int64_t)blockIdx.x * 4 + wave;
  if (t >= T) return;
  float* s = reinterpret_cast<float*>(route_lds) + (size_t)wave * (2 * E + rule.group_count);
  select_token(logits, t, E, rule, s, s + E, s + 2 * E, ids, weights);
}

// logits: float32 [T, E] working memory.
static bool route_rule(RouteRule& r, int E, int top, int group_count, int group_keep, int group_top, int sigmoid, int normalise,
                       float scale, const float* correction) {
  r.top = top; r.group_count = group_count; r.group_keep = group_keep; r.group_top = group_top; r.sigmoid = sigmoid;
  r.normalise = normalise; r.scale = scale; r.correction = correction;
  return E >= 1 && E <= MOE_MAX_EXPERTS && top >= 1 && top <= 64 && top <= E && group_count >= 1 && E % group_count == 0 &&
         group_keep >= 1 && group_keep <= group_count && group_keep * (E / group_count) >= top && group_top >= 1;
}

extern "C" int me_moe_route(const void* x, int64_t ldx, int dtype, const float* w, int64_t T, int n, int E, int top,
                            int group_count, int group_keep, float* logits, int32_t* ids, float* weights, int select,
                            int group_top, int sigmoid, int normalise, float scale, const float* correction,
                            hipStream_t stream) {
  if (T == 0) return 0;
  RouteRule rule;
  ME_CHECK(route_rule(rule, E, top, group_count, group_keep, group_top, sigmoid, normalise, scale, correction),
           "moe_route: bad routing sizes (%d experts, top %d, %d groups, keep %d, %d of a group)", E, top, group_count, group_keep, group_top);
  ME_CHECK(E >= 1 && E <= MOE_MAX_EXPERTS && top >= 1 && top <= 64 && top <= E, "moe_route: %d experts, top %d", E, top);
  ME_CHECK(group_count >= 1 && E % group_count == 0 && group_keep >= 1 && group_keep <= group_count,
           "moe_route: %d groups (keep %d) over %d experts", group_count, group_keep, E);
  ME_CHECK(group_keep * (E / group_count) >= top, "moe_route: the kept groups hold fewer than top experts");
  const size_t es = dtype == ME_F32 ? 4 : 2;
  int TT = 8;
  while (TT > 1 && ((size_t)TT * n * es > 32 * 1024 || TT / 2 >= T)) TT >>= 1;       // as many as fit, and no more than there are
  ME_CHECK((size_t)TT * n * es <= 64 * 1024, "moe_route: a row of %d does not fit a workgroup's memory", n);
  const int64_t groups = (T + TT - 1) / TT;
  ME_CHECK(groups < (1ll << 31) && (T + 3) / 4 < (1ll << 31), "moe_route: too many tokens");
  // few tokens: the experts spread over as many workgroups as possible; many: a workgroup keeps its rows for 8 experts
  // (two per wave: enough workgroups to a compute unit to hide each other's waits; 32 per workgroup took twice as long)
  const int per_group = groups <= 64 ? 4 : 8;
  const dim3 grid((unsigned)groups, (unsigned)((E + per_group - 1) / per_group));
  if (dtype == ME_F32)
    moe_logits_kernel<float><<<grid, dim3(256), (size_t)TT * n * es, stream>>>((const float*)x, ldx, w, T, n, E, TT, per_group, logits);
  else
    moe_logits_kernel<bf16_t><<<grid, dim3(256), (size_t)TT * n * es, stream>>>((const bf16_t*)x, ldx, w, T, n, E, TT, per_group, logits);
  ME_LAUNCH_CHECK();
  if (!select) return 0;           // the caller lets `me_moe_sort` choose (few tokens: one launch less)
  const size_t lds = (size_t)4 * (2 * E + group_count) * 4;
  ME_CHECK(lds <= 64 * 1024, "moe_route: %d experts do not fit a workgroup's memory", E);
  moe_select_kernel<<<dim3((unsigned)((T + 3) / 4)), dim3(256), lds, stream>>>(logits, T, E, rule, ids, weights);
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ pairs by expert
// One workgroup. order[p']: the pair at sorted place p'; offsets[e]: where expert e's pairs begin; tile_expert / tile_row:
// expert and first sorted place of every tile of up to `tile_rows` pairs (expert -1: a tile nobody needs).
// With `logits` (few tokens) the workgroup first makes the choice itself, a wave per token in turn, and writes ids and
// weights: the launch of `moe_select` is saved.
__global__ void __launch_bounds__(1024)
moe_sort_kernel(int32_t* __restrict__ ids, int P, int E, int max_tiles, int tile_rows, int32_t* __restrict__ order,
                int32_t* __restrict__ offsets, int32_t* __restrict__ tile_expert, int32_t* __restrict__ tile_row,
                const float* __restrict__ logits, float* __restrict__ weights, RouteRule rule) {
  __shared__ int count[MOE_MAX_EXPERTS], begin[MOE_MAX_EXPERTS + 1], tile_at[MOE_MAX_EXPERTS + 1], cursor[MOE_MAX_EXPERTS];
  extern __shared__ __align__(16) unsigned char route_lds[];
  for (int e = threadIdx.x; e < E; e += blockDim.x) { count[e] = 0; cursor[e] = 0; }
  if (logits) {
    const int wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    float* s = reinterpret_cast<float*>(route_lds) + (size_t)wave * (2 * E + rule.group_count);
    for (int t = wave; t < P / rule.top; t += waves) select_token(logits, t, E, rule, s, s + E, s + 2 * E, ids, weights);
    __threadfence_block();
  }
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) atomicAdd(&count[ids[p]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, tiles = 0;
    for (int e = 0; e < E; ++e) {
      begin[e] = at; tile_at[e] = tiles;
      at += count[e];
      tiles += (count[e] + tile_rows - 1) / tile_rows;
    }
    begin[E] = at; tile_at[E] = tiles;
  }
  __syncthreads();
  for (int e = threadIdx.x; e <= E; e += blockDim.x) offsets[e] = begin[e];
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int e = ids[p];
    order[begin[e] + atomicAdd(&cursor[e], 1)] = p;
  }
  for (int e = threadIdx.x; e < E; e += blockDim.x)
    for (int i = tile_at[e]; i < tile_at[e + 1] && i < max_tiles; ++i) {
      tile_expert[i] = e;
      tile_row[i] = begin[e] + (i - tile_at[e]) * tile_rows;
    }
  for (int i = tile_at[E] + threadIdx.x; i < max_tiles; i += blockDim.x) { tile_expert[i] = -1; tile_row[i] = 0; }
}

// logits: null, or the router's float32 [T, E] with the choice still to be made (`me_moe_route` with select 0): ids and
// weights are then written here (`moe_sort_chooses` says when that fits).
extern "C" int me_moe_sort(int32_t* ids, int64_t P, int E, int max_tiles, int tile_rows, int32_t* order, int32_t* offsets,
                           int32_t* tile_expert, int32_t* tile_row, const float* logits, float* weights, int top, int group_count,
                           int group_keep, int group_top, int sigmoid, int normalise, float scale, const float* correction,
                           hipStream_t stream) {
  if (P == 0) return 0;
  ME_CHECK(E >= 1 && E <= MOE_MAX_EXPERTS && P < (1ll << 30), "moe_sort: %d experts, %lld pairs", E, (long long)P);
  ME_CHECK(tile_rows == 16 || tile_rows == 64 || tile_rows == 128, "moe_sort: tiles of 16, 64 or 128 rows");
  ME_CHECK(max_tiles >= P / tile_rows + (P < E ? P : E), "moe_sort: %d tiles cannot hold every expert's last tile", max_tiles);
  size_t lds = 0;
  RouteRule rule;
  route_rule(rule, E, top, group_count, group_keep, group_top, sigmoid, normalise, scale, correction);
  if (logits) {
    ME_CHECK(weights && route_rule(rule, E, top, group_count, group_keep, group_top, sigmoid, normalise, scale, correction) && P % top == 0,
             "moe_sort: bad routing sizes");
    lds = (size_t)16 * (2 * E + group_count) * 4;
    ME_CHECK(lds <= 40 * 1024, "moe_sort: %d experts are too many to choose here", E);
  }
  moe_sort_kernel<<<dim3(1), dim3(1024), lds, stream>>>(ids, (int)P, E, max_tiles, tile_rows, order, offsets, tile_expert, tile_row,
                                                        logits, weights, rule);
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ tiled products
// A stage in LDS: TM B rows (pairs) then TN A rows (weights), 128 bytes each. A workgroup's 4 waves are 2 x 2
// sub-tiles of TM/2 x TN/2, each MJ x MI matrix-instruction tiles of 16 x 16: 64 x 64 (2 x 2 per wave) for a few
// hundred rows per expert, 128 x 128 (4 x 4 per wave: twice the products per operand read from LDS) beyond.
// ACT 1: the tile's weight rows are TN/2 gate rows and the TN/2 up rows that go with them; the result is silu(gate) * up.
// ACT 2: experts without a gate: the tile's TN weight rows are up rows and the result is relu(up)^2. ACT 0: the down product,
// times the pair's weight, into the pair's partial sum.
//   x: [T, K] token rows (ACT 1, 2) or [P, K] rows at sorted places (ACT 0); w: [E * rows_per_expert, K]
template <int ACT, int TM, int TN>
__global__ void __launch_bounds__(256)
moe_tile_kernel(const bf16_t* __restrict__ x, int64_t ldx, const bf16_t* __restrict__ w, int64_t ldw,
                const int32_t* __restrict__ order, const int32_t* __restrict__ offsets, const int32_t* __restrict__ tile_expert,
                const int32_t* __restrict__ tile_row, const float* __restrict__ pair_weight, void* __restrict__ out,
                int64_t T, int top, int N, int K) {
  constexpr int ROWS = TM + TN, NQ = ROWS / 32, MI = TN / 32, MJ = TM / 32, STAGE = ROWS * 128;
  extern __shared__ __align__(16) unsigned char lds[];        // [2][STAGE]
  const int e = tile_expert[blockIdx.y];
  if (e < 0) return;
  const int row0 = tile_row[blockIdx.y];
  const int rows = min(TM, offsets[e + 1] - row0);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * (ACT == 1 ? TN / 2 : TN);      // first feature of the tile
  // the pieces this thread brings per stage: rows tid / 8 + 32 q, piece tid % 8
  const bf16_t* src[NQ];
  uint32_t dst[NQ];
  const int c = tid & 7;
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const int R = (tid >> 3) + 32 * q;
    if (R < TM) {
      const int p = row0 + min(R, rows - 1);
      const int64_t from = ACT ? (int64_t)(order[p] / top) : (int64_t)p;
      src[q] = x + from * ldx;
    } else {
      const int wr = R - TM;
      int64_t row;
      if (ACT == 1) row = (int64_t)e * 2 * N + (wr < TN / 2 ? min(n0 + wr, N - 1) : N + min(n0 + wr - TN / 2, N - 1));
      else row = (int64_t)e * N + min(n0 + wr, N - 1);
      src[q] = w + row * ldw;
    }
    dst[q] = R * 128 + ((c ^ ((R >> 1) & 7)) * 16);
  }
  uint4 piece[NQ];
  auto fetch = [&](int k0) {
    const int k = k0 + 8 * c;
#pragma unroll
    for (int q = 0; q < NQ; ++q) piece[q] = k < K ? *reinterpret_cast<const uint4*>(src[q] + k) : make_uint4(0u, 0u, 0u, 0u);
  };
  auto put = [&](int b) {
#pragma unroll
    for (int q = 0; q < NQ; ++q) *reinterpret_cast<uint4*>(lds + b * STAGE + dst[q]) = piece[q];
  };
  const int wm = wave >> 1, wn = wave & 1;
  const int swz = (n >> 1) & 7;
  // rows of the wave's operand tiles: pairs wm * TM/2 + 16 j + n; weights (ACT: half of them gates, half their ups)
  int a_row[MI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
    a_row[i] = TM + (ACT == 1 ? (i < MI / 2 ? wn * (TN / 4) + 16 * i : TN / 2 + wn * (TN / 4) + 16 * (i - MI / 2)) : wn * (TN / 2) + 16 * i) + n;
  f32x4 acc[MI][MJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < MJ; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int steps = (K + 63) / 64;
  fetch(0);
  put(0);
  __syncthreads();
  for (int k = 0; k < steps; ++k) {
    if (k + 1 < steps) fetch((k + 1) * 64);
    const unsigned char* buf = lds + (k & 1) * STAGE;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int col = ((4 * s + g) ^ swz) * 16;
      bf16x8 a[MI], b[MJ];
#pragma unroll
      for (int i = 0; i < MI; ++i) a[i] = *reinterpret_cast<const bf16x8*>(buf + a_row[i] * 128 + col);
#pragma unroll
      for (int j = 0; j < MJ; ++j) b[j] = *reinterpret_cast<const bf16x8*>(buf + (wm * (TM / 2) + 16 * j + n) * 128 + col);
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < MJ; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    if (k + 1 < steps) put((k + 1) & 1);
    __syncthreads();
  }
  // lane (n, g) of tile (i, j): 4 consecutive features from 4 g of pair row wm * TM/2 + 16 j + n
#pragma unroll
  for (int j = 0; j < MJ; ++j) {
    const int r = wm * (TM / 2) + 16 * j + n;
    if (r >= rows) continue;
    const int p = row0 + r;
    if constexpr (ACT == 2) {
      bf16_t* o = (bf16_t*)out + (int64_t)p * N;
#pragma unroll
      for (int i = 0; i < MI; ++i) {
        const int f = n0 + wn * (TN / 2) + 16 * i + 4 * g;
        bf16x4 r;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float up = fmaxf(acc[i][j][q], 0.f);
          r[q] = from_f32<bf16_t>(up * up);
        }
        if (f + 3 < N && (N & 3) == 0) {
          *reinterpret_cast<bf16x4*>(o + f) = r;
        } else {
#pragma unroll
          for (int q = 0; q < 4; ++q)
            if (f + q < N) o[f + q] = r[q];
        }
      }
    } else if constexpr (ACT == 1) {
      bf16_t* o = (bf16_t*)out + (int64_t)p * N;
#pragma unroll
      for (int i = 0; i < MI / 2; ++i) {
        const int f = n0 + wn * (TN / 4) + 16 * i + 4 * g;
        bf16x4 r;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float gate = acc[i][j][q];
          r[q] = from_f32<bf16_t>(gate / (1.f + __expf(-gate)) * acc[i + MI / 2][j][q]);
        }
        if (f + 3 < N && (N & 3) == 0) {
          *reinterpret_cast<bf16x4*>(o + f) = r;          // 4 neighbours, 8 bytes
        } else {
#pragma unroll
          for (int q = 0; q < 4; ++q)
            if (f + q < N) o[f + q] = r[q];
        }
      }
    } else {
      const int pair = order[p];
      const int64_t tok = pair / top, choice = pair - tok * top;
      const float pw = pair_weight[pair];
      float* o = (float*)out + (choice * T + tok) * N;
#pragma unroll
      for (int i = 0; i < MI; ++i) {
        const int f = n0 + wn * (TN / 2) + 16 * i + 4 * g;
        if (f + 3 < N && (N & 3) == 0) {
          *reinterpret_cast<float4*>(o + f) = make_float4(acc[i][j][0] * pw, acc[i][j][1] * pw, acc[i][j][2] * pw, acc[i][j][3] * pw);
        } else {
#pragma unroll
          for (int q = 0; q < 4; ++q)
            if (f + q < N) o[f + q] = acc[i][j][q] * pw;
        }
      }
    }
  }
}

template <int ACT, int TM>
static int launch_moe_tile(const bf16_t* x, int64_t ldx, const bf16_t* w, int64_t ldw, const int32_t* order, const int32_t* offsets,
                           const int32_t* tile_expert, const int32_t* tile_row, const float* pair_weight, void* out, int64_t T,
                           int top, int N, int K, int max_tiles, hipStream_t stream) {
  constexpr int TN = TM;
  const size_t lds = 2 * (size_t)(TM + TN) * 128;
  static bool allowed = false;                     // 64 KB of LDS for the large tiles: more than a kernel may have unasked
  if (!allowed && lds > 48 * 1024) {
    hipError_t err = hipFuncSetAttribute((const void*)moe_tile_kernel<ACT, TM, TN>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    ME_CHECK(err == hipSuccess, "routed experts: cannot get %zu bytes of LDS: %s", lds, hipGetErrorString(err));
    allowed = true;
  }
  const int per = ACT == 1 ? TN / 2 : TN;
  moe_tile_kernel<ACT, TM, TN><<<dim3((unsigned)((N + per - 1) / per), (unsigned)max_tiles), dim3(256), lds, stream>>>(
      x, ldx, w, ldw, order, offsets, tile_expert, tile_row, pair_weight, out, T, top, N, K);
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ few rows per expert
// Tiles of up to 16 pair rows (a decode step: a handful of tokens per expert). What such a step costs is the stream of
// the chosen experts' weights, so a workgroup takes 16 features only and cuts K over its 4 waves: a wave walks every
// fourth step of 32, its lanes asking memory for their operand pieces directly (no LDS on the way in), four steps in
// flight; the waves' sums meet in LDS.
template <int ACT>
__global__ void __launch_bounds__(256)
moe_skinny_kernel(const bf16_t* __restrict__ x, int64_t ldx, const bf16_t* __restrict__ w, const int32_t* __restrict__ order,
                  const int32_t* __restrict__ offsets, const int32_t* __restrict__ tile_expert, const int32_t* __restrict__ tile_row,
                  const float* __restrict__ pair_weight, void* __restrict__ out, int64_t T, int top, int N, int K) {
  __shared__ float part[4][ACT == 1 ? 2 : 1][64][4];
  const int e = tile_expert[blockIdx.y];
  if (e < 0) return;
  const int row0 = tile_row[blockIdx.y];
  const int rows = min(16, offsets[e + 1] - row0);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int p = row0 + min(n, rows - 1);
  const bf16_t* xr = x + (ACT ? (int64_t)(order[p] / top) : (int64_t)p) * ldx + 8 * g;
  const int f = min(n0 + n, N - 1);
  const bf16_t* wr = w + ((int64_t)e * (ACT == 1 ? 2 : 1) * N + f) * K + 8 * g;
  const bf16_t* ur = wr + (int64_t)N * K;            // ACT 1: the up row of the same feature
  f32x4 acc_g = {0.f, 0.f, 0.f, 0.f}, acc_u = {0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int k0 = wave * 32; k0 < K; k0 += 4 * 128) {
    bf16x8 a[4], u[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + i * 128;
      const bool in = k + 8 * g < K;
      a[i] = in ? *reinterpret_cast<const bf16x8*>(wr + k) : zero;
      if (ACT == 1) u[i] = in ? *reinterpret_cast<const bf16x8*>(ur + k) : zero;
      b[i] = in ? *reinterpret_cast<const bf16x8*>(xr + k) : zero;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      acc_g = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[i], acc_g, 0, 0, 0);
      if (ACT == 1) acc_u = __builtin_amdgcn_mfma_f32_16x16x32_bf16(u[i], b[i], acc_u, 0, 0, 0);
    }
  }
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    part[wave][0][lane][q] = acc_g[q];
    if constexpr (ACT == 1) part[wave][1][lane][q] = acc_u[q];
  }
  __syncthreads();
  if (wave != 0 || n >= rows) return;
  // lane (n, g): features n0 + 4 g .. + 3 of pair row n
  const int pr = row0 + n;
  float sg[4], su[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    sg[q] = part[0][0][lane][q] + part[1][0][lane][q] + part[2][0][lane][q] + part[3][0][lane][q];
    if constexpr (ACT == 1) su[q] = part[0][1][lane][q] + part[1][1][lane][q] + part[2][1][lane][q] + part[3][1][lane][q];
  }
  if constexpr (ACT == 2) {
    bf16_t* o = (bf16_t*)out + (int64_t)pr * N;
#pragma unroll
    for (int q = 0; q < 4; ++q)
      if (n0 + 4 * g + q < N) { const float up = fmaxf(sg[q], 0.f); o[n0 + 4 * g + q] = from_f32<bf16_t>(up * up); }
  } else if constexpr (ACT == 1) {
    bf16_t* o = (bf16_t*)out + (int64_t)pr * N;
#pragma unroll
    for (int q = 0; q < 4; ++q)
      if (n0 + 4 * g + q < N) o[n0 + 4 * g + q] = from_f32<bf16_t>(sg[q] / (1.f + __expf(-sg[q])) * su[q]);
  } else {
    const int pair = order[pr];
    const int64_t tok = pair / top, choice = pair - tok * top;
    const float pw = pair_weight[pair];
    float* o = (float*)out + (choice * T + tok) * N;
#pragma unroll
    for (int q = 0; q < 4; ++q)
      if (n0 + 4 * g + q < N) o[n0 + 4 * g + q] = sg[q] * pw;
  }
}

// act: bfloat16 [P, F] at sorted places; gate_up: [E * 2 F, K] (an expert's gate rows, then its up rows), or with `gated` 0
// [E * F, K] (up rows only: the result is relu(up)^2)
// tile_rows: 16 (tiles of `moe_sort` with 16 rows: the skinny kernel) or 64
extern "C" int me_moe_gate_up(const void* x, int64_t ldx, const void* gate_up, const int32_t* order, const int32_t* offsets,
                              const int32_t* tile_expert, const int32_t* tile_row, void* act, int64_t T, int top, int F, int K,
                              int max_tiles, int tile_rows, int gated, hipStream_t stream) {
  if (T == 0) return 0;
  ME_CHECK(K % 8 == 0 && ldx % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(gate_up) % 16 == 0,
           "moe_gate_up: rows must be whole 16-byte pieces (K = %d)", K);
  ME_CHECK(max_tiles >= 1 && max_tiles <= 65535 && F >= 1, "moe_gate_up: %d tiles", max_tiles);
  if (!gated) {
    if (tile_rows == 16) {
      moe_skinny_kernel<2><<<dim3((unsigned)((F + 15) / 16), (unsigned)max_tiles), dim3(256), 0, stream>>>(
          (const bf16_t*)x, ldx, (const bf16_t*)gate_up, order, offsets, tile_expert, tile_row, nullptr, act, T, top, F, K);
      ME_LAUNCH_CHECK();
      return 0;
    }
    if (tile_rows == 128)
      return launch_moe_tile<2, 128>((const bf16_t*)x, ldx, (const bf16_t*)gate_up, (int64_t)K, order, offsets, tile_expert, tile_row,
                                     nullptr, act, T, top, F, K, max_tiles, stream);
    ME_CHECK(tile_rows == 64, "moe_gate_up: tiles of 16, 64 or 128 rows");
    return launch_moe_tile<2, 64>((const bf16_t*)x, ldx, (const bf16_t*)gate_up, (int64_t)K, order, offsets, tile_expert, tile_row,
                                  nullptr, act, T, top, F, K, max_tiles, stream);
  }
  if (tile_rows == 16) {
    moe_skinny_kernel<1><<<dim3((unsigned)((F + 15) / 16), (unsigned)max_tiles), dim3(256), 0, stream>>>(
        (const bf16_t*)x, ldx, (const bf16_t*)gate_up, order, offsets, tile_expert, tile_row, nullptr, act, T, top, F, K);
    ME_LAUNCH_CHECK();
    return 0;
  }
  if (tile_rows == 128)
    return launch_moe_tile<1, 128>((const bf16_t*)x, ldx, (const bf16_t*)gate_up, (int64_t)K, order, offsets, tile_expert, tile_row,
                                      nullptr, act, T, top, F, K, max_tiles, stream);
  ME_CHECK(tile_rows == 64, "moe_gate_up: tiles of 16, 64 or 128 rows");
  return launch_moe_tile<1, 64>((const bf16_t*)x, ldx, (const bf16_t*)gate_up, (int64_t)K, order, offsets, tile_expert, tile_row,
                                   nullptr, act, T, top, F, K, max_tiles, stream);
}

// out: float32 [top, T, N]; down: [E * N, F]
extern "C" int me_moe_down(const void* act, const void* down, const int32_t* order, const int32_t* offsets,
                           const int32_t* tile_expert, const int32_t* tile_row, const float* pair_weight, float* out, int64_t T,
                           int top, int N, int F, int max_tiles, int tile_rows, hipStream_t stream) {
  if (T == 0) return 0;
  ME_CHECK(F % 8 == 0 && reinterpret_cast<uintptr_t>(act) % 16 == 0 && reinterpret_cast<uintptr_t>(down) % 16 == 0,
           "moe_down: rows must be whole 16-byte pieces (F = %d)", F);
  ME_CHECK(max_tiles >= 1 && max_tiles <= 65535 && N >= 1, "moe_down: %d tiles", max_tiles);
  if (tile_rows == 16) {
    moe_skinny_kernel<0><<<dim3((unsigned)((N + 15) / 16), (unsigned)max_tiles), dim3(256), 0, stream>>>(
        (const bf16_t*)act, (int64_t)F, (const bf16_t*)down, order, offsets, tile_expert, tile_row, pair_weight, out, T, top, N, F);
    ME_LAUNCH_CHECK();
    return 0;
  }
  if (tile_rows == 128)
    return launch_moe_tile<0, 128>((const bf16_t*)act, (int64_t)F, (const bf16_t*)down, (int64_t)F, order, offsets, tile_expert,
                                       tile_row, pair_weight, out, T, top, N, F, max_tiles, stream);
  ME_CHECK(tile_rows == 64, "moe_down: tiles of 16, 64 or 128 rows");
  return launch_moe_tile<0, 64>((const bf16_t*)act, (int64_t)F, (const bf16_t*)down, (int64_t)F, order, offsets, tile_expert,
                                    tile_row, pair_weight, out, T, top, N, F, max_tiles, stream);
}

// ------------------------------------------------------------------ one wave per output element
// act [P, F] in pair order (pair = token * top + choice): needs no sorting.
template <typename TX, bool GATED>
__global__ void __launch_bounds__(256)
moe_gate_up_simple_kernel(const TX* __restrict__ x, int64_t ldx, const TX* __restrict__ gate_up, const int32_t* __restrict__ ids,
                          TX* __restrict__ act, int64_t P, int top, int F, int K) {
  const int lane = threadIdx.x & 63;
  const int64_t at = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (at >= P * F) return;
  const int64_t pair = at / F;
  const int f = (int)(at - pair * F);
  const TX* xr = x + (pair / top) * ldx;
  const TX* gr = gate_up + ((int64_t)ids[pair] * (GATED ? 2 : 1) * F + f) * K;
  const TX* ur = gr + (int64_t)F * K;
  float sg = 0.f, su = 0.f;
  for (int k = lane; k < K; k += 64) {
    const float v = to_f32<TX>(xr[k]);
    sg += v * to_f32<TX>(gr[k]);
    if (GATED) su += v * to_f32<TX>(ur[k]);
  }
  sg = wave_sum(sg);
  if (GATED) su = wave_sum(su);
  const float up = fmaxf(sg, 0.f);
  if (lane == 0) act[at] = from_f32<TX>(GATED ? sg / (1.f + expf(-sg)) * su : up * up);
}

template <typename TX>
__global__ void __launch_bounds__(256)
moe_down_simple_kernel(const TX* __restrict__ act, const TX* __restrict__ down, const int32_t* __restrict__ ids,
                       const float* __restrict__ pair_weight, float* __restrict__ out, int64_t T, int top, int N, int F) {
  const int lane = threadIdx.x & 63;
  const int64_t at = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (at >= T * top * N) return;
  const int64_t pair = at / N;
  const int f = (int)(at - pair * N);
  const TX* ar = act + pair * F;
  const TX* dr = down + ((int64_t)ids[pair] * N + f) * F;
  float s = 0.f;
  for (int k = lane; k < F; k += 64) s += to_f32<TX>(ar[k]) * to_f32<TX>(dr[k]);
  s = wave_sum(s);
  const int64_t tok = pair / top, choice = pair - tok * top;
  if (lane == 0) out[(choice * T + tok) * N + f] = s * pair_weight[pair];
}

extern "C" int me_moe_experts_simple(const void* x, int64_t ldx, int dtype, const void* gate_up, const void* down,
                                     const int32_t* ids, const float* pair_weight, void* act, float* out, int64_t T, int top,
                                     int N, int F, int K, int gated, hipStream_t stream) {
  if (T == 0) return 0;
  const int64_t P = T * top;
  const int64_t g1 = (P * F + 3) / 4, g2 = (P * N + 3) / 4;
  ME_CHECK(g1 < (1ll << 31) && g2 < (1ll << 31), "moe_experts_simple: too many outputs");
  if (dtype == ME_F32) {
    if (gated) moe_gate_up_simple_kernel<float, true><<<dim3((unsigned)g1), dim3(256), 0, stream>>>((const float*)x, ldx, (const float*)gate_up, ids,
                                                                                                    (float*)act, P, top, F, K);
    else moe_gate_up_simple_kernel<float, false><<<dim3((unsigned)g1), dim3(256), 0, stream>>>((const float*)x, ldx, (const float*)gate_up, ids,
                                                                                               (float*)act, P, top, F, K);
    moe_down_simple_kernel<float><<<dim3((unsigned)g2), dim3(256), 0, stream>>>((const float*)act, (const float*)down, ids, pair_weight,
                                                                                out, T, top, N, F);
  } else {
    if (gated) moe_gate_up_simple_kernel<bf16_t, true><<<dim3((unsigned)g1), dim3(256), 0, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)gate_up, ids,
                                                                                                     (bf16_t*)act, P, top, F, K);
    else moe_gate_up_simple_kernel<bf16_t, false><<<dim3((unsigned)g1), dim3(256), 0, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)gate_up, ids,
                                                                                                (bf16_t*)act, P, top, F, K);
    moe_down_simple_kernel<bf16_t><<<dim3((unsigned)g2), dim3(256), 0, stream>>>((const bf16_t*)act, (const bf16_t*)down, ids,
                                                                                 pair_weight, out, T, top, N, F);
  }
  ME_LAUNCH_CHECK();
  return 0;
}
