// A feed-forward of many small experts of which every token uses a few.
//
//   route:    float32 router logits [T, E] -> the `top` largest per token (ties: the lower index) and their weights:
//             the softmax over those `top` logits alone, or every chosen logit's sigmoid (as it is, or divided by the
//             sum of the chosen ones).
//   group:    the T * top (token, choice) pairs sorted by expert, cut into tiles of 16 rows that belong to one expert
//             each.  It runs on the device, in one block, so a step never waits for the host (and can be captured).
//   gate_up:  for every tile, hidden = clamp-gated activation of (x Wg_e^T, x Wu_e^T)
//   down:     for every tile, y[pair] = hidden Wd_e^T, float32, at the pair's own place (token * top + choice)
//   combine:  out[t] = sum_j weight[t, j] y[t * top + j]  (+ sigmoid(shared_gate[t]) * shared[t]), summed in the order
//             of j: a token's result does not depend on what else is in the batch.
//
// The products take their rows through tile_product.h: float32 FMA for the 32-bit path, MFMA 16x16x32 for bfloat16.
// The grids are sized for the worst case (every expert with a ragged last tile); tiles that do not exist leave at once.
#include "common.h"
#include "fmsamd.h"
#include "tile_product.h"

#define ROUTE_MAX_EXPERTS 1024
#define ROUTE_MAX_TOP 64

// One wave per token.
__global__ void __launch_bounds__(256)
    route_kernel(const float* __restrict__ logits, long ld, int n_tokens, int n_experts, int top, int score, int* __restrict__ ids,
                 float* __restrict__ weights) {
  extern __shared__ float lds[];  // 4 waves x (n_experts + top)
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + wave;
  if (t >= n_tokens) return;
  float* z = lds + (size_t)wave * (n_experts + top);
  float* chosen = z + n_experts;
  for (int e = lane; e < n_experts; e += WAVE) z[e] = logits[(size_t)t * ld + e];
  __builtin_amdgcn_wave_barrier();
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < n_experts; e += WAVE) {
      const float v = z[e];
      if (v > best || (v == best && e < at)) best = v, at = e;
    }
    if (at == 0x7fffffff) at = lane < n_experts ? lane : 0;  // only NaNs or -inf left in this lane's share
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) {
      const float ov = __shfl_xor(best, off, WAVE);
      const int oa = __shfl_xor(at, off, WAVE);
      if (ov > best || (ov == best && oa < at)) best = ov, at = oa;
    }
    if (lane == 0) {
      ids[(size_t)t * top + j] = at;
      chosen[j] = best;
      z[at] = -INFINITY;
    }
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
  }
  if (lane == 0) {
    if (score == FMS_ROUTE_SOFTMAX) {
      const float m = chosen[0];  // the largest comes first
      float sum = 0.f;
      for (int j = 0; j < top; ++j) sum += expf(chosen[j] - m);
      for (int j = 0; j < top; ++j) weights[(size_t)t * top + j] = expf(chosen[j] - m) / sum;
    } else {  // sigmoid scores (the order of the logits is the order of their sigmoids)
      float sum = 0.f;
      for (int j = 0; j < top; ++j) sum += 1.f / (1.f + expf(-chosen[j]));
      const float norm = score == FMS_ROUTE_SIGMOID_NORMED ? 1.f / sum : 1.f;
      for (int j = 0; j < top; ++j) weights[(size_t)t * top + j] = norm / (1.f + expf(-chosen[j]));
    }
  }
}

extern "C" int fmsamd_moe_route(const float* logits, long ld, int n_tokens, int n_experts, int top, int score, int* ids,
                                float* weights, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  FMS_REQUIRE(n_tokens > 0 && n_experts > 0 && n_experts <= ROUTE_MAX_EXPERTS && top > 0 && top <= n_experts && top <= ROUTE_MAX_TOP,
              "moe_route: %d experts (at most %d), top %d (at most %d and the experts)", n_experts, ROUTE_MAX_EXPERTS, top, ROUTE_MAX_TOP);
  FMS_REQUIRE(ld >= n_experts, "moe_route: rows of %ld for %d experts", ld, n_experts);
  FMS_REQUIRE(score >= FMS_ROUTE_SOFTMAX && score <= FMS_ROUTE_SIGMOID_NORMED, "moe_route: unknown score %d", score);
  const size_t lds = 4 * (size_t)(n_experts + top) * sizeof(float);
  route_kernel<<<ceil_div(n_tokens, 4), 256, lds, stream>>>(logits, ld, n_tokens, n_experts, top, score, ids, weights);
  FMS_LAUNCH_CHECK("moe_route");
  return 0;
}

// The wave's largest value and where it is (ties: the lower index); every lane gets both.
__device__ __forceinline__ void wave_argmax(float& best, int& at) {
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(best, off, WAVE);
    const int oa = __shfl_xor(at, off, WAVE);
    if (ov > best || (ov == best && oa < at)) best = ov, at = oa;
  }
}

__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_wave_barrier();
  __threadfence_block();
}

// Routing over groups of experts.  s = softmax over all n router outputs; an output is chosen by s + correction, but
// weighted by s.  The outputs form `groups` equal runs of neighbours; a group's score is its largest choice score, and
// only outputs of the `keep` best groups can be chosen (the others count as minus infinity).  The weights of the `top`
// chosen are their s divided by their sum (+ 1e-20), times `scale`.  One wave per token; ties go to the lower index.
__global__ void __launch_bounds__(256)
    route_grouped_kernel(const float* __restrict__ logits, long ld, int n_tokens, int n, int top, const float* __restrict__ correction,
                         int groups, int keep, float scale, int* __restrict__ ids, float* __restrict__ weights) {
  extern __shared__ float lds[];  // 4 waves x (2 n + 2 groups + top)
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + wave;
  if (t >= n_tokens) return;
  float* s = lds + (size_t)wave * (2 * n + 2 * groups + top);
  float* choice = s + n;
  float* gscore = choice + n;
  float* kept = gscore + groups;
  float* chosen = kept + groups;
  float m = -INFINITY;
  for (int e = lane; e < n; e += WAVE) {
    const float z = logits[(size_t)t * ld + e];
    s[e] = z;
    m = fmaxf(m, z);
  }
  m = wave_max(m);
  float sum = 0.f;
  for (int e = lane; e < n; e += WAVE) {
    const float p = expf(s[e] - m);
    s[e] = p;
    sum += p;
  }
  sum = wave_sum(sum);
  for (int e = lane; e < n; e += WAVE) {
    const float p = s[e] / sum;
    float c = p + (correction ? correction[e] : 0.f);
    if (!(c >= -3.0e38f)) c = -3.0e38f;  // not a number (a padding row's logits): still a candidate, the last of all
    s[e] = p;
    choice[e] = c;
  }
  wave_lds_fence();
  if (groups > 1) {
    const int per = n / groups;
    for (int g = lane; g < groups; g += WAVE) {
      float best = -INFINITY;
      for (int e = g * per; e < (g + 1) * per; ++e) best = fmaxf(best, choice[e]);
      gscore[g] = best;
      kept[g] = 0.f;
    }
    wave_lds_fence();
    for (int j = 0; j < keep; ++j) {
      float best = -INFINITY;
      int at = 0x7fffffff;
      for (int g = lane; g < groups; g += WAVE) {
        const float v = gscore[g];
        if (v > best || (v == best && g < at)) best = v, at = g;
      }
      wave_argmax(best, at);
      if (lane == 0 && at < groups) kept[at] = 1.f, gscore[at] = -INFINITY;
      wave_lds_fence();
    }
    for (int e = lane; e < n; e += WAVE)
      if (kept[e / per] == 0.f) choice[e] = -INFINITY;
    wave_lds_fence();
  }
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < n; e += WAVE) {
      const float v = choice[e];
      if (v > best || (v == best && e < at)) best = v, at = e;
    }
    wave_argmax(best, at);
    if (at >= n) at = 0;  // nothing left to choose from: the configuration allows fewer outputs than `top`
    if (lane == 0) {
      ids[(size_t)t * top + j] = at;
      chosen[j] = s[at];
      choice[at] = -INFINITY;
    }
    wave_lds_fence();
  }
  if (lane == 0) {
    float total = 0.f;
    for (int j = 0; j < top; ++j) total += chosen[j];
    const float norm = scale / (total + 1e-20f);
    for (int j = 0; j < top; ++j) weights[(size_t)t * top + j] = chosen[j] * norm;
  }
}

extern "C" int fmsamd_moe_route_grouped(const float* logits, long ld, int n_tokens, int n_outputs, int top, const float* correction,
                                        int groups, int keep, float scale, int* ids, float* weights, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  FMS_REQUIRE(n_tokens > 0 && n_outputs > 0 && n_outputs <= ROUTE_MAX_EXPERTS && top > 0 && top <= n_outputs && top <= ROUTE_MAX_TOP,
              "moe_route_grouped: %d outputs (at most %d), top %d (at most %d and the outputs)", n_outputs, ROUTE_MAX_EXPERTS, top,
              ROUTE_MAX_TOP);
  FMS_REQUIRE(ld >= n_outputs, "moe_route_grouped: rows of %ld for %d outputs", ld, n_outputs);
  FMS_REQUIRE(groups >= 1 && n_outputs % groups == 0 && keep >= 1 && keep <= groups && (long)keep * (n_outputs / groups) >= top,
              "moe_route_grouped: %d groups of %d outputs, %d kept, cannot give %d choices", groups, n_outputs / (groups > 0 ? groups : 1),
              keep, top);
  const size_t lds = 4 * (size_t)(2 * n_outputs + 2 * groups + top) * sizeof(float);
  route_grouped_kernel<<<ceil_div(n_tokens, 4), 256, lds, stream>>>(logits, ld, n_tokens, n_outputs, top, correction, groups, keep, scale,
                                                                    ids, weights);
  FMS_LAUNCH_CHECK("moe_route_grouped");
  return 0;
}

// --------------------------------------------------------------------------
// group: order[0 .. n) = the pairs sorted by expert; tiles[i] = (expert, first row in order, rows), rows 0: no tile
// --------------------------------------------------------------------------
__global__ void __launch_bounds__(1024)
    group_kernel(const int* __restrict__ ids, int n_pairs, int n_experts, int* __restrict__ order, int* __restrict__ tiles,
                 int max_tiles, int tile_rows) {
  __shared__ int counts[ROUTE_MAX_EXPERTS];
  __shared__ int cursor[ROUTE_MAX_EXPERTS];
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) counts[e] = 0;
  __syncthreads();
  for (int a = threadIdx.x; a < n_pairs; a += blockDim.x) {
    const int e = ids[a];
    if (e >= 0 && e < n_experts) atomicAdd(&counts[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, nt = 0;
    for (int e = 0; e < n_experts; ++e) {
      cursor[e] = at;
      const int c = counts[e];
      for (int r = 0; r < c && nt < max_tiles; r += tile_rows, ++nt) {
        tiles[3 * nt] = e;
        tiles[3 * nt + 1] = at + r;
        tiles[3 * nt + 2] = c - r < tile_rows ? c - r : tile_rows;
      }
      at += c;
    }
    for (; nt < max_tiles; ++nt) tiles[3 * nt] = 0, tiles[3 * nt + 1] = 0, tiles[3 * nt + 2] = 0;
  }
  __syncthreads();
  for (int a = threadIdx.x; a < n_pairs; a += blockDim.x) {
    const int e = ids[a];
    if (e >= 0 && e < n_experts) order[atomicAdd(&cursor[e], 1)] = a;
  }
}

// Rows of a tile: 64 where the experts have that many rows on average (prompts) and the matrix-core kernel can run
// (wide_ok: bfloat16, rows aligned to 16 bytes), else 16.
extern "C" int fmsamd_moe_tile_rows(int n_pairs, int n_experts, int wide_ok) {
  return (wide_ok && n_pairs >= (long)TILE_WIDE_ROWS * n_experts) ? TILE_WIDE_ROWS : TILE_ROWS;
}

extern "C" int fmsamd_moe_max_tiles(int n_pairs, int n_experts, int tile_rows) {
  if (tile_rows <= 0) return 0;
  return (n_pairs + tile_rows - 1) / tile_rows + (n_experts < n_pairs ? n_experts : n_pairs);
}

extern "C" int fmsamd_moe_group(const int* ids, int n_pairs, int n_experts, int* order, int* tiles, int max_tiles,
                                int tile_rows, hipStream_t stream) {
  if (n_pairs == 0) return 0;
  FMS_REQUIRE(n_pairs > 0 && n_experts > 0 && n_experts <= ROUTE_MAX_EXPERTS, "moe_group: %d pairs, %d experts (at most %d)", n_pairs,
              n_experts, ROUTE_MAX_EXPERTS);
  FMS_REQUIRE(tile_rows == TILE_ROWS || tile_rows == TILE_WIDE_ROWS, "moe_group: tiles of %d rows", tile_rows);
  FMS_REQUIRE(max_tiles >= fmsamd_moe_max_tiles(n_pairs, n_experts, tile_rows), "moe_group: room for %d tiles, %d may be needed", max_tiles,
              fmsamd_moe_max_tiles(n_pairs, n_experts, tile_rows));
  group_kernel<<<1, 1024, 0, stream>>>(ids, n_pairs, n_experts, order, tiles, max_tiles, tile_rows);
  FMS_LAUNCH_CHECK("moe_group");
  return 0;
}

// --------------------------------------------------------------------------
// the experts' products
// --------------------------------------------------------------------------
struct ExpertArgs {
  const void* x;  // gate_up: [T, ldx] token rows; down: hidden [pairs, ldx] in sorted order
  long ldx;
  const void* w1;  // gate_up: gate weights [E, N, K]; down: down weights [E, N, K]
  const void* w2;  // gate_up: up weights [E, N, K]
  void* y;  // gate_up: hidden [pairs, N] in sorted order; down: float32 [pairs, N] by pair
  const int* order;
  const int* tiles;
  int top, N, K;
  float limit, alpha, shift;
  const float* in_scale;  // gate_up: a factor per pair on the expert's input (applied to both float32 sums), or null
  int act;  // gate_up without up weights (w2 null): hidden = act(x W1^T), one of FMS_ACT_*
};

__device__ __forceinline__ float pair_scale(const ExpertArgs& a, int sorted_row) {
  return a.in_scale ? a.in_scale[a.order[sorted_row]] : 1.f;
}

__device__ __forceinline__ float clamp_gated(float g, float u, float limit, float alpha, float shift) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.f + expf(-alpha * g)) * (u + shift);
}

// what an expert keeps between its two products: the clamped gated activation of (gate, up), or act(the one product)
__device__ __forceinline__ float hidden_value(const ExpertArgs& a, bool gated, float g, float u) {
  return gated ? clamp_gated(g, u, a.limit, a.alpha, a.shift) : fms_activate(g, a.act);
}

template <typename T>
__global__ void __launch_bounds__(TILE_THREADS) expert_gate_up_fma_kernel(ExpertArgs a) {
  const int e = a.tiles[3 * blockIdx.x], start = a.tiles[3 * blockIdx.x + 1], rows = a.tiles[3 * blockIdx.x + 2];
  if (rows == 0) return;
  const int n0 = blockIdx.y * TILE_FMA_COLS;
  const T* x = (const T*)a.x;
  const T* wg = (const T*)a.w1 + (size_t)e * a.N * a.K;
  const T* wu = (const T*)a.w2 + (size_t)e * a.N * a.K;
  auto a_row = [&](int m) { return m < rows ? x + (size_t)(a.order[start + m] / a.top) * a.ldx : (const T*)nullptr; };
  const bool gated = a.w2 != nullptr;
  float g[4], u[4] = {0.f, 0.f, 0.f, 0.f};
  tile_product_fma<T>(a_row, [&](int n) { return n0 + n < a.N ? wg + (size_t)(n0 + n) * a.K : (const T*)nullptr; }, a.K, g);
  if (gated) tile_product_fma<T>(a_row, [&](int n) { return n0 + n < a.N ? wu + (size_t)(n0 + n) * a.K : (const T*)nullptr; }, a.K, u);
  const int n = n0 + threadIdx.x % 64;
  if (n >= a.N) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = (threadIdx.x / 64) * 4 + i;
    if (m < rows) {
      const float sc = pair_scale(a, start + m);
      ((T*)a.y)[(size_t)(start + m) * a.N + n] = from_f32<T>(hidden_value(a, gated, g[i] * sc, u[i] * sc));
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(TILE_THREADS) expert_down_fma_kernel(ExpertArgs a) {
  const int e = a.tiles[3 * blockIdx.x], start = a.tiles[3 * blockIdx.x + 1], rows = a.tiles[3 * blockIdx.x + 2];
  if (rows == 0) return;
  const int n0 = blockIdx.y * TILE_FMA_COLS;
  const T* x = (const T*)a.x;
  const T* w = (const T*)a.w1 + (size_t)e * a.N * a.K;
  float acc[4];
  tile_product_fma<T>([&](int m) { return m < rows ? x + (size_t)(start + m) * a.ldx : (const T*)nullptr; },
                      [&](int n) { return n0 + n < a.N ? w + (size_t)(n0 + n) * a.K : (const T*)nullptr; }, a.K, acc);
  const int n = n0 + threadIdx.x % 64;
  if (n >= a.N) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = (threadIdx.x / 64) * 4 + i;
    if (m < rows) ((float*)a.y)[(size_t)a.order[start + m] * a.N + n] = acc[i];
  }
}

__global__ void __launch_bounds__(TILE_THREADS) expert_gate_up_mfma_kernel(ExpertArgs a) {
  const int e = a.tiles[3 * blockIdx.x], start = a.tiles[3 * blockIdx.x + 1], rows = a.tiles[3 * blockIdx.x + 2];
  if (rows == 0) return;
  const int n0 = blockIdx.y * TILE_MFMA_COLS;
  const bf16* x = (const bf16*)a.x;
  const bf16* wg = (const bf16*)a.w1 + (size_t)e * a.N * a.K;
  const bf16* wu = (const bf16*)a.w2 + (size_t)e * a.N * a.K;
  auto a_row = [&](int m) { return m < rows ? x + (size_t)(a.order[start + m] / a.top) * a.ldx : (const bf16*)nullptr; };
  const bool gated = a.w2 != nullptr;
  f32x4 g[TILE_MFMA_WAVE_TILES], u[TILE_MFMA_WAVE_TILES];
#pragma unroll
  for (int tl = 0; tl < TILE_MFMA_WAVE_TILES; ++tl) u[tl] = f32x4{0.f, 0.f, 0.f, 0.f};
  tile_product_mfma(a_row, [&](int n) { return n0 + n < a.N ? wg + (size_t)(n0 + n) * a.K : (const bf16*)nullptr; }, a.K, g);
  if (gated) tile_product_mfma(a_row, [&](int n) { return n0 + n < a.N ? wu + (size_t)(n0 + n) * a.K : (const bf16*)nullptr; }, a.K, u);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = (lane >> 4) * 4 + i;
    if (m >= rows) continue;
    const float sc = pair_scale(a, start + m);
#pragma unroll
    for (int tl = 0; tl < TILE_MFMA_WAVE_TILES; ++tl) {
      const int n = n0 + wave * (16 * TILE_MFMA_WAVE_TILES) + tl * 16 + (lane & 15);
      if (n < a.N) ((bf16*)a.y)[(size_t)(start + m) * a.N + n] = (bf16)hidden_value(a, gated, g[tl][i] * sc, u[tl][i] * sc);
    }
  }
}

__global__ void __launch_bounds__(TILE_THREADS) expert_down_mfma_kernel(ExpertArgs a) {
  const int e = a.tiles[3 * blockIdx.x], start = a.tiles[3 * blockIdx.x + 1], rows = a.tiles[3 * blockIdx.x + 2];
  if (rows == 0) return;
  const int n0 = blockIdx.y * TILE_MFMA_COLS;
  const bf16* x = (const bf16*)a.x;
  const bf16* w = (const bf16*)a.w1 + (size_t)e * a.N * a.K;
  f32x4 acc[TILE_MFMA_WAVE_TILES];
  tile_product_mfma([&](int m) { return m < rows ? x + (size_t)(start + m) * a.ldx : (const bf16*)nullptr; },
                    [&](int n) { return n0 + n < a.N ? w + (size_t)(n0 + n) * a.K : (const bf16*)nullptr; }, a.K, acc);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = (lane >> 4) * 4 + i;
    if (m >= rows) continue;
    float* yrow = (float*)a.y + (size_t)a.order[start + m] * a.N;
#pragma unroll
    for (int tl = 0; tl < TILE_MFMA_WAVE_TILES; ++tl) {
      const int n = n0 + wave * (16 * TILE_MFMA_WAVE_TILES) + tl * 16 + (lane & 15);
      if (n < a.N) yrow[n] = acc[tl][i];
    }
  }
}

// The same two products on tiles of 64 rows (tile_product_mfma_wide).
__global__ void __launch_bounds__(TILE_THREADS) expert_gate_up_wide_kernel(ExpertArgs a) {
  const int e = a.tiles[3 * blockIdx.x], start = a.tiles[3 * blockIdx.x + 1], rows = a.tiles[3 * blockIdx.x + 2];
  if (rows == 0) return;
  const int n0 = blockIdx.y * TILE_MFMA_COLS;
  const bf16* x = (const bf16*)a.x;
  const bf16* wg = (const bf16*)a.w1 + (size_t)e * a.N * a.K;
  const bf16* wu = (const bf16*)a.w2 + (size_t)e * a.N * a.K;
  auto a_row = [&](int m) { return m < rows ? x + (size_t)(a.order[start + m] / a.top) * a.ldx : (const bf16*)nullptr; };
  const bool gated = a.w2 != nullptr;
  f32x4 g[2][4], u[2][4];
#pragma unroll
  for (int mt = 0; mt < 2; ++mt)
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) u[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};
  tile_product_mfma_wide(a_row, [&](int n) { return n0 + n < a.N ? wg + (size_t)(n0 + n) * a.K : (const bf16*)nullptr; }, a.K, g);
  if (gated) tile_product_mfma_wide(a_row, [&](int n) { return n0 + n < a.N ? wu + (size_t)(n0 + n) * a.K : (const bf16*)nullptr; }, a.K, u);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = (wave >> 1) * 32 + mt * 16 + (lane >> 4) * 4 + i;
      if (m >= rows) continue;
      const float sc = pair_scale(a, start + m);
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        const int n = n0 + (wave & 1) * 64 + nt * 16 + (lane & 15);
        if (n < a.N) ((bf16*)a.y)[(size_t)(start + m) * a.N + n] = (bf16)hidden_value(a, gated, g[mt][nt][i] * sc, u[mt][nt][i] * sc);
      }
    }
  }
}

__global__ void __launch_bounds__(TILE_THREADS) expert_down_wide_kernel(ExpertArgs a) {
  const int e = a.tiles[3 * blockIdx.x], start = a.tiles[3 * blockIdx.x + 1], rows = a.tiles[3 * blockIdx.x + 2];
  if (rows == 0) return;
  const int n0 = blockIdx.y * TILE_MFMA_COLS;
  const bf16* x = (const bf16*)a.x;
  const bf16* w = (const bf16*)a.w1 + (size_t)e * a.N * a.K;
  f32x4 acc[2][4];
  tile_product_mfma_wide([&](int m) { return m < rows ? x + (size_t)(start + m) * a.ldx : (const bf16*)nullptr; },
                         [&](int n) { return n0 + n < a.N ? w + (size_t)(n0 + n) * a.K : (const bf16*)nullptr; }, a.K, acc);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = (wave >> 1) * 32 + mt * 16 + (lane >> 4) * 4 + i;
      if (m >= rows) continue;
      float* yrow = (float*)a.y + (size_t)a.order[start + m] * a.N;
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        const int n = n0 + (wave & 1) * 64 + nt * 16 + (lane & 15);
        if (n < a.N) yrow[n] = acc[mt][nt][i];
      }
    }
  }
}

// stage 0: hidden = act(x Wg^T, x Wu^T) for the tiles' rows; stage 1: y = hidden Wd^T
// tile_rows: what fmsamd_moe_tile_rows said when the tiles were made
extern "C" int fmsamd_moe_experts(int stage, const void* x, long ldx, const void* w1, const void* w2, void* y, int dtype,
                                  const int* order, const int* tiles, int max_tiles, int tile_rows, int top, int N, int K,
                                  float limit, float alpha, float shift, const float* in_scale, int act, hipStream_t stream) {
  if (max_tiles == 0) return 0;
  FMS_REQUIRE(act >= 0 && act <= FMS_ACT_LAST, "moe_experts: unknown activation %d", act);
  FMS_REQUIRE(stage == 0 || stage == 1, "moe_experts: stage %d", stage);
  FMS_REQUIRE(tile_rows == TILE_ROWS || tile_rows == TILE_WIDE_ROWS, "moe_experts: tiles of %d rows", tile_rows);
  FMS_REQUIRE(max_tiles > 0 && top > 0 && N > 0 && K > 0 && ldx >= K, "moe_experts: bad sizes tiles=%d top=%d N=%d K=%d ldx=%ld", max_tiles,
              top, N, K, ldx);
  ExpertArgs a{x, ldx, w1, w2, y, order, tiles, top, N, K, limit, alpha, shift, stage == 0 ? in_scale : nullptr, act};
  const bool mfma = dtype == FMS_BF16 && K % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)w1 % 16) == 0 &&
                    (w2 == nullptr || ((uintptr_t)w2 % 16) == 0);
  const dim3 grid(max_tiles, ceil_div(N, mfma ? TILE_MFMA_COLS : TILE_FMA_COLS));
  FMS_REQUIRE(grid.y <= 65535, "moe_experts: %d columns are too many for one launch", N);
  if (tile_rows == TILE_WIDE_ROWS) {
    // tiles of 64 rows are made for the matrix-core kernel only
    FMS_REQUIRE(mfma, "moe_experts: tiles of %d rows need bfloat16 rows aligned to 16 bytes", tile_rows);
    if (stage == 0) expert_gate_up_wide_kernel<<<grid, TILE_THREADS, 0, stream>>>(a);
    else expert_down_wide_kernel<<<grid, TILE_THREADS, 0, stream>>>(a);
  } else if (dtype == FMS_F32) {
    if (stage == 0) expert_gate_up_fma_kernel<float><<<grid, TILE_THREADS, 0, stream>>>(a);
    else expert_down_fma_kernel<float><<<grid, TILE_THREADS, 0, stream>>>(a);
  } else if (dtype == FMS_BF16) {
    if (mfma) {
      if (stage == 0) expert_gate_up_mfma_kernel<<<grid, TILE_THREADS, 0, stream>>>(a);
      else expert_down_mfma_kernel<<<grid, TILE_THREADS, 0, stream>>>(a);
    } else {
      if (stage == 0) expert_gate_up_fma_kernel<bf16><<<grid, TILE_THREADS, 0, stream>>>(a);
      else expert_down_fma_kernel<bf16><<<grid, TILE_THREADS, 0, stream>>>(a);
    }
  } else {
    FMS_REQUIRE(false, "moe_experts: unknown dtype %d", dtype);
  }
  FMS_LAUNCH_CHECK("moe_experts");
  return 0;
}

// --------------------------------------------------------------------------
// combine
// --------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
    combine_kernel(const float* __restrict__ y, const float* __restrict__ weights, int top, const T* __restrict__ shared,
                   const float* __restrict__ shared_gate, long ldg, T* __restrict__ out, int width, const int* __restrict__ ids,
                   int n_experts, const T* __restrict__ x_in, long ldx) {
  const int t = blockIdx.x;
  const float sg = shared ? (shared_gate ? 1.f / (1.f + expf(-shared_gate[(size_t)t * ldg])) : 1.f) : 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = 0.f;
    for (int j = 0; j < top; ++j) {
      // a choice past the experts is an identity expert: its output is the token's input
      const bool same = ids != nullptr && ids[(size_t)t * top + j] >= n_experts;
      const float yj = same ? to_f32(x_in[(size_t)t * ldx + i]) : y[((size_t)t * top + j) * width + i];
      v = fmaf(weights ? weights[(size_t)t * top + j] : 1.f, yj, v);
    }
    if (shared) v = fmaf(sg, to_f32(shared[(size_t)t * width + i]), v);
    out[(size_t)t * width + i] = from_f32<T>(v);
  }
}

// The same for rows of at most 1024 * KEEP elements (a multiple of 4): a thread's elements wait in registers, four a
// load, and every choice's row is asked for at once, so the kernel pays the memory's latency once a choice instead of
// once an element and choice.
template <typename T, int KEEP>
__global__ void __launch_bounds__(256)
    combine_small_kernel(const float* __restrict__ y, const float* __restrict__ weights, int top, const T* __restrict__ shared,
                         const float* __restrict__ shared_gate, long ldg, T* __restrict__ out, int width, const int* __restrict__ ids,
                         int n_experts, const T* __restrict__ x_in, long ldx) {
  const int t = blockIdx.x;
  f32x4 acc[KEEP], sh[KEEP];
#pragma unroll
  for (int n = 0; n < KEEP; ++n) {
    const int i = (threadIdx.x + n * 256) * 4;
    acc[n] = f32x4{0.f, 0.f, 0.f, 0.f};
    sh[n] = acc[n];
    if (shared && i < width) {
      if constexpr (sizeof(T) == 4) {
        sh[n] = *reinterpret_cast<const f32x4*>(shared + (size_t)t * width + i);
      } else {
        const bf16x4 v = *reinterpret_cast<const bf16x4*>(shared + (size_t)t * width + i);
        sh[n] = f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
      }
    }
  }
  const float sg = shared ? (shared_gate ? 1.f / (1.f + expf(-shared_gate[(size_t)t * ldg])) : 1.f) : 0.f;
  for (int j = 0; j < top; ++j) {
    const float wj = weights ? weights[(size_t)t * top + j] : 1.f;  // no weights: the plain sum
    const float* row = y + ((size_t)t * top + j) * width;
    // a choice past the experts is an identity expert: its output is the token's input
    const bool same = ids != nullptr && ids[(size_t)t * top + j] >= n_experts;
#pragma unroll
    for (int n = 0; n < KEEP; ++n) {
      const int i = (threadIdx.x + n * 256) * 4;
      if (i < width) {
        f32x4 v;
        if (same) {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = to_f32(x_in[(size_t)t * ldx + i + e]);
        } else {
          v = *reinterpret_cast<const f32x4*>(row + i);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[n][e] = fmaf(wj, v[e], acc[n][e]);
      }
    }
  }
#pragma unroll
  for (int n = 0; n < KEEP; ++n) {
    const int i = (threadIdx.x + n * 256) * 4;
    if (i < width) {
      f32x4 r;
#pragma unroll
      for (int e = 0; e < 4; ++e) r[e] = fmaf(sg, sh[n][e], acc[n][e]);
      if constexpr (sizeof(T) == 4) {
        *reinterpret_cast<f32x4*>(out + (size_t)t * width + i) = r;
      } else {
        *reinterpret_cast<bf16x4*>(out + (size_t)t * width + i) = bf16x4{(bf16)r[0], (bf16)r[1], (bf16)r[2], (bf16)r[3]};
      }
    }
  }
}

extern "C" int fmsamd_moe_combine(const float* y, const float* weights, int top, const void* shared, const float* shared_gate,
                                  long ldg, void* out, int dtype, int n_tokens, int width, const int* ids, int n_experts,
                                  const void* x_in, long ldx, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  FMS_REQUIRE(n_tokens > 0 && top > 0 && width > 0, "moe_combine: bad sizes T=%d top=%d width=%d", n_tokens, top, width);
  FMS_REQUIRE(ids == nullptr || (x_in != nullptr && ldx >= width && n_experts >= 0), "moe_combine: identity experts need the tokens' inputs");
  if (width <= 1024 * 4 && width % 4 == 0 && dtype == FMS_F32)
    combine_small_kernel<float, 4><<<n_tokens, 256, 0, stream>>>(y, weights, top, (const float*)shared, shared_gate, ldg, (float*)out, width, ids, n_experts, (const float*)x_in, ldx);
  else if (width <= 1024 * 4 && width % 4 == 0 && dtype == FMS_BF16)
    combine_small_kernel<bf16, 4><<<n_tokens, 256, 0, stream>>>(y, weights, top, (const bf16*)shared, shared_gate, ldg, (bf16*)out, width, ids, n_experts, (const bf16*)x_in, ldx);
  else if (dtype == FMS_F32)
    combine_kernel<float><<<n_tokens, 256, 0, stream>>>(y, weights, top, (const float*)shared, shared_gate, ldg, (float*)out, width, ids, n_experts, (const float*)x_in, ldx);
  else if (dtype == FMS_BF16)
    combine_kernel<bf16><<<n_tokens, 256, 0, stream>>>(y, weights, top, (const bf16*)shared, shared_gate, ldg, (bf16*)out, width, ids, n_experts, (const bf16*)x_in, ldx);
  else
    FMS_REQUIRE(false, "moe_combine: unknown dtype %d", dtype);
  FMS_LAUNCH_CHECK("moe_combine");
  return 0;
}
