// Attention over a latent cache: every token leaves one row [latent (R) | rotated shared key part (P)] in the
// cache, and all query heads read that one row.  With per-head matrices Uk [D, R] (keys) and Uv [V, R] (values)
//   score(t, j, h) = (q_plain . Uk_h c_j + q_rot . k_rot_j) * scale = ((Uk_h^T q_plain) . c_j + q_rot . k_rot_j) * scale
//   out(t, h)      = Uv_h sum_j p_j c_j
// so the kernels never expand keys or values: the query goes into the latent space once per token and head, attention
// runs as one shared "kv head" with keys of R + P and values of R elements (the first R of the same row), and the
// result leaves the latent space once per token and head.  Whole prompts, portions and single tokens run the same way.
//
// The softmax may have a sink: a learned logit per head that counts once in the denominator and has no value.  It is
// the state in which the running maximum and sum start.
//
//   latent_kv_write:      RMS norm of the latent, rotation of the shared key part, row written into its page
//   latent_q_rotate:      the rotated part of every head's query into its place behind the latent part
//   headwise_linear:      y[t, h, :] = W_h x[t, h, :] (optionally times sigmoid(gate[t, h])), FMA or MFMA
//   latent_attn_generic:  float32 arithmetic on any storage type; one block per (head, token)
//   latent_attn_mfma:     bfloat16, MFMA 16x16x32; a wave owns 16 heads of one token (+ merge of partial results)
//
// Cache layout: rows [page][token in page][R + P]; for the MFMA kernel also the latent transposed, [page][R][token in
// page], so that both products read their contraction index contiguously, straight from global memory.
#include "common.h"
#include "fmsamd.h"
#include "tile_product.h"

// --------------------------------------------------------------------------
// cache write
// --------------------------------------------------------------------------
template <typename CT>
__global__ void __launch_bounds__(256)
    latent_kv_write_kernel(const float* __restrict__ down, long ld, int col0, int rank, int rot, const void* __restrict__ w,
                           int w_dtype, float eps, const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                           const int* __restrict__ block_table, int table_stride, const float* __restrict__ cos_t,
                           const float* __restrict__ sin_t, CT* __restrict__ cache, CT* __restrict__ vt_cache) {
  __shared__ float scratch[17];
  const int t = blockIdx.x;
  const int seq = seq_of_token[t];
  if (seq < 0) return;
  const int pos = positions[t];
  const int page = block_table[(size_t)seq * table_stride + pos / PAGE_TOKENS];
  if (page < 0) return;
  const float* x = down + (size_t)t * ld + col0;
  CT* row = cache + ((size_t)page * PAGE_TOKENS + pos % PAGE_TOKENS) * (rank + rot);
  float sq = 0.f;
  for (int i = threadIdx.x; i < rank; i += blockDim.x) sq = fmaf(x[i], x[i], sq);
  const float rs = rsqrtf(block_sum(sq, scratch) / (float)rank + eps);
  for (int i = threadIdx.x; i < rank; i += blockDim.x) {
    const float wi = w == nullptr ? 1.f : (w_dtype == FMS_F32 ? ((const float*)w)[i] : (float)((const bf16*)w)[i]);
    const CT c = from_f32<CT>(x[i] * rs * wi);
    row[i] = c;
    // the latent once more with the tokens of a page side by side, [page][rank][token]: the layout from which the
    // second product of the MFMA kernel loads its operand without a transposition
    if (vt_cache) vt_cache[((size_t)page * rank + i) * PAGE_TOKENS + pos % PAGE_TOKENS] = c;
  }
  const int half = rot / 2;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const float c = cos_t[(size_t)pos * half + i], s = sin_t[(size_t)pos * half + i];
    const float u = x[rank + 2 * i], v = x[rank + 2 * i + 1];
    row[rank + 2 * i] = from_f32<CT>(u * c - v * s);
    row[rank + 2 * i + 1] = from_f32<CT>(v * c + u * s);
  }
}

extern "C" int fmsamd_latent_kv_write(const float* down, long ld, int col0, int rank, int rot, const void* norm_weight,
                                      int weight_dtype, float eps, const int* positions, const int* seq_of_token,
                                      const int* block_table, int table_stride, const float* cos_t, const float* sin_t,
                                      int max_pos, void* cache, void* vt_cache, int cache_dtype, int n_tokens,
                                      hipStream_t stream) {
  if (n_tokens == 0) return 0;
  FMS_REQUIRE(n_tokens > 0 && rank > 0 && rot >= 0 && rot % 2 == 0 && col0 >= 0 && ld >= col0 + rank + rot,
              "latent_kv_write: bad sizes T=%d rank=%d rot=%d col0=%d ld=%ld", n_tokens, rank, rot, col0, ld);
  FMS_REQUIRE(rot == 0 || (cos_t != nullptr && sin_t != nullptr && max_pos > 0), "latent_kv_write: a rotation needs its tables");
  if (cache_dtype == FMS_F32)
    latent_kv_write_kernel<float><<<n_tokens, 256, 0, stream>>>(down, ld, col0, rank, rot, norm_weight, weight_dtype, eps,
                                                                positions, seq_of_token, block_table, table_stride, cos_t,
                                                                sin_t, (float*)cache, (float*)vt_cache);
  else if (cache_dtype == FMS_BF16)
    latent_kv_write_kernel<bf16><<<n_tokens, 256, 0, stream>>>(down, ld, col0, rank, rot, norm_weight, weight_dtype, eps,
                                                               positions, seq_of_token, block_table, table_stride, cos_t,
                                                               sin_t, (bf16*)cache, (bf16*)vt_cache);
  else
    FMS_REQUIRE(false, "latent_kv_write: unknown dtype %d", cache_dtype);
  FMS_LAUNCH_CHECK("latent_kv_write");
  return 0;
}

// --------------------------------------------------------------------------
// queries: q [T, H, D + P] -> qa[t, h, R : R + P] = rotate(q[t, h, D : D + P])
// --------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
    latent_q_rotate_kernel(const T* __restrict__ q, long ldq, int nheads, int dim, int rot, T* __restrict__ qa, long ldqa,
                           int rank, const int* __restrict__ positions, const float* __restrict__ cos_t,
                           const float* __restrict__ sin_t) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int half = rot / 2;
  for (int i = threadIdx.x; i < nheads * half; i += blockDim.x) {
    const int h = i / half, p = i % half;
    const T* src = q + (size_t)t * ldq + (size_t)h * (dim + rot) + dim + 2 * p;
    T* dst = qa + (size_t)t * ldqa + (size_t)h * (rank + rot) + rank + 2 * p;
    const float c = cos_t[(size_t)pos * half + p], s = sin_t[(size_t)pos * half + p];
    const float u = to_f32(src[0]), v = to_f32(src[1]);
    dst[0] = from_f32<T>(u * c - v * s);
    dst[1] = from_f32<T>(v * c + u * s);
  }
}

extern "C" int fmsamd_latent_q_rotate(const void* q, long ldq, int dtype, int nheads, int dim, int rot, void* qa, long ldqa,
                                      int rank, const int* positions, const float* cos_t, const float* sin_t, int max_pos,
                                      int n_tokens, hipStream_t stream) {
  if (n_tokens == 0 || rot == 0) return 0;
  FMS_REQUIRE(n_tokens > 0 && nheads > 0 && dim >= 0 && rot > 0 && rot % 2 == 0 && rank > 0, "latent_q_rotate: bad sizes");
  FMS_REQUIRE(ldq >= (long)nheads * (dim + rot) && ldqa >= (long)nheads * (rank + rot), "latent_q_rotate: rows too short");
  FMS_REQUIRE(cos_t != nullptr && sin_t != nullptr && max_pos > 0, "latent_q_rotate: a rotation needs its tables");
  if (dtype == FMS_F32)
    latent_q_rotate_kernel<float><<<n_tokens, 256, 0, stream>>>((const float*)q, ldq, nheads, dim, rot, (float*)qa, ldqa, rank,
                                                                positions, cos_t, sin_t);
  else if (dtype == FMS_BF16)
    latent_q_rotate_kernel<bf16><<<n_tokens, 256, 0, stream>>>((const bf16*)q, ldq, nheads, dim, rot, (bf16*)qa, ldqa, rank,
                                                               positions, cos_t, sin_t);
  else
    FMS_REQUIRE(false, "latent_q_rotate: unknown dtype %d", dtype);
  FMS_LAUNCH_CHECK("latent_q_rotate");
  return 0;
}

// --------------------------------------------------------------------------
// y[t, h, n] = sum_k x[t, h, k] W[h, n, k]  (* sigmoid(gate[t, h]))
// --------------------------------------------------------------------------
struct HeadwiseArgs {
  const void* x;
  long ldx, xs;  // row stride, head stride of x (elements)
  const void* w;  // [H, N, K]
  void* y;
  long ldy, ys;
  const float* gate;  // logits [T, ldg] or null
  long ldg;
  int T, H, N, K;
};

template <typename T>
__global__ void __launch_bounds__(TILE_THREADS) headwise_fma_kernel(HeadwiseArgs a) {
  const int t0 = blockIdx.x * TILE_ROWS, h = blockIdx.y, n0 = blockIdx.z * TILE_FMA_COLS;
  const T* x = (const T*)a.x + (size_t)h * a.xs;
  const T* w = (const T*)a.w + (size_t)h * a.N * a.K;
  float acc[4];
  tile_product_fma<T>([&](int m) { return t0 + m < a.T ? x + (size_t)(t0 + m) * a.ldx : (const T*)nullptr; },
                      [&](int n) { return n0 + n < a.N ? w + (size_t)(n0 + n) * a.K : (const T*)nullptr; }, a.K, acc);
  const int n = n0 + threadIdx.x % 64;
  if (n >= a.N) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = t0 + (threadIdx.x / 64) * 4 + i;
    if (t < a.T) {
      float v = acc[i];
      if (a.gate) v *= 1.f / (1.f + expf(-a.gate[(size_t)t * a.ldg + h]));
      ((T*)a.y)[(size_t)t * a.ldy + (size_t)h * a.ys + n] = from_f32<T>(v);
    }
  }
}

__global__ void __launch_bounds__(TILE_THREADS) headwise_mfma_kernel(HeadwiseArgs a) {
  const int t0 = blockIdx.x * TILE_ROWS, h = blockIdx.y, n0 = blockIdx.z * TILE_MFMA_COLS;
  const bf16* x = (const bf16*)a.x + (size_t)h * a.xs;
  const bf16* w = (const bf16*)a.w + (size_t)h * a.N * a.K;
  f32x4 acc[TILE_MFMA_WAVE_TILES];
  tile_product_mfma([&](int m) { return t0 + m < a.T ? x + (size_t)(t0 + m) * a.ldx : (const bf16*)nullptr; },
                    [&](int n) { return n0 + n < a.N ? w + (size_t)(n0 + n) * a.K : (const bf16*)nullptr; }, a.K, acc);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = t0 + (lane >> 4) * 4 + i;
    if (t >= a.T) continue;
    const float g = a.gate ? 1.f / (1.f + expf(-a.gate[(size_t)t * a.ldg + h])) : 1.f;
#pragma unroll
    for (int tl = 0; tl < TILE_MFMA_WAVE_TILES; ++tl) {
      const int n = n0 + wave * (16 * TILE_MFMA_WAVE_TILES) + tl * 16 + (lane & 15);
      if (n < a.N) ((bf16*)a.y)[(size_t)t * a.ldy + (size_t)h * a.ys + n] = (bf16)(acc[tl][i] * g);
    }
  }
}

// The same on tiles of 64 tokens (a wave 32 x 64), for steps of many tokens: a head's weights are read once for 64
// tokens instead of once for 16.
__global__ void __launch_bounds__(TILE_THREADS) headwise_mfma_wide_kernel(HeadwiseArgs a) {
  const int t0 = blockIdx.x * TILE_WIDE_ROWS, h = blockIdx.y, n0 = blockIdx.z * TILE_MFMA_COLS;
  const bf16* x = (const bf16*)a.x + (size_t)h * a.xs;
  const bf16* w = (const bf16*)a.w + (size_t)h * a.N * a.K;
  f32x4 acc[2][4];
  tile_product_mfma_wide([&](int m) { return t0 + m < a.T ? x + (size_t)(t0 + m) * a.ldx : (const bf16*)nullptr; },
                         [&](int n) { return n0 + n < a.N ? w + (size_t)(n0 + n) * a.K : (const bf16*)nullptr; }, a.K, acc);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int t = t0 + (wave >> 1) * 32 + mt * 16 + (lane >> 4) * 4 + i;
      if (t >= a.T) continue;
      const float g = a.gate ? 1.f / (1.f + expf(-a.gate[(size_t)t * a.ldg + h])) : 1.f;
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        const int n = n0 + (wave & 1) * 64 + nt * 16 + (lane & 15);
        if (n < a.N) ((bf16*)a.y)[(size_t)t * a.ldy + (size_t)h * a.ys + n] = (bf16)(acc[mt][nt][i] * g);
      }
    }
  }
}

extern "C" int fmsamd_headwise_linear(const void* x, long ldx, long x_head_stride, const void* w, void* y, long ldy,
                                      long y_head_stride, const float* gate, long ldg, int dtype, int n_tokens, int nheads,
                                      int N, int K, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  FMS_REQUIRE(n_tokens > 0 && nheads > 0 && nheads <= 65535 && N > 0 && K > 0, "headwise_linear: bad sizes T=%d H=%d N=%d K=%d",
              n_tokens, nheads, N, K);
  FMS_REQUIRE(ldx >= (nheads - 1) * x_head_stride + K && ldy >= (nheads - 1) * y_head_stride + N,
              "headwise_linear: rows too short for %d heads", nheads);
  HeadwiseArgs a{x, ldx, x_head_stride, w, y, ldy, y_head_stride, gate, ldg, n_tokens, nheads, N, K};
  const int row_tiles = ceil_div(n_tokens, TILE_ROWS);
  if (dtype == FMS_F32) {
    headwise_fma_kernel<float><<<dim3(row_tiles, nheads, ceil_div(N, TILE_FMA_COLS)), TILE_THREADS, 0, stream>>>(a);
  } else if (dtype == FMS_BF16) {
    const bool aligned = K % 8 == 0 && ldx % 8 == 0 && x_head_stride % 8 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0;
    if (aligned && n_tokens >= 2 * TILE_WIDE_ROWS)
      headwise_mfma_wide_kernel<<<dim3(ceil_div(n_tokens, TILE_WIDE_ROWS), nheads, ceil_div(N, TILE_MFMA_COLS)), TILE_THREADS, 0, stream>>>(a);
    else if (aligned)
      headwise_mfma_kernel<<<dim3(row_tiles, nheads, ceil_div(N, TILE_MFMA_COLS)), TILE_THREADS, 0, stream>>>(a);
    else
      headwise_fma_kernel<bf16><<<dim3(row_tiles, nheads, ceil_div(N, TILE_FMA_COLS)), TILE_THREADS, 0, stream>>>(a);
  } else {
    FMS_REQUIRE(false, "headwise_linear: unknown dtype %d", dtype);
  }
  FMS_LAUNCH_CHECK("headwise_linear");
  return 0;
}

// --------------------------------------------------------------------------
// generic attention: one block per (head, token), keys 256 at a time
// --------------------------------------------------------------------------
#define LAT_THREADS 256
#define LAT_MAX_RANK 1024  // 4 output elements a thread

template <typename T>
__global__ void __launch_bounds__(LAT_THREADS)
    latent_attn_generic_kernel(const T* __restrict__ qa, long ldq, T* __restrict__ out, long ldo,
                               const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                               const int* __restrict__ block_table, int table_stride, const T* __restrict__ cache,
                               const float* __restrict__ sink, int rank, int rot, float scale, int window) {
  extern __shared__ float qs[];  // rank + rot
  __shared__ float ps[LAT_THREADS];
  __shared__ float scratch[17];
  const int h = blockIdx.x, t = blockIdx.y;
  const int width = rank + rot;
  const int seq = seq_of_token[t];
  T* o = out + (size_t)t * ldo + (size_t)h * rank;
  if (seq < 0) {
    for (int d = threadIdx.x; d < rank; d += blockDim.x) o[d] = from_f32<T>(0.f);
    return;
  }
  const int pos = positions[t];
  const int lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;
  const int* bt = block_table + (size_t)seq * table_stride;
  const T* qrow = qa + (size_t)t * ldq + (size_t)h * width;
  for (int d = threadIdx.x; d < width; d += blockDim.x) qs[d] = to_f32(qrow[d]);
  __syncthreads();

  // the sink is where the softmax starts: a logit that is already in the denominator, with no value
  float m_run = sink ? sink[h] : -1e30f, l_run = sink ? 1.f : 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  const int first = lo - lo % PAGE_TOKENS;  // chunks begin at a page's first token
  for (int base = first; base <= pos; base += LAT_THREADS) {
    const int j = base + threadIdx.x;
    float s = -INFINITY;
    if (j >= lo && j <= pos) {
      const T* krow = cache + (readable_page(bt[j / PAGE_TOKENS]) * PAGE_TOKENS + j % PAGE_TOKENS) * width;
      float dot = 0.f;
      for (int d = 0; d < width; ++d) dot = fmaf(qs[d], to_f32(krow[d]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m_run, block_max(s, scratch));
    const float p = (j >= lo && j <= pos) ? expf(s - m_new) : 0.f;
    const float alpha = expf(m_run - m_new);
    ps[threadIdx.x] = p;
    const float psum = block_sum(p, scratch);  // has the barriers that publish ps
    l_run = l_run * alpha + psum;
    m_run = m_new;
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] *= alpha;
    const int n = pos - base + 1 < LAT_THREADS ? pos - base + 1 : LAT_THREADS;
    for (int pg = 0; pg * PAGE_TOKENS < n; ++pg) {
      const T* prow = cache + readable_page(bt[base / PAGE_TOKENS + pg]) * PAGE_TOKENS * width;
      const int cnt = n - pg * PAGE_TOKENS < PAGE_TOKENS ? n - pg * PAGE_TOKENS : PAGE_TOKENS;
      for (int i = 0; i < cnt; ++i) {
        const float pi = ps[pg * PAGE_TOKENS + i];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int d = threadIdx.x + e * LAT_THREADS;
          if (d < rank) acc[e] = fmaf(pi, to_f32(prow[(size_t)i * width + d]), acc[e]);
        }
      }
    }
    __syncthreads();  // ps is overwritten by the next chunk
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int d = threadIdx.x + e * LAT_THREADS;
    if (d < rank) o[d] = from_f32<T>(l_run > 0.f ? acc[e] / l_run : 0.f);
  }
}

extern "C" int fmsamd_latent_attn_generic(const void* qa, long ldq, void* out, long ldo, int dtype, const int* positions,
                                          const int* seq_of_token, const int* block_table, int table_stride,
                                          const void* cache, const float* sink, int n_tokens, int nheads, int rank, int rot,
                                          float scale, int window, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  FMS_REQUIRE(n_tokens > 0 && n_tokens <= 65535 && nheads > 0, "latent_attn_generic: %d tokens, %d heads (at most 65535 tokens a launch)",
              n_tokens, nheads);
  FMS_REQUIRE(rank > 0 && rank <= LAT_MAX_RANK && rot >= 0 && rank + rot <= 2048, "latent_attn_generic: latent size %d (at most %d), rotated size %d",
              rank, LAT_MAX_RANK, rot);
  FMS_REQUIRE(ldq >= (long)nheads * (rank + rot) && ldo >= (long)nheads * rank, "latent_attn_generic: rows too short");
  FMS_REQUIRE(window >= 0, "latent_attn_generic: window %d", window);
  const dim3 grid(nheads, n_tokens);
  const size_t lds = (size_t)(rank + rot) * sizeof(float);
  if (dtype == FMS_F32)
    latent_attn_generic_kernel<float><<<grid, LAT_THREADS, lds, stream>>>((const float*)qa, ldq, (float*)out, ldo, positions,
                                                                          seq_of_token, block_table, table_stride,
                                                                          (const float*)cache, sink, rank, rot, scale, window);
  else if (dtype == FMS_BF16)
    latent_attn_generic_kernel<bf16><<<grid, LAT_THREADS, lds, stream>>>((const bf16*)qa, ldq, (bf16*)out, ldo, positions,
                                                                         seq_of_token, block_table, table_stride,
                                                                         (const bf16*)cache, sink, rank, rot, scale, window);
  else
    FMS_REQUIRE(false, "latent_attn_generic: unknown dtype %d", dtype);
  FMS_LAUNCH_CHECK("latent_attn_generic");
  return 0;
}


// --------------------------------------------------------------------------
// bfloat16 MFMA kernel.  A wave owns one token and 16 of its heads (the columns of its tiles) and walks over tiles of
// 32 keys.  S^T = K Q^T (rows: keys, columns: heads) leaves the probabilities in the accumulator in the operand
// layout of O^T = C^T P^T, so nothing goes through LDS.  The 32 keys of a tile are dealt to the two score tiles so
// that a lane's eight probabilities are eight consecutive keys: tile a has the keys 8g + i, tile b the keys
// 8g + 4 + i (g, i < 4).
//
// Two ways to share the work of a block's four waves:
//   * prompts: each wave another (token, head group); every wave walks all keys of its token (the waves of a block
//     read the same rows, which the caches serve);
//   * single tokens: all waves of a block, and the blocks of several splits, share one (token, head group) and deal
//     its key tiles out in turn; every part leaves (maximum, sum, unnormalised result) in a workspace and a second
//     kernel merges them.
// The sink starts the maximum of every part and is counted in the sum of part 0 only.
// --------------------------------------------------------------------------
#define LAT_EMPTY -1e30f

// The state of a wave's 16 columns, and one tile of 32 keys worked into it.  load_k(which, c) gives this lane's eight
// elements c * 32 + grp * 8 .. of its row of score tile a (which 0) or b (1); load_v(dt) its eight keys grp * 8 .. of
// latent element dt * 16 + col.  Loads are asked for in groups (KG steps of K, VG tiles of the latent) before the
// first of a group is multiplied: with the accumulators of a large latent a wave has a SIMD to itself, and the loads
// it keeps in flight are all that hides the memory's latency.
template <int RT, int WC>
struct LatentState {
  f32x4 acc[RT];
  float m, l;
};

// EXACT: the latent has exactly RT * 16 elements and a row exactly WC * 32, so no product of the loops below has
// to be asked whether it exists (each such question is a branch around a matrix instruction).
template <int RT, int WC, int KG, int VG, bool EXACT, typename LoadQ, typename LoadK, typename LoadV>
__device__ __forceinline__ void latent_tile(LatentState<RT, WC>& st, LoadQ load_q, LoadK load_k, LoadV load_v, int base,
                                            int lo, int pos, int rank, int width, float scale, int grp) {
  f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int c0 = 0; c0 < WC; c0 += KG) {
    bf16x8 ka[KG], kb[KG];
#pragma unroll
    for (int c = 0; c < KG; ++c) {
      if (c0 + c < WC && (EXACT || (c0 + c) * 32 < width)) ka[c] = load_k(0, c0 + c), kb[c] = load_k(1, c0 + c);
    }
#pragma unroll
    for (int c = 0; c < KG; ++c) {
      if (c0 + c < WC && (EXACT || (c0 + c) * 32 < width)) {
        const bf16x8 q = load_q(c0 + c);
        sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[c], q, sa, 0, 0, 0);
        sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb[c], q, sb, 0, 0, 0);
      }
    }
  }
  // this lane's scores: keys base + 8 grp + i (sa) and base + 8 grp + 4 + i (sb) of its column
  float s[8];
  float top = -INFINITY;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int ja = base + 8 * grp + i, jb = ja + 4;
    s[i] = (ja >= lo && ja <= pos) ? sa[i] * scale : -INFINITY;
    s[4 + i] = (jb >= lo && jb <= pos) ? sb[i] * scale : -INFINITY;
    top = fmaxf(top, fmaxf(s[i], s[4 + i]));
  }
  top = fmaxf(top, __shfl_xor(top, 16, WAVE));
  top = fmaxf(top, __shfl_xor(top, 32, WAVE));
  const float m_new = fmaxf(st.m, top);
  const float alpha = __expf(st.m - m_new);
  float psum = 0.f;
  bf16x8 pmat;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float p = __expf(s[i] - m_new);  // exp(-inf) = 0 for the keys that are not seen
    psum += p;
    pmat[i] = (bf16)p;
  }
  st.l = st.l * alpha + psum;
  st.m = m_new;
  // Once a column's maximum has settled, alpha is one: the accumulators (which live in the matrix unit's registers
  // and have to be moved out and back to be scaled) are left alone unless some column's maximum rose.
  const bool rescale = __any(alpha != 1.f);
#pragma unroll
  for (int d0 = 0; d0 < RT; d0 += VG) {
    bf16x8 v[VG];
#pragma unroll
    for (int dt = 0; dt < VG; ++dt) {
      if (d0 + dt < RT && (EXACT || (d0 + dt) * 16 < rank)) v[dt] = load_v(d0 + dt);
    }
#pragma unroll
    for (int dt = 0; dt < VG; ++dt) {
      if (d0 + dt < RT && (EXACT || (d0 + dt) * 16 < rank)) {
        if (rescale) {
#pragma unroll
          for (int i = 0; i < 4; ++i) st.acc[d0 + dt][i] *= alpha;
        }
        st.acc[d0 + dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v[dt], pmat, st.acc[d0 + dt], 0, 0, 0);
      }
    }
  }
}

// What a wave leaves: the normalised result (one part) or its part's maximum, sum and unnormalised result.
template <int RT, int WC, bool EXACT>
__device__ __forceinline__ void latent_finish(LatentState<RT, WC>& st, bf16* __restrict__ out, long ldo, float* __restrict__ ws, int t,
                                              int head, int nheads, int rank, int n_parts, int part, int grp) {
  st.l += __shfl_xor(st.l, 16, WAVE);
  st.l += __shfl_xor(st.l, 32, WAVE);
  if (head >= nheads) return;
  // acc[dt][i] is element d = dt * 16 + grp * 4 + i of this lane's column
  if (n_parts == 1) {
    const float inv = st.l > 0.f ? 1.f / st.l : 0.f;
    bf16* o = out + (size_t)t * ldo + (size_t)head * rank;
#pragma unroll
    for (int dt = 0; dt < RT; ++dt) {
      if (EXACT || dt * 16 < rank) {
        bf16x4 r = {(bf16)(st.acc[dt][0] * inv), (bf16)(st.acc[dt][1] * inv), (bf16)(st.acc[dt][2] * inv), (bf16)(st.acc[dt][3] * inv)};
        *reinterpret_cast<bf16x4*>(o + dt * 16 + grp * 4) = r;
      }
    }
  } else {
    float* w = ws + (((size_t)t * nheads + head) * n_parts + part) * (rank + 4);
    if (grp == 0) w[0] = st.m, w[1] = st.l;
#pragma unroll
    for (int dt = 0; dt < RT; ++dt) {
      if (EXACT || dt * 16 < rank) *reinterpret_cast<f32x4*>(w + 4 + dt * 16 + grp * 4) = st.acc[dt];
    }
  }
}

// LDS: the four waves of a block (four consecutive tiles of one sequence: neighbouring tokens, or the head groups of
// one token) share every tile of keys through LDS, so a tile comes from the caches once a block instead of once a
// wave; a block whose tiles lie in different sequences, and every block of a decode step, loads straight from
// global memory.
template <int RT, int WC, bool LDS, bool EXACT>
__global__ void __launch_bounds__(256)
    latent_attn_mfma_kernel(const bf16* __restrict__ qa, long ldq, bf16* __restrict__ out, long ldo, float* __restrict__ ws,
                            const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                            const int* __restrict__ block_table, int table_stride, const bf16* __restrict__ cache,
                            const bf16* __restrict__ vt_cache, const float* __restrict__ sink, int n_tokens, int nheads,
                            int rank, int width, float scale, int window, int tiles_per_token, int n_parts) {
  extern __shared__ __attribute__((aligned(16))) bf16 lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int n_tiles = n_tokens * tiles_per_token;
  int tile, part;
  if (n_parts == 1) {
    tile = blockIdx.x * 4 + wave;
    part = 0;
  } else {
    tile = blockIdx.x;
    part = blockIdx.y * 4 + wave;
  }
  // do the block's four tiles share their keys?  (every wave works that out for itself, and all agree)
  bool together = false;
  int seq = -1, pos = -1, t = 0;
  if (tile < n_tiles) {
    t = tile / tiles_per_token;
    seq = uniform_load(seq_of_token + t);
    pos = seq >= 0 ? uniform_load(positions + t) : -1;
  }
  int first_pos = 0x7fffffff, last_pos = -1;
  if (LDS) {
    together = true;
    int common = -2;
    for (int w = 0; w < 4; ++w) {
      const int tl = blockIdx.x * 4 + w;
      if (tl >= n_tiles) continue;
      const int tt = tl / tiles_per_token;
      const int sq = uniform_load(seq_of_token + tt);
      if (sq < 0) continue;
      if (common == -2) common = sq;
      together = together && sq == common;
      const int p = uniform_load(positions + tt);
      first_pos = p < first_pos ? p : first_pos;
      last_pos = p > last_pos ? p : last_pos;
    }
    together = together && common >= 0;
  }
  const int head = (tile % tiles_per_token) * 16 + col;
  const bool valid = tile < n_tiles && seq >= 0 && head < nheads;
  if (!(LDS && together)) {
    if (tile >= n_tiles) return;
    if (seq < 0) {
      if (n_parts == 1 && head < nheads) {
        for (int d = grp; d < rank; d += 4) out[(size_t)t * ldo + (size_t)head * rank + d] = (bf16)0.f;
      }
      return;
    }
  }
  const int lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;

  // The wave's queries wait in LDS, each lane's eight elements of every step of K in a slot of its own (written and
  // read by the same lane: no barrier): in registers they would crowd out the loads that have to be in flight.
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  bf16* q_lds = lds + ((size_t)wave * WC * 64 + lane) * 8;
  {
    const bf16* qrow = qa + (size_t)t * ldq + (size_t)(valid ? head : 0) * width;
#pragma unroll
    for (int c = 0; c < WC; ++c) {
      const int k = c * 32 + grp * 8;
      *reinterpret_cast<bf16x8*>(q_lds + c * 64 * 8) = (valid && (EXACT || k < width)) ? *reinterpret_cast<const bf16x8*>(qrow + k) : zero8;
    }
  }
  auto load_q = [&](int c) { return *reinterpret_cast<const bf16x8*>(q_lds + c * 64 * 8); };
  LatentState<RT, WC> st;
#pragma unroll
  for (int dt = 0; dt < RT; ++dt) st.acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  st.m = (sink && valid) ? sink[head] : LAT_EMPTY;
  st.l = (sink && valid && part == 0 && grp == 0) ? 1.f : 0.f;
  const int key_a = 8 * (col >> 2) + (col & 3);  // the key of this lane's row in score tile a; tile b: + 4

  if (LDS && together) {
    // all four waves walk the keys that any of them sees; a wave's own mask hides what it must not see
    const int ks = width + 8, vs = 32 + 8;  // row strides in LDS (elements): 16 bytes of padding against bank conflicts
    bf16* k_lds = lds + 4 * WC * 64 * 8;  // behind the four waves' queries
    bf16* v_lds = k_lds + 32 * ks;
    const int first_lo = window > 0 ? (first_pos - window + 1 > 0 ? first_pos - window + 1 : 0) : 0;
    const int common_seq = uniform_load(seq_of_token + (blockIdx.x * 4 < n_tiles ? (blockIdx.x * 4) / tiles_per_token : 0));
    int any_seq = common_seq;
    if (any_seq < 0) any_seq = seq;  // the block's first tile may be a padding row
    for (int w = 0; w < 4 && any_seq < 0; ++w) {
      const int tl = blockIdx.x * 4 + w;
      if (tl < n_tiles) any_seq = uniform_load(seq_of_token + tl / tiles_per_token);
    }
    const int* bt = block_table + (size_t)any_seq * table_stride;
    const int chunks_k = width / 8;  // 16-byte pieces in a key row
    // A thread's pieces of a tile: KP 16-byte pieces of the key rows, VP of the transposed latent.  The next tile's
    // pieces are asked for before this tile is worked on and wait in registers until every wave is done with it.
    constexpr int KP = (32 * WC * 4 + 255) / 256, VP = (RT * 16 * 4 + 255) / 256;
    bf16x8 kpre[KP], vpre[VP];
    // where this thread's pieces lie in a tile of the cache and in LDS: the same for every tile (the divisions are
    // done once; -1: this thread has no such piece)
    int k_from[KP], k_to[KP], v_from[VP], v_to[VP];
#pragma unroll
    for (int n = 0; n < KP; ++n) {
      const int i = threadIdx.x + n * 256;
      const bool has = i < 32 * chunks_k;
      k_from[n] = has ? (i / chunks_k) * width + (i % chunks_k) * 8 : -1;
      k_to[n] = has ? (i / chunks_k) * ks + (i % chunks_k) * 8 : -1;
    }
#pragma unroll
    for (int n = 0; n < VP; ++n) {
      const int i = threadIdx.x + n * 256;
      const bool has = i < rank * 4;
      v_from[n] = has ? (i >> 2) * PAGE_TOKENS + (i & 3) * 8 : -1;
      v_to[n] = has ? (i >> 2) * vs + (i & 3) * 8 : -1;
    }
    auto fetch = [&](int base) {
      const size_t page = readable_page(uniform_load(bt + base / PAGE_TOKENS));
      const int in_page = base % PAGE_TOKENS;
      const bf16* kp = cache + (page * PAGE_TOKENS + in_page) * width;
      const bf16* vp = vt_cache + page * rank * PAGE_TOKENS + in_page;
#pragma unroll
      for (int n = 0; n < KP; ++n) {
        if (k_from[n] >= 0) kpre[n] = *reinterpret_cast<const bf16x8*>(kp + k_from[n]);
      }
#pragma unroll
      for (int n = 0; n < VP; ++n) {
        if (v_from[n] >= 0) vpre[n] = *reinterpret_cast<const bf16x8*>(vp + v_from[n]);
      }
    };
    const int first_base = (first_lo / 32) * 32;
    if (first_base <= last_pos) fetch(first_base);
    for (int base = first_base; base <= last_pos; base += 32) {
      __syncthreads();  // the tile before this one has been read by every wave
#pragma unroll
      for (int n = 0; n < KP; ++n) {
        if (k_to[n] >= 0) *reinterpret_cast<bf16x8*>(k_lds + k_to[n]) = kpre[n];
      }
#pragma unroll
      for (int n = 0; n < VP; ++n) {
        if (v_to[n] >= 0) *reinterpret_cast<bf16x8*>(v_lds + v_to[n]) = vpre[n];
      }
      __syncthreads();
      if (base + 32 <= last_pos) fetch(base + 32);
      // (a condition that all lanes of the wave share: matrix instructions take their operands from every lane)
      if (tile < n_tiles && seq >= 0 && base <= pos) {
        latent_tile<RT, WC, (WC <= 10 ? WC : (WC % 8 == 0 ? 8 : 6)), (RT <= 16 ? RT : 8), EXACT>(
            st, load_q,
            [&](int which, int c) {
              return (EXACT || c * 32 + grp * 8 < width) ? *reinterpret_cast<const bf16x8*>(k_lds + (key_a + 4 * which) * ks + c * 32 + grp * 8) : zero8;
            },
            [&](int dt) { return *reinterpret_cast<const bf16x8*>(v_lds + (dt * 16 + col) * vs + grp * 8); }, base, lo, pos, rank, width,
            scale, grp);
      }
    }
    if (tile >= n_tiles) return;
    if (seq < 0) {
      if (head < nheads) {
        for (int d = grp; d < rank; d += 4) out[(size_t)t * ldo + (size_t)head * rank + d] = (bf16)0.f;
      }
      return;
    }
  } else {
    const int* bt = block_table + (size_t)seq * table_stride;
    for (int kt = lo / 32 + part; kt * 32 <= pos; kt += n_parts) {
      const int base = kt * 32;
      const size_t page = readable_page(uniform_load(bt + base / PAGE_TOKENS));
      const int in_page = base % PAGE_TOKENS;
      const bf16* ka = cache + (page * PAGE_TOKENS + in_page + key_a) * width + grp * 8;
      const bf16* vt = vt_cache + (page * rank + col) * PAGE_TOKENS + in_page + grp * 8;
      // straight from global memory: half a tile of key loads, then half its latent loads, in flight at once (all of them up to medium sizes)
      latent_tile<RT, WC, (WC <= 10 ? WC : (WC % 8 == 0 ? 8 : 9)), (RT <= 16 ? RT : 16), EXACT>(
          st, load_q,
          [&](int which, int c) {
            return (EXACT || c * 32 + grp * 8 < width) ? *reinterpret_cast<const bf16x8*>(ka + which * 4 * (size_t)width + c * 32) : zero8;
          },
          [&](int dt) { return *reinterpret_cast<const bf16x8*>(vt + (size_t)dt * 16 * PAGE_TOKENS); }, base, lo, pos, rank, width, scale,
          grp);
    }
  }
  latent_finish<RT, WC, EXACT>(st, out, ldo, ws, t, head, nheads, rank, n_parts, part, grp);
}

// out[t, h, :] = sum_i acc_i exp(m_i - M) / sum_i l_i exp(m_i - M) over the parts i.  The parts' maxima and sums are
// loaded side by side (a thread a part) and their weights left in LDS: no chain of dependent loads.
#define LAT_MAX_PARTS 256
__global__ void __launch_bounds__(256)
    latent_attn_merge_kernel(const float* __restrict__ ws, bf16* __restrict__ out, long ldo, const int* __restrict__ seq_of_token,
                             int nheads, int rank, int n_parts) {
  __shared__ float weight[LAT_MAX_PARTS];
  __shared__ float inv_total;
  const int h = blockIdx.x, t = blockIdx.y;
  bf16* o = out + (size_t)t * ldo + (size_t)h * rank;
  if (seq_of_token[t] < 0) {
    for (int d = threadIdx.x; d < rank; d += blockDim.x) o[d] = (bf16)0.f;
    return;
  }
  const float* w = ws + ((size_t)t * nheads + h) * n_parts * (rank + 4);
  if (threadIdx.x < WAVE) {  // the first wave weighs the parts
    float top = LAT_EMPTY;
    for (int i = threadIdx.x; i < n_parts; i += WAVE) top = fmaxf(top, w[(size_t)i * (rank + 4)]);
    top = wave_max(top);
    float total = 0.f;
    for (int i = threadIdx.x; i < n_parts; i += WAVE) {
      const float e = __expf(w[(size_t)i * (rank + 4)] - top);
      weight[i] = e;
      total += w[(size_t)i * (rank + 4) + 1] * e;
    }
    total = wave_sum(total);
    if (threadIdx.x == 0) inv_total = total > 0.f ? 1.f / total : 0.f;
  }
  __syncthreads();
  const float inv = inv_total;
  for (int d = threadIdx.x; d < rank; d += blockDim.x) {
    float v = 0.f;
#pragma unroll 8
    for (int i = 0; i < n_parts; ++i) v = fmaf(w[(size_t)i * (rank + 4) + 4 + d], weight[i], v);
    o[d] = (bf16)(v * inv);
  }
}

// bytes of the workspace for n_splits blocks of four parts each (0: one block per four tiles, no workspace)
extern "C" long fmsamd_latent_attn_workspace(int n_tokens, int nheads, int rank, int n_splits) {
  return n_splits <= 0 ? 0 : (long)n_tokens * nheads * n_splits * 4 * (rank + 4) * (long)sizeof(float);
}

// 1 if the MFMA kernel takes these sizes
extern "C" int fmsamd_latent_attn_mfma_fits(int rank, int rot) {
  return rank > 0 && rank % 16 == 0 && rot >= 0 && (rank + rot) % 8 == 0 && rank <= 512 && rank + rot <= 576;
}

// n_splits 0: prompts (a wave per tile, every wave all keys); n_splits >= 1: single tokens (n_splits blocks of four
// waves deal a tile's keys out; workspace as fmsamd_latent_attn_workspace says)
extern "C" int fmsamd_latent_attn_mfma(const void* qa, long ldq, void* out, long ldo, void* workspace, long workspace_bytes,
                                       const int* positions, const int* seq_of_token, const int* block_table,
                                       int table_stride, const void* cache, const void* vt_cache, const float* sink,
                                       int n_tokens, int nheads, int rank, int rot, float scale, int window, int n_splits,
                                       hipStream_t stream) {
  if (n_tokens == 0) return 0;
  const int width = rank + rot;
  FMS_REQUIRE(n_tokens > 0 && nheads > 0 && fmsamd_latent_attn_mfma_fits(rank, rot), "latent_attn_mfma: sizes T=%d H=%d rank=%d rot=%d do not fit",
              n_tokens, nheads, rank, rot);
  FMS_REQUIRE(ldq >= (long)nheads * width && ldq % 8 == 0 && ldo >= (long)nheads * rank && ldo % 4 == 0 && ((uintptr_t)qa % 16) == 0,
              "latent_attn_mfma: rows too short or not aligned");
  FMS_REQUIRE(cache != nullptr && vt_cache != nullptr && window >= 0 && n_splits >= 0 && n_splits * 4 <= LAT_MAX_PARTS, "latent_attn_mfma: bad arguments (at most 64 splits)");
  const int tiles_per_token = ceil_div(nheads, 16);
  const long tiles = (long)n_tokens * tiles_per_token;
  const int n_parts = n_splits == 0 ? 1 : n_splits * 4;
  FMS_REQUIRE(n_splits == 0 || (workspace != nullptr && workspace_bytes >= fmsamd_latent_attn_workspace(n_tokens, nheads, rank, n_splits)),
              "latent_attn_mfma: the workspace is too small");
  const dim3 grid(n_splits == 0 ? ceil_div(tiles, 4) : (unsigned)tiles, n_splits == 0 ? 1 : n_splits);
  FMS_REQUIRE(tiles <= 0x7fffffffL && grid.y <= 65535, "latent_attn_mfma: too many tiles for one launch");
  // LDS: every wave's queries; for prompts also a tile of 32 key rows and the same keys' latent, transposed, which the
  // waves of a block share
#define LAUNCH_LATENT(RT, WC, EXACT)                                                                                               \
  const size_t q_lds = (size_t)4 * WC * 64 * 8 * sizeof(bf16); /* the four waves' queries */                                       \
  const size_t lds = q_lds + (size_t)(32 * (width + 8) + rank * 40) * sizeof(bf16);                                                \
  static bool allowed = false; /* more than 64 KB of LDS a block has to be asked for, once a kernel */                             \
  if (!allowed) {                                                                                                                  \
    hipError_t e1 = hipFuncSetAttribute((const void*)latent_attn_mfma_kernel<RT, WC, true, EXACT>,                                 \
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);                                   \
    hipError_t e2 = hipFuncSetAttribute((const void*)latent_attn_mfma_kernel<RT, WC, false, EXACT>,                                \
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);                                   \
    FMS_REQUIRE(e1 == hipSuccess && e2 == hipSuccess, "latent_attn_mfma: the kernel's LDS could not be sized: %s",                 \
                hipGetErrorString(e1 != hipSuccess ? e1 : e2));                                                                    \
    allowed = true;                                                                                                                \
  }                                                                                                                                \
  FMS_REQUIRE(lds <= 160 * 1024, "latent_attn_mfma: %zu bytes of LDS", lds);                                                       \
  if (n_splits == 0)                                                                                                               \
    latent_attn_mfma_kernel<RT, WC, true, EXACT><<<grid, 256, lds, stream>>>(                                                      \
        (const bf16*)qa, ldq, (bf16*)out, ldo, (float*)workspace, positions, seq_of_token, block_table, table_stride,              \
        (const bf16*)cache, (const bf16*)vt_cache, sink, n_tokens, nheads, rank, width, scale, window, tiles_per_token, n_parts);  \
  else                                                                                                                             \
    latent_attn_mfma_kernel<RT, WC, false, EXACT><<<grid, 256, q_lds, stream>>>(                                                   \
        (const bf16*)qa, ldq, (bf16*)out, ldo, (float*)workspace, positions, seq_of_token, block_table, table_stride,              \
        (const bf16*)cache, (const bf16*)vt_cache, sink, n_tokens, nheads, rank, width, scale, window, tiles_per_token, n_parts)
  // the sizes of the largest configuration exactly (a latent of 512 with a rotated part of 64, or with none) and the
  // smaller latents without a rotated part run without a question around any product; everything else in the smallest
  // configuration that holds it
  if (rank == 512 && width == 576) {
    LAUNCH_LATENT(32, 18, true);
  } else if (rank == 512 && width == 512) {
    LAUNCH_LATENT(32, 16, true);
  } else if (rank == 256 && width == 256) {
    LAUNCH_LATENT(16, 8, true);
  } else if (rank == 128 && width == 128) {
    LAUNCH_LATENT(8, 4, true);
  } else if (rank <= 128 && width <= 192) {
    LAUNCH_LATENT(8, 6, false);
  } else if (rank <= 256 && width <= 320) {
    LAUNCH_LATENT(16, 10, false);
  } else {
    LAUNCH_LATENT(32, 18, false);
  }
#undef LAUNCH_LATENT
  FMS_LAUNCH_CHECK("latent_attn_mfma");
  if (n_parts > 1) {
    latent_attn_merge_kernel<<<dim3(nheads, n_tokens), rank > 128 ? 256 : 64, 0, stream>>>((const float*)workspace, (bf16*)out, ldo, seq_of_token, nheads,
                                                                         rank, n_parts);
    FMS_LAUNCH_CHECK("latent_attn_merge");
  }
  return 0;
}
