// The real-gated linear recurrent unit: a recurrence of its own for every channel,
//
//   r = sigmoid(Ra u + ba),  i = sigmoid(Ri u + bi)      Ra, Ri block-diagonal: `blocks` square matrices
//   log a = -c r softplus(lam),  a = exp(log a)
//   S <- a S + sqrt(1 - a^2) (i u),   out = S * act(y)
//
// Two kernels run a step of any number of tokens per sequence, all in float32:
//   rglru_gates: both gates of a tile of tokens and one block of channels; it leaves a and b = sqrt(1 - a^2) i u.
//                sqrt(1 - a^2) is formed as sqrt(-expm1(2 log a)), which keeps its digits where a is close to one.
//                The matrices are given transposed, [block][in][out], so that neighbouring threads read neighbouring
//                weights; the tile's inputs wait in LDS and every weight is used for all its tokens.
//                A step of few tokens has too few tiles to fill the chip: there a block takes 64 outputs of a block of
//                channels and deals the inputs out over its eight waves, whose partial sums meet in LDS.
//   rglru_scan:  S <- a S + b over the tokens of every sequence, from and into the state of its slot, times the
//                activation of the other branch, rounded once.  A thread owns a channel of a sequence and asks for
//                the operands of several tokens before it walks over them.
//   Long sequences (prompts) are cut into chunks of token rows that run side by side, in two kernels: the first leaves
//                for every chunk and channel the product of its a and the state it ends in when it starts from zero
//                (or from the sequence's stored state, if the sequence starts inside the chunk: then the product
//                counts as zero, nothing before matters); the second folds the chunks before its own back to the
//                sequence's start, which gives the state its chunk starts from, and walks the chunk again for the
//                outputs.  S_end = (prod a) S_start + L holds for every run of tokens, so the result differs from
//                the token-by-token walk by rounding only.
#include "common.h"
#include "fmsamd.h"

#define GATE_TOKENS 8
#define SCAN_AHEAD 8

__device__ __forceinline__ float rg_softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float rg_sigmoid(float z) { return 1.f / (1.f + expf(-z)); }

template <typename W>
__global__ void __launch_bounds__(256)
    rglru_gates_kernel(const float* __restrict__ u, long ldu, const W* __restrict__ ra_t, const float* __restrict__ ra_b,
                       const W* __restrict__ ri_t, const float* __restrict__ ri_b, const float* __restrict__ lam, float c,
                       const int* __restrict__ seq_of_token, float* __restrict__ a_out, float* __restrict__ b_out, int n_tokens,
                       int channels, int bw) {
  extern __shared__ float us[];  // [GATE_TOKENS][bw]
  const int t0 = blockIdx.x * GATE_TOKENS, blk = blockIdx.y;
  const int nt = min(GATE_TOKENS, n_tokens - t0);
  for (int i = threadIdx.x; i < GATE_TOKENS * bw; i += blockDim.x) {
    const int tt = i / bw, k = i - tt * bw;
    // a padding row holds nothing that anybody reads: zeros, so that its gates are numbers
    us[i] = (tt < nt && seq_of_token[t0 + tt] >= 0) ? u[(size_t)(t0 + tt) * ldu + (size_t)blk * bw + k] : 0.f;
  }
  __syncthreads();
  const W* wa = ra_t + (size_t)blk * bw * bw;
  const W* wi = ri_t + (size_t)blk * bw * bw;
  for (int o = threadIdx.x; o < bw; o += blockDim.x) {
    float ra[GATE_TOKENS], ri[GATE_TOKENS];
#pragma unroll
    for (int tt = 0; tt < GATE_TOKENS; ++tt) ra[tt] = ri[tt] = 0.f;
    for (int k = 0; k < bw; ++k) {
      const float va = to_f32(wa[(size_t)k * bw + o]), vi = to_f32(wi[(size_t)k * bw + o]);
#pragma unroll
      for (int tt = 0; tt < GATE_TOKENS; ++tt) {
        const float x = us[tt * bw + k];
        ra[tt] = fmaf(va, x, ra[tt]);
        ri[tt] = fmaf(vi, x, ri[tt]);
      }
    }
    const int ch = blk * bw + o;
    const float rate = -c * rg_softplus(lam[ch]);
    const float ba = ra_b[ch], bi = ri_b[ch];
#pragma unroll
    for (int tt = 0; tt < GATE_TOKENS; ++tt) {
      if (tt >= nt) break;
      const float log_a = rate * rg_sigmoid(ra[tt] + ba);
      const float gate = rg_sigmoid(ri[tt] + bi);
      a_out[(size_t)(t0 + tt) * channels + ch] = expf(log_a);
      b_out[(size_t)(t0 + tt) * channels + ch] = sqrtf(-expm1f(2.f * log_a)) * gate * us[tt * bw + o];
    }
  }
}

#define GATE_SLICES 8
static_assert(GATE_SLICES == GATE_TOKENS, "the waves that summed the slices finish one token each");

// Few tokens: a block of 8 waves takes 64 outputs of one block of channels for a tile of tokens; wave w sums over the
// inputs w, w + 8, ... and the eight partial sums of every (gate, token, output) meet in LDS.
template <typename W>
__global__ void __launch_bounds__(64 * GATE_SLICES)
    rglru_gates_small_kernel(const float* __restrict__ u, long ldu, const W* __restrict__ ra_t, const float* __restrict__ ra_b,
                             const W* __restrict__ ri_t, const float* __restrict__ ri_b, const float* __restrict__ lam, float c,
                             const int* __restrict__ seq_of_token, float* __restrict__ a_out, float* __restrict__ b_out,
                             int n_tokens, int channels, int bw) {
  extern __shared__ float us[];                 // [GATE_TOKENS][bw]
  float* part = us + (size_t)GATE_TOKENS * bw;  // [GATE_SLICES][2][GATE_TOKENS][64]
  const int t0 = blockIdx.x * GATE_TOKENS, blk = blockIdx.y, o0 = blockIdx.z * 64;
  const int nt = min(GATE_TOKENS, n_tokens - t0);
  for (int i = threadIdx.x; i < GATE_TOKENS * bw; i += blockDim.x) {
    const int tt = i / bw, k = i - tt * bw;
    us[i] = (tt < nt && seq_of_token[t0 + tt] >= 0) ? u[(size_t)(t0 + tt) * ldu + (size_t)blk * bw + k] : 0.f;
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, slice = threadIdx.x >> 6;
  const int o = o0 + lane;
  float ra[GATE_TOKENS], ri[GATE_TOKENS];
#pragma unroll
  for (int tt = 0; tt < GATE_TOKENS; ++tt) ra[tt] = ri[tt] = 0.f;
  if (o < bw) {
    const W* wa = ra_t + (size_t)blk * bw * bw + o;
    const W* wi = ri_t + (size_t)blk * bw * bw + o;
#pragma unroll 4
    for (int k = slice; k < bw; k += GATE_SLICES) {
      const float va = to_f32(wa[(size_t)k * bw]), vi = to_f32(wi[(size_t)k * bw]);
#pragma unroll
      for (int tt = 0; tt < GATE_TOKENS; ++tt) {
        const float x = us[tt * bw + k];
        ra[tt] = fmaf(va, x, ra[tt]);
        ri[tt] = fmaf(vi, x, ri[tt]);
      }
    }
  }
#pragma unroll
  for (int tt = 0; tt < GATE_TOKENS; ++tt) {
    part[((slice * 2 + 0) * GATE_TOKENS + tt) * 64 + lane] = ra[tt];
    part[((slice * 2 + 1) * GATE_TOKENS + tt) * 64 + lane] = ri[tt];
  }
  __syncthreads();
  const int tt = slice;  // GATE_SLICES == GATE_TOKENS: wave w finishes token w of the tile
  if (tt >= nt || o >= bw) return;
  float sa = 0.f, si = 0.f;
#pragma unroll
  for (int w = 0; w < GATE_SLICES; ++w) {
    sa += part[((w * 2 + 0) * GATE_TOKENS + tt) * 64 + lane];
    si += part[((w * 2 + 1) * GATE_TOKENS + tt) * 64 + lane];
  }
  const int ch = blk * bw + o;
  const float log_a = -c * rg_softplus(lam[ch]) * rg_sigmoid(sa + ra_b[ch]);
  const float gate = rg_sigmoid(si + ri_b[ch]);
  a_out[(size_t)(t0 + tt) * channels + ch] = expf(log_a);
  b_out[(size_t)(t0 + tt) * channels + ch] = sqrtf(-expm1f(2.f * log_a)) * gate * us[tt * bw + o];
}

extern "C" int fmsamd_rglru_gates(const float* u, long ldu, const void* ra_t, const float* ra_b, const void* ri_t,
                                  const float* ri_b, int weight_dtype, const float* lam, float c, const int* seq_of_token,
                                  float* a_out, float* b_out, int n_tokens, int channels, int blocks, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  FMS_REQUIRE(n_tokens > 0 && channels > 0 && blocks > 0 && channels % blocks == 0 && ldu >= channels,
              "rglru_gates: %d channels in %d blocks, rows of %ld", channels, blocks, ldu);
  const int bw = channels / blocks;
  FMS_REQUIRE((size_t)GATE_TOKENS * bw * sizeof(float) <= 64 * 1024, "rglru_gates: blocks of %d channels do not fit the LDS", bw);
  FMS_REQUIRE(blocks <= 65535, "rglru_gates: %d blocks are too many for one launch", blocks);
  const dim3 grid(ceil_div(n_tokens, GATE_TOKENS), blocks);
  const size_t lds = (size_t)GATE_TOKENS * bw * sizeof(float);
  const size_t small_lds = lds + (size_t)GATE_SLICES * 2 * GATE_TOKENS * 64 * sizeof(float);
  if ((long)grid.x * blocks < 1024 && small_lds <= 64 * 1024 && ceil_div(bw, 64) <= 65535) {  // too few tiles to fill the chip
    const dim3 sgrid(grid.x, blocks, ceil_div(bw, 64));
    if (weight_dtype == FMS_F32)
      rglru_gates_small_kernel<float><<<sgrid, 64 * GATE_SLICES, small_lds, stream>>>(u, ldu, (const float*)ra_t, ra_b, (const float*)ri_t,
                                                                                     ri_b, lam, c, seq_of_token, a_out, b_out, n_tokens,
                                                                                     channels, bw);
    else if (weight_dtype == FMS_BF16)
      rglru_gates_small_kernel<bf16><<<sgrid, 64 * GATE_SLICES, small_lds, stream>>>(u, ldu, (const bf16*)ra_t, ra_b, (const bf16*)ri_t, ri_b,
                                                                                    lam, c, seq_of_token, a_out, b_out, n_tokens, channels,
                                                                                    bw);
    else
      FMS_REQUIRE(false, "rglru_gates: unknown dtype %d", weight_dtype);
    FMS_LAUNCH_CHECK("rglru_gates_small");
    return 0;
  }
  if (weight_dtype == FMS_F32)
    rglru_gates_kernel<float><<<grid, 256, lds, stream>>>(u, ldu, (const float*)ra_t, ra_b, (const float*)ri_t, ri_b, lam, c,
                                                          seq_of_token, a_out, b_out, n_tokens, channels, bw);
  else if (weight_dtype == FMS_BF16)
    rglru_gates_kernel<bf16><<<grid, 256, lds, stream>>>(u, ldu, (const bf16*)ra_t, ra_b, (const bf16*)ri_t, ri_b, lam, c,
                                                         seq_of_token, a_out, b_out, n_tokens, channels, bw);
  else
    FMS_REQUIRE(false, "rglru_gates: unknown dtype %d", weight_dtype);
  FMS_LAUNCH_CHECK("rglru_gates");
  return 0;
}

template <typename T>
__global__ void __launch_bounds__(256)
    rglru_scan_kernel(const float* __restrict__ a, const float* __restrict__ b, const float* __restrict__ y, long ldy, int act,
                      float* __restrict__ state, const int* __restrict__ seq_starts, const int* __restrict__ seq_of_token,
                      const int* __restrict__ slot_ids, T* __restrict__ out, long ldo, int channels) {
  const int s = blockIdx.x;
  const int first = seq_starts[s], last = seq_starts[s + 1];
  const int ch = blockIdx.y * blockDim.x + threadIdx.x;
  if (first >= last || ch >= channels) return;
  if (seq_of_token[first] < 0) {  // a padding row of a step of fixed shape
    for (int t = first; t < last; ++t) out[(size_t)t * ldo + ch] = from_f32<T>(0.f);
    return;
  }
  float* sp = state + (size_t)slot_ids[s] * channels + ch;
  float S = *sp;
  for (int t0 = first; t0 < last; t0 += SCAN_AHEAD) {
    float av[SCAN_AHEAD], bv[SCAN_AHEAD], yv[SCAN_AHEAD];
#pragma unroll
    for (int e = 0; e < SCAN_AHEAD; ++e) {
      const int t = t0 + e;
      av[e] = bv[e] = yv[e] = 0.f;
      if (t < last) {
        av[e] = a[(size_t)t * channels + ch];
        bv[e] = b[(size_t)t * channels + ch];
        yv[e] = y[(size_t)t * ldy + ch];
      }
    }
#pragma unroll
    for (int e = 0; e < SCAN_AHEAD; ++e) {
      const int t = t0 + e;
      if (t < last) {
        S = fmaf(av[e], S, bv[e]);
        out[(size_t)t * ldo + ch] = from_f32<T>(S * fms_activate(yv[e], act));
      }
    }
  }
  *sp = S;
}

extern "C" int fmsamd_rglru_scan(const float* a, const float* b, const float* y, long ldy, int act, float* state,
                                 const int* seq_starts, const int* seq_of_token, const int* slot_ids, void* out, int out_dtype,
                                 long ldo, int n_seqs, int channels, hipStream_t stream) {
  if (n_seqs == 0) return 0;
  FMS_REQUIRE(n_seqs > 0 && channels > 0 && ldy >= channels && ldo >= channels, "rglru_scan: bad sizes seqs=%d channels=%d", n_seqs,
              channels);
  FMS_REQUIRE(act >= 0 && act <= FMS_ACT_LAST, "rglru_scan: unknown activation %d", act);
  const int threads = channels >= 256 ? 256 : 64;
  const dim3 grid(n_seqs, ceil_div(channels, threads));
  FMS_REQUIRE(grid.y <= 65535, "rglru_scan: %d channels are too many for one launch", channels);
  if (out_dtype == FMS_F32)
    rglru_scan_kernel<float><<<grid, threads, 0, stream>>>(a, b, y, ldy, act, state, seq_starts, seq_of_token, slot_ids, (float*)out,
                                                           ldo, channels);
  else if (out_dtype == FMS_BF16)
    rglru_scan_kernel<bf16><<<grid, threads, 0, stream>>>(a, b, y, ldy, act, state, seq_starts, seq_of_token, slot_ids, (bf16*)out,
                                                          ldo, channels);
  else
    FMS_REQUIRE(false, "rglru_scan: unknown dtype %d", out_dtype);
  FMS_LAUNCH_CHECK("rglru_scan");
  return 0;
}

// ---- long sequences: chunks of token rows side by side ----------------------------------------------------------------
// How many token rows a chunk of the chunked walk has; 0: the step is walked sequence by sequence (few tokens a sequence).
extern "C" int fmsamd_rglru_scan_chunk(int n_tokens, int n_seqs) {
  if (n_seqs <= 0 || n_tokens < 256 || (long)n_tokens < 128L * n_seqs) return 0;
  return n_tokens <= 8192 ? 64 : (n_tokens <= 32768 ? 128 : 256);
}

// Chunk j = token rows j * chunk .. ; a thread owns a channel of it.  Leaves P = the product of the chunk's a (0 if a
// sequence starts inside) and L = the state at the chunk's end when what came before the chunk counts as zero (from the
// stored state of a sequence that starts inside, which is also copied to init [sequence][channel] for the second kernel:
// that one overwrites the stored state).
__global__ void __launch_bounds__(256)
    rglru_chunk_sums_kernel(const float* __restrict__ a, const float* __restrict__ b, const float* __restrict__ state,
                            const int* __restrict__ seq_of_token, const int* __restrict__ slot_ids, float* __restrict__ P_ws,
                            float* __restrict__ L_ws, float* __restrict__ init, int n_tokens, int channels, int chunk) {
  const int j = blockIdx.x, ch = blockIdx.y * blockDim.x + threadIdx.x;
  if (ch >= channels) return;
  const int first = j * chunk, last = min(first + chunk, n_tokens);
  int prev = first > 0 ? seq_of_token[first - 1] : -2;
  float S = 0.f, P = 1.f;
  for (int t0 = first; t0 < last; t0 += SCAN_AHEAD) {
    float av[SCAN_AHEAD], bv[SCAN_AHEAD];
#pragma unroll
    for (int e = 0; e < SCAN_AHEAD; ++e) {
      const int t = t0 + e;
      av[e] = 1.f, bv[e] = 0.f;
      if (t < last) av[e] = a[(size_t)t * channels + ch], bv[e] = b[(size_t)t * channels + ch];
    }
#pragma unroll
    for (int e = 0; e < SCAN_AHEAD; ++e) {
      const int t = t0 + e;
      if (t >= last) break;
      const int sq = seq_of_token[t];
      if (sq >= 0) {
        if (sq != prev) {
          const float s0 = state[(size_t)slot_ids[sq] * channels + ch];
          init[(size_t)sq * channels + ch] = s0;
          S = s0, P = 0.f;
        }
        S = fmaf(av[e], S, bv[e]);
        P *= av[e];
      }
      prev = sq;
    }
  }
  P_ws[(size_t)j * channels + ch] = P;
  L_ws[(size_t)j * channels + ch] = S;
}

template <typename T>
__global__ void __launch_bounds__(256)
    rglru_chunk_walk_kernel(const float* __restrict__ a, const float* __restrict__ b, const float* __restrict__ y, long ldy, int act,
                            float* __restrict__ state, const int* __restrict__ seq_starts, const int* __restrict__ seq_of_token,
                            const int* __restrict__ slot_ids, const float* __restrict__ P_ws, const float* __restrict__ L_ws,
                            const float* __restrict__ init, T* __restrict__ out, long ldo, int n_tokens, int channels, int chunk) {
  const int j = blockIdx.x, ch = blockIdx.y * blockDim.x + threadIdx.x;
  if (ch >= channels) return;
  const int first = j * chunk, last = min(first + chunk, n_tokens);
  int prev = first > 0 ? seq_of_token[first - 1] : -2;
  // the state the chunk starts from: the chunks before it, back to the one in which its first token's sequence starts
  float S = 0.f;
  const int sq0 = seq_of_token[first];
  if (sq0 >= 0 && sq0 == prev) {
    const int k0 = seq_starts[sq0] / chunk;
    float m = 1.f;
    for (int k = j - 1; k >= k0; --k) {
      S = fmaf(m, L_ws[(size_t)k * channels + ch], S);
      m *= P_ws[(size_t)k * channels + ch];
    }
  }
  for (int t0 = first; t0 < last; t0 += SCAN_AHEAD) {
    float av[SCAN_AHEAD], bv[SCAN_AHEAD], yv[SCAN_AHEAD];
#pragma unroll
    for (int e = 0; e < SCAN_AHEAD; ++e) {
      const int t = t0 + e;
      av[e] = 1.f, bv[e] = yv[e] = 0.f;
      if (t < last) av[e] = a[(size_t)t * channels + ch], bv[e] = b[(size_t)t * channels + ch], yv[e] = y[(size_t)t * ldy + ch];
    }
#pragma unroll
    for (int e = 0; e < SCAN_AHEAD; ++e) {
      const int t = t0 + e;
      if (t >= last) break;
      const int sq = seq_of_token[t];
      if (sq < 0) {  // a padding row
        out[(size_t)t * ldo + ch] = from_f32<T>(0.f);
      } else {
        if (sq != prev) S = init[(size_t)sq * channels + ch];
        S = fmaf(av[e], S, bv[e]);
        out[(size_t)t * ldo + ch] = from_f32<T>(S * fms_activate(yv[e], act));
        if (t + 1 == n_tokens || seq_of_token[t + 1] != sq) state[(size_t)slot_ids[sq] * channels + ch] = S;  // the sequence's last token
      }
      prev = sq;
    }
  }
}

// workspace: float32 [(2 * ceil(n_tokens / chunk) + n_seqs) * channels]
extern "C" int fmsamd_rglru_scan_chunked(const float* a, const float* b, const float* y, long ldy, int act, float* state,
                                         const int* seq_starts, const int* seq_of_token, const int* slot_ids, void* out,
                                         int out_dtype, long ldo, int n_tokens, int n_seqs, int channels, int chunk, float* workspace,
                                         hipStream_t stream) {
  if (n_tokens == 0) return 0;
  FMS_REQUIRE(n_tokens > 0 && n_seqs > 0 && channels > 0 && chunk > 0 && ldy >= channels && ldo >= channels && workspace != nullptr,
              "rglru_scan_chunked: bad sizes tokens=%d seqs=%d channels=%d chunk=%d", n_tokens, n_seqs, channels, chunk);
  FMS_REQUIRE(act >= 0 && act <= FMS_ACT_LAST, "rglru_scan_chunked: unknown activation %d", act);
  const int n_chunks = ceil_div(n_tokens, chunk);
  const int threads = channels >= 256 ? 256 : 64;
  const dim3 grid(n_chunks, ceil_div(channels, threads));
  FMS_REQUIRE(grid.y <= 65535, "rglru_scan_chunked: %d channels are too many for one launch", channels);
  float* P_ws = workspace;
  float* L_ws = P_ws + (size_t)n_chunks * channels;
  float* init = L_ws + (size_t)n_chunks * channels;
  rglru_chunk_sums_kernel<<<grid, threads, 0, stream>>>(a, b, state, seq_of_token, slot_ids, P_ws, L_ws, init, n_tokens, channels, chunk);
  FMS_LAUNCH_CHECK("rglru_chunk_sums");
  if (out_dtype == FMS_F32)
    rglru_chunk_walk_kernel<float><<<grid, threads, 0, stream>>>(a, b, y, ldy, act, state, seq_starts, seq_of_token, slot_ids, P_ws, L_ws,
                                                                 init, (float*)out, ldo, n_tokens, channels, chunk);
  else if (out_dtype == FMS_BF16)
    rglru_chunk_walk_kernel<bf16><<<grid, threads, 0, stream>>>(a, b, y, ldy, act, state, seq_starts, seq_of_token, slot_ids, P_ws, L_ws,
                                                                init, (bf16*)out, ldo, n_tokens, channels, chunk);
  else
    FMS_REQUIRE(false, "rglru_scan_chunked: unknown dtype %d", out_dtype);
  FMS_LAUNCH_CHECK("rglru_chunk_walk");
  return 0;
}
