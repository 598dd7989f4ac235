// The gated delta rule: a recurrent mixer whose state is a matrix S [key channels, value channels] per head.
//
//   S <- g * S           g: one decay per head, or one per head and key channel (it scales rows of S)
//   u  = beta (v - S^T k)
//   S <- S + k u^T
//   o  = S^T q           the read-out sees the token's own write
//
// Three kernels run a step of any number of tokens per sequence, all in float32:
//   delta_prepare:  the short causal convolution over time of the q, k and v channels (inputs before the step come
//                   from the sequence's state, zeros before its start), silu, unit vectors per q and k head, q's scale,
//                   beta = sigmoid, g = exp(-exp(A_log) softplus(a + dt_bias)).
//   conv_state:     the last (taps - 1) inputs of every sequence go into its state.
//   delta_rule:     the recurrence.  Columns of S never mix (each value channel is a recurrence of its own), so a wave
//                   owns a few columns of one head of one sequence: 16 (or 32) lanes share a column, each with a run of
//                   its rows in registers.  The wave walks over the sequence's tokens; q, k and g of a run of tokens are
//                   staged in LDS for all its lanes (the next run's are asked for before this one is worked on).  With
//                   kg = g k and qg = g q, both inner products of a token read the state as the token found it,
//                   u = beta (v - S^T kg),  o = S^T qg + (k . q) u,  and are summed over the column's lanes together, in
//                   the vector unit; then S <- g S + k u^T.  (A decay per head leaves the sums: g S^T k.)
//   gated_head_norm: o / rms(o) * weight * act(gate) per head, rounded once to the activation type.
//
// The state is kept transposed, [slot][head][value channel][key channel], so that a lane's rows are contiguous.
#include "common.h"
#include "fmsamd.h"
#include "short_conv.h"

#define DELTA_MAX_TAPS CONV_MAX_TAPS

__device__ __forceinline__ float softplus_f32(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float sigmoid_f32(float z) { return 1.f / (1.f + expf(-z)); }

// Blocks of 1024 threads for steps of few tokens (a decode step has a block per token and nothing else to hide a
// load's latency behind: the fewer passes a thread makes, the fewer round trips to memory follow one another).
template <typename W>
__global__ void __launch_bounds__(1024)
    delta_prepare_kernel(const float* __restrict__ proj, long ld, int col_b, const float* __restrict__ a, long lda, int col_a,
                         const W* __restrict__ conv_w, int taps, const float* __restrict__ a_log,
                         const float* __restrict__ dt_bias, const float* __restrict__ conv_state,
                         const int* __restrict__ seq_of_token, const int* __restrict__ slot_ids, float* __restrict__ qkv,
                         float* __restrict__ beta, float* __restrict__ decay, float* __restrict__ kq, int H, int G, int D, int Dv,
                         int per_channel, float q_scale) {
  extern __shared__ float y[];  // the C convolved channels of this token
  const int t = blockIdx.x;
  const int seq = seq_of_token[t];
  if (seq < 0) return;
  const int slot = slot_ids[seq];
  const int C = 2 * G * D + H * Dv;
  const int have = tokens_before(seq_of_token, t, seq, taps);
  const float* state = conv_state + (size_t)slot * (taps - 1) * C;
  // two channels a thread and pass, all their taps asked for before any is used: a decode step has a block per token
  // and nothing else to hide a load's latency behind
  for (int c0 = threadIdx.x; c0 < C; c0 += 2 * blockDim.x) {
    float x[2][DELTA_MAX_TAPS], w[2][DELTA_MAX_TAPS];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int c = c0 + e * blockDim.x;
#pragma unroll
      for (int j = 0; j < DELTA_MAX_TAPS; ++j) {
        const int d = taps - 1 - j;  // how far back this tap reaches
        x[e][j] = w[e][j] = 0.f;
        if (j < taps && c < C) {
          x[e][j] = d <= have ? proj[(size_t)(t - d) * ld + c] : state[(size_t)(taps - 1 + have - d) * C + c];
          w[e][j] = to_f32(conv_w[(size_t)c * taps + j]);
        }
      }
    }
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int c = c0 + e * blockDim.x;
      float acc = 0.f;
#pragma unroll
      for (int j = 0; j < DELTA_MAX_TAPS; ++j) acc = fmaf(w[e][j], x[e][j], acc);
      if (c < C) y[c] = acc / (1.f + expf(-acc));
    }
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  for (int head = wave; head < 2 * G; head += nwaves) {
    float* v = y + (size_t)head * D;
    float s = 0.f;
    for (int i = lane; i < D; i += WAVE) s = fmaf(v[i], v[i], s);
    s = wave_sum(s);
    const float inv = (head < G ? q_scale : 1.f) / sqrtf(s + 1e-6f);
    for (int i = lane; i < D; i += WAVE) v[i] *= inv;
  }
  __syncthreads();
  for (int head = wave; head < G; head += nwaves) {  // k . q of the finished vectors, which the recurrence's read-out needs
    float s = 0.f;
    for (int i = lane; i < D; i += WAVE) s = fmaf(y[(size_t)head * D + i], y[(size_t)(G + head) * D + i], s);
    s = wave_sum(s);
    if (lane == 0) kq[(size_t)t * G + head] = s;
  }
  for (int c = threadIdx.x; c < C; c += blockDim.x) qkv[(size_t)t * C + c] = y[c];
  for (int h = threadIdx.x; h < H; h += blockDim.x) beta[(size_t)t * H + h] = sigmoid_f32(proj[(size_t)t * ld + col_b + h]);
  const int per_head = per_channel ? D : 1;
  for (int i = threadIdx.x; i < H * per_head; i += blockDim.x) {
    const float z = a[(size_t)t * lda + col_a + i] + dt_bias[i];
    decay[(size_t)t * H * per_head + i] = expf(-expf(a_log[i / per_head]) * softplus_f32(z));
  }
}

// --------------------------------------------------------------------------
// the recurrence
// --------------------------------------------------------------------------
#define DELTA_WAVES 4                       // waves of a block: they share the staged tokens
#define DELTA_THREADS (DELTA_WAVES * WAVE)

struct DeltaArgs {
  const float* qkv;    // [T, C]: q [G*D] | k [G*D] | v [H*Dv]
  const float* beta;   // [T, H]
  const float* decay;  // [T, H] or [T, H*D]
  const float* kq;     // [T, G]: k . q
  float* state;        // [slots][H][Dv][D]
  float* out;          // [T, H*Dv]
  const int* seq_starts;
  const int* seq_of_token;
  const int* slot_ids;
  int H, G, D, Dv, per_channel;
};

// The sum over the 16 lanes of a row, in all of them, in the vector unit: two swaps inside quads, then the mirror of
// a half row and of the row (a shuffle through LDS would put four round trips to LDS into every token's chain).
__device__ __forceinline__ float row16_sum(float v) {
#define FMS_DPP_ADD(ctrl) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xF, 0xF, true))
  FMS_DPP_ADD(0xB1);   // quad_perm [1, 0, 3, 2]
  FMS_DPP_ADD(0x4E);   // quad_perm [2, 3, 0, 1]
  FMS_DPP_ADD(0x141);  // row_half_mirror
  FMS_DPP_ADD(0x140);  // row_mirror
#undef FMS_DPP_ADD
  return v;
}

// The sum over the PARTS lanes that share a column: a row of 16 lanes, or two rows (the second step swaps the odd rows
// of one copy with the even rows of another, so that their sum is the pair's sum in both).
template <int PARTS>
__device__ __forceinline__ float row_sum(float v) {
  v = row16_sum(v);
  if constexpr (PARTS == 32) {
    const unsigned u = __float_as_uint(v);
    const auto rows = __builtin_amdgcn_permlane16_swap(u, u, false, false);  // rows [0, 0, 2, 2] and [1, 1, 3, 3]
    v = __uint_as_float(rows[0]) + __uint_as_float(rows[1]);
  }
  return v;
}

// PARTS: lanes that share a column of S (16, or 32 where a step has few sequences and heads: twice the blocks, half the
// work a token and lane).  R: rows of S per lane (D <= PARTS R).  TC: tokens staged at a time.  A block's four waves own
// 256 / PARTS columns of one head and share the staged tokens (staging costs instructions, and four waves split them).
// The next run's q, k and g are asked for from global memory before this run is worked on and wait in registers meanwhile.
template <int PARTS, int R, int TC, bool PER_CHANNEL>
__global__ void __launch_bounds__(DELTA_THREADS) delta_rule_kernel(DeltaArgs a) {
  constexpr int DELTA_COLS = DELTA_THREADS / PARTS;  // columns of S the block owns
  constexpr int DELTA_PARTS = PARTS;
  constexpr int DP = R * DELTA_PARTS;          // padded key size
  constexpr int NI = TC * DP / DELTA_THREADS;  // staged elements a thread
  static_assert(TC * DP % DELTA_THREADS == 0 && TC * DELTA_COLS <= DELTA_THREADS, "the staging loops assume this");
  // With a decay per channel: qg = g q, kg = g k, k and g.  With one decay per head the factor leaves the inner products
  // (S^T (g k) = g S^T k): q and k alone are staged, and g as one number a token; half the LDS traffic.
  constexpr int CH = PER_CHANNEL ? TC : 1;
  __shared__ __attribute__((aligned(16))) float qg[TC][DP];
  __shared__ __attribute__((aligned(16))) float kg[CH][DP];
  __shared__ __attribute__((aligned(16))) float kk[TC][DP];
  __shared__ __attribute__((aligned(16))) float gg[CH][DP];
  __shared__ float vv[TC][DELTA_COLS];
  __shared__ float gs[TC];
  __shared__ float bb[TC];
  __shared__ float kqs[TC];
  __shared__ float oo[TC][DELTA_COLS];

  const int b = blockIdx.x, h = blockIdx.y;
  const int t0 = a.seq_starts[b], t1 = a.seq_starts[b + 1];
  if (t0 >= t1 || a.seq_of_token[t0] < 0) return;
  const int slot = a.slot_ids[b];
  const int lane = threadIdx.x;  // of the block
  const int part = lane % DELTA_PARTS, col = lane / DELTA_PARTS;
  const int j = blockIdx.z * DELTA_COLS + col;  // this lane's column of S
  const int H = a.H, G = a.G, D = a.D, Dv = a.Dv;
  const int C = 2 * G * D + H * Dv;
  const int kh = h / (H / G);
  const bool live = j < Dv;

  float S[R];
  float* srow = a.state + (((size_t)slot * H + h) * Dv + (live ? j : 0)) * D + part * R;
#pragma unroll
  for (int r = 0; r < R; ++r) S[r] = (live && part * R + r < D) ? srow[r] : 0.f;

  // what a lane fetches of a run: NI (q, k, g) triples, one value, and beta and k . q of one token
  float pq[NI], pk[NI], pg[PER_CHANNEL ? NI : 1], pv = 0.f, pb = 0.f, pkq = 0.f, pgs = 1.f;
  const int vt = lane / DELTA_COLS, vc = lane % DELTA_COLS;  // the (token, column) whose value and output this lane moves
  const int vj = blockIdx.z * DELTA_COLS + vc;
  auto fetch = [&](int tb) {
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      const int idx = it * DELTA_THREADS + lane;
      const int tt = idx / DP, i = idx % DP;
      const int t = tb + tt;
      // past the run's last token (and past the key channels) a token that changes nothing: k = 0, g = 1
      pq[it] = pk[it] = 0.f;
      if constexpr (PER_CHANNEL) pg[it] = 1.f;
      if (t < t1 && i < D) {
        const float* row = a.qkv + (size_t)t * C;
        pq[it] = row[kh * D + i];
        pk[it] = row[G * D + kh * D + i];
        if constexpr (PER_CHANNEL) pg[it] = a.decay[((size_t)t * H + h) * D + i];
      }
    }
    pgs = 1.f;
    pb = 0.f;
    pv = (vt < TC && tb + vt < t1 && vj < Dv) ? a.qkv[(size_t)(tb + vt) * C + 2 * G * D + h * Dv + vj] : 0.f;
    if (lane < TC && tb + lane < t1) {
      pb = a.beta[(size_t)(tb + lane) * H + h];
      pkq = a.kq[(size_t)(tb + lane) * G + kh];
      if constexpr (!PER_CHANNEL) pgs = a.decay[(size_t)(tb + lane) * H + h];
    }
  };
  fetch(t0);

  for (int tb = t0; tb < t1; tb += TC) {
    const int n = t1 - tb < TC ? t1 - tb : TC;
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      const int idx = it * DELTA_THREADS + lane;
      const int tt = idx / DP, i = idx % DP;
      kk[tt][i] = pk[it];
      if constexpr (PER_CHANNEL) {
        qg[tt][i] = pq[it] * pg[it];
        kg[tt][i] = pk[it] * pg[it];
        gg[tt][i] = pg[it];
      } else {
        qg[tt][i] = pq[it];
      }
    }
    if (vt < TC) vv[vt][vc] = pv;
    if (lane < TC) bb[lane] = pb, kqs[lane] = pkq, gs[lane] = pgs;
    block_sync_lds();
    if (tb + TC < t1) fetch(tb + TC);  // under way while this run is worked on

    // a token's operands are read from LDS into registers while the token before it is worked on (two sets, in turn)
    struct Operands {
      float kg[PER_CHANNEL ? R : 1], qg[R], kk[R], gg[PER_CHANNEL ? R : 1], g, beta, v, kq;
    };
    auto load = [&](Operands& x, int tt) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        x.qg[r] = qg[tt][part * R + r];
        x.kk[r] = kk[tt][part * R + r];
        if constexpr (PER_CHANNEL) {
          x.kg[r] = kg[tt][part * R + r];
          x.gg[r] = gg[tt][part * R + r];
        }
      }
      x.g = gs[tt];
      x.beta = bb[tt];
      x.v = vv[tt][col];
      x.kq = kqs[tt];
    };
    auto work = [&](const Operands& x, int tt) {
      float du0 = 0.f, du1 = 0.f, dq0 = 0.f, dq1 = 0.f;
#pragma unroll
      for (int r = 0; r < R; r += 2) {
        du0 = fmaf(S[r], PER_CHANNEL ? x.kg[PER_CHANNEL ? r : 0] : x.kk[r], du0);
        dq0 = fmaf(S[r], x.qg[r], dq0);
        du1 = fmaf(S[r + 1], PER_CHANNEL ? x.kg[PER_CHANNEL ? r + 1 : 0] : x.kk[r + 1], du1);
        dq1 = fmaf(S[r + 1], x.qg[r + 1], dq1);
      }
      float du = row_sum<PARTS>(du0 + du1), dq = row_sum<PARTS>(dq0 + dq1);
      if constexpr (!PER_CHANNEL) du *= x.g, dq *= x.g;  // the head's decay, taken out of the sums
      const float u = x.beta * (x.v - du);
#pragma unroll
      for (int r = 0; r < R; ++r) S[r] = fmaf(x.kk[r], u, (PER_CHANNEL ? x.gg[PER_CHANNEL ? r : 0] : x.g) * S[r]);
      if (part == 0) oo[tt][col] = fmaf(x.kq, u, dq);
    };
    // Tokens go in pairs, and a run of an odd number works on one staged token that changes nothing (beta = 0, k = 0,
    // g = 1; its output is not copied out): the loop's body then has no branch around its loads, and the compiler can
    // let a token's work wait for its own operands only, not for the ones just asked for.
    Operands xa, xb;
    load(xa, 0);
    const int n2 = TC > 1 ? (n + 1) & ~1 : 1;
    for (int tt = 0; tt < n2; tt += 2) {
      load(xb, tt + 1 < TC ? tt + 1 : tt);
      work(xa, tt);
      if constexpr (TC > 1) {
        load(xa, tt + 2 < TC ? tt + 2 : tt);
        work(xb, tt + 1);
      }
    }
    block_sync_lds();
    if (vt < n && vj < Dv) a.out[(size_t)(tb + vt) * H * Dv + h * Dv + vj] = oo[vt][vc];
    block_sync_lds();  // the run's reads are done before the next one is written
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (part * R + r < D) srow[r] = S[r];
  }
}

// out[t, h, j] = o / rms_j(o) * weight[j] * act(gate[t, h, j]) * out_scale; one wave per (token, head)
template <typename T, typename W>
__global__ void __launch_bounds__(256)
    gated_head_norm_kernel(const float* __restrict__ o, const float* __restrict__ gate, long ldg, const W* __restrict__ weight,
                           float eps, int act, float out_scale, T* __restrict__ out, long ldo, const int* __restrict__ seq_of_token,
                           int n_tokens, int H, int Dv) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const long pair = (long)blockIdx.x * 4 + wave;
  if (pair >= (long)n_tokens * H) return;
  const int t = (int)(pair / H), h = (int)(pair % H);
  if (seq_of_token[t] < 0) return;
  const float* row = o + ((size_t)t * H + h) * Dv;
  float s = 0.f;
  for (int j = lane; j < Dv; j += WAVE) s = fmaf(row[j], row[j], s);
  s = wave_sum(s);
  const float inv = 1.f / sqrtf(s / (float)Dv + eps);
  for (int j = lane; j < Dv; j += WAVE) {
    const float g = fms_activate(gate[(size_t)t * ldg + (size_t)h * Dv + j], act);
    out[(size_t)t * ldo + (size_t)h * Dv + j] = from_f32<T>(row[j] * inv * to_f32(weight[j]) * g * out_scale);
  }
}

// --------------------------------------------------------------------------
extern "C" int fmsamd_delta_prepare(const float* proj, long ld, int col_b, const float* a, long lda, int col_a, const void* conv_w,
                                    int conv_dtype, int taps, const float* a_log, const float* dt_bias, float* conv_state,
                                    const int* seq_of_token, const int* slot_ids, float* qkv, float* beta, float* decay,
                                    float* kq, int n_tokens, int heads, int kv_heads, int dim, int vdim, int per_channel,
                                    float q_scale, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  FMS_REQUIRE(n_tokens > 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0,
              "delta_prepare: bad sizes heads=%d kv_heads=%d dim=%d vdim=%d", heads, kv_heads, dim, vdim);
  FMS_REQUIRE(taps >= 1 && taps <= DELTA_MAX_TAPS, "delta_prepare: %d taps (1 to %d)", taps, DELTA_MAX_TAPS);
  const long C = 2L * kv_heads * dim + (long)heads * vdim;
  FMS_REQUIRE(ld >= C && col_b >= 0 && col_b + heads <= ld, "delta_prepare: rows of %ld for %ld channels", ld, C);
  FMS_REQUIRE(C * 4 <= 64 * 1024, "delta_prepare: %ld channels do not fit one block's LDS", C);
  FMS_REQUIRE(col_a >= 0 && col_a + heads * (per_channel ? dim : 1) <= lda, "delta_prepare: the decay's columns leave its rows");
  const size_t lds = (size_t)C * sizeof(float);
  const int threads = n_tokens <= 64 ? 1024 : 256;
#define FMS_PREP(W)                                                                                                   \
  delta_prepare_kernel<W><<<n_tokens, threads, lds, stream>>>(proj, ld, col_b, a, lda, col_a, (const W*)conv_w, taps, a_log, \
                                                          dt_bias, conv_state, seq_of_token, slot_ids, qkv, beta, decay, \
                                                          kq, heads, kv_heads, dim, vdim, per_channel, q_scale)
  if (conv_dtype == FMS_F32) FMS_PREP(float);
  else if (conv_dtype == FMS_BF16) FMS_PREP(bf16);
  else FMS_REQUIRE(false, "delta_prepare: unknown dtype %d", conv_dtype);
#undef FMS_PREP
  FMS_LAUNCH_CHECK("delta_prepare");
  if (taps > 1) {
    conv_state_kernel<<<n_tokens, threads, 0, stream>>>(proj, ld, taps, conv_state, seq_of_token, slot_ids, n_tokens, (int)C);
    FMS_LAUNCH_CHECK("conv_state");
  }
  return 0;
}

extern "C" int fmsamd_delta_rule(const float* qkv, const float* beta, const float* decay, const float* kq, float* state,
                                 float* out, const int* seq_starts, const int* seq_of_token, const int* slot_ids, int n_seqs, int heads,
                                 int kv_heads, int dim, int vdim, int per_channel, int single_tokens, hipStream_t stream) {
  if (n_seqs == 0) return 0;
  FMS_REQUIRE(n_seqs > 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0,
              "delta_rule: bad sizes heads=%d kv_heads=%d dim=%d vdim=%d", heads, kv_heads, dim, vdim);
  FMS_REQUIRE(dim <= 256, "delta_rule: %d key channels (at most 256)", dim);
  DeltaArgs a{qkv, beta, decay, kq, state, out, seq_starts, seq_of_token, slot_ids, heads, kv_heads, dim, vdim, per_channel};
  // Few sequences and heads (a prompt alone): 32 lanes a column instead of 16, so that the step has twice the blocks and a
  // token costs every wave half the work; with many blocks anyway, 16 lanes (fewer reduction steps a token).
  const bool wide = !single_tokens && dim > 32 && (long)n_seqs * heads * ceil_div(vdim, 16) <= 512;
  const int cols = DELTA_THREADS / (wide ? 32 : 16);
  FMS_REQUIRE(heads <= 65535 && ceil_div(vdim, cols) <= 65535, "delta_rule: too many heads or value channels for one launch");
  const dim3 grid(n_seqs, heads, ceil_div(vdim, cols));
#define FMS_DR(P, R, TC)                                                                        \
  do {                                                                                          \
    if (per_channel) delta_rule_kernel<P, R, TC, true><<<grid, DELTA_THREADS, 0, stream>>>(a);  \
    else delta_rule_kernel<P, R, TC, false><<<grid, DELTA_THREADS, 0, stream>>>(a);             \
  } while (0)
  // single_tokens: every sequence brings one token (a decode step).  Staging room for one pass of the block's threads
  // is then enough, and a block that small leaves the compute unit's LDS to many more blocks.
  if (single_tokens) {
    if (dim <= 32) FMS_DR(16, 2, 8);
    else if (dim <= 64) FMS_DR(16, 4, 4);
    else if (dim <= 128) FMS_DR(16, 8, 2);
    else FMS_DR(16, 16, 1);
  } else if (wide) {
    if (dim <= 64) FMS_DR(32, 2, 16);
    else if (dim <= 128) FMS_DR(32, 4, 16);
    else FMS_DR(32, 8, 8);
  } else if (dim <= 32) FMS_DR(16, 2, 16);
  else if (dim <= 64) FMS_DR(16, 4, 16);
  else if (dim <= 128) FMS_DR(16, 8, 16);
  else FMS_DR(16, 16, 8);
#undef FMS_DR
  FMS_LAUNCH_CHECK("delta_rule");
  return 0;
}

extern "C" int fmsamd_gated_head_norm(const float* o, const float* gate, long ldg, const void* weight, int weight_dtype, float eps,
                                      int act, float out_scale, void* out, int out_dtype, long ldo, const int* seq_of_token,
                                      int n_tokens, int heads, int vdim, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  FMS_REQUIRE(n_tokens > 0 && heads > 0 && vdim > 0 && ldg >= (long)heads * vdim && ldo >= (long)heads * vdim,
              "gated_head_norm: bad sizes heads=%d vdim=%d", heads, vdim);
  FMS_REQUIRE(act >= 0 && act <= FMS_ACT_LAST, "gated_head_norm: unknown activation %d", act);
  const int blocks = ceil_div((long)n_tokens * heads, 4);
#define FMS_GHN(T, W)                                                                                                          \
  gated_head_norm_kernel<T, W><<<blocks, 256, 0, stream>>>(o, gate, ldg, (const W*)weight, eps, act, out_scale, (T*)out, ldo, \
                                                           seq_of_token, n_tokens, heads, vdim)
  if (out_dtype == FMS_F32 && weight_dtype == FMS_F32) FMS_GHN(float, float);
  else if (out_dtype == FMS_BF16 && weight_dtype == FMS_F32) FMS_GHN(bf16, float);
  else if (out_dtype == FMS_BF16 && weight_dtype == FMS_BF16) FMS_GHN(bf16, bf16);
  else if (out_dtype == FMS_F32 && weight_dtype == FMS_BF16) FMS_GHN(float, bf16);
  else FMS_REQUIRE(false, "gated_head_norm: unknown dtypes %d, %d", out_dtype, weight_dtype);
#undef FMS_GHN
  FMS_LAUNCH_CHECK("gated_head_norm");
  return 0;
}
