// What a block needs whose norms sit behind its branches only, and whose branches read the stream itself.
//
//   group_norm_chain: stream += gnorm_b(branch) * wb (or the branch as it is);   out = nothing | the stream as it is | gnorm(stream) * w
//     gnorm splits a row into `groups` equal consecutive parts and divides each by its own root mean square
//     (eps inside the root); one group is the plain RMS norm.  Both statistics and the sum are float32.
//   short_conv: out = (x +) conv(x) (+ bias): a causal convolution over time on every channel, the inputs before the
//     step taken from the sequence's state; then the state is moved on (short_conv.h).
#include "common.h"
#include "fmsamd.h"
#include "short_conv.h"

__device__ __forceinline__ float scale_at(const void* w, int dtype, int i) {
  if (w == nullptr) return 1.f;
  return dtype == FMS_F32 ? ((const float*)w)[i] : (float)((const bf16*)w)[i];
}

// inv[g] = rsqrt(mean(row[g's part]^2) + eps): a wave a group, the lanes strided over the part, so that the order of the
// sum depends on nothing but the sizes.
__device__ __forceinline__ void group_scales(const float* row, float* inv, int width, int groups, float eps) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  const int part = width / groups;
  for (int g = wave; g < groups; g += nwaves) {
    const float* p = row + (size_t)g * part;
    float sq = 0.f;
    for (int i = lane; i < part; i += WAVE) sq = fmaf(p[i], p[i], sq);
    sq = wave_sum(sq);
    if (lane == 0) inv[g] = rsqrtf(sq / (float)part + eps);
  }
}

// One block per output row; the row waits in LDS (width floats, then the groups' scales).
template <typename T>
__global__ void __launch_bounds__(256)
    group_norm_chain_kernel(float* __restrict__ resid, const T* __restrict__ branch, const void* __restrict__ wb, int wb_dtype,
                            int groups_b, float eps_b, const void* __restrict__ w, int w_dtype, int groups, float eps,
                            T* __restrict__ out, int out_mode, const int* __restrict__ rows, int width) {
  extern __shared__ float lds[];
  float* row = lds;
  float* inv = lds + width;
  const int r = rows ? rows[blockIdx.x] : blockIdx.x;
  float* x = resid + (size_t)r * width;
  if (branch != nullptr) {
    const T* b = branch + (size_t)r * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) row[i] = to_f32(b[i]);
    if (groups_b > 0) {
      __syncthreads();
      group_scales(row, inv, width, groups_b, eps_b);
      __syncthreads();
    }
    const int part = groups_b > 0 ? width / groups_b : width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
      const float v = x[i] + (groups_b > 0 ? row[i] * inv[i / part] * scale_at(wb, wb_dtype, i) : row[i]);
      row[i] = v;
      if (!rows) x[i] = v;
    }
  } else {
    for (int i = threadIdx.x; i < width; i += blockDim.x) row[i] = x[i];
  }
  if (out_mode == FMS_CHAIN_NONE) return;
  T* o = out + (size_t)blockIdx.x * width;
  if (out_mode == FMS_CHAIN_CAST) {
    for (int i = threadIdx.x; i < width; i += blockDim.x) o[i] = from_f32<T>(row[i]);  // a thread reads what it wrote
    return;
  }
  __syncthreads();
  group_scales(row, inv, width, groups, eps);
  __syncthreads();
  const int part = width / groups;
  for (int i = threadIdx.x; i < width; i += blockDim.x) o[i] = from_f32<T>(row[i] * inv[i / part] * scale_at(w, w_dtype, i));
}

// Four consecutive elements of a row, or of a weight given with its type's code, as floats in one load; and back.
template <typename T>
__device__ __forceinline__ f32x4 row4(const T* p) {
  if constexpr (sizeof(T) == 4) {
    return *reinterpret_cast<const f32x4*>(p);
  } else {
    const bf16x4 t = *reinterpret_cast<const bf16x4*>(p);
    return f32x4{(float)t[0], (float)t[1], (float)t[2], (float)t[3]};
  }
}
__device__ __forceinline__ f32x4 weight4(const void* w, int dtype, int i) {
  return dtype == FMS_F32 ? row4((const float*)w + i) : row4((const bf16*)w + i);
}
template <typename T>
__device__ __forceinline__ void put4(T* p, f32x4 v) {
  if constexpr (sizeof(T) == 4) {
    *reinterpret_cast<f32x4*>(p) = v;
  } else {
    *reinterpret_cast<bf16x4*>(p) = bf16x4{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
  }
}

// The same for rows of at most 1024 * KEEP elements whose groups are multiples of 256 elements: branch, stream and both
// weights are asked for at once, four elements a load, and wait in registers, so the kernel pays the memory's latency
// once (a decode step's rows are few, and nothing else hides it) and reads every row once.  A wave's 256 elements of a
// pass lie in one group: the waves leave their sums of squares in LDS, and a group's scale is the sum of its waves' in
// a fixed order.  Rows of a prompt and of a decode step run this same kernel.
template <typename T, int KEEP>
__global__ void __launch_bounds__(256)
    group_norm_chain_small_kernel(float* __restrict__ resid, const T* __restrict__ branch, const void* __restrict__ wb, int wb_dtype,
                                  int groups_b, float eps_b, const void* __restrict__ w, int w_dtype, int groups, float eps,
                                  T* __restrict__ out, int out_mode, const int* __restrict__ rows, int width) {
  __shared__ float partial[4 * KEEP];
  const int r = rows ? rows[blockIdx.x] : blockIdx.x;
  float* x = resid + (size_t)r * width;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const f32x4 ones = {1.f, 1.f, 1.f, 1.f}, zeros = {0.f, 0.f, 0.f, 0.f};
  f32x4 bv[KEEP], xv[KEEP], wbv[KEEP], wv[KEEP];
#pragma unroll
  for (int n = 0; n < KEEP; ++n) {
    const int i = (threadIdx.x + n * 256) * 4;
    bv[n] = zeros, xv[n] = zeros, wbv[n] = ones, wv[n] = ones;
    if (i < width) {
      xv[n] = row4(x + i);
      if (branch) bv[n] = row4(branch + (size_t)r * width + i);
      if (branch && groups_b > 0 && wb) wbv[n] = weight4(wb, wb_dtype, i);
      if (out_mode == FMS_CHAIN_NORM && w) wv[n] = weight4(w, w_dtype, i);
    }
  }
  if (branch != nullptr) {
    if (groups_b > 0) {
#pragma unroll
      for (int n = 0; n < KEEP; ++n) {
        float sq = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) sq = fmaf(bv[n][e], bv[n][e], sq);
        sq = wave_sum(sq);
        if (lane == 0) partial[n * 4 + wave] = sq;
      }
      __syncthreads();
      const int part = width / groups_b, per = part / 256;
#pragma unroll
      for (int n = 0; n < KEEP; ++n) {
        const int i = (threadIdx.x + n * 256) * 4;
        if (i < width) {
          const int p0 = (i / part) * per;
          float sum = 0.f;
          for (int p = p0; p < p0 + per; ++p) sum += partial[p];
          const float inv = rsqrtf(sum / (float)part + eps_b);
#pragma unroll
          for (int e = 0; e < 4; ++e) xv[n][e] = xv[n][e] + bv[n][e] * inv * wbv[n][e];
        }
      }
      __syncthreads();  // the sums are read: the next norm may write its own
    } else {
#pragma unroll
      for (int n = 0; n < KEEP; ++n)
#pragma unroll
        for (int e = 0; e < 4; ++e) xv[n][e] += bv[n][e];
    }
    if (!rows) {
#pragma unroll
      for (int n = 0; n < KEEP; ++n) {
        const int i = (threadIdx.x + n * 256) * 4;
        if (i < width) put4(x + i, xv[n]);
      }
    }
  }
  if (out_mode == FMS_CHAIN_NONE) return;
  T* o = out + (size_t)blockIdx.x * width;
  if (out_mode == FMS_CHAIN_CAST) {
#pragma unroll
    for (int n = 0; n < KEEP; ++n) {
      const int i = (threadIdx.x + n * 256) * 4;
      if (i < width) put4(o + i, xv[n]);
    }
    return;
  }
#pragma unroll
  for (int n = 0; n < KEEP; ++n) {
    float sq = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) sq = fmaf(xv[n][e], xv[n][e], sq);
    sq = wave_sum(sq);
    if (lane == 0) partial[n * 4 + wave] = sq;
  }
  __syncthreads();
  const int part = width / groups, per = part / 256;
#pragma unroll
  for (int n = 0; n < KEEP; ++n) {
    const int i = (threadIdx.x + n * 256) * 4;
    if (i < width) {
      const int p0 = (i / part) * per;
      float sum = 0.f;
      for (int p = p0; p < p0 + per; ++p) sum += partial[p];
      const float inv = rsqrtf(sum / (float)part + eps);
      f32x4 y;
#pragma unroll
      for (int e = 0; e < 4; ++e) y[e] = xv[n][e] * inv * wv[n][e];
      put4(o + i, y);
    }
  }
}

extern "C" int fmsamd_group_norm_chain(float* resid, const void* branch, int act_dtype, const void* branch_weight,
                                       int branch_weight_dtype, int branch_groups, float branch_eps, const void* weight,
                                       int weight_dtype, int groups, float eps, void* out, int out_mode, const int* rows,
                                       int n_out, int width, hipStream_t stream) {
  if (n_out == 0) return 0;
  FMS_REQUIRE(n_out > 0 && width > 0 && width <= 15360, "group_norm_chain: bad sizes rows=%d width=%d", n_out, width);
  FMS_REQUIRE(resid != nullptr, "group_norm_chain: the stream is needed");
  FMS_REQUIRE(out_mode >= FMS_CHAIN_NONE && out_mode <= FMS_CHAIN_NORM && (out_mode == FMS_CHAIN_NONE || out != nullptr),
              "group_norm_chain: output mode %d", out_mode);
  FMS_REQUIRE(branch == nullptr || branch_groups == 0 || (branch_groups > 0 && branch_groups <= 1024 && width % branch_groups == 0),
              "group_norm_chain: %d groups do not divide the branch's %d channels", branch_groups, width);
  FMS_REQUIRE(out_mode != FMS_CHAIN_NORM || (groups > 0 && groups <= 1024 && width % groups == 0),
              "group_norm_chain: %d groups do not divide %d channels", groups, width);
  const bool branch_fits = branch == nullptr || branch_groups == 0 || (width / branch_groups) % 256 == 0;
  const bool norm_fits = out_mode != FMS_CHAIN_NORM || (width / groups) % 256 == 0;
  const bool types_fit = (branch_weight == nullptr || branch_weight_dtype == FMS_F32 || branch_weight_dtype == FMS_BF16) &&
                         (weight == nullptr || weight_dtype == FMS_F32 || weight_dtype == FMS_BF16);
  if (width <= 1024 * 4 && width % 4 == 0 && branch_fits && norm_fits && types_fit && (act_dtype == FMS_F32 || act_dtype == FMS_BF16)) {
    if (act_dtype == FMS_F32)
      group_norm_chain_small_kernel<float, 4><<<n_out, 256, 0, stream>>>(resid, (const float*)branch, branch_weight, branch_weight_dtype,
                                                                         branch_groups, branch_eps, weight, weight_dtype, groups, eps,
                                                                         (float*)out, out_mode, rows, width);
    else
      group_norm_chain_small_kernel<bf16, 4><<<n_out, 256, 0, stream>>>(resid, (const bf16*)branch, branch_weight, branch_weight_dtype,
                                                                        branch_groups, branch_eps, weight, weight_dtype, groups, eps,
                                                                        (bf16*)out, out_mode, rows, width);
    FMS_LAUNCH_CHECK("group_norm_chain_small");
    return 0;
  }
  const size_t lds = ((size_t)width + 1024) * sizeof(float);
  if (act_dtype == FMS_F32)
    group_norm_chain_kernel<float><<<n_out, 256, lds, stream>>>(resid, (const float*)branch, branch_weight, branch_weight_dtype,
                                                                branch_groups, branch_eps, weight, weight_dtype, groups, eps,
                                                                (float*)out, out_mode, rows, width);
  else if (act_dtype == FMS_BF16)
    group_norm_chain_kernel<bf16><<<n_out, 256, lds, stream>>>(resid, (const bf16*)branch, branch_weight, branch_weight_dtype,
                                                               branch_groups, branch_eps, weight, weight_dtype, groups, eps,
                                                               (bf16*)out, out_mode, rows, width);
  else
    FMS_REQUIRE(false, "group_norm_chain: unknown dtype %d", act_dtype);
  FMS_LAUNCH_CHECK("group_norm_chain");
  return 0;
}

// A block per token, a thread per channel and pass; all taps of a channel are asked for before any is used.
template <typename W, typename T>
__global__ void __launch_bounds__(1024)
    short_conv_kernel(const float* __restrict__ x, long ld, int C, const W* __restrict__ conv_w, const W* __restrict__ bias,
                      int taps, float* __restrict__ conv_state, const int* __restrict__ seq_of_token,
                      const int* __restrict__ slot_ids, int add_input, T* __restrict__ out, long ldo, int move_state) {
  const int t = blockIdx.x;
  const int seq = seq_of_token[t];
  T* o = out + (size_t)t * ldo;
  if (seq < 0) {  // a padding row: zeros, so that whatever reads the row reads numbers
    for (int c = threadIdx.x; c < C; c += blockDim.x) o[c] = from_f32<T>(0.f);
    return;
  }
  const int have = tokens_before(seq_of_token, t, seq, taps);
  float* state = conv_state + (size_t)slot_ids[seq] * (taps - 1) * C;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float xs[CONV_MAX_TAPS], ws[CONV_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j) {
      const int d = taps - 1 - j;  // how far back this tap reaches
      xs[j] = ws[j] = 0.f;
      if (j < taps) {
        xs[j] = d <= have ? x[(size_t)(t - d) * ld + c] : state[(size_t)(taps - 1 + have - d) * C + c];
        ws[j] = to_f32(conv_w[(size_t)c * taps + j]);
      }
    }
    float acc = bias ? to_f32(bias[c]) : 0.f;
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j) acc = fmaf(ws[j], xs[j], acc);
    if (add_input) acc += x[(size_t)t * ld + c];
    o[c] = from_f32<T>(acc);
    if (move_state) {
      // every sequence brings one token (have == 0): xs[0 .. taps - 2] are the channel's old entries, all read above by
      // this thread, which is their only reader in the step; the new ones are the old ones moved up and the token's own
#pragma unroll
      for (int j = 0; j < CONV_MAX_TAPS - 1; ++j)
        if (j < taps - 1) state[(size_t)j * C + c] = xs[j + 1];
    }
  }
}

// Steps of many tokens: a block takes CONV_TILE consecutive token rows and a thread VEC neighbouring channels, whose last
// inputs it carries from row to row in registers, so every input is loaded once.  A sequence's start inside the tile (and
// the tile's first row) fills the registers from the rows before, or from the state where the step holds no more.  The
// convolution is run as one of CONV_MAX_TAPS taps whose first weights are zero: every register has a fixed place.
#define CONV_TILE 16

template <typename W, typename T, int VEC>
__global__ void __launch_bounds__(256)
    short_conv_tile_kernel(const float* __restrict__ x, long ld, int C, const W* __restrict__ conv_w, const W* __restrict__ bias,
                           int taps, const float* __restrict__ conv_state, const int* __restrict__ seq_of_token,
                           const int* __restrict__ slot_ids, int add_input, T* __restrict__ out, long ldo, int n_tokens) {
  const int c0 = (blockIdx.y * blockDim.x + threadIdx.x) * VEC;
  if (c0 >= C) return;
  const int first = blockIdx.x * CONV_TILE, last = min(first + CONV_TILE, n_tokens);
  // back[d][v]: the weight of the input d rows back (d = 0: the row's own), hist[d - 1][v]: that input
  float back[CONV_MAX_TAPS][VEC], hist[CONV_MAX_TAPS - 1][VEC], bv[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    bv[v] = bias ? to_f32(bias[c0 + v]) : 0.f;
#pragma unroll
    for (int d = 0; d < CONV_MAX_TAPS; ++d) back[d][v] = d < taps ? to_f32(conv_w[(size_t)(c0 + v) * taps + (taps - 1 - d)]) : 0.f;
#pragma unroll
    for (int d = 0; d < CONV_MAX_TAPS - 1; ++d) hist[d][v] = 0.f;
  }
  float xs[CONV_TILE][VEC];  // the tile's rows, asked for together
#pragma unroll
  for (int e = 0; e < CONV_TILE; ++e) {
    const int t = first + e;
#pragma unroll
    for (int v = 0; v < VEC; ++v) xs[e][v] = 0.f;
    if (t < last) {
      if (VEC == 4) {
        const float4 q = *reinterpret_cast<const float4*>(x + (size_t)t * ld + c0);
        xs[e][0] = q.x, xs[e][1] = q.y, xs[e][2] = q.z, xs[e][3] = q.w;
      } else {
#pragma unroll
        for (int v = 0; v < VEC; ++v) xs[e][v] = x[(size_t)t * ld + c0 + v];
      }
    }
  }
  int prev = -2;
#pragma unroll
  for (int e = 0; e < CONV_TILE; ++e) {
    const int t = first + e;
    if (t >= last) break;
    const int seq = seq_of_token[t];
    T* o = out + (size_t)t * ldo + c0;
    if (seq < 0) {  // a padding row
#pragma unroll
      for (int v = 0; v < VEC; ++v) o[v] = from_f32<T>(0.f);
      prev = seq;
      continue;
    }
    if (seq != prev) {  // the tile's first row, or a sequence's first row of the step
      const int have = tokens_before(seq_of_token, t, seq, taps);
      const float* state = conv_state + (size_t)slot_ids[seq] * (taps - 1) * C;
#pragma unroll
      for (int d = 1; d < CONV_MAX_TAPS; ++d) {
        if (d < taps) {
#pragma unroll
          for (int v = 0; v < VEC; ++v)
            hist[d - 1][v] = d <= have ? x[(size_t)(t - d) * ld + c0 + v] : state[(size_t)(taps - 1 + have - d) * C + c0 + v];
        }
      }
    }
    prev = seq;
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      float acc = bv[v];
#pragma unroll
      for (int d = CONV_MAX_TAPS - 1; d > 0; --d) acc = fmaf(back[d][v], hist[d - 1][v], acc);  // the oldest input first
      acc = fmaf(back[0][v], xs[e][v], acc);
      if (add_input) acc += xs[e][v];
      o[v] = from_f32<T>(acc);  // the same sums in the same order as the kernel of short steps
    }
#pragma unroll
    for (int d = CONV_MAX_TAPS - 2; d > 0; --d) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) hist[d][v] = hist[d - 1][v];
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) hist[0][v] = xs[e][v];
  }
}

extern "C" int fmsamd_short_conv(const float* x, long ld, int channels, const void* conv_w, const void* bias, int weight_dtype,
                                 int taps, float* conv_state, const int* seq_of_token, const int* slot_ids, int add_input,
                                 void* out, int out_dtype, long ldo, int n_tokens, int single_tokens, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  FMS_REQUIRE(n_tokens > 0 && channels > 0 && ld >= channels && ldo >= channels, "short_conv: bad sizes T=%d C=%d ld=%ld ldo=%ld",
              n_tokens, channels, ld, ldo);
  FMS_REQUIRE(taps >= 1 && taps <= CONV_MAX_TAPS, "short_conv: %d taps (1 to %d)", taps, CONV_MAX_TAPS);
  FMS_REQUIRE(taps == 1 || conv_state != nullptr, "short_conv: a convolution of %d taps needs the sequences' state", taps);
  const int threads = n_tokens <= 64 ? 1024 : 256;
  // a step in which every sequence brings one token: the kernel that convolves also moves the state on
  // (of any number of sequences: a tile of rows would walk 16 sequences one after the other, each with its own state)
  const int move_state = single_tokens && taps > 1;
  if (n_tokens >= 4 * CONV_TILE && !single_tokens) {  // many rows: tiles of rows, every input loaded once
    const bool wide = channels % 4 == 0 && ld % 4 == 0 && ((uintptr_t)x % 16) == 0;
    const int per_block = 256 * (wide ? 4 : 1);
    const dim3 grid(ceil_div(n_tokens, CONV_TILE), ceil_div(channels, per_block));
    FMS_REQUIRE(grid.y <= 65535, "short_conv: %d channels are too many for one launch", channels);
#define FMS_CONV_TILE(W, T)                                                                                                          \
  do {                                                                                                                               \
    if (wide)                                                                                                                        \
      short_conv_tile_kernel<W, T, 4><<<grid, 256, 0, stream>>>(x, ld, channels, (const W*)conv_w, (const W*)bias, taps, conv_state, \
                                                                seq_of_token, slot_ids, add_input, (T*)out, ldo, n_tokens);          \
    else                                                                                                                             \
      short_conv_tile_kernel<W, T, 1><<<grid, 256, 0, stream>>>(x, ld, channels, (const W*)conv_w, (const W*)bias, taps, conv_state, \
                                                                seq_of_token, slot_ids, add_input, (T*)out, ldo, n_tokens);          \
  } while (0)
    if (weight_dtype == FMS_F32 && out_dtype == FMS_F32) FMS_CONV_TILE(float, float);
    else if (weight_dtype == FMS_F32 && out_dtype == FMS_BF16) FMS_CONV_TILE(float, bf16);
    else if (weight_dtype == FMS_BF16 && out_dtype == FMS_F32) FMS_CONV_TILE(bf16, float);
    else if (weight_dtype == FMS_BF16 && out_dtype == FMS_BF16) FMS_CONV_TILE(bf16, bf16);
    else FMS_REQUIRE(false, "short_conv: unknown dtypes %d %d", weight_dtype, out_dtype);
#undef FMS_CONV_TILE
    FMS_LAUNCH_CHECK("short_conv_tile");
    if (taps > 1) {
      conv_state_kernel<<<n_tokens, threads, 0, stream>>>(x, ld, taps, conv_state, seq_of_token, slot_ids, n_tokens, channels);
      FMS_LAUNCH_CHECK("conv_state");
    }
    return 0;
  }
#define FMS_CONV(W, T)                                                                                                     \
  short_conv_kernel<W, T><<<n_tokens, threads, 0, stream>>>(x, ld, channels, (const W*)conv_w, (const W*)bias, taps, conv_state, \
                                                            seq_of_token, slot_ids, add_input, (T*)out, ldo, move_state)
  if (weight_dtype == FMS_F32 && out_dtype == FMS_F32) FMS_CONV(float, float);
  else if (weight_dtype == FMS_F32 && out_dtype == FMS_BF16) FMS_CONV(float, bf16);
  else if (weight_dtype == FMS_BF16 && out_dtype == FMS_F32) FMS_CONV(bf16, float);
  else if (weight_dtype == FMS_BF16 && out_dtype == FMS_BF16) FMS_CONV(bf16, bf16);
  else FMS_REQUIRE(false, "short_conv: unknown dtypes %d %d", weight_dtype, out_dtype);
#undef FMS_CONV
  FMS_LAUNCH_CHECK("short_conv");
  if (taps > 1 && !move_state) {
    conv_state_kernel<<<n_tokens, threads, 0, stream>>>(x, ld, taps, conv_state, seq_of_token, slot_ids, n_tokens, channels);
    FMS_LAUNCH_CHECK("conv_state");
  }
  return 0;
}
