// Norms that sit behind a branch, and activations of feed-forwards that are not "act(gate) * up".
//
//   norm_add_norm: a block whose branches are normed before they join the stream,
//       stream += branch / rms(branch) * wb;   out = stream / rms(stream) * w
//     in one pass over the row: two row norms and the residual sum, all float32.
//   rms_norm_cols: the RMS norm of a run of columns of float32 rows (a slice of a fused projection).
//   poly_norm: a sum of the RMS-normed first three powers of a token's values.
//   activate: out = act(x), the activations of common.h.
//   clamped_gated_act: out = g' * sigmoid(alpha g') * (u' + shift), g' = min(g, limit), u' = clamp(u, -limit, limit).
#include "common.h"
#include "fmsamd.h"

__device__ __forceinline__ float load_scale(const void* w, int dtype, int i) {
  if (w == nullptr) return 1.f;
  return dtype == FMS_F32 ? ((const float*)w)[i] : (float)((const bf16*)w)[i];
}

// One block per output row; the row waits in LDS (width floats) between the two reductions.
template <typename T>
__global__ void __launch_bounds__(256)
    norm_add_norm_kernel(float* __restrict__ resid, const T* __restrict__ branch, const void* __restrict__ wb, float eps_b,
                         const void* __restrict__ w, int w_dtype, float eps, T* __restrict__ out,
                         const int* __restrict__ rows, int width) {
  extern __shared__ float row[];
  __shared__ float scratch[17];
  const int r = rows ? rows[blockIdx.x] : blockIdx.x;
  float* x = resid + (size_t)r * width;
  const T* b = branch + (size_t)r * width;
  float sq = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = to_f32(b[i]);
    row[i] = v;
    sq = fmaf(v, v, sq);
  }
  const float rb = rsqrtf(block_sum(sq, scratch) / (float)width + eps_b);
  sq = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = x[i] + row[i] * rb * load_scale(wb, w_dtype, i);
    row[i] = v;
    if (!rows) x[i] = v;
    sq = fmaf(v, v, sq);
  }
  if (out == nullptr) return;
  const float rs = rsqrtf(block_sum(sq, scratch) / (float)width + eps);
  T* o = out + (size_t)blockIdx.x * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) o[i] = from_f32<T>(row[i] * rs * load_scale(w, w_dtype, i));
}

// Four consecutive elements as floats, from float or bfloat16 storage, in one load; and back.
template <typename T>
__device__ __forceinline__ f32x4 load4(const T* p) {
  if constexpr (sizeof(T) == 4) {
    return *reinterpret_cast<const f32x4*>(p);
  } else {
    const bf16x4 t = *reinterpret_cast<const bf16x4*>(p);
    return f32x4{(float)t[0], (float)t[1], (float)t[2], (float)t[3]};
  }
}
template <typename T>
__device__ __forceinline__ void store4(T* p, f32x4 v) {
  if constexpr (sizeof(T) == 4) {
    *reinterpret_cast<f32x4*>(p) = v;
  } else {
    *reinterpret_cast<bf16x4*>(p) = bf16x4{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
  }
}

// The same for rows of at most 1024 * KEEP elements (a multiple of 4): branch, stream and both weights are asked for
// at once, four elements a load, and wait in registers, so the kernel pays the memory's latency once instead of four
// times (a decode step's rows are few, and nothing else hides it).  The loops over what is kept have compile-time
// trip counts.
template <typename T, typename WT, int KEEP>
__global__ void __launch_bounds__(256)
    norm_add_norm_small_kernel(float* __restrict__ resid, const T* __restrict__ branch, const WT* __restrict__ wb, float eps_b,
                               const WT* __restrict__ w, float eps, T* __restrict__ out, const int* __restrict__ rows, int width) {
  __shared__ float scratch[17];
  const int r = rows ? rows[blockIdx.x] : blockIdx.x;
  float* x = resid + (size_t)r * width;
  const T* b = branch + (size_t)r * width;
  const f32x4 ones = {1.f, 1.f, 1.f, 1.f}, zeros = {0.f, 0.f, 0.f, 0.f};
  f32x4 bv[KEEP], xv[KEEP], wbv[KEEP], wv[KEEP];
  float sq = 0.f;
#pragma unroll
  for (int n = 0; n < KEEP; ++n) {
    const int i = (threadIdx.x + n * 256) * 4;
    bv[n] = zeros, xv[n] = zeros, wbv[n] = ones, wv[n] = ones;
    if (i < width) {
      bv[n] = load4(b + i);
      xv[n] = load4(x + i);
      if (wb) wbv[n] = load4(wb + i);
      if (w) wv[n] = load4(w + i);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) sq = fmaf(bv[n][e], bv[n][e], sq);
  }
  const float rb = rsqrtf(block_sum(sq, scratch) / (float)width + eps_b);
  sq = 0.f;
#pragma unroll
  for (int n = 0; n < KEEP; ++n) {
    const int i = (threadIdx.x + n * 256) * 4;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      xv[n][e] = xv[n][e] + bv[n][e] * rb * wbv[n][e];
      sq = fmaf(xv[n][e], xv[n][e], sq);  // elements past the row are zero
    }
    if (i < width && !rows) store4(x + i, xv[n]);
  }
  if (out == nullptr) return;
  const float rs = rsqrtf(block_sum(sq, scratch) / (float)width + eps);
  T* o = out + (size_t)blockIdx.x * width;
#pragma unroll
  for (int n = 0; n < KEEP; ++n) {
    const int i = (threadIdx.x + n * 256) * 4;
    if (i < width) {
      f32x4 y;
#pragma unroll
      for (int e = 0; e < 4; ++e) y[e] = xv[n][e] * rs * wv[n][e];
      store4(o + i, y);
    }
  }
}

extern "C" int fmsamd_norm_add_norm(float* resid, const void* branch, int act_dtype, const void* branch_weight,
                                    float branch_eps, const void* weight, int weight_dtype, float eps, void* out,
                                    const int* rows, int n_out, int width, hipStream_t stream) {
  if (n_out == 0) return 0;
  FMS_REQUIRE(n_out > 0 && width > 0 && width <= 16384, "norm_add_norm: bad sizes rows=%d width=%d", n_out, width);
  FMS_REQUIRE(resid != nullptr && branch != nullptr, "norm_add_norm: the stream and the branch are needed");
  const size_t lds = (size_t)width * sizeof(float);
  const bool no_weights = branch_weight == nullptr && weight == nullptr;
  if (width <= 1024 * 4 && width % 4 == 0 && (act_dtype == FMS_F32 || act_dtype == FMS_BF16) &&
      (no_weights || weight_dtype == FMS_F32 || weight_dtype == FMS_BF16)) {
#define SMALL(T, WT)                                                                                                    \
  norm_add_norm_small_kernel<T, WT, 4><<<n_out, 256, 0, stream>>>(resid, (const T*)branch, (const WT*)branch_weight, branch_eps, \
                                                                  (const WT*)weight, eps, (T*)out, rows, width)
    if (act_dtype == FMS_F32 && (no_weights || weight_dtype == FMS_F32)) SMALL(float, float);
    else if (act_dtype == FMS_F32) SMALL(float, bf16);
    else if (no_weights || weight_dtype == FMS_BF16) SMALL(bf16, bf16);
    else SMALL(bf16, float);
#undef SMALL
    FMS_LAUNCH_CHECK("norm_add_norm");
    return 0;
  }
  if (act_dtype == FMS_F32)
    norm_add_norm_kernel<float><<<n_out, 256, lds, stream>>>(resid, (const float*)branch, branch_weight, branch_eps,
                                                             weight, weight_dtype, eps, (float*)out, rows, width);
  else if (act_dtype == FMS_BF16)
    norm_add_norm_kernel<bf16><<<n_out, 256, lds, stream>>>(resid, (const bf16*)branch, branch_weight, branch_eps,
                                                            weight, weight_dtype, eps, (bf16*)out, rows, width);
  else
    FMS_REQUIRE(false, "norm_add_norm: unknown dtype %d", act_dtype);
  FMS_LAUNCH_CHECK("norm_add_norm");
  return 0;
}

// out[t, 0:n] = x[t, col0 : col0 + n] / rms * w, x float32 with rows ldx apart
template <typename T>
__global__ void __launch_bounds__(256)
    rms_norm_cols_kernel(const float* __restrict__ x, long ldx, int col0, int n, const void* __restrict__ w, int w_dtype,
                         float eps, T* __restrict__ out, long ldo) {
  __shared__ float scratch[17];
  const float* xr = x + (size_t)blockIdx.x * ldx + col0;
  float sq = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) sq = fmaf(xr[i], xr[i], sq);
  const float rs = rsqrtf(block_sum(sq, scratch) / (float)n + eps);
  T* o = out + (size_t)blockIdx.x * ldo;
  for (int i = threadIdx.x; i < n; i += blockDim.x) o[i] = from_f32<T>(xr[i] * rs * load_scale(w, w_dtype, i));
}

extern "C" int fmsamd_rms_norm_cols(const float* x, long ldx, int col0, int n, const void* weight, int weight_dtype,
                                    float eps, void* out, int out_dtype, long ldo, int rows, hipStream_t stream) {
  if (rows == 0) return 0;
  FMS_REQUIRE(rows > 0 && n > 0 && col0 >= 0 && ldx >= col0 + n && ldo >= n, "rms_norm_cols: bad sizes rows=%d n=%d col0=%d ldx=%ld",
              rows, n, col0, ldx);
  if (out_dtype == FMS_F32)
    rms_norm_cols_kernel<float><<<rows, 256, 0, stream>>>(x, ldx, col0, n, weight, weight_dtype, eps, (float*)out, ldo);
  else if (out_dtype == FMS_BF16)
    rms_norm_cols_kernel<bf16><<<rows, 256, 0, stream>>>(x, ldx, col0, n, weight, weight_dtype, eps, (bf16*)out, ldo);
  else
    FMS_REQUIRE(false, "rms_norm_cols: unknown dtype %d", out_dtype);
  FMS_LAUNCH_CHECK("rms_norm_cols");
  return 0;
}

// out[t, :] = a z / rms(z) + b z^2 / rms(z^2) + c z^3 / rms(z^3) + e over a token's n values (powers element by element,
// eps inside every root): z float32 rows ldz apart.  One block per row; the three sums of squares are float32.
template <typename T>
__global__ void __launch_bounds__(256)
    poly_norm_kernel(const float* __restrict__ z, long ldz, int n, float a, float b, float c, float e, float eps,
                     T* __restrict__ out, long ldo) {
  __shared__ float scratch[17];
  const float* zr = z + (size_t)blockIdx.x * ldz;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float v = zr[i], v2 = v * v, v3 = v2 * v;
    s2 = fmaf(v, v, s2);
    s4 = fmaf(v2, v2, s4);
    s6 = fmaf(v3, v3, s6);
  }
  const float r1 = a * rsqrtf(block_sum(s2, scratch) / (float)n + eps);
  const float r2 = b * rsqrtf(block_sum(s4, scratch) / (float)n + eps);
  const float r3 = c * rsqrtf(block_sum(s6, scratch) / (float)n + eps);
  T* o = out + (size_t)blockIdx.x * ldo;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float v = zr[i], v2 = v * v;
    o[i] = from_f32<T>(fmaf(r1, v, fmaf(r2, v2, fmaf(r3, v2 * v, e))));
  }
}

// Rows of at most THREADS * 4 * NV elements (a multiple of 4, rows 16 bytes aligned): a thread keeps its NV groups of four
// elements in registers, so the row is read once, and the three sums are reduced together.
template <typename T, int NV>
__global__ void __launch_bounds__(1024)
    poly_norm_reg_kernel(const float* __restrict__ z, long ldz, int n, float a, float b, float c, float e, float eps,
                         T* __restrict__ out, long ldo) {
  __shared__ float sums[3][16];
  const float* zr = z + (size_t)blockIdx.x * ldz;
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE, nwaves = blockDim.x / WAVE;
  float4 v[NV];
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int i = (k * blockDim.x + threadIdx.x) * 4;
    v[k] = i < n ? *reinterpret_cast<const float4*>(zr + i) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const float q[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float v2 = q[j] * q[j], v3 = v2 * q[j];
      s2 = fmaf(q[j], q[j], s2);
      s4 = fmaf(v2, v2, s4);
      s6 = fmaf(v3, v3, s6);
    }
  }
  s2 = wave_sum(s2), s4 = wave_sum(s4), s6 = wave_sum(s6);
  if (lane == 0) sums[0][wave] = s2, sums[1][wave] = s4, sums[2][wave] = s6;
  __syncthreads();
  float t2 = 0.f, t4 = 0.f, t6 = 0.f;
  for (int w = 0; w < nwaves; ++w) t2 += sums[0][w], t4 += sums[1][w], t6 += sums[2][w];  // the same order in every thread
  const float r1 = a * rsqrtf(t2 / (float)n + eps), r2 = b * rsqrtf(t4 / (float)n + eps), r3 = c * rsqrtf(t6 / (float)n + eps);
  T* o = out + (size_t)blockIdx.x * ldo;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int i = (k * blockDim.x + threadIdx.x) * 4;
    if (i < n) {
      const float q[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
      f32x4 r;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float v2 = q[j] * q[j];
        r[j] = fmaf(r1, q[j], fmaf(r2, v2, fmaf(r3, v2 * q[j], e)));
      }
      store4(o + i, r);
    }
  }
}

extern "C" int fmsamd_poly_norm(const float* z, long ldz, int n, float a, float b, float c, float e, float eps, void* out,
                                int out_dtype, long ldo, int rows, hipStream_t stream) {
  if (rows == 0) return 0;
  FMS_REQUIRE(rows > 0 && n > 0 && ldz >= n && ldo >= n, "poly_norm: bad sizes rows=%d n=%d ldz=%ld ldo=%ld", rows, n, ldz, ldo);
  // a step of few rows has few blocks: more threads a row
  const int threads = rows <= 128 ? 1024 : 256;
  const int nv = ceil_div(n, threads * 4);
  const size_t esize = out_dtype == FMS_F32 ? 4 : 2;
  if (n % 4 == 0 && ldz % 4 == 0 && ldo % 4 == 0 && ((uintptr_t)z % 16) == 0 && ((uintptr_t)out % (4 * esize)) == 0 && nv <= 8 &&
      (out_dtype == FMS_F32 || out_dtype == FMS_BF16)) {
#define FMS_POLY(NV)                                                                                                       \
  do {                                                                                                                     \
    if (out_dtype == FMS_F32)                                                                                              \
      poly_norm_reg_kernel<float, NV><<<rows, threads, 0, stream>>>(z, ldz, n, a, b, c, e, eps, (float*)out, ldo);         \
    else                                                                                                                   \
      poly_norm_reg_kernel<bf16, NV><<<rows, threads, 0, stream>>>(z, ldz, n, a, b, c, e, eps, (bf16*)out, ldo);           \
  } while (0)
    if (nv <= 1) FMS_POLY(1);
    else if (nv <= 2) FMS_POLY(2);
    else if (nv <= 4) FMS_POLY(4);
    else FMS_POLY(8);
#undef FMS_POLY
    FMS_LAUNCH_CHECK("poly_norm_reg");
    return 0;
  }
  if (out_dtype == FMS_F32)
    poly_norm_kernel<float><<<rows, 256, 0, stream>>>(z, ldz, n, a, b, c, e, eps, (float*)out, ldo);
  else if (out_dtype == FMS_BF16)
    poly_norm_kernel<bf16><<<rows, 256, 0, stream>>>(z, ldz, n, a, b, c, e, eps, (bf16*)out, ldo);
  else
    FMS_REQUIRE(false, "poly_norm: unknown dtype %d", out_dtype);
  FMS_LAUNCH_CHECK("poly_norm");
  return 0;
}

template <typename T>
__global__ void activate_kernel(const T* __restrict__ x, T* __restrict__ out, long n, int act) {
  const long stride = (long)gridDim.x * blockDim.x;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    out[i] = from_f32<T>(fms_activate(to_f32(x[i]), act));
}

// four elements a thread and step, for element counts that are multiples of 4
template <typename T>
__global__ void activate4_kernel(const T* __restrict__ x, T* __restrict__ out, long n4, int act) {
  const long stride = (long)gridDim.x * blockDim.x;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
    f32x4 v = load4(x + 4 * i);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = fms_activate(v[e], act);
    store4(out + 4 * i, v);
  }
}

extern "C" int fmsamd_activate(const void* x, void* out, int dtype, long n, int act, hipStream_t stream) {
  if (n == 0) return 0;
  FMS_REQUIRE(n > 0 && act >= 0 && act <= FMS_ACT_LAST, "activate: bad arguments n=%ld act=%d", n, act);
  if (n % 4 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)out % 16) == 0 && (dtype == FMS_F32 || dtype == FMS_BF16)) {
    const long n4 = n / 4;
    const int blocks4 = (int)((n4 + 255) / 256 < 8192 ? (n4 + 255) / 256 : 8192);
    if (dtype == FMS_F32)
      activate4_kernel<float><<<blocks4, 256, 0, stream>>>((const float*)x, (float*)out, n4, act);
    else
      activate4_kernel<bf16><<<blocks4, 256, 0, stream>>>((const bf16*)x, (bf16*)out, n4, act);
    FMS_LAUNCH_CHECK("activate");
    return 0;
  }
  const int blocks = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
  if (dtype == FMS_F32)
    activate_kernel<float><<<blocks, 256, 0, stream>>>((const float*)x, (float*)out, n, act);
  else if (dtype == FMS_BF16)
    activate_kernel<bf16><<<blocks, 256, 0, stream>>>((const bf16*)x, (bf16*)out, n, act);
  else
    FMS_REQUIRE(false, "activate: unknown dtype %d", dtype);
  FMS_LAUNCH_CHECK("activate");
  return 0;
}

__device__ __forceinline__ float clamped_gate(float g, float u, float limit, float alpha, float shift) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.f + expf(-alpha * g)) * (u + shift);
}

// gu [T, 2 * hidden] (gate first), out [T, hidden]; hidden a multiple of 4: four elements a thread and step
template <typename T>
__global__ void clamped_gated_act4_kernel(const T* __restrict__ gu, T* __restrict__ out, int hidden, float limit, float alpha,
                                          float shift) {
  const T* g = gu + (size_t)blockIdx.x * 2 * hidden;
  T* o = out + (size_t)blockIdx.x * hidden;
  for (int i = threadIdx.x * 4; i < hidden; i += blockDim.x * 4) {
    const f32x4 gv = load4(g + i), uv = load4(g + hidden + i);
    f32x4 r;
#pragma unroll
    for (int e = 0; e < 4; ++e) r[e] = clamped_gate(gv[e], uv[e], limit, alpha, shift);
    store4(o + i, r);
  }
}

template <typename T>
__global__ void clamped_gated_act_kernel(const T* __restrict__ gu, T* __restrict__ out, int hidden, float limit,
                                         float alpha, float shift) {
  const T* g = gu + (size_t)blockIdx.x * 2 * hidden;
  T* o = out + (size_t)blockIdx.x * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x)
    o[i] = from_f32<T>(clamped_gate(to_f32(g[i]), to_f32(g[hidden + i]), limit, alpha, shift));
}

extern "C" int fmsamd_clamped_gated_act(const void* gu, void* out, int dtype, int n_tokens, int hidden, float limit,
                                        float alpha, float shift, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  FMS_REQUIRE(n_tokens > 0 && hidden > 0 && limit > 0.f, "clamped_gated_act: bad arguments T=%d hidden=%d limit=%g", n_tokens,
              hidden, (double)limit);
  if (hidden % 4 == 0 && ((uintptr_t)gu % 16) == 0 && ((uintptr_t)out % 16) == 0 && (dtype == FMS_F32 || dtype == FMS_BF16)) {
    if (dtype == FMS_F32)
      clamped_gated_act4_kernel<float><<<n_tokens, 256, 0, stream>>>((const float*)gu, (float*)out, hidden, limit, alpha, shift);
    else
      clamped_gated_act4_kernel<bf16><<<n_tokens, 256, 0, stream>>>((const bf16*)gu, (bf16*)out, hidden, limit, alpha, shift);
    FMS_LAUNCH_CHECK("clamped_gated_act");
    return 0;
  }
  if (dtype == FMS_F32)
    clamped_gated_act_kernel<float><<<n_tokens, 256, 0, stream>>>((const float*)gu, (float*)out, hidden, limit, alpha, shift);
  else if (dtype == FMS_BF16)
    clamped_gated_act_kernel<bf16><<<n_tokens, 256, 0, stream>>>((const bf16*)gu, (bf16*)out, hidden, limit, alpha, shift);
  else
    FMS_REQUIRE(false, "clamped_gated_act: unknown dtype %d", dtype);
  FMS_LAUNCH_CHECK("clamped_gated_act");
  return 0;
}

// --------------------------------------------------------------------------
// The chain for norms that may take the mean off and add a shift (layer norms on both sides of a branch):
//   stream += N(branch; wb, bb);  out = N(stream; w, b),  N(v; w, b) = (v - mean) / sqrt(var + eps) * w + b,
// var the mean of the squared deviations (without `mean`: no mean is taken off and var is the mean square).  One block
// per output row; the row waits in LDS between the reductions; the mean is found first and the deviations are squared
// afterwards, so nothing is lost where the mean is large against the spread.  All float32.
// --------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
    norm_add_norm_affine_kernel(float* __restrict__ resid, const T* __restrict__ branch, const void* __restrict__ wb,
                                const void* __restrict__ bb, float eps_b, int mean_b, const void* __restrict__ w,
                                const void* __restrict__ b, int w_dtype, float eps, int use_mean, T* __restrict__ out,
                                const int* __restrict__ rows, int width) {
  extern __shared__ float row[];
  __shared__ float scratch[17];
  const int r = rows ? rows[blockIdx.x] : blockIdx.x;
  float* x = resid + (size_t)r * width;
  const T* br = branch + (size_t)r * width;
  const float inv_n = 1.f / (float)width;
  float s = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = to_f32(br[i]);
    row[i] = v;
    s += v;
  }
  float mean = mean_b ? block_sum(s, scratch) * inv_n : 0.f;
  float sq = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float d = row[i] - mean;
    sq = fmaf(d, d, sq);
  }
  float rs = rsqrtf(block_sum(sq, scratch) * inv_n + eps_b);
  s = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = (row[i] - mean) * rs * load_scale(wb, w_dtype, i);
    if (bb != nullptr) v += load_scale(bb, w_dtype, i);
    v += x[i];
    row[i] = v;
    if (!rows) x[i] = v;
    s += v;
  }
  if (out == nullptr) return;
  mean = use_mean ? block_sum(s, scratch) * inv_n : 0.f;
  sq = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float d = row[i] - mean;
    sq = fmaf(d, d, sq);
  }
  rs = rsqrtf(block_sum(sq, scratch) * inv_n + eps);
  T* o = out + (size_t)blockIdx.x * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = (row[i] - mean) * rs * load_scale(w, w_dtype, i);
    if (b != nullptr) v += load_scale(b, w_dtype, i);
    o[i] = from_f32<T>(v);
  }
}

// The same for rows of at most 1024 * KEEP elements (a multiple of 4): branch, stream and the four vectors are asked for
// at once, four elements a load, and wait in registers, so the kernel pays the memory's latency once (a decode step's
// rows are few, and nothing else hides it: with the row in LDS and every vector loaded where it is used the kernel took
// 18.6 microseconds for eight rows of 2048).
template <typename T, typename WT, int KEEP>
__global__ void __launch_bounds__(256)
    norm_add_norm_affine_small_kernel(float* __restrict__ resid, const T* __restrict__ branch, const WT* __restrict__ wb,
                                      const WT* __restrict__ bb, float eps_b, int mean_b, const WT* __restrict__ w,
                                      const WT* __restrict__ b, float eps, int use_mean, T* __restrict__ out,
                                      const int* __restrict__ rows, int width) {
  __shared__ float scratch[17];
  const int r = rows ? rows[blockIdx.x] : blockIdx.x;
  float* x = resid + (size_t)r * width;
  const T* br = branch + (size_t)r * width;
  const f32x4 ones = {1.f, 1.f, 1.f, 1.f}, zeros = {0.f, 0.f, 0.f, 0.f};
  f32x4 bv[KEEP], xv[KEEP], wbv[KEEP], bbv[KEEP], wv[KEEP], sv[KEEP];
  const float inv_n = 1.f / (float)width;
  float s = 0.f;
#pragma unroll
  for (int n = 0; n < KEEP; ++n) {
    const int i = (threadIdx.x + n * 256) * 4;
    bv[n] = zeros, xv[n] = zeros, wbv[n] = ones, bbv[n] = zeros, wv[n] = ones, sv[n] = zeros;
    if (i < width) {
      bv[n] = load4(br + i);
      xv[n] = load4(x + i);
      if (wb) wbv[n] = load4(wb + i);
      if (bb) bbv[n] = load4(bb + i);
      if (w) wv[n] = load4(w + i);
      if (b) sv[n] = load4(b + i);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) s += bv[n][e];
  }
  float mean = mean_b ? block_sum(s, scratch) * inv_n : 0.f;
  float sq = 0.f;
#pragma unroll
  for (int n = 0; n < KEEP; ++n) {
    const bool in = (threadIdx.x + n * 256) * 4 < width;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float d = in ? bv[n][e] - mean : 0.f;  // elements past the row count for nothing
      bv[n][e] = d;
      sq = fmaf(d, d, sq);
    }
  }
  float rs = rsqrtf(block_sum(sq, scratch) * inv_n + eps_b);
  s = 0.f;
#pragma unroll
  for (int n = 0; n < KEEP; ++n) {
    const int i = (threadIdx.x + n * 256) * 4;
    const bool in = i < width;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      xv[n][e] = in ? xv[n][e] + (bv[n][e] * rs * wbv[n][e] + bbv[n][e]) : 0.f;
      s += xv[n][e];
    }
    if (in && !rows) store4(x + i, xv[n]);
  }
  if (out == nullptr) return;
  mean = use_mean ? block_sum(s, scratch) * inv_n : 0.f;
  sq = 0.f;
#pragma unroll
  for (int n = 0; n < KEEP; ++n) {
    const bool in = (threadIdx.x + n * 256) * 4 < width;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float d = in ? xv[n][e] - mean : 0.f;
      xv[n][e] = d;
      sq = fmaf(d, d, sq);
    }
  }
  rs = rsqrtf(block_sum(sq, scratch) * inv_n + eps);
  T* o = out + (size_t)blockIdx.x * width;
#pragma unroll
  for (int n = 0; n < KEEP; ++n) {
    const int i = (threadIdx.x + n * 256) * 4;
    if (i < width) {
      f32x4 y;
#pragma unroll
      for (int e = 0; e < 4; ++e) y[e] = xv[n][e] * rs * wv[n][e] + sv[n][e];
      store4(o + i, y);
    }
  }
}

extern "C" int fmsamd_norm_add_norm_affine(float* resid, const void* branch, int act_dtype, const void* branch_weight,
                                           const void* branch_bias, float branch_eps, int branch_mean, const void* weight,
                                           const void* bias, int weight_dtype, float eps, int use_mean, void* out,
                                           const int* rows, int n_out, int width, hipStream_t stream) {
  if (n_out == 0) return 0;
  FMS_REQUIRE(n_out > 0 && width > 0 && width <= 16384, "norm_add_norm_affine: bad sizes rows=%d width=%d", n_out, width);
  FMS_REQUIRE(resid != nullptr && branch != nullptr, "norm_add_norm_affine: the stream and the branch are needed");
  const bool vectors = branch_weight || branch_bias || weight || bias;
  FMS_REQUIRE(!vectors || weight_dtype == FMS_F32 || weight_dtype == FMS_BF16, "norm_add_norm_affine: unknown weight dtype %d", weight_dtype);
  if (width <= 1024 * 4 && width % 4 == 0 && (act_dtype == FMS_F32 || act_dtype == FMS_BF16)) {
#define SMALL(T, WT)                                                                                                          \
  norm_add_norm_affine_small_kernel<T, WT, 4><<<n_out, 256, 0, stream>>>(resid, (const T*)branch, (const WT*)branch_weight,   \
                                                                         (const WT*)branch_bias, branch_eps, branch_mean,     \
                                                                         (const WT*)weight, (const WT*)bias, eps, use_mean,   \
                                                                         (T*)out, rows, width)
    if (act_dtype == FMS_F32 && (!vectors || weight_dtype == FMS_F32)) SMALL(float, float);
    else if (act_dtype == FMS_F32) SMALL(float, bf16);
    else if (!vectors || weight_dtype == FMS_BF16) SMALL(bf16, bf16);
    else SMALL(bf16, float);
#undef SMALL
    FMS_LAUNCH_CHECK("norm_add_norm_affine");
    return 0;
  }
  const size_t lds = (size_t)width * sizeof(float);
  if (act_dtype == FMS_F32)
    norm_add_norm_affine_kernel<float><<<n_out, 256, lds, stream>>>(resid, (const float*)branch, branch_weight, branch_bias, branch_eps,
                                                                    branch_mean, weight, bias, weight_dtype, eps, use_mean,
                                                                    (float*)out, rows, width);
  else if (act_dtype == FMS_BF16)
    norm_add_norm_affine_kernel<bf16><<<n_out, 256, lds, stream>>>(resid, (const bf16*)branch, branch_weight, branch_bias, branch_eps,
                                                                   branch_mean, weight, bias, weight_dtype, eps, use_mean,
                                                                   (bf16*)out, rows, width);
  else
    FMS_REQUIRE(false, "norm_add_norm_affine: unknown dtype %d", act_dtype);
  FMS_LAUNCH_CHECK("norm_add_norm_affine");
  return 0;
}
