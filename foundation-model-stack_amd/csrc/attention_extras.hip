// Steps around attention that some mixers have and others do not:
//   qk_projection_norm: an RMS norm over the whole query projection and one over the whole key projection (all heads
//                       at once, before they are cut into heads and rotated), or head by head with one weight for all
//                       heads, from the float32 sums of the projection; the values are copied, or blended with the values
//                       that an earlier layer left for the same token.  One rounding to the activation type.
//   gate_mul:           out = x * act(gate) * scale (gate: float32 logits, one a column or one a run of columns, or none),
//                       into rows of any stride.
//   cast_cols:          a run of columns of float32 rows as rows of their own, in the activation type.
//   scale_f32:          x *= s in place.
#include "common.h"
#include "fmsamd.h"

// the values of a row: copied, or blended with the values another layer left for the same token
template <typename T>
__device__ __forceinline__ void copy_values(const float* __restrict__ row, T* __restrict__ o, int nv, const T* __restrict__ first,
                                            const float* __restrict__ lambda) {
  if (first != nullptr) {
    const float lam = *lambda;
    for (int i = threadIdx.x; i < nv; i += blockDim.x) o[i] = from_f32<T>((1.f - lam) * row[i] + lam * to_f32(first[i]));
  } else {
    for (int i = threadIdx.x; i < nv; i += blockDim.x) o[i] = from_f32<T>(row[i]);
  }
}

template <typename T, typename W>
__global__ void __launch_bounds__(1024)
    qk_projection_norm_kernel(const float* __restrict__ proj, long ld, int nq, int nk, int nv, const W* __restrict__ wq,
                              const W* __restrict__ wk, float eps, T* __restrict__ out, long ldo,
                              const int* __restrict__ seq_of_token, const T* __restrict__ v_first, long ld_first,
                              const float* __restrict__ v_lambda) {
  __shared__ float scratch[17];
  const int t = blockIdx.x;
  if (seq_of_token != nullptr && seq_of_token[t] < 0) return;
  const float* row = proj + (size_t)t * ld;
  T* o = out + (size_t)t * ldo;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < nq; i += blockDim.x) sq = fmaf(row[i], row[i], sq);
  for (int i = threadIdx.x; i < nk; i += blockDim.x) sk = fmaf(row[nq + i], row[nq + i], sk);
  sq = block_sum(sq, scratch);
  sk = block_sum(sk, scratch);
  const float iq = 1.f / sqrtf(sq / (float)nq + eps), ik = 1.f / sqrtf(sk / (float)nk + eps);
  for (int i = threadIdx.x; i < nq; i += blockDim.x) o[i] = from_f32<T>(row[i] * iq * (wq ? to_f32(wq[i]) : 1.f));
  for (int i = threadIdx.x; i < nk; i += blockDim.x) o[nq + i] = from_f32<T>(row[nq + i] * ik * (wk ? to_f32(wk[i]) : 1.f));
  copy_values<T>(row + nq + nk, o + nq + nk, nv, v_first ? v_first + (size_t)t * ld_first : nullptr, v_lambda);
}

// The norms head by head: a wave takes the heads of queries and keys in turn (a head is dim consecutive columns), so the
// sums are wave reductions and no barrier is needed.  The weights have dim entries and serve every head.
template <typename T, typename W>
__global__ void __launch_bounds__(1024)
    qk_head_norm_kernel(const float* __restrict__ proj, long ld, int nq, int nk, int nv, int dim, const W* __restrict__ wq,
                        const W* __restrict__ wk, float eps, T* __restrict__ out, long ldo, const int* __restrict__ seq_of_token,
                        const T* __restrict__ v_first, long ld_first, const float* __restrict__ v_lambda) {
  const int t = blockIdx.x;
  if (seq_of_token != nullptr && seq_of_token[t] < 0) return;
  const float* row = proj + (size_t)t * ld;
  T* o = out + (size_t)t * ldo;
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE, n_waves = blockDim.x / WAVE;
  const int q_heads = nq / dim, heads = (nq + nk) / dim;
  for (int head = wave; head < heads; head += n_waves) {
    const float* x = row + (size_t)head * dim;
    const W* w = head < q_heads ? wq : wk;
    float s = 0.f;
    for (int i = lane; i < dim; i += WAVE) s = fmaf(x[i], x[i], s);
    const float inv = 1.f / sqrtf(wave_sum(s) / (float)dim + eps);
    for (int i = lane; i < dim; i += WAVE) o[(size_t)head * dim + i] = from_f32<T>(x[i] * inv * (w ? to_f32(w[i]) : 1.f));
  }
  copy_values<T>(row + nq + nk, o + nq + nk, nv, v_first ? v_first + (size_t)t * ld_first : nullptr, v_lambda);
}

extern "C" int fmsamd_qk_projection_norm(const float* proj, long ld, int nq, int nk, int nv, const void* wq, const void* wk,
                                         int weight_dtype, float eps, void* out, int out_dtype, long ldo, const int* seq_of_token,
                                         int n_tokens, int norm_dim, const void* v_first, long ld_first, const void* v_lambda,
                                         hipStream_t stream) {
  if (n_tokens == 0) return 0;
  FMS_REQUIRE(n_tokens > 0 && nq > 0 && nk > 0 && nv >= 0 && ld >= (long)nq + nk + nv && ldo >= (long)nq + nk + nv,
              "qk_projection_norm: bad sizes q=%d k=%d v=%d", nq, nk, nv);
  FMS_REQUIRE(norm_dim >= 0 && (norm_dim == 0 || (nq % norm_dim == 0 && nk % norm_dim == 0)),
              "qk_projection_norm: heads of %d do not divide queries (%d) and keys (%d)", norm_dim, nq, nk);
  FMS_REQUIRE(v_first == nullptr || (v_lambda != nullptr && ld_first >= nv), "qk_projection_norm: blended values need a factor and rows of %d", nv);
  const int threads = n_tokens <= 64 ? 1024 : 256;
#define FMS_QKN(T, W)                                                                                                        \
  do {                                                                                                                       \
    if (norm_dim > 0)                                                                                                        \
      qk_head_norm_kernel<T, W><<<n_tokens, threads, 0, stream>>>(proj, ld, nq, nk, nv, norm_dim, (const W*)wq, (const W*)wk, eps, \
                                                                  (T*)out, ldo, seq_of_token, (const T*)v_first, ld_first,  \
                                                                  (const float*)v_lambda);                                       \
    else                                                                                                                     \
      qk_projection_norm_kernel<T, W><<<n_tokens, threads, 0, stream>>>(proj, ld, nq, nk, nv, (const W*)wq, (const W*)wk, eps, \
                                                                        (T*)out, ldo, seq_of_token, (const T*)v_first,      \
                                                                        ld_first, (const float*)v_lambda);                       \
  } while (0)
  if (out_dtype == FMS_F32 && weight_dtype == FMS_F32) FMS_QKN(float, float);
  else if (out_dtype == FMS_BF16 && weight_dtype == FMS_F32) FMS_QKN(bf16, float);
  else if (out_dtype == FMS_BF16 && weight_dtype == FMS_BF16) FMS_QKN(bf16, bf16);
  else if (out_dtype == FMS_F32 && weight_dtype == FMS_BF16) FMS_QKN(float, bf16);
  else FMS_REQUIRE(false, "qk_projection_norm: unknown dtypes %d, %d", out_dtype, weight_dtype);
#undef FMS_QKN
  FMS_LAUNCH_CHECK("qk_projection_norm");
  return 0;
}

template <typename T>
__global__ void __launch_bounds__(1024)
    gate_mul_kernel(const T* __restrict__ x, long ldx, const float* __restrict__ gate, long ldg, int act, float scale,
                    T* __restrict__ out, long ldo, int cols, int group) {
  const int t = blockIdx.x;
  for (int i = threadIdx.x; i < cols; i += blockDim.x) {
    float v = to_f32(x[(size_t)t * ldx + i]) * scale;
    if (gate != nullptr) v *= fms_activate(gate[(size_t)t * ldg + i / group], act);
    out[(size_t)t * ldo + i] = from_f32<T>(v);
  }
}

extern "C" int fmsamd_gate_mul(const void* x, long ldx, const float* gate, long ldg, int act, float scale, void* out, long ldo,
                               int dtype, int n_tokens, int cols, int group, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  FMS_REQUIRE(group >= 1 && cols % group == 0, "gate_mul: runs of %d columns do not divide %d", group, cols);
  FMS_REQUIRE(n_tokens > 0 && cols > 0 && ldx >= cols && ldo >= cols && (gate == nullptr || ldg >= cols / group), "gate_mul: bad sizes");
  FMS_REQUIRE(act >= 0 && act <= FMS_ACT_LAST, "gate_mul: unknown activation %d", act);
  const int threads = n_tokens <= 64 ? 1024 : 256;  // few tokens: fewer passes a thread, fewer round trips in a row
  if (dtype == FMS_F32)
    gate_mul_kernel<float><<<n_tokens, threads, 0, stream>>>((const float*)x, ldx, gate, ldg, act, scale, (float*)out, ldo, cols, group);
  else if (dtype == FMS_BF16)
    gate_mul_kernel<bf16><<<n_tokens, threads, 0, stream>>>((const bf16*)x, ldx, gate, ldg, act, scale, (bf16*)out, ldo, cols, group);
  else
    FMS_REQUIRE(false, "gate_mul: unknown dtype %d", dtype);
  FMS_LAUNCH_CHECK("gate_mul");
  return 0;
}

// out[t, 0:n] = x[t, col0 : col0 + n] in another type
template <typename T>
__global__ void __launch_bounds__(1024) cast_cols_kernel(const float* __restrict__ x, long ldx, T* __restrict__ out, long ldo, int n) {
  const int t = blockIdx.x;
  for (int i = threadIdx.x; i < n; i += blockDim.x) out[(size_t)t * ldo + i] = from_f32<T>(x[(size_t)t * ldx + i]);
}

extern "C" int fmsamd_cast_cols(const float* x, long ldx, void* out, int out_dtype, long ldo, int n_tokens, int n, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  FMS_REQUIRE(n_tokens > 0 && n > 0 && ldx >= n && ldo >= n, "cast_cols: bad sizes");
  const int threads = n >= 1024 ? 1024 : (n >= 256 ? 256 : 64);
  if (out_dtype == FMS_F32) cast_cols_kernel<float><<<n_tokens, threads, 0, stream>>>(x, ldx, (float*)out, ldo, n);
  else if (out_dtype == FMS_BF16) cast_cols_kernel<bf16><<<n_tokens, threads, 0, stream>>>(x, ldx, (bf16*)out, ldo, n);
  else FMS_REQUIRE(false, "cast_cols: unknown dtype %d", out_dtype);
  FMS_LAUNCH_CHECK("cast_cols");
  return 0;
}

__global__ void __launch_bounds__(256) scale_f32_kernel(float* __restrict__ x, size_t n, float s) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) x[i] *= s;
}

extern "C" int fmsamd_scale_f32(float* x, long n, float s, hipStream_t stream) {
  if (n == 0) return 0;
  FMS_REQUIRE(n > 0, "scale_f32: negative count");
  const int blocks = ceil_div(n, 256) > 4096 ? 4096 : ceil_div(n, 256);
  scale_f32_kernel<<<blocks, 256, 0, stream>>>(x, (size_t)n, s);
  FMS_LAUNCH_CHECK("scale_f32");
  return 0;
}
