// Kernels of a routed feed-forward (a mixture of experts whose router's scores are a softmax, with a correction
// added for the choice only, and whose last outputs may be experts that hand their input through), of a dense
// feed-forward with biases and the exact gelu, and of layers with a norm on either side of every branch.
#include "common.h"

namespace {

__device__ __forceinline__ float silu_r(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float sigmoid_r(float z) { return 1.0f / (1.0f + expf(-z)); }

// ----------------------------------------------------------------------------- router
// One wave a token.  z [n, z_stride]: 32-bit router outputs, the first n_out of a row.  s = softmax(z); the `top`
// largest of s + correction are chosen (of equal ones the lower index), and the weights are their s.
constexpr int kRouterPerLane = 8;  // outputs a lane holds: up to 512 experts
__global__ void __launch_bounds__(256)
router_topk_kernel(const float* __restrict__ z, int z_stride, const float* __restrict__ correction, int n, int n_out, int top,
                   int32_t* __restrict__ ids, float* __restrict__ weights) {
  const int t = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  if (t >= n) return;
  const float* zr = z + (size_t)t * z_stride;
  float s[kRouterPerLane], c[kRouterPerLane];
  float mx = -INFINITY;
#pragma unroll
  for (int u = 0; u < kRouterPerLane; ++u) {
    const int e = lane + u * kWave;
    s[u] = e < n_out ? zr[e] : -INFINITY;
    mx = fmaxf(mx, s[u]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int u = 0; u < kRouterPerLane; ++u) {
    const int e = lane + u * kWave;
    s[u] = e < n_out ? expf(s[u] - mx) : 0.f;
    sum += s[u];
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int u = 0; u < kRouterPerLane; ++u) {
    const int e = lane + u * kWave;
    s[u] = s[u] / sum;
    c[u] = e < n_out ? s[u] + correction[e] : -INFINITY;
  }
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY, best_s = 0.f;
    int best_e = 0x7fffffff;
#pragma unroll
    for (int u = 0; u < kRouterPerLane; ++u) {
      const int e = lane + u * kWave;
      if (e < n_out && (c[u] > best || (c[u] == best && e < best_e))) { best = c[u]; best_e = e; best_s = s[u]; }
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, kWave), os = __shfl_xor(best_s, off, kWave);
      const int oe = __shfl_xor(best_e, off, kWave);
      if (ob > best || (ob == best && oe < best_e)) { best = ob; best_e = oe; best_s = os; }
    }
    if (lane == 0) {
      ids[(size_t)t * top + k] = best_e;
      weights[(size_t)t * top + k] = best_s;
    }
#pragma unroll
    for (int u = 0; u < kRouterPerLane; ++u)
      if (lane + u * kWave == best_e) c[u] = -INFINITY;
  }
}

// ----------------------------------------------------------------------------- experts, a (token, choice) at a time
// mid[p, f] = T(silu(Wg[e] x) * (Wu[e] x)) for the pair p = (token t, choice j), e = ids[p] < n_experts; pairs whose
// expert hands its input through are left alone.  w_gu [E][2F][D] (an expert's gate rows, then its up rows).  A wave
// takes an output at a time, its lanes the row's elements V at a time; the sums have an order fixed by D alone.
constexpr int kPairThreads = 256;
template <typename T, int V>
__global__ void __launch_bounds__(kPairThreads)
expert_glu_pairs_kernel(const T* __restrict__ x, const T* __restrict__ w_gu, const int32_t* __restrict__ ids, int top, int n_experts,
                        T* __restrict__ mid, int D, int F, int f_per_block) {
  extern __shared__ __attribute__((aligned(16))) float x_l[];
  const int p = blockIdx.x;
  const int e = ids[p];
  if (e >= n_experts) return;
  const T* xr = x + (size_t)(p / top) * D;
  for (int d = threadIdx.x; d < D; d += kPairThreads) x_l[d] = to_f32(xr[d]);
  __syncthreads();
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int f_end = min(F, (blockIdx.y + 1) * f_per_block);
  const T* wg = w_gu + (size_t)e * 2 * F * D;
  for (int f = blockIdx.y * f_per_block + wave; f < f_end; f += kPairThreads / kWave) {
    const T* g_row = wg + (size_t)f * D;
    const T* u_row = wg + (size_t)(F + f) * D;
    float ag = 0.f, au = 0.f;
    for (int d0 = lane * V; d0 < D; d0 += kWave * V) {
      struct alignas(sizeof(T) * V) Vec { T e[V]; };
      const Vec gv = *reinterpret_cast<const Vec*>(g_row + d0);
      const Vec uv = *reinterpret_cast<const Vec*>(u_row + d0);
#pragma unroll
      for (int i = 0; i < V; ++i) {
        ag = fmaf(to_f32(gv.e[i]), x_l[d0 + i], ag);
        au = fmaf(to_f32(uv.e[i]), x_l[d0 + i], au);
      }
    }
    ag = wave_sum(ag);
    au = wave_sum(au);
    if (lane == 0) mid[(size_t)p * F + f] = from_f32<T>(silu_r(ag) * au);
  }
}

// out[t, d] = T(sum_j w[t, j] * (e_j < n_experts ? Wd[e_j][d] . mid[t, j] : x[t, d]) + sigmoid(sg[t]) * shared[t, d]);
// w_d [E][D][F]; shared (or null) [n, D] with its gate's 32-bit pre-activation sg[t * sg_stride].  The pairs of a token
// are added in the order of its choices.
template <typename T, int V>
__global__ void __launch_bounds__(kPairThreads)
expert_down_pairs_kernel(const T* __restrict__ mid, const T* __restrict__ w_d, const int32_t* __restrict__ ids,
                         const float* __restrict__ weights, int top, int n_experts, const T* __restrict__ x,
                         const T* __restrict__ shared, const float* __restrict__ sg, int sg_stride, T* __restrict__ out, int D,
                         int F, int d_per_block) {
  extern __shared__ __attribute__((aligned(16))) float mid_l[];  // [top][F]
  const int t = blockIdx.x;
  for (int i = threadIdx.x; i < top * F; i += kPairThreads) {
    const int j = i / F;
    mid_l[i] = ids[(size_t)t * top + j] < n_experts ? to_f32(mid[(size_t)t * top * F + i]) : 0.f;
  }
  __syncthreads();
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int d_end = min(D, (blockIdx.y + 1) * d_per_block);
  const float share = shared ? sigmoid_r(sg[(size_t)t * sg_stride]) : 0.f;
  for (int d = blockIdx.y * d_per_block + wave; d < d_end; d += kPairThreads / kWave) {
    float total = 0.f;
    for (int j = 0; j < top; ++j) {
      const int e = ids[(size_t)t * top + j];
      const float wj = weights[(size_t)t * top + j];
      if (e >= n_experts) {
        total += wj * to_f32(x[(size_t)t * D + d]);
        continue;
      }
      const T* row = w_d + ((size_t)e * D + d) * F;
      const float* m = mid_l + j * F;
      float acc = 0.f;
      for (int f0 = lane * V; f0 < F; f0 += kWave * V) {
        struct alignas(sizeof(T) * V) Vec { T e[V]; };
        const Vec wv = *reinterpret_cast<const Vec*>(row + f0);
#pragma unroll
        for (int i = 0; i < V; ++i) acc = fmaf(to_f32(wv.e[i]), m[f0 + i], acc);
      }
      total += wj * wave_sum(acc);
    }
    if (shared) total += share * to_f32(shared[(size_t)t * D + d]);
    if (lane == 0) out[(size_t)t * D + d] = from_f32<T>(total);
  }
}

// ----------------------------------------------------------------------------- dense feed-forward with biases
// x[r, c] <- T(gelu(x[r, c] + b[c])), gelu(z) = z/2 (1 + erf(z / sqrt 2)), in 32-bit.
template <typename T>
__global__ void __launch_bounds__(256)
bias_gelu_kernel(T* __restrict__ x, const T* __restrict__ b, size_t total, int width) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    const float z = to_f32(x[i]) + to_f32(b[i % width]);
    x[i] = from_f32<T>(0.5f * z * (1.0f + erff(z * 0.70710678118654752440f)));
  }
}

// out[i] = T(sa * a[i] + sb * b[i]) in 32-bit: two branches that read the same rows, weighted and added.
template <typename T>
__global__ void __launch_bounds__(256)
weighted_pair_kernel(const T* __restrict__ a, float sa, const T* __restrict__ b, float sb, T* __restrict__ out, size_t total) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x)
    out[i] = from_f32<T>(sa * to_f32(a[i]) + sb * to_f32(b[i]));
}

// ----------------------------------------------------------------------------- a branch's result into the stream, and the next norm
// stream[r] += y[r] / sqrt(mean(y[r]^2) + eps) * w_post (32-bit, in place), and, where w_next is given,
// rows[r] = T(stream[r] / sqrt(mean(stream[r]^2) + eps_next) * w_next): the norm behind a branch and the norm before
// the next one in a single pass over the row, which stays in LDS in between.
constexpr int kSandwichThreads = 256;
template <typename T>
__global__ void __launch_bounds__(kSandwichThreads)
post_norm_add_norm_kernel(float* __restrict__ stream, const T* __restrict__ y, const float* __restrict__ w_post, float eps,
                          const float* __restrict__ w_next, float eps_next, T* __restrict__ rows, int hidden) {
#pragma clang fp contract(off)
  extern __shared__ __attribute__((aligned(16))) float row_l[];
  __shared__ float scratch[kSandwichThreads / kWave];
  const size_t r = blockIdx.x;
  const T* yr = y + r * hidden;
  float* sr = stream + r * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += kSandwichThreads) {
    const float v = to_f32(yr[i]);
    row_l[i] = v;
    ss += v * v;
  }
  ss = block_sum<kSandwichThreads / kWave>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)hidden + eps);
  float s2 = 0.f;
  for (int i = threadIdx.x; i < hidden; i += kSandwichThreads) {
    const float h = sr[i] + row_l[i] * inv * w_post[i];
    sr[i] = h;
    row_l[i] = h;
    s2 += h * h;
  }
  if (w_next == nullptr) return;
  s2 = block_sum<kSandwichThreads / kWave>(s2, scratch);
  const float inv2 = 1.0f / sqrtf(s2 / (float)hidden + eps_next);
  for (int i = threadIdx.x; i < hidden; i += kSandwichThreads) rows[r * hidden + i] = from_f32<T>(row_l[i] * inv2 * w_next[i]);
}

}  // namespace

// ============================================================================= C interface
TL_EXPORT int tl_router_topk(const float* z, int z_stride, const float* correction, int n, int n_out, int top, int32_t* ids,
                             float* weights, hipStream_t stream) {
  TL_REQUIRE(n >= 0 && n_out > 0 && top > 0 && top <= n_out && z_stride >= n_out, "router_topk: bad sizes");
  if (n_out > kRouterPerLane * kWave)
    return tl_fail(TL_ERR_UNSUPPORTED, "router_topk: %d router outputs, at most %d", n_out, kRouterPerLane * kWave);
  if (n == 0) return TL_OK;
  const int per_block = 256 / kWave;
  router_topk_kernel<<<(n + per_block - 1) / per_block, 256, 0, stream>>>(z, z_stride, correction, n, n_out, top, ids, weights);
  return tl_check_launch("router_topk");
}

TL_EXPORT int tl_expert_glu_pairs(const void* x, const void* w_gu, const int32_t* ids, int top, int n_experts, void* mid, int n,
                                  int D, int F, int dtype, hipStream_t stream) {
  TL_REQUIRE(n >= 0 && top > 0 && n_experts >= 0 && D > 0 && F > 0, "expert_glu_pairs: bad sizes");
  TL_REQUIRE((long long)n * top <= 0x7fffffff, "expert_glu_pairs: too many pairs a step");
  if (n == 0 || n_experts == 0) return TL_OK;
  const size_t lds = (size_t)D * sizeof(float);
  if (lds > (size_t)tl_device_facts().lds_bytes)
    return tl_fail(TL_ERR_UNSUPPORTED, "expert_glu_pairs: rows of %d elements do not fit the LDS", D);
  // blocks: enough to fill the GPU with few pairs, not more outputs a block than that needs
  const int pairs = n * top;
  int f_per_block = F;
  const int want_blocks = 4 * tl_device_facts().compute_units;
  if (pairs < want_blocks) f_per_block = max(kPairThreads / kWave, (int)(((long long)F * pairs + want_blocks - 1) / want_blocks));
  const dim3 grid(pairs, (F + f_per_block - 1) / f_per_block);
#define TL_GLU(T, V) expert_glu_pairs_kernel<T, V><<<grid, kPairThreads, lds, stream>>>((const T*)x, (const T*)w_gu, ids, top, n_experts, (T*)mid, D, F, f_per_block)
  if (dtype == TL_F32) {
    if (D % 4 == 0) TL_GLU(float, 4);
    else TL_GLU(float, 1);
  } else if (dtype == TL_BF16) {
    if (D % 8 == 0) TL_GLU(bf16_t, 8);
    else TL_GLU(bf16_t, 1);
  } else {
    return tl_fail(TL_ERR_ARG, "expert_glu_pairs: unknown dtype %d", dtype);
  }
#undef TL_GLU
  return tl_check_launch("expert_glu_pairs");
}

TL_EXPORT int tl_expert_down_pairs(const void* mid, const void* w_d, const int32_t* ids, const float* weights, int top,
                                   int n_experts, const void* x, const void* shared, const float* sg, int sg_stride, void* out,
                                   int n, int D, int F, int dtype, hipStream_t stream) {
  TL_REQUIRE(n >= 0 && top > 0 && n_experts >= 0 && D > 0 && F > 0, "expert_down_pairs: bad sizes");
  TL_REQUIRE(shared == nullptr || sg != nullptr, "expert_down_pairs: a shared expert without its gate");
  if (n == 0) return TL_OK;
  const size_t lds = (size_t)top * F * sizeof(float);
  if (lds > (size_t)tl_device_facts().lds_bytes)
    return tl_fail(TL_ERR_UNSUPPORTED, "expert_down_pairs: %d choices of %d elements do not fit the LDS", top, F);
  int d_per_block = D;
  const int want_blocks = 4 * tl_device_facts().compute_units;
  if (n < want_blocks) d_per_block = max(kPairThreads / kWave, (int)(((long long)D * n + want_blocks - 1) / want_blocks));
  const dim3 grid(n, (D + d_per_block - 1) / d_per_block);
#define TL_DOWN(T, V)                                                                                                        \
  expert_down_pairs_kernel<T, V><<<grid, kPairThreads, lds, stream>>>((const T*)mid, (const T*)w_d, ids, weights, top, n_experts, \
                                                                      (const T*)x, (const T*)shared, sg, sg_stride, (T*)out, D, F, d_per_block)
  if (dtype == TL_F32) {
    if (F % 4 == 0) TL_DOWN(float, 4);
    else TL_DOWN(float, 1);
  } else if (dtype == TL_BF16) {
    if (F % 8 == 0) TL_DOWN(bf16_t, 8);
    else TL_DOWN(bf16_t, 1);
  } else {
    return tl_fail(TL_ERR_ARG, "expert_down_pairs: unknown dtype %d", dtype);
  }
#undef TL_DOWN
  return tl_check_launch("expert_down_pairs");
}

TL_EXPORT int tl_bias_gelu(void* x, const void* bias, int n, int width, int dtype, hipStream_t stream) {
  TL_REQUIRE(n >= 0 && width > 0, "bias_gelu: bad sizes");
  if (n == 0) return TL_OK;
  const size_t total = (size_t)n * width;
  const int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
  if (dtype == TL_F32) bias_gelu_kernel<float><<<blocks, 256, 0, stream>>>((float*)x, (const float*)bias, total, width);
  else if (dtype == TL_BF16) bias_gelu_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)x, (const bf16_t*)bias, total, width);
  else return tl_fail(TL_ERR_ARG, "bias_gelu: unknown dtype %d", dtype);
  return tl_check_launch("bias_gelu");
}

TL_EXPORT int tl_weighted_pair(const void* a, float sa, const void* b, float sb, void* out, long long total, int dtype,
                               hipStream_t stream) {
  TL_REQUIRE(total >= 0, "weighted_pair: bad size");
  if (total == 0) return TL_OK;
  const int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
  if (dtype == TL_F32) weighted_pair_kernel<float><<<blocks, 256, 0, stream>>>((const float*)a, sa, (const float*)b, sb, (float*)out, (size_t)total);
  else if (dtype == TL_BF16) weighted_pair_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)a, sa, (const bf16_t*)b, sb, (bf16_t*)out, (size_t)total);
  else return tl_fail(TL_ERR_ARG, "weighted_pair: unknown dtype %d", dtype);
  return tl_check_launch("weighted_pair");
}

TL_EXPORT int tl_post_norm_add_norm(float* stream_rows, const void* y, const float* w_post, float eps, const float* w_next,
                                    float eps_next, void* rows, int n, int hidden, int dtype, hipStream_t stream) {
  TL_REQUIRE(n >= 0 && hidden > 0, "post_norm_add_norm: bad sizes");
  TL_REQUIRE(w_next == nullptr || rows != nullptr, "post_norm_add_norm: the next norm's rows have nowhere to go");
  if (n == 0) return TL_OK;
  const size_t lds = (size_t)hidden * sizeof(float);
  if (lds + 64 > (size_t)tl_device_facts().lds_bytes)
    return tl_fail(TL_ERR_UNSUPPORTED, "post_norm_add_norm: rows of %d elements do not fit the LDS", hidden);
  if (dtype == TL_F32)
    post_norm_add_norm_kernel<float><<<n, kSandwichThreads, lds, stream>>>(stream_rows, (const float*)y, w_post, eps, w_next, eps_next,
                                                                         (float*)rows, hidden);
  else if (dtype == TL_BF16)
    post_norm_add_norm_kernel<bf16_t><<<n, kSandwichThreads, lds, stream>>>(stream_rows, (const bf16_t*)y, w_post, eps, w_next, eps_next,
                                                                          (bf16_t*)rows, hidden);
  else return tl_fail(TL_ERR_ARG, "post_norm_add_norm: unknown dtype %d", dtype);
  return tl_check_launch("post_norm_add_norm");
}
