// Layers over several residual streams (hyper-connections) with a norm that takes no statistics (dynamic tanh), and
// the joining of the two softmax maps of differential attention.
//
// The streams x_1 .. x_S are 32-bit planes [S][n][D].  A sublayer reads u = sum_s in[s] x_s, works on
// norm(u) = tanh(alpha u) * w + b, and its result y goes back as x_r <- sum_s mix[s][r] x_s + out[r] y for all r at
// once.  Every element (token, channel) is on its own, so one kernel does a sublayer's write and the next
// sublayer's read and norm in one trip over the planes; all sums run over s ascending, in 32-bit.
#include "common.h"

namespace {

constexpr int kMaxStreams = 16;  // (the weights of all pairs are one entry a thread of a block)

struct StreamWeights {
  float mix[kMaxStreams][kMaxStreams];  // [from][to]
  float out[kMaxStreams];
  float in[kMaxStreams];
};

// One thread an element (V of them side by side).  branch (BT) given: the planes are updated in place.  w given: the
// normed read goes to rows (T); with `gather` the tokens read are gather[0 .. n) (no update then).
// MAXS: the most streams this instantiation holds in registers (4, 8 or 16: few streams leave room for many waves).
template <typename T, typename BT, int V, int MAXS>
__global__ void __launch_bounds__(256)
streams_update_kernel(float* __restrict__ x, int S, long long plane, int n, int D, const BT* __restrict__ branch,
                      const float* __restrict__ mix, const float* __restrict__ out_w, const float* __restrict__ in_w,
                      const float* __restrict__ alpha, const float* __restrict__ w, const float* __restrict__ b,
                      const int32_t* __restrict__ gather, T* __restrict__ rows) {
#pragma clang fp contract(off)
  __shared__ StreamWeights sw;
  if (threadIdx.x < kMaxStreams * kMaxStreams) {
    const int s = threadIdx.x / kMaxStreams, r = threadIdx.x % kMaxStreams;
    sw.mix[s][r] = (mix && s < S && r < S) ? mix[s * S + r] : 0.f;
    if (r == 0) {
      sw.out[s] = (out_w && s < S) ? out_w[s] : 0.f;
      sw.in[s] = s < S ? (in_w ? in_w[s] : 1.f) : 0.f;
    }
  }
  __syncthreads();
  const int per_row = D / V;
  const long long total = (long long)n * per_row;
  const float a = w ? alpha[0] : 0.f;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x) {
    const int t_out = (int)(i / per_row), d0 = (int)(i % per_row) * V;
    const int t = gather ? gather[t_out] : t_out;
    float xs[MAXS][V];
#pragma unroll
    for (int s = 0; s < MAXS; ++s)
      if (s < S) {
        const float* p = x + s * plane + (long long)t * D + d0;
        if constexpr (V == 4) {
          const float4 v4 = *reinterpret_cast<const float4*>(p);
          xs[s][0] = v4.x; xs[s][1] = v4.y; xs[s][2] = v4.z; xs[s][3] = v4.w;
        } else {
#pragma unroll
          for (int e = 0; e < V; ++e) xs[s][e] = p[e];
        }
      }
    if (branch) {
      float y[V];
#pragma unroll
      for (int e = 0; e < V; ++e) y[e] = to_f32(branch[(long long)t * D + d0 + e]);
      float nx[MAXS][V];
#pragma unroll
      for (int r = 0; r < MAXS; ++r)
        if (r < S) {
#pragma unroll
          for (int e = 0; e < V; ++e) {
            float acc = 0.f;
#pragma unroll
            for (int s = 0; s < MAXS; ++s)
              if (s < S) acc += sw.mix[s][r] * xs[s][e];
            nx[r][e] = acc + sw.out[r] * y[e];
          }
        }
#pragma unroll
      for (int r = 0; r < MAXS; ++r)
        if (r < S) {
          float* p = x + r * plane + (long long)t * D + d0;
#pragma unroll
          for (int e = 0; e < V; ++e) xs[r][e] = nx[r][e];
          if constexpr (V == 4) *reinterpret_cast<float4*>(p) = float4{nx[r][0], nx[r][1], nx[r][2], nx[r][3]};
          else {
#pragma unroll
            for (int e = 0; e < V; ++e) p[e] = nx[r][e];
          }
        }
    }
    if (w) {
#pragma unroll
      for (int e = 0; e < V; ++e) {
        float u = 0.f;
#pragma unroll
        for (int s = 0; s < MAXS; ++s)
          if (s < S) u += sw.in[s] * xs[s][e];
        rows[(long long)t_out * D + d0 + e] = from_f32<T>(tanhf(a * u) * w[d0 + e] + b[d0 + e]);
      }
    }
  }
}

// The streams' first filling: every plane a copy of the rows h [n][D].
__global__ void __launch_bounds__(256)
streams_open_kernel(const float* __restrict__ h, float* __restrict__ x, int S, long long plane) {
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < plane; i += (long long)gridDim.x * blockDim.x) {
    const float v = h[i];
    for (int s = 0; s < S; ++s) x[s * plane + i] = v;
  }
}

// Differential attention: a [n][M = 2][H][dv] holds the two maps' outputs (map 0 of all heads, then map 1);
// out[t, h, :] = T(o / sqrt(mean(o^2) + eps) * gain) with o = a_0 - lambda a_1, one wave a (token, head), 32-bit.
constexpr int kJoinWaves = 4;
template <typename T>
__global__ void __launch_bounds__(kJoinWaves* kWave)
maps_join_kernel(const T* __restrict__ a, int a_stride, T* __restrict__ out, int H, int dv, float lambda, float eps, float gain) {
#pragma clang fp contract(off)
  const int t = blockIdx.x;
  const int h = blockIdx.y * kJoinWaves + threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  if (h >= H) return;
  const T* a0 = a + (size_t)t * a_stride + (size_t)h * dv;
  const T* a1 = a0 + (size_t)H * dv;
  float ss = 0.f;
  for (int d = lane; d < dv; d += kWave) {
    const float o = to_f32(a0[d]) - lambda * to_f32(a1[d]);
    ss += o * o;
  }
  ss = wave_sum(ss);
  const float inv = gain / sqrtf(ss / (float)dv + eps);
  T* op = out + ((size_t)t * H + h) * dv;
  for (int d = lane; d < dv; d += kWave) op[d] = from_f32<T>((to_f32(a0[d]) - lambda * to_f32(a1[d])) * inv);
}

int grid_for(long long total) {
  const long long blocks = (total + 255) / 256;
  return (int)(blocks < 1 ? 1 : (blocks > 16384 ? 16384 : blocks));
}

}  // namespace

// x: S planes of n_all * D floats each (plane = n_all * D).  branch [n][D] (dtype branch_dtype; null: the planes are
// only read), mix [S][S] ([from][to]) and out_w [S] go with it.  w (null: no normed read), b, alpha (one float on
// the device) and in_w [S] (null: ones) give rows [n][D] of `dtype` = tanh(alpha u) w + b, u = sum_s in_w[s] x_s;
// gather (only without branch): the n tokens that are read.
TL_EXPORT int tl_streams_update(float* x, int S, long long plane, int n, int D, const void* branch, int branch_dtype,
                                const float* mix, const float* out_w, const float* in_w, const float* alpha, const float* w,
                                const float* b, const int32_t* gather, void* rows, int dtype, hipStream_t stream) {
  TL_REQUIRE(S > 0 && n >= 0 && D > 0 && plane >= 0, "streams_update: bad sizes");
  if (S > kMaxStreams) return tl_fail(TL_ERR_UNSUPPORTED, "streams_update: %d streams, at most %d", S, kMaxStreams);
  TL_REQUIRE(branch == nullptr || (mix != nullptr && out_w != nullptr && gather == nullptr), "streams_update: a branch needs mix and out and all tokens");
  TL_REQUIRE(w == nullptr || (b != nullptr && alpha != nullptr && rows != nullptr), "streams_update: a normed read needs weight, bias, alpha and a place for the rows");
  TL_REQUIRE(branch != nullptr || w != nullptr, "streams_update: nothing to do");
  if (n == 0) return TL_OK;
  if (dtype != TL_F32 && dtype != TL_BF16) return tl_fail(TL_ERR_ARG, "streams_update: unknown dtype %d", dtype);
  if (branch && branch_dtype != TL_F32 && branch_dtype != dtype) return tl_fail(TL_ERR_ARG, "streams_update: the branch is 32-bit or of the rows' dtype");
  const bool vec = D % 4 == 0 && ((uintptr_t)x % 16) == 0 && plane % 4 == 0;
  const int blocks = grid_for((long long)n * (vec ? D / 4 : D));
#define TL_SU_M(T, BT, V, M) \
  streams_update_kernel<T, BT, V, M><<<blocks, 256, 0, stream>>>(x, S, plane, n, D, (const BT*)branch, mix, out_w, in_w, alpha, w, b, gather, (T*)rows)
#define TL_SU(T, BT, V) do { if (S <= 4) TL_SU_M(T, BT, V, 4); else if (S <= 8) TL_SU_M(T, BT, V, 8); else TL_SU_M(T, BT, V, 16); } while (0)
#define TL_SU_V(T, BT) do { if (vec) TL_SU(T, BT, 4); else TL_SU(T, BT, 1); } while (0)
  if (dtype == TL_F32) TL_SU_V(float, float);
  else if (branch && branch_dtype == TL_F32) TL_SU_V(bf16_t, float);
  else TL_SU_V(bf16_t, bf16_t);
#undef TL_SU_V
#undef TL_SU
#undef TL_SU_M
  return tl_check_launch("streams_update");
}

TL_EXPORT int tl_streams_open(const float* h, float* x, int S, long long plane, hipStream_t stream) {
  TL_REQUIRE(S > 0 && plane >= 0, "streams_open: bad sizes");
  if (plane == 0) return TL_OK;
  streams_open_kernel<<<grid_for(plane), 256, 0, stream>>>(h, x, S, plane);
  return tl_check_launch("streams_open");
}

TL_EXPORT int tl_maps_join(const void* a, int a_stride, void* out, int n, int H, int dv, float lambda, float eps, float gain,
                           int dtype, hipStream_t stream) {
  TL_REQUIRE(n >= 0 && H > 0 && dv > 0 && a_stride >= 2 * H * dv, "maps_join: bad sizes");
  TL_REQUIRE(n <= 0x7fffffff / 2, "maps_join: too many tokens");
  if (n == 0) return TL_OK;
  for (int t0 = 0; t0 < n; t0 += 65535) {
    const int nt = n - t0 < 65535 ? n - t0 : 65535;
    const dim3 grid(nt, (H + kJoinWaves - 1) / kJoinWaves);
    if (dtype == TL_F32)
      maps_join_kernel<float><<<grid, kJoinWaves * kWave, 0, stream>>>((const float*)a + (size_t)t0 * a_stride, a_stride,
                                                                        (float*)out + (size_t)t0 * H * dv, H, dv, lambda, eps, gain);
    else if (dtype == TL_BF16)
      maps_join_kernel<bf16_t><<<grid, kJoinWaves * kWave, 0, stream>>>((const bf16_t*)a + (size_t)t0 * a_stride, a_stride,
                                                                         (bf16_t*)out + (size_t)t0 * H * dv, H, dv, lambda, eps, gain);
    else return tl_fail(TL_ERR_ARG, "maps_join: unknown dtype %d", dtype);
  }
  return tl_check_launch("maps_join");
}
