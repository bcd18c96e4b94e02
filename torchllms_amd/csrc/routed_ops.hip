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
// correction may be null.  n_groups > 0: the outputs form that many equal groups of neighbours, a group's score is
// the largest s in it, and only outputs of the keep_groups best groups (of equal ones the lower) can be chosen.
// normalize: the weights are divided by their sum (+ 1e-20); then they are multiplied by route_scale.
constexpr int kRouterPerLane = 8;  // outputs a lane holds: up to 512 experts
__global__ void __launch_bounds__(256)
router_topk_kernel(const float* __restrict__ z, int z_stride, const float* __restrict__ correction, int n, int n_out, int top,
                   int32_t* __restrict__ ids, float* __restrict__ weights, int n_groups, int keep_groups, int normalize,
                   float route_scale) {
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
    c[u] = e < n_out ? (correction ? s[u] + correction[e] : s[u]) : -INFINITY;
  }
  if (n_groups > 0) {
    const int per = n_out / n_groups;
    float mine = -INFINITY;  // lane g: the score of group g (n_groups <= 64)
    for (int g = 0; g < n_groups; ++g) {
      float best = -INFINITY;
#pragma unroll
      for (int u = 0; u < kRouterPerLane; ++u) {
        const int e = lane + u * kWave;
        if (e < n_out && e / per == g) best = fmaxf(best, s[u]);
      }
      best = wave_max(best);
      if (lane == g) mine = best;
    }
    unsigned long long open = 0ull;  // the groups that stay, one bit each
    for (int k = 0; k < keep_groups; ++k) {
      float best = mine;
      int best_g = lane < n_groups ? lane : 0x7fffffff;
#pragma unroll
      for (int off = kWave / 2; off > 0; off >>= 1) {
        const float ob = __shfl_xor(best, off, kWave);
        const int og = __shfl_xor(best_g, off, kWave);
        if (ob > best || (ob == best && og < best_g)) { best = ob; best_g = og; }
      }
      open |= 1ull << best_g;
      if (lane == best_g) mine = -INFINITY;
    }
#pragma unroll
    for (int u = 0; u < kRouterPerLane; ++u) {
      const int e = lane + u * kWave;
      if (e < n_out && !((open >> (e / per)) & 1ull)) c[u] = -INFINITY;
    }
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
  if ((normalize || route_scale != 1.0f) && lane == 0) {  // (the lane that wrote them reads them back)
    float* w = weights + (size_t)t * top;
    float total = 0.f;
    for (int k = 0; k < top; ++k) total += w[k];
    for (int k = 0; k < top; ++k) w[k] = (normalize ? w[k] / (total + 1e-20f) : w[k]) * route_scale;
  }
}

// ----------------------------------------------------------------------------- experts over their gathered rows
// The (token, choice) pairs lie in the order of their experts (expert_gather below): rows[offsets[e] .. offsets[e + 1]]
// are the inputs of expert e.  A block takes some outputs of one expert and walks that expert's rows R at a time: the
// rows go to LDS, a wave takes an output at a time, reads its weights once (V elements a lane) and multiplies them
// with all R rows, so an expert's weights are read once per R rows however many tokens chose it.  Every row's sum has
// an order fixed by the row's width alone, whatever lies beside it.
constexpr int kRowsThreads = 256;
constexpr int kRowsAtOnce = 8;

// mid[r, f] = T(silu(Wg[e][f] . x_r) * (Wu[e][f] . x_r)); w_gu [E][2F][D] (an expert's gate rows, then its up rows).
template <typename T, int V>
__global__ void __launch_bounds__(kRowsThreads)
expert_glu_rows_kernel(const T* __restrict__ rows, const T* __restrict__ w_gu, const int32_t* __restrict__ offsets,
                       T* __restrict__ mid, int D, int F, int f_per_block, int at_once) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  T* x_l = reinterpret_cast<T*>(lds_raw);  // [at_once][D]
  const int e = blockIdx.x;
  const int lo = offsets[e], hi = offsets[e + 1];
  if (lo == hi) return;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int f_begin = blockIdx.y * f_per_block, f_end = min(F, f_begin + f_per_block);
  const T* wg = w_gu + (size_t)e * 2 * F * D;
  struct alignas(sizeof(T) * V) Vec { T e[V]; };
  for (int r0 = lo; r0 < hi; r0 += at_once) {
    const int nr = min(at_once, hi - r0);
    __syncthreads();
    for (int i = threadIdx.x * V; i < nr * D; i += kRowsThreads * V)
      *reinterpret_cast<Vec*>(x_l + i) = *reinterpret_cast<const Vec*>(rows + (size_t)r0 * D + i);
    __syncthreads();
    for (int f = f_begin + wave; f < f_end; f += kRowsThreads / kWave) {
      const T* g_row = wg + (size_t)f * D;
      const T* u_row = wg + (size_t)(F + f) * D;
      float ag[kRowsAtOnce], au[kRowsAtOnce];
#pragma unroll
      for (int r = 0; r < kRowsAtOnce; ++r) ag[r] = au[r] = 0.f;
#pragma unroll 4
      for (int d0 = lane * V; d0 < D; d0 += kWave * V) {  // (unrolled: the loads of four rounds are asked for together)
        const Vec gv = *reinterpret_cast<const Vec*>(g_row + d0);
        const Vec uv = *reinterpret_cast<const Vec*>(u_row + d0);
        float gf[V], uf[V];
#pragma unroll
        for (int i = 0; i < V; ++i) { gf[i] = to_f32(gv.e[i]); uf[i] = to_f32(uv.e[i]); }
#pragma unroll
        for (int r = 0; r < kRowsAtOnce; ++r) {
          if (r < nr) {
            const Vec xv = *reinterpret_cast<const Vec*>(x_l + r * D + d0);
#pragma unroll
            for (int i = 0; i < V; ++i) {
              const float xe = to_f32(xv.e[i]);
              ag[r] = fmaf(gf[i], xe, ag[r]);
              au[r] = fmaf(uf[i], xe, au[r]);
            }
          }
        }
      }
#pragma unroll
      for (int r = 0; r < kRowsAtOnce; ++r) {
        if (r < nr) {
          const float g = wave_sum(ag[r]), u = wave_sum(au[r]);
          if (lane == 0) mid[(size_t)(r0 + r) * F + f] = from_f32<T>(silu_r(g) * u);
        }
      }
    }
  }
}

// y[r, d] = Wd[e][d] . mid_r in 32-bit; w_d [E][D][F].
template <typename T, int V>
__global__ void __launch_bounds__(kRowsThreads)
expert_down_rows_kernel(const T* __restrict__ mid, const T* __restrict__ w_d, const int32_t* __restrict__ offsets,
                        float* __restrict__ y, int D, int F, int d_per_block, int at_once) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  T* m_l = reinterpret_cast<T*>(lds_raw);  // [at_once][F]
  const int e = blockIdx.x;
  const int lo = offsets[e], hi = offsets[e + 1];
  if (lo == hi) return;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int d_begin = blockIdx.y * d_per_block, d_end = min(D, d_begin + d_per_block);
  struct alignas(sizeof(T) * V) Vec { T e[V]; };
  for (int r0 = lo; r0 < hi; r0 += at_once) {
    const int nr = min(at_once, hi - r0);
    __syncthreads();
    for (int i = threadIdx.x * V; i < nr * F; i += kRowsThreads * V)
      *reinterpret_cast<Vec*>(m_l + i) = *reinterpret_cast<const Vec*>(mid + (size_t)r0 * F + i);
    __syncthreads();
    for (int d = d_begin + wave; d < d_end; d += kRowsThreads / kWave) {
      const T* row = w_d + ((size_t)e * D + d) * F;
      float acc[kRowsAtOnce];
#pragma unroll
      for (int r = 0; r < kRowsAtOnce; ++r) acc[r] = 0.f;
#pragma unroll 4
      for (int f0 = lane * V; f0 < F; f0 += kWave * V) {
        const Vec wv = *reinterpret_cast<const Vec*>(row + f0);
        float wf[V];
#pragma unroll
        for (int i = 0; i < V; ++i) wf[i] = to_f32(wv.e[i]);
#pragma unroll
        for (int r = 0; r < kRowsAtOnce; ++r) {
          if (r < nr) {
            const Vec mv = *reinterpret_cast<const Vec*>(m_l + r * F + f0);
#pragma unroll
            for (int i = 0; i < V; ++i) acc[r] = fmaf(wf[i], to_f32(mv.e[i]), acc[r]);
          }
        }
      }
#pragma unroll
      for (int r = 0; r < kRowsAtOnce; ++r) {
        if (r < nr) {
          const float v = wave_sum(acc[r]);
          if (lane == 0) y[(size_t)(r0 + r) * D + d] = v;
        }
      }
    }
  }
}

// The same two products for bfloat16 rows of up to NI * 512 elements, with the weights held in registers: a wave takes
// one output, asks for its whole weight row (gate and up row) at once, 16 bytes a lane and round, and then walks the
// expert's rows.  The weights are read once however many rows the expert has, and every load of a wave is in flight
// together.  GLU: w [E][2N][K], mid[r, n] = silu(gate) * up; else w [E][N][K], y[r, n] in 32-bit.
// Each row's sum is taken in the order of the kernels above (a lane its rounds in ascending order, then the lanes).
typedef __bf16 bf16x8_r __attribute__((ext_vector_type(8)));
template <int NI, bool GLU>
__global__ void __launch_bounds__(kRowsThreads)
expert_rows_held_kernel(const bf16_t* __restrict__ rows, const bf16_t* __restrict__ w, const int32_t* __restrict__ offsets,
                        bf16_t* __restrict__ mid, float* __restrict__ y, int K, int N) {
  const int e = blockIdx.x;
  const int lo = offsets[e], hi = offsets[e + 1];
  if (lo == hi) return;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int n = blockIdx.y * (kRowsThreads / kWave) + wave;
  const bool live = n < N;
  const bf16_t* g_row = w + ((size_t)e * (GLU ? 2 : 1) * N + (live ? n : 0)) * K;
  const bf16_t* u_row = g_row + (size_t)N * K;
  bf16x8_r gw[NI], uw[GLU ? NI : 1];
#pragma unroll
  for (int it = 0; it < NI; ++it) {
    const int d0 = (it * kWave + lane) * 8;
    const int at = d0 < K ? d0 : 0;
    gw[it] = *reinterpret_cast<const bf16x8_r*>(g_row + at);
    if (GLU) uw[it] = *reinterpret_cast<const bf16x8_r*>(u_row + at);
  }
  // the expert's rows one after the other, each straight from memory (they are few and lie in the caches): the first
  // row's pieces are asked for together with the weights, no LDS and no barrier
  for (int r = lo; r < hi; ++r) {
    const bf16_t* x_row = rows + (size_t)r * K;
    bf16x8_r xv[NI];
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      const int d0 = (it * kWave + lane) * 8;
      xv[it] = *reinterpret_cast<const bf16x8_r*>(x_row + (d0 < K ? d0 : 0));
    }
    float ag = 0.f, au = 0.f;
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      const int d0 = (it * kWave + lane) * 8;
      if (d0 < K) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float xe = (float)xv[it][i];
          ag = fmaf((float)gw[it][i], xe, ag);
          if (GLU) au = fmaf((float)uw[it][i], xe, au);
        }
      }
    }
    const float g = wave_sum(ag);
    if (GLU) {
      const float u = wave_sum(au);
      if (live && lane == 0) mid[(size_t)r * N + n] = from_f32<bf16_t>(silu_r(g) * u);
    } else {
      if (live && lane == 0) y[(size_t)r * N + n] = g;
    }
  }
}

// The same two products on the matrix cores, for experts with many rows: a wave takes 16 outputs of one expert and up
// to 32 of its rows at a time, and walks K in steps of 128: a lane asks for four neighbouring 16-byte pieces of its
// weight row (and of its up row) and of its one or two rows of x, straight from memory (the rows are small and come from
// the caches; no LDS, no barrier), and every piece is one MFMA 16x16x32 (which k a lane holds does not matter as long as
// both operands hold the same).  acc[i] = C[row 16 c + lane % 16][output n0 + 4 (lane / 16) + i].
typedef float float4_r __attribute__((ext_vector_type(4)));
constexpr int kRowsMfmaFrom = 8;  // pairs of a step above which the experts' products run on the matrix cores
template <bool GLU>
__global__ void __launch_bounds__(kRowsThreads)
expert_rows_mfma_kernel(const bf16_t* __restrict__ rows, const bf16_t* __restrict__ w, const int32_t* __restrict__ offsets,
                        bf16_t* __restrict__ mid, float* __restrict__ y, int K, int N) {
  const int e = blockIdx.x;
  const int lo = offsets[e], hi = offsets[e + 1];
  if (lo == hi) return;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int n16 = lane & 15, g4 = lane >> 4;
  const int n0 = (blockIdx.y * (kRowsThreads / kWave) + wave) * 16;
  if (n0 >= N) return;
  const int n_mine = n0 + n16 < N ? n0 + n16 : N - 1;
  const bf16_t* g_row = w + ((size_t)e * (GLU ? 2 : 1) * N + n_mine) * K;
  const bf16_t* u_row = g_row + (size_t)N * K;
  bf16x8_r zero;
#pragma unroll
  for (int i = 0; i < 8; ++i) zero[i] = (__bf16)0.0f;
  for (int r0 = lo; r0 < hi; r0 += 32) {
    const bool two = r0 + 16 < hi;
    const bf16_t* x0 = rows + (size_t)min(r0 + n16, hi - 1) * K;
    const bf16_t* x1 = rows + (size_t)min(r0 + 16 + n16, hi - 1) * K;
    float4_r ag0 = {0.f, 0.f, 0.f, 0.f}, ag1 = ag0, au0 = ag0, au1 = ag0;
    for (int k0 = 0; k0 < K; k0 += 128) {
      bf16x8_r gw[4], uw[4], xa[4], xb[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int kk = k0 + 8 * (4 * g4 + u);
        const bool in = kk < K;
        const int at = in ? kk : 0;
        gw[u] = *reinterpret_cast<const bf16x8_r*>(g_row + at);
        if (GLU) uw[u] = *reinterpret_cast<const bf16x8_r*>(u_row + at);
        xa[u] = *reinterpret_cast<const bf16x8_r*>(x0 + at);
        if (two) xb[u] = *reinterpret_cast<const bf16x8_r*>(x1 + at);
        if (!in) { xa[u] = zero; xb[u] = zero; }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        ag0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(gw[u], xa[u], ag0, 0, 0, 0);
        if (GLU) au0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uw[u], xa[u], au0, 0, 0, 0);
        if (two) {
          ag1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(gw[u], xb[u], ag1, 0, 0, 0);
          if (GLU) au1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uw[u], xb[u], au1, 0, 0, 0);
        }
      }
    }
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const int r = r0 + 16 * c + n16;
      if (r < hi && (c == 0 || two)) {
        const float4_r g = c == 0 ? ag0 : ag1, uu = c == 0 ? au0 : au1;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int n = n0 + 4 * g4 + i;
          if (n < N) {
            if (GLU) mid[(size_t)r * N + n] = from_f32<bf16_t>(silu_r(g[i]) * uu[i]);
            else y[(size_t)r * N + n] = g[i];
          }
        }
      }
    }
  }
}

template <bool GLU>
static int launch_rows_held(const void* rows, const void* w, const int32_t* offsets, int n_experts, void* mid, float* y, int K, int N,
                            int max_rows, hipStream_t stream) {
  if (max_rows > kRowsMfmaFrom) {
    // more rows than a few: the matrix cores (an expert can have that many; one that has not pays little for it)
    const dim3 mgrid(n_experts, (N + 16 * (kRowsThreads / kWave) - 1) / (16 * (kRowsThreads / kWave)));
    expert_rows_mfma_kernel<GLU><<<mgrid, kRowsThreads, 0, stream>>>((const bf16_t*)rows, (const bf16_t*)w, offsets, (bf16_t*)mid, y, K, N);
    return tl_check_launch("expert_rows_mfma");
  }
  const dim3 grid(n_experts, (N + kRowsThreads / kWave - 1) / (kRowsThreads / kWave));
  const int rounds = (K + kWave * 8 - 1) / (kWave * 8);
#define TL_HELD(NI) expert_rows_held_kernel<NI, GLU><<<grid, kRowsThreads, 0, stream>>>((const bf16_t*)rows, (const bf16_t*)w, offsets, (bf16_t*)mid, y, K, N)
  if (rounds <= 1) TL_HELD(1);
  else if (rounds <= 2) TL_HELD(2);
  else if (rounds <= 4) TL_HELD(4);
  else if (rounds <= 8) TL_HELD(8);
  else TL_HELD(16);
#undef TL_HELD
  return tl_check_launch("expert_rows_held");
}
// The widest rows the kernel with held weights takes, in elements (bfloat16, a multiple of 8).
constexpr int kHeldMaxWidth = 16 * kWave * 8;

// ----------------------------------------------------------------------------- experts, the rows of each side by side
// The (token, choice) pairs are put in the order of their experts, so that an expert's rows lie side by side and its
// weights are read once for all of them.  counts[e]: how many pairs chose output e.
__global__ void __launch_bounds__(256)
expert_count_kernel(const int32_t* __restrict__ ids, int pairs, int32_t* __restrict__ counts) {
  for (int p = blockIdx.x * blockDim.x + threadIdx.x; p < pairs; p += gridDim.x * blockDim.x) atomicAdd(&counts[ids[p]], 1);
}

// offsets[e] = counts[0] + .. + counts[e - 1] (and the total at n_out); cursor[e] = 0.  One thread: n_out is small.
__global__ void expert_offsets_kernel(const int32_t* __restrict__ counts, int n_out, int32_t* __restrict__ offsets,
                                      int32_t* __restrict__ cursor) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  int total = 0;
  for (int e = 0; e < n_out; ++e) {
    offsets[e] = total;
    cursor[e] = 0;
    total += counts[e];
  }
  offsets[n_out] = total;
}

// A block a pair: the pair takes the next free row of its expert's range (which of an expert's pairs gets which row
// depends on timing; a row's result does not depend on where it lies), remembers it in pos[p], and its token's row of
// x is copied there.
template <typename T>
__global__ void __launch_bounds__(256)
expert_gather_kernel(const T* __restrict__ x, const int32_t* __restrict__ ids, const int32_t* __restrict__ offsets,
                     int32_t* __restrict__ cursor, int top, int32_t* __restrict__ pos, T* __restrict__ rows, int D) {
  __shared__ int at_l;
  const int p = blockIdx.x;
  if (threadIdx.x == 0) {
    const int e = ids[p];
    at_l = offsets[e] + atomicAdd(&cursor[e], 1);
    pos[p] = at_l;
  }
  __syncthreads();
  const T* src = x + (size_t)(p / top) * D;
  T* dst = rows + (size_t)at_l * D;
  for (int d = threadIdx.x; d < D; d += blockDim.x) dst[d] = src[d];
}

// out[t, d] = T(sum_j w[t, j] * (e_j < n_experts ? y[pos[t, j], d] : x[t, d]) + sigmoid(sg[t]) * shared[t, d]): the
// experts' results (32-bit, or of the tensors' dtype) back in the order of the tokens, weighted and added in the order of a token's choices.
template <typename T, typename YT>
__global__ void __launch_bounds__(256)
expert_combine_kernel(const YT* __restrict__ y, const int32_t* __restrict__ pos, const int32_t* __restrict__ ids,
                      const float* __restrict__ weights, int top, int n_experts, const T* __restrict__ x,
                      const T* __restrict__ shared, const float* __restrict__ sg, int sg_stride, T* __restrict__ out, int D) {
  // a block a token and 256 columns: a token's few columns are spread over many blocks, so that a step of few tokens is
  // not one block's walk along the row
  const int t = blockIdx.x;
  const int d = blockIdx.y * blockDim.x + threadIdx.x;
  if (d >= D) return;
  const float share = shared ? (sg ? sigmoid_r(sg[(size_t)t * sg_stride]) : 1.f) : 0.f;  // (no gate: added as it is)
  float total = 0.f;
  for (int j = 0; j < top; ++j) {
    const int e = ids[(size_t)t * top + j];
    const float wj = weights[(size_t)t * top + j];
    total += wj * (e < n_experts ? to_f32(y[(size_t)pos[(size_t)t * top + j] * D + d]) : to_f32(x[(size_t)t * D + d]));
  }
  if (shared) total += share * to_f32(shared[(size_t)t * D + d]);
  out[(size_t)t * D + d] = from_f32<T>(total);
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


// The same for few rows of up to HELD * 256 elements: a launch is then as long as a row's trips to memory, so everything
// a thread needs is asked for at once (an element past the end is the row's first once more, and not used).  Operation
// for operation the kernel above: the same bits.
template <typename T, int HELD>
__global__ void __launch_bounds__(kSandwichThreads)
post_norm_add_norm_held_kernel(float* __restrict__ stream, const T* __restrict__ y, const float* __restrict__ w_post, float eps,
                               const float* __restrict__ w_next, float eps_next, T* __restrict__ rows, int hidden) {
#pragma clang fp contract(off)
  __shared__ float scratch[kSandwichThreads / kWave];
  const size_t r = blockIdx.x;
  const T* yr = y + r * hidden;
  float* sr = stream + r * hidden;
  T yraw[HELD];
  float sv[HELD], wp[HELD], wn[HELD];
#pragma unroll
  for (int c = 0; c < HELD; ++c) {
    const int i = threadIdx.x + c * kSandwichThreads;
    const int at = i < hidden ? i : 0;
    yraw[c] = yr[at];
    sv[c] = sr[at];
    wp[c] = w_post[at];
    wn[c] = w_next ? w_next[at] : 0.f;
  }
  float yv[HELD];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < HELD; ++c) {
    yv[c] = threadIdx.x + c * kSandwichThreads < hidden ? to_f32(yraw[c]) : 0.f;
    ss += yv[c] * yv[c];
  }
  ss = block_sum<kSandwichThreads / kWave>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)hidden + eps);
  float s2 = 0.f;
#pragma unroll
  for (int c = 0; c < HELD; ++c) {
    const int i = threadIdx.x + c * kSandwichThreads;
    if (i < hidden) {
      sv[c] = sv[c] + yv[c] * inv * wp[c];
      sr[i] = sv[c];
      s2 += sv[c] * sv[c];
    }
  }
  if (w_next == nullptr) return;
  s2 = block_sum<kSandwichThreads / kWave>(s2, scratch);
  const float inv2 = 1.0f / sqrtf(s2 / (float)hidden + eps_next);
#pragma unroll
  for (int c = 0; c < HELD; ++c) {
    const int i = threadIdx.x + c * kSandwichThreads;
    if (i < hidden) rows[r * hidden + i] = from_f32<T>(sv[c] * inv2 * wn[c]);
  }
}

}  // namespace

// ============================================================================= C interface
TL_EXPORT int tl_router_topk(const float* z, int z_stride, const float* correction, int n, int n_out, int top, int32_t* ids,
                             float* weights, int n_groups, int keep_groups, int normalize, float route_scale, hipStream_t stream) {
  TL_REQUIRE(n >= 0 && n_out > 0 && top > 0 && top <= n_out && z_stride >= n_out, "router_topk: bad sizes");
  TL_REQUIRE(n_groups >= 0 && (n_groups == 0 || (n_groups <= kWave && n_out % n_groups == 0 && keep_groups > 0 && keep_groups <= n_groups
                                                 && (long long)keep_groups * (n_out / n_groups) >= top)),
             "router_topk: %d groups of which %d stay do not fit %d outputs and %d choices (at most 64 groups)", n_groups, keep_groups, n_out, top);
  if (n_out > kRouterPerLane * kWave)
    return tl_fail(TL_ERR_UNSUPPORTED, "router_topk: %d router outputs, at most %d", n_out, kRouterPerLane * kWave);
  if (n == 0) return TL_OK;
  const int per_block = 256 / kWave;
  router_topk_kernel<<<(n + per_block - 1) / per_block, 256, 0, stream>>>(z, z_stride, correction, n, n_out, top, ids, weights, n_groups,
                                                                         keep_groups, normalize, route_scale);
  return tl_check_launch("router_topk");
}

// How many of an expert's rows a block holds in LDS at once: no more than any expert can have (`max_rows`, the step's
// pairs), and no more than 32 KB of them, so that several blocks share a CU and hide each other's trips to memory (an
// expert with more rows is walked in several passes; a block's few weight rows come from the caches then).
static int rows_at_once(int width, int elem, int max_rows) {
  int r = 1;
  while (r < kRowsAtOnce && r < max_rows) r *= 2;
  while (r > 1 && (size_t)r * width * elem > 32 * 1024) r /= 2;
  return r;
}
// Outputs a block takes: as few as leave eight blocks a CU among the experts that can be in use.
static int outputs_per_block(int n_experts, int n_out, int max_rows) {
  const int active = max_rows < n_experts ? (max_rows > 0 ? max_rows : 1) : n_experts;
  const int want_blocks = 8 * tl_device_facts().compute_units;
  int per = (int)(((long long)n_out * active + want_blocks - 1) / want_blocks);
  const int waves = kRowsThreads / kWave;
  per = (per + waves - 1) / waves * waves;
  return per < waves ? waves : per;
}

// rows [pairs, D] in the order of their experts, offsets [n_experts + 1 ..]; mid [pairs, F].
TL_EXPORT int tl_expert_glu_rows(const void* rows, const void* w_gu, const int32_t* offsets, int n_experts, void* mid, int D, int F,
                                 int max_rows, int dtype, hipStream_t stream) {
  TL_REQUIRE(n_experts >= 0 && D > 0 && F > 0 && max_rows >= 0, "expert_glu_rows: bad sizes");
  if (n_experts == 0 || max_rows == 0) return TL_OK;
  if (dtype != TL_F32 && dtype != TL_BF16) return tl_fail(TL_ERR_ARG, "expert_glu_rows: unknown dtype %d", dtype);
  if (dtype == TL_BF16 && D % 8 == 0 && D <= kHeldMaxWidth)
    return launch_rows_held<true>(rows, w_gu, offsets, n_experts, mid, nullptr, D, F, max_rows, stream);
  const int elem = dtype == TL_F32 ? 4 : 2;
  const int at_once = rows_at_once(D, elem, max_rows);
  const size_t lds = (size_t)at_once * D * elem;
  if (lds > (size_t)tl_device_facts().lds_bytes)
    return tl_fail(TL_ERR_UNSUPPORTED, "expert_glu_rows: rows of %d elements do not fit the LDS", D);
  const int per = outputs_per_block(n_experts, F, max_rows);
  const dim3 grid(n_experts, (F + per - 1) / per);
#define TL_GLU(T, V) expert_glu_rows_kernel<T, V><<<grid, kRowsThreads, lds, stream>>>((const T*)rows, (const T*)w_gu, offsets, (T*)mid, D, F, per, at_once)
  if (dtype == TL_F32) {
    if (D % 4 == 0) TL_GLU(float, 4);
    else TL_GLU(float, 1);
  } else {
    if (D % 8 == 0) TL_GLU(bf16_t, 8);
    else TL_GLU(bf16_t, 1);
  }
#undef TL_GLU
  return tl_check_launch("expert_glu_rows");
}

// mid [pairs, F] in the order of their experts; y [pairs, D] float.
TL_EXPORT int tl_expert_down_rows(const void* mid, const void* w_d, const int32_t* offsets, int n_experts, float* y, int D, int F,
                                  int max_rows, int dtype, hipStream_t stream) {
  TL_REQUIRE(n_experts >= 0 && D > 0 && F > 0 && max_rows >= 0, "expert_down_rows: bad sizes");
  if (n_experts == 0 || max_rows == 0) return TL_OK;
  if (dtype != TL_F32 && dtype != TL_BF16) return tl_fail(TL_ERR_ARG, "expert_down_rows: unknown dtype %d", dtype);
  if (dtype == TL_BF16 && F % 8 == 0 && F <= kHeldMaxWidth)
    return launch_rows_held<false>(mid, w_d, offsets, n_experts, nullptr, y, F, D, max_rows, stream);
  const int elem = dtype == TL_F32 ? 4 : 2;
  const int at_once = rows_at_once(F, elem, max_rows);
  const size_t lds = (size_t)at_once * F * elem;
  if (lds > (size_t)tl_device_facts().lds_bytes)
    return tl_fail(TL_ERR_UNSUPPORTED, "expert_down_rows: rows of %d elements do not fit the LDS", F);
  const int per = outputs_per_block(n_experts, D, max_rows);
  const dim3 grid(n_experts, (D + per - 1) / per);
#define TL_DOWN(T, V) expert_down_rows_kernel<T, V><<<grid, kRowsThreads, lds, stream>>>((const T*)mid, (const T*)w_d, offsets, y, D, F, per, at_once)
  if (dtype == TL_F32) {
    if (F % 4 == 0) TL_DOWN(float, 4);
    else TL_DOWN(float, 1);
  } else {
    if (F % 8 == 0) TL_DOWN(bf16_t, 8);
    else TL_DOWN(bf16_t, 1);
  }
#undef TL_DOWN
  return tl_check_launch("expert_down_rows");
}

// counts, cursor: n_out int32 each (counts zeroed by the caller); offsets: n_out + 1; pos: n * top; rows [n * top, D].
TL_EXPORT int tl_expert_gather(const void* x, const int32_t* ids, int n, int top, int n_out, int32_t* counts, int32_t* offsets,
                               int32_t* cursor, int32_t* pos, void* rows, int D, int dtype, hipStream_t stream) {
  TL_REQUIRE(n >= 0 && top > 0 && n_out > 0 && D > 0, "expert_gather: bad sizes");
  TL_REQUIRE((long long)n * top <= 0x7fffffff, "expert_gather: too many pairs a step");
  if (n == 0) return TL_OK;
  if (dtype != TL_F32 && dtype != TL_BF16) return tl_fail(TL_ERR_ARG, "expert_gather: unknown dtype %d", dtype);
  const int pairs = n * top;
  expert_count_kernel<<<(pairs + 255) / 256 < 1024 ? (pairs + 255) / 256 : 1024, 256, 0, stream>>>(ids, pairs, counts);
  expert_offsets_kernel<<<1, 64, 0, stream>>>(counts, n_out, offsets, cursor);
  if (dtype == TL_F32) expert_gather_kernel<float><<<pairs, 256, 0, stream>>>((const float*)x, ids, offsets, cursor, top, pos, (float*)rows, D);
  else expert_gather_kernel<bf16_t><<<pairs, 256, 0, stream>>>((const bf16_t*)x, ids, offsets, cursor, top, pos, (bf16_t*)rows, D);
  return tl_check_launch("expert_gather");
}

// y: the experts' results in the order of the gathered rows, 32-bit (y_f32) or of the tensors' dtype.
TL_EXPORT int tl_expert_combine(const void* y, int y_f32, const int32_t* pos, const int32_t* ids, const float* weights, int top,
                                int n_experts, const void* x, const void* shared, const float* sg, int sg_stride, void* out, int n,
                                int D, int dtype, hipStream_t stream) {
  TL_REQUIRE(n >= 0 && n <= 0x7fffffff && top > 0 && n_experts >= 0 && D > 0 && (D + 255) / 256 <= 65535, "expert_combine: bad sizes");
  if (n == 0) return TL_OK;
  const dim3 cgrid(n, (D + 255) / 256);
#define TL_COMBINE(T, YT)                                                                                                   \
  expert_combine_kernel<T, YT><<<cgrid, 256, 0, stream>>>((const YT*)y, pos, ids, weights, top, n_experts, (const T*)x, (const T*)shared, \
                                                      sg, sg_stride, (T*)out, D)
  if (dtype == TL_F32) TL_COMBINE(float, float);
  else if (dtype == TL_BF16 && y_f32) TL_COMBINE(bf16_t, float);
  else if (dtype == TL_BF16) TL_COMBINE(bf16_t, bf16_t);
  else return tl_fail(TL_ERR_ARG, "expert_combine: unknown dtype %d", dtype);
#undef TL_COMBINE
  return tl_check_launch("expert_combine");
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
  if (dtype != TL_F32 && dtype != TL_BF16) return tl_fail(TL_ERR_ARG, "post_norm_add_norm: unknown dtype %d", dtype);
  const bool few = n <= 2 * tl_device_facts().compute_units;
#define TL_SANDWICH(T)                                                                                                         \
  do {                                                                                                                         \
    if (few && hidden <= 4 * kSandwichThreads)                                                                                 \
      post_norm_add_norm_held_kernel<T, 4><<<n, kSandwichThreads, 0, stream>>>(stream_rows, (const T*)y, w_post, eps, w_next, eps_next, (T*)rows, hidden);  \
    else if (few && hidden <= 16 * kSandwichThreads)                                                                           \
      post_norm_add_norm_held_kernel<T, 16><<<n, kSandwichThreads, 0, stream>>>(stream_rows, (const T*)y, w_post, eps, w_next, eps_next, (T*)rows, hidden); \
    else                                                                                                                       \
      post_norm_add_norm_kernel<T><<<n, kSandwichThreads, lds, stream>>>(stream_rows, (const T*)y, w_post, eps, w_next, eps_next, (T*)rows, hidden);        \
  } while (0)
  if (dtype == TL_F32) TL_SANDWICH(float);
  else TL_SANDWICH(bf16_t);
#undef TL_SANDWICH
  return tl_check_launch("post_norm_add_norm");
}
