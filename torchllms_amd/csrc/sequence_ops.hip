// Kernels of layers that are not plain pre-norm attention: a scaled embedding into a 32-bit residual
// stream, layer norm fused with a scaled residual sum of two branches, gated activations other than
// silu, rotation + unit RMS norm of queries and keys with the cache write (keys and values of different
// head sizes), short causal convolutions with their history kept per request, the selective scan of a
// diagonal state-space layer and the gated delta rule.  Everything that the recurrences carry is 32-bit,
// and every sum has an order fixed by the element it belongs to, so that a result does not depend on how
// a sequence was cut into steps or on what else ran in the batch.
#include <limits.h>

#include "common.h"

namespace {

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// Sum over groups of `width` neighbouring lanes (width a power of two, at most 64): every lane of a
// group gets the group's sum, added in a fixed butterfly order.
__device__ __forceinline__ float group_sum(float v, int width) {
  for (int off = 1; off < width; off <<= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

// ----------------------------------------------------------------------------- scaled embedding
// out[t, :] = float(table[tokens[t], :]) * scale, 32-bit.
template <typename T>
__global__ void embed_scaled_kernel(const int32_t* __restrict__ tokens, const T* __restrict__ table,
                                    float* __restrict__ out, int hidden, float scale) {
  const int t = blockIdx.x;
  const T* src = table + (size_t)tokens[t] * hidden;
  float* dst = out + (size_t)t * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_f32(src[i]) * scale;
}

// ----------------------------------------------------------------------------- layer norm
// For output row r (source row s = rows ? rows[r] : r):
//   h = HT(float(x[s]) + mult * (float(d0[s]) + float(d1[s])))      (d0, d1 optional)
//   y = T((h - mean(h)) / sqrt(mean((h - mean(h))^2) + eps) * w + b)
// h is written to h_out (which may be x itself) when given.  Statistics in 32-bit, two passes over the
// row kept in LDS, fixed reduction order.
constexpr int kNormThreads = 256;

template <typename HT, typename T>
__global__ void __launch_bounds__(kNormThreads)
layernorm_kernel(const HT* x, const T* __restrict__ d0, const T* __restrict__ d1, float mult,
                 const int32_t* __restrict__ rows, const float* __restrict__ w, const float* __restrict__ b,
                 HT* h_out, T* __restrict__ y, int hidden, float eps) {
  __shared__ float scratch[kNormThreads / kWave];
  extern __shared__ float row_cache[];
  const int r = blockIdx.x;
  const size_t s = rows ? (size_t)rows[r] : (size_t)r;
  const HT* xr = x + s * hidden;
  const T* d0r = d0 ? d0 + s * hidden : nullptr;
  const T* d1r = d1 ? d1 + s * hidden : nullptr;
  HT* hr = h_out ? h_out + (size_t)r * hidden : nullptr;
  float sum = 0.f;
  for (int i = threadIdx.x; i < hidden; i += kNormThreads) {
    float v = to_f32(xr[i]);
    if (d0r) {
      float add = to_f32(d0r[i]);
      if (d1r) add += to_f32(d1r[i]);
      v = to_f32(from_f32<HT>(fmaf(mult, add, v)));
    }
    row_cache[i] = v;
    if (hr) hr[i] = from_f32<HT>(v);
    sum += v;
  }
  const float mean = block_sum<kNormThreads / kWave>(sum, scratch) / (float)hidden;
  float sq = 0.f;
  for (int i = threadIdx.x; i < hidden; i += kNormThreads) {
    const float dv = row_cache[i] - mean;
    sq += dv * dv;
  }
  const float var = block_sum<kNormThreads / kWave>(sq, scratch) / (float)hidden;
  const float inv = 1.0f / sqrtf(var + eps);
  T* yr = y + (size_t)r * hidden;
  for (int i = threadIdx.x; i < hidden; i += kNormThreads)
    yr[i] = from_f32<T>(fmaf((row_cache[i] - mean) * inv, w[i], b[i]));
}

template <typename HT, typename T>
int layernorm_launch(const void* x, const void* d0, const void* d1, float mult, const int32_t* rows, const float* w,
                     const float* b, void* h_out, void* y, int n, int hidden, float eps, hipStream_t stream) {
  const size_t lds = (size_t)hidden * sizeof(float);
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)layernorm_kernel<HT, T>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return tl_fail(TL_ERR_HIP, "layernorm: %s", hipGetErrorString(e));
  }
  layernorm_kernel<HT, T><<<n, kNormThreads, lds, stream>>>((const HT*)x, (const T*)d0, (const T*)d1, mult, rows, w, b,
                                                            (HT*)h_out, (T*)y, hidden, eps);
  return tl_check_launch("layernorm");
}

// ----------------------------------------------------------------------------- gated activation
// gate_up: [n, 2F] = gate | up.  out[n, F] = T(act(float(gate)) * float(up)); act 1: gelu in its tanh form.
// A thread takes V consecutive columns of one row (V elements = 16 bytes when the row allows it).
template <typename T, int V>
__global__ void gelu_mul_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int n, int inter) {
  const int c0 = (blockIdx.x * blockDim.x + threadIdx.x) * V;
  if (c0 >= inter) return;
  struct alignas(sizeof(T) * V) Vec { T e[V]; };
  for (int r = blockIdx.y; r < n; r += gridDim.y) {
    const T* gp = gate_up + (size_t)r * 2 * inter + c0;
    const Vec g = *reinterpret_cast<const Vec*>(gp);
    const Vec u = *reinterpret_cast<const Vec*>(gp + inter);
    Vec o;
#pragma unroll
    for (int i = 0; i < V; ++i) o.e[i] = from_f32<T>(gelu_tanh_f(to_f32(g.e[i])) * to_f32(u.e[i]));
    *reinterpret_cast<Vec*>(out + (size_t)r * inter + c0) = o;
  }
}

template <typename T>
int gelu_mul_launch(const T* gate_up, T* out, int n, int inter, hipStream_t stream) {
  constexpr int kVec = 16 / sizeof(T);
  const bool wide = inter % kVec == 0 && ((uintptr_t)gate_up % 16) == 0 && ((uintptr_t)out % 16) == 0;
  const int per_block = 256 * (wide ? kVec : 1);
  const dim3 grid((inter + per_block - 1) / per_block, n < 65535 ? n : 65535);
  if (wide) gelu_mul_kernel<T, kVec><<<grid, 256, 0, stream>>>(gate_up, out, n, inter);
  else gelu_mul_kernel<T, 1><<<grid, 256, 0, stream>>>(gate_up, out, n, inter);
  return tl_check_launch("gelu_mul");
}

// ----------------------------------------------------------------------------- rotation, unit norm, cache write
// qkv: [n_tokens, row] with row = (Hq + Hkv) * dk + Hkv * dv: query heads | key heads | value heads.
// Query and key heads are rotated (pairing 0: channels (2i, 2i+1); 1: (i, i + rot/2); channels from
// rot on pass), then, with norm_eps > 0, divided by sqrt(mean(x^2) + norm_eps) over the head; all in
// 32-bit with one rounding at the end.  Queries go back in place; keys go to their page
// [page][Hkv][P][dk] at slot_mapping[t] and values to [page][Hkv][P][dv] (without pages keys go back in
// place too).  One wave a head.
constexpr int kHeadWaves = 4;
constexpr int kHeadChan = 4;  // channels a lane holds: heads of up to 256

constexpr int kHeadsPerWave = 2;  // heads a wave takes, all their loads asked for before anything waits for one

template <typename T>
__global__ void __launch_bounds__(kHeadWaves* kWave)
rope_norm_kv_write_kernel(T* qkv, int row, int n_q, int n_kv, int dk, int dv, const float2* __restrict__ cos_sin,
                          int rot, int pairing, float norm_eps, T* __restrict__ k_pages, T* __restrict__ v_pages,
                          const int32_t* __restrict__ slot_mapping, int page_size) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int unit0 = (blockIdx.y * kHeadWaves + wave) * kHeadsPerWave;
  const int n_units = n_q + 2 * n_kv;
  if (unit0 >= n_units) return;
  T* base = qkv + (size_t)t * row;
  const int slot = slot_mapping ? slot_mapping[t] : -1;
  const bool store = k_pages != nullptr && slot >= 0;
  const size_t page = store ? slot / page_size : 0;
  const int off = store ? slot % page_size : 0;
  const int rh = rot / 2;
  // a unit is a query head, a key head or a value head (copied); units past the last do nothing
  float val[kHeadsPerWave][kHeadChan];
  float ss[kHeadsPerWave];
#pragma unroll
  for (int u = 0; u < kHeadsPerWave; ++u) {
    const int unit = unit0 + u;
    ss[u] = 0.f;
    const bool rotated = unit < n_q + n_kv;
    const bool value = !rotated && unit < n_units;
    const T* head = rotated ? base + (size_t)unit * dk : base + (size_t)(n_q + n_kv) * dk + (size_t)(value ? unit - n_q - n_kv : 0) * dv;
    const int width = rotated ? dk : dv;
#pragma unroll
    for (int c = 0; c < kHeadChan; ++c) {
      const int d = lane + c * kWave;
      val[u][c] = 0.f;
      if ((rotated || value) && d < width) {
        const float a = to_f32(head[d]);
        float v = a;
        if (rotated && d < rot) {
          int i, partner;
          bool first;
          if (pairing == 0) {
            i = d / 2; first = (d % 2) == 0; partner = first ? d + 1 : d - 1;
          } else {
            first = d < rh; i = first ? d : d - rh; partner = first ? d + rh : d - rh;
          }
          const float o = to_f32(head[partner]);
          const float2 cs = cos_sin[(size_t)t * rh + i];
          v = first ? a * cs.x - o * cs.y : a * cs.x + o * cs.y;
        }
        val[u][c] = v;
        ss[u] += v * v;
      }
    }
  }
#pragma unroll
  for (int u = 0; u < kHeadsPerWave; ++u) ss[u] = wave_sum(ss[u]);  // (every load lies before these exchanges, every store behind)
#pragma unroll
  for (int u = 0; u < kHeadsPerWave; ++u) {
    const int unit = unit0 + u;
    if (unit >= n_units) continue;
    if (unit >= n_q + n_kv) {  // a value head: copied into its page
      if (!store || v_pages == nullptr) continue;
      T* dst = v_pages + ((page * n_kv + (unit - n_q - n_kv)) * page_size + off) * dv;
#pragma unroll
      for (int c = 0; c < kHeadChan; ++c) {
        const int d = lane + c * kWave;
        if (d < dv) dst[d] = from_f32<T>(val[u][c]);
      }
      continue;
    }
    const float inv = norm_eps > 0.f ? 1.0f / sqrtf(ss[u] / (float)dk + norm_eps) : 1.0f;
    const bool is_q = unit < n_q;
    if (!is_q && k_pages != nullptr && !store) continue;  // a token without a slot keeps nothing
    T* dst = base + (size_t)unit * dk;
    if (!is_q && store) dst = k_pages + ((page * n_kv + (unit - n_q)) * page_size + off) * dk;
#pragma unroll
    for (int c = 0; c < kHeadChan; ++c) {
      const int d = lane + c * kWave;
      if (d < dk) dst[d] = from_f32<T>(val[u][c] * inv);
    }
  }
}

// ----------------------------------------------------------------------------- short causal convolution
// x: element (t, c) at x + t * x_stride + c, c < C (a slice of a projection's output).  Tokens of a
// request are consecutive (qo_indptr); the request's K - 1 inputs before them are its history, 32-bit,
// hist[k][c] at state + slot * state_stride + k * C + c, oldest first, zero for a new request.
//   out[t, c] = act(bias[c] + sum_j taps[j][c] * in(t - (K - 1 - j))),  j ascending, 32-bit (taps: [K][C])
// act 0: none, 1: silu.  The history is brought up to date by a second kernel, after every token has read it.
template <typename T, int V>
__global__ void __launch_bounds__(256)
causal_conv_kernel(const T* __restrict__ x, int x_stride, const float* __restrict__ taps, const float* __restrict__ bias,
                   const float* __restrict__ state, long long state_stride, const int32_t* __restrict__ token_seq,
                   const int32_t* __restrict__ qo_indptr, const int32_t* __restrict__ slot_ids, T* __restrict__ out,
                   int out_stride, int C, int K, int act, int t0) {
  // a thread takes V neighbouring channels of one token (V elements = 16 bytes where the rows allow it)
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * V;
  if (c >= C) return;
  const int t = t0 + blockIdx.y;
  const int row = token_seq[t];
  const int start = qo_indptr[row];
  const int i = t - start;
  const float* hist = state + (long long)slot_ids[row] * state_stride;
  struct alignas(sizeof(T) * V) Vec { T e[V]; };
  float acc[V];
#pragma unroll
  for (int e = 0; e < V; ++e) acc[e] = bias ? bias[c + e] : 0.f;
  for (int j = 0; j < K; ++j) {
    const int src = i - (K - 1 - j);
    float v[V];
    if (src >= 0) {
      const Vec in = *reinterpret_cast<const Vec*>(x + (size_t)(start + src) * x_stride + c);
#pragma unroll
      for (int e = 0; e < V; ++e) v[e] = to_f32(in.e[e]);
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) v[e] = hist[(size_t)(K - 1 + src) * C + c + e];
    }
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = fmaf(taps[(size_t)j * C + c + e], v[e], acc[e]);
  }
  Vec o;
#pragma unroll
  for (int e = 0; e < V; ++e) o.e[e] = from_f32<T>(act == 1 ? silu_f(acc[e]) : acc[e]);
  *reinterpret_cast<Vec*>(out + (size_t)t * out_stride + c) = o;
}

// A step in which every request brings one token (decode): convolution and new history in one kernel.  A thread
// owns V channels of one request: it reads their history, adds the token, and writes the history back one place on.
template <typename T, int V>
__global__ void __launch_bounds__(256)
conv_step_kernel(const T* __restrict__ x, int x_stride, const float* __restrict__ taps, const float* __restrict__ bias,
                 float* __restrict__ state, long long state_stride, const int32_t* __restrict__ qo_indptr,
                 const int32_t* __restrict__ slot_ids, T* __restrict__ out, int out_stride, int C, int K, int act) {
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * V;
  if (c >= C) return;
  const int row = blockIdx.y;
  const int t = qo_indptr[row];
  float* hist = state + (long long)slot_ids[row] * state_stride;
  struct alignas(sizeof(T) * V) Vec { T e[V]; };
  const Vec in = *reinterpret_cast<const Vec*>(x + (size_t)t * x_stride + c);
  float acc[V];
#pragma unroll
  for (int e = 0; e < V; ++e) acc[e] = bias ? bias[c + e] : 0.f;
  // eight entries of the history are asked for at once (a store between two loads of the same array makes the
  // second wait for the first); entry j moves to place j - 1, which has been read before
  constexpr int kAhead = 8;
  for (int j0 = 0; j0 < K - 1; j0 += kAhead) {
    float hv[kAhead][V];
#pragma unroll
    for (int u = 0; u < kAhead; ++u)
#pragma unroll
      for (int e = 0; e < V; ++e) hv[u][e] = j0 + u < K - 1 ? hist[(size_t)(j0 + u) * C + c + e] : 0.f;
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      const int j = j0 + u;
      if (j < K - 1) {
#pragma unroll
        for (int e = 0; e < V; ++e) {
          acc[e] = fmaf(taps[(size_t)j * C + c + e], hv[u][e], acc[e]);
          if (j > 0) hist[(size_t)(j - 1) * C + c + e] = hv[u][e];
        }
      }
    }
  }
  Vec o;
#pragma unroll
  for (int e = 0; e < V; ++e) {
    const float v = to_f32(in.e[e]);
    acc[e] = fmaf(taps[(size_t)(K - 1) * C + c + e], v, acc[e]);
    if (K > 1) hist[(size_t)(K - 2) * C + c + e] = v;
    o.e[e] = from_f32<T>(act == 1 ? silu_f(acc[e]) : acc[e]);
  }
  *reinterpret_cast<Vec*>(out + (size_t)t * out_stride + c) = o;
}

// New history of every request of the step: the last K - 1 entries of (old history, the step's inputs).
template <typename T>
__global__ void __launch_bounds__(256)
conv_history_kernel(const T* __restrict__ x, int x_stride, float* __restrict__ state, long long state_stride,
                    const int32_t* __restrict__ qo_indptr, const int32_t* __restrict__ slot_ids, int C, int K) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int row = blockIdx.y;
  const int start = qo_indptr[row];
  const int n = qo_indptr[row + 1] - start;
  float* hist = state + (long long)slot_ids[row] * state_stride;
  // entry k of the new history is entry n + k of the old one while that exists (n >= 1: read before
  // anything at or above it is written), else the step's input n - (K - 1) + k
  for (int k = 0; k < K - 1; ++k) {
    const int idx = n - (K - 1) + k;
    const float v = idx >= 0 ? to_f32(x[(size_t)(start + idx) * x_stride + c]) : hist[(size_t)(K - 1 + idx) * C + c];
    hist[(size_t)k * C + c] = v;
  }
}

// ----------------------------------------------------------------------------- selective scan
// Per request, channel c and state n (32-bit, carried in state[slot][c][n]):
//   dt = softplus(dt_pre[t, c] + dt_bias[c]);  S[n] = exp(dt * A[c][n]) * S[n] + dt * x[t, c] * B[t, n]
//   y  = sum_n S[n] * C[t, n] + D[c] * x[t, c]  (n ascending within a lane, lanes in butterfly order)
//   out[t, c] = T(y * silu(z[t, c]))
// bc: [n_tokens, bc_stride] with B at column b_off and C at c_off.  LPC neighbouring lanes share a channel,
// each holding NB states.  A block takes kScanThreads / LPC channels of one request and walks its tokens
// in order; the rows of B and C reach LDS a tile of tokens at a time.
constexpr int kScanThreads = 128;
constexpr int kScanTile = 8;

// MODE 0: a block walks all tokens of its request, from the request's state to the request's state.
// For long prompts the walk is cut into segments of tokens that run side by side (``segs``: first and
// last token of every segment): MODE 1 walks a segment from a zero state, emits nothing and leaves the
// state it ends with and the sum of its step sizes (the decay of state n over the segment is
// exp(A[c][n] * that sum)); a carry kernel then goes over each request's segments in order and puts the
// state that enters each in its place; MODE 2 walks the segment again from there and emits.
template <typename T, typename DT, int NB, int MODE>
__global__ void __launch_bounds__(kScanThreads)
selective_scan_kernel(const T* __restrict__ x, const DT* __restrict__ dt_pre, const T* __restrict__ bc, int bc_stride,
                      int b_off, int c_off, const T* __restrict__ z, int z_stride, const float* __restrict__ dt_bias,
                      const float* __restrict__ A, const float* __restrict__ D, float* __restrict__ state,
                      long long state_stride, const int32_t* __restrict__ qo_indptr, const int32_t* __restrict__ slot_ids,
                      T* __restrict__ out, int inner, int N, int lpc, const int32_t* __restrict__ segs,
                      float* __restrict__ seg_dt) {
  extern __shared__ __attribute__((aligned(16))) float bc_lds[];  // [kScanTile][2 * N]
  constexpr bool kFastExp = sizeof(T) == 2;
  const bool vec4 = N % 4 == 0;
  const int row = blockIdx.y;  // (MODE 1, 2: the segment)
  const int start = MODE == 0 ? qo_indptr[row] : segs[2 * row], end = MODE == 0 ? qo_indptr[row + 1] : segs[2 * row + 1];
  const int per_block = kScanThreads / lpc;
  const int c_raw = blockIdx.x * per_block + threadIdx.x / lpc;
  const int part = threadIdx.x % lpc;
  const bool live = c_raw < inner;
  const int c = live ? c_raw : inner - 1;
  const int n0 = part * NB;
  float* st = state + (MODE == 0 ? (long long)slot_ids[row] : (long long)row) * state_stride + (size_t)c * N;
  float s[NB], a[NB];
#pragma unroll
  for (int n = 0; n < NB; ++n) {
    const bool in = n0 + n < N;
    s[n] = in && MODE != 1 ? st[n0 + n] : 0.f;
    a[n] = in ? A[(size_t)c * N + n0 + n] : 0.f;
    // with 16-bit activations the decay is one hardware exponential of a prescaled exponent (the kernel's time
    // is its exponentials); with 32-bit ones the library's exp of the product as it is written
    if (kFastExp) a[n] *= 1.4426950408889634f;
  }
  const float bias = dt_bias[c], dd = D[c];
  float dt_sum = 0.f;
  for (int t0 = start; t0 < end; t0 += kScanTile) {
    const int nt = min(kScanTile, end - t0);
    // the tile's own inputs are asked for at once, before anything waits for one of them
    T x_t[kScanTile], z_t[kScanTile];
    DT dt_t[kScanTile];
#pragma unroll
    for (int tt = 0; tt < kScanTile; ++tt) {
      const size_t t = (size_t)(t0 + (tt < nt ? tt : 0));
      x_t[tt] = x[t * inner + c];
      dt_t[tt] = dt_pre[t * inner + c];
      if (MODE != 1) z_t[tt] = z[t * z_stride + c];
    }
    __syncthreads();  // everybody has finished with the tile before
    for (int tt = 0; tt < nt; ++tt) {
      const T* src = bc + (size_t)(t0 + tt) * bc_stride;
      for (int e = threadIdx.x; e < 2 * N; e += kScanThreads)
        bc_lds[tt * 2 * N + e] = to_f32(e < N ? src[b_off + e] : src[c_off + e - N]);
    }
    __syncthreads();
#pragma unroll
    for (int tt = 0; tt < kScanTile; ++tt) {
      if (tt >= nt) break;
      const size_t t = (size_t)(t0 + tt);
      const float xv = to_f32(x_t[tt]);
      const float dt = softplus_f(to_f32(dt_t[tt]) + bias);
      const float zv = MODE == 1 ? 0.f : to_f32(z_t[tt]);
      const float dx = dt * xv;
      dt_sum += dt;
      const float* Bt = bc_lds + tt * 2 * N + n0;
      const float* Ct = Bt + N;
      float y = 0.f;
      if (vec4) {  // N is a multiple of 4: four states' B and C a read (the same for every lane of a channel group)
#pragma unroll
        for (int n = 0; n < NB; n += 4) {
          if (n0 + n < N) {
            const float4 b4 = *reinterpret_cast<const float4*>(Bt + n), c4 = *reinterpret_cast<const float4*>(Ct + n);
            const float bb[4] = {b4.x, b4.y, b4.z, b4.w}, cc[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              s[n + e] = fmaf(kFastExp ? __builtin_amdgcn_exp2f(dt * a[n + e]) : expf(dt * a[n + e]), s[n + e], dx * bb[e]);
              y = fmaf(s[n + e], cc[e], y);
            }
          }
        }
      } else {
#pragma unroll
        for (int n = 0; n < NB; ++n) {
          if (n0 + n < N) {
            s[n] = fmaf(kFastExp ? __builtin_amdgcn_exp2f(dt * a[n]) : expf(dt * a[n]), s[n], dx * Bt[n]);
            y = fmaf(s[n], Ct[n], y);
          }
        }
      }
      if (MODE != 1) {
        y = group_sum(y, lpc);
        y = fmaf(dd, xv, y);
        if (live && part == 0) out[t * inner + c] = from_f32<T>(y * silu_f(zv));
      }
    }
  }
  if (live && MODE != 2) {
#pragma unroll
    for (int n = 0; n < NB; ++n)
      if (n0 + n < N) st[n0 + n] = s[n];
    if (MODE == 1 && part == 0) seg_dt[(size_t)row * inner + c] = dt_sum;
  }
}

// The carry between the segments of a request: element (c, n) of the state goes through the request's
// segments in order; ws[seg] holds the state a segment ends with when it starts from zero and receives
// the state that enters it.  The request's state row takes what the last segment leaves.
__global__ void __launch_bounds__(256)
scan_carry_kernel(float* __restrict__ ws, const float* __restrict__ seg_dt, const float* __restrict__ A,
                  float* __restrict__ state, long long state_stride, const int32_t* __restrict__ row_seg,
                  const int32_t* __restrict__ slot_ids, int inner, int N) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t per = (size_t)inner * N;
  if (idx >= per) return;
  const int row = blockIdx.y;
  const int c = (int)(idx / N);
  float* st = state + (long long)slot_ids[row] * state_stride + idx;
  float s = *st;
  const float a = A[idx];
  for (int seg = row_seg[row]; seg < row_seg[row + 1]; ++seg) {
    float* w = ws + (size_t)seg * per + idx;
    const float local = *w;
    *w = s;
    s = fmaf(expf(a * seg_dt[(size_t)seg * inner + c]), s, local);
  }
  *st = s;
}

// ----------------------------------------------------------------------------- gated delta rule
// Per request and head h (key/query head g = h / (H / G)), state S [dk][dv] in 32-bit, kept transposed in
// state[slot][h][j][i] (column j of S is contiguous).  For every token, in order:
//   k^ = k / sqrt(sum k^2 + 1e-6);  q^ = q / sqrt(sum q^2 + 1e-6) * dk^-1/2
//   beta = sigmoid(b);  decay = exp(-exp(A_log[h]) * softplus(a + dt_bias[h]))
//   S <- decay * S;  u = beta * (v - S^T k^);  S <- S + k^ u^T;  o = S^T q^
// and, in a second kernel, out[t, h, :] = T(o / sqrt(mean(o^2) + eps) * norm_w * silu(gate[t, h, :])).
// qkv: the convolved and activated q | k | v channels, [n_tokens, qkv_stride]; proj: the layer's input
// projection, of which gate (H * dv columns from gate_off), b and a (H columns each) are read.
//
// The columns of S do not depend on each other, so a block takes kDeltaCols columns of one (request,
// head): a prompt of one request fills the GPU with heads * dv / kDeltaCols blocks.  lpc neighbouring
// lanes share a column, each holding 16 rows of it in registers.  The tokens come in tiles of kDeltaTile:
// the raw keys, queries and values of the next tile travel from memory into registers while the current
// tile is worked on; in LDS the keys and queries are made unit vectors once per tile; then the tile's
// tokens follow each other without a barrier (sums over a column's lanes by lane-to-lane moves).
constexpr int kDeltaTile = 16;
__device__ __forceinline__ float log_sigmoid_f(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }
// kDeltaCols, a template argument: 16 or 32 columns a block.  The time of a token is the block's multiply-adds, so
// a launch of few blocks (a prompt of one request: heads * dv / 16 blocks, 256 for 32 heads of 128 columns) takes 16;
// a launch that fills the GPU anyway (decode steps of many requests) takes 32 and has half the blocks to start.

// Sum over groups of `width` neighbouring lanes (1, 2, 4, 8 or 16) by data-parallel moves inside a row
// of 16 lanes: every lane of a group gets the same bits.
__device__ __forceinline__ float dpp_xor1(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, false));
}
__device__ __forceinline__ float dpp_xor2(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, false));
}
__device__ __forceinline__ float dpp_half_mirror(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, false));
}
__device__ __forceinline__ float dpp_mirror(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, false));
}
__device__ __forceinline__ float row_group_sum(float v, int width) {
  if (width >= 2) v += dpp_xor1(v);
  if (width >= 4) v += dpp_xor2(v);
  if (width >= 8) v += dpp_half_mirror(v);
  if (width >= 16) v += dpp_mirror(v);
  return v;
}

// kDeltaRows: rows of a column that a lane holds (8 for keys of up to 128 channels, else 16; a column's lanes lie
// in one row of 16 lanes).
// CH: a decay of its own for every key channel (row of S) of a head: the pre-activations come as 32-bit rows
// a_ch [n_tokens, a_stride] with H * dk columns, dt_bias has H * dk entries, and a token's decays lie in LDS beside
// its key; the column a_off of proj is not read.
// RULE 0: the delta rule with a decay per head; 1: with a decay per key channel (CH); 2: no delta and no unit
// vectors, S <- diag(decay) S + k v^T with q times dk^-1/2 and decay = sigmoid(a_ch + dt_bias)^plain_rate per key
// channel (gated linear attention; proj and A_log are not read).
template <typename T, bool VEC, int kDeltaRows, int kDeltaCols, int RULE>
// (Held to 128 registers, so that more of a decode step's many short blocks share a CU, the compiler spills 400 to
// 1,000 bytes a lane: what the tile's pipeline carries is more than that.  It is left its 233 to 256.)
__global__ void __launch_bounds__(512)
gated_delta_kernel(const T* __restrict__ qkv, int qkv_stride, const T* __restrict__ proj, int proj_stride, int b_off,
                   int a_off, const float* __restrict__ A_log, const float* __restrict__ dt_bias,
                   float* __restrict__ state, long long state_stride, const int32_t* __restrict__ qo_indptr,
                   const int32_t* __restrict__ slot_ids, float* __restrict__ o_raw, int H, int G, int dk, int dv, int lpc,
                   int col_groups, const float* __restrict__ a_ch, int a_stride, float plain_rate) {
  constexpr bool CH = RULE >= 1, PLAIN = RULE == 2;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  // per token of the tile: k [dk], q [dk] (raw, then unit), v [kDeltaCols], o [kDeltaCols]; then six scalars
  const int dkp = dk + dk / 16 * 4;  // a token's keys in LDS: four floats of padding after every sixteen, so that
                                     // the lanes of a column, sixteen rows apart, read different banks
  float* k_l = lds;
  float* q_l = k_l + kDeltaTile * dkp;
  float* v_l = q_l + kDeltaTile * dkp;
  float* o_l = v_l + kDeltaTile * kDeltaCols;
  float* sc_l = o_l + kDeltaTile * kDeltaCols;  // [kDeltaTile][6]: beta, decay, 1/|k|, scale/|q|, k^ . q^
  float* g_l = sc_l + kDeltaTile * 6;           // (CH) [kDeltaTile][dkp]: a token's decays, padded as its key
  const int row = blockIdx.y;
  const int h = blockIdx.x / col_groups, cg = blockIdx.x % col_groups;
  const int g = h / (H / G);
  const int start = qo_indptr[row], end = qo_indptr[row + 1];
  const int n_threads = blockDim.x;
  const int j_loc = threadIdx.x / lpc, part = threadIdx.x % lpc;
  const int j_raw = cg * kDeltaCols + j_loc;
  const bool live = j_loc < kDeltaCols && j_raw < dv;
  const int j = j_raw < dv ? j_raw : dv - 1;
  const int i0 = part * kDeltaRows;
  float* st = state + (long long)slot_ids[row] * state_stride + ((size_t)h * dv + j) * dk;
  float S[kDeltaRows];
  if (VEC) {
#pragma unroll
    for (int r = 0; r < kDeltaRows; r += 4) {
      const float4 s4 = i0 + r < dk ? *reinterpret_cast<const float4*>(st + i0 + r) : float4{0.f, 0.f, 0.f, 0.f};
      S[r] = s4.x; S[r + 1] = s4.y; S[r + 2] = s4.z; S[r + 3] = s4.w;
    }
  } else {
#pragma unroll
    for (int r = 0; r < kDeltaRows; ++r) S[r] = i0 + r < dk ? st[i0 + r] : 0.f;
  }
  const float neg_rate = PLAIN ? 0.f : -expf(A_log[h]), bias = CH ? 0.f : dt_bias[h];
  const float q_scale = 1.0f / sqrtf((float)dk);
  const int q_col = g * dk, k_col = G * dk + g * dk, v_col = 2 * G * dk + h * dv + cg * kDeltaCols;
  const int v_cols = min(kDeltaCols, dv - cg * kDeltaCols);

  // what a thread fetches of a tile: element e of the tile's keys and queries (e = tt * 2 dk + d, d < dk a
  // key's channel, else a query's) for e = tid, tid + threads, ...; likewise of the values
  // (element e = tt * 2 dk + d of a tile without a division: from one pass to the next a thread's element moves on
  // by the block's threads, which are less than two tokens' worth)
  const int two_dk = 2 * dk;
  const int tt_first = threadIdx.x / two_dk, d_first = threadIdx.x % two_dk;
  const int tt_step = n_threads / two_dk, d_step = n_threads % two_dk;
  constexpr int kPreKQ = kDeltaRows == 16 && kDeltaCols == 16 ? 32 : 16, kPreV = 8;  // (a tile's elements over the block's threads, at most)
  T pre_kq[kPreKQ], pre_v[kPreV], pre_b = from_f32<T>(0.f), pre_a = from_f32<T>(0.f);
  auto fetch = [&](int t0) {
    const int nt = min(kDeltaTile, end - t0);
    if (!PLAIN && threadIdx.x < nt) {
      const T* pr = proj + (size_t)(t0 + threadIdx.x) * proj_stride;
      pre_b = pr[b_off + h];
      if (!CH) pre_a = pr[a_off + h];
    }
    int tt = tt_first, d = d_first;
#pragma unroll
    for (int u = 0; u < kPreKQ; ++u) {
      if (tt < nt) pre_kq[u] = qkv[(size_t)(t0 + tt) * qkv_stride + (d < dk ? k_col + d : q_col + d - dk)];
      tt += tt_step;
      d += d_step;
      if (d >= two_dk) { d -= two_dk; ++tt; }
    }
#pragma unroll
    for (int u = 0; u < kPreV; ++u) {
      const int e = threadIdx.x + u * n_threads;
      const int tt = e / kDeltaCols, d = e % kDeltaCols;
      if (tt < nt && d < v_cols) pre_v[u] = qkv[(size_t)(t0 + tt) * qkv_stride + v_col + d];
    }
  };
  if (start < end) fetch(start);
  for (int t0 = start; t0 < end; t0 += kDeltaTile) {
    const int nt = min(kDeltaTile, end - t0);
    __syncthreads();  // the tile before has been read to its end
    {
      int tt = tt_first, d = d_first;
#pragma unroll
      for (int u = 0; u < kPreKQ; ++u) {
        const int dd = d < dk ? d : d - dk;
        if (tt < nt) (d < dk ? k_l : q_l)[tt * dkp + dd + dd / 16 * 4] = to_f32(pre_kq[u]);
        tt += tt_step;
        d += d_step;
        if (d >= two_dk) { d -= two_dk; ++tt; }
      }
    }
#pragma unroll
    for (int u = 0; u < kPreV; ++u) {
      const int e = threadIdx.x + u * n_threads;
      const int tt = e / kDeltaCols, d = e % kDeltaCols;
      if (tt < nt && d < v_cols) v_l[tt * kDeltaCols + d] = to_f32(pre_v[u]);
    }
    if (threadIdx.x < nt) {
      sc_l[6 * threadIdx.x] = PLAIN ? 1.f : sigmoid_f(to_f32(pre_b));
      if (!CH) sc_l[6 * threadIdx.x + 1] = expf(neg_rate * softplus_f(to_f32(pre_a) + bias));
    }
    if (CH) {
      for (int e = threadIdx.x; e < nt * dk; e += n_threads) {
        const int tt = e / dk, d = e % dk;
        const float pre = a_ch[(size_t)(t0 + tt) * a_stride + h * dk + d] + dt_bias[h * dk + d];
        g_l[tt * dkp + d + d / 16 * 4] = PLAIN ? expf(plain_rate * log_sigmoid_f(pre)) : expf(neg_rate * softplus_f(pre));
      }
    }
    if (t0 + kDeltaTile < end) fetch(t0 + kDeltaTile);  // on its way while this tile is worked on
    __syncthreads();
    // per token the sums of squares of its key and its query and their product, each by eight neighbouring
    // lanes (a lane its channels in ascending order, the lanes by moves in a fixed order)
    for (int v0 = 0; v0 < kDeltaTile; v0 += n_threads / 8) {
      const int tt = v0 + threadIdx.x / 8, sub = threadIdx.x % 8;
      float kk2 = 0.f, qq2 = 0.f, kq = 0.f;
      if (tt < nt) {
        for (int d = sub; d < dk; d += 8) {
          const float ke = k_l[tt * dkp + d + d / 16 * 4], qe = q_l[tt * dkp + d + d / 16 * 4];
          kk2 = fmaf(ke, ke, kk2);
          qq2 = fmaf(qe, qe, qq2);
          kq = fmaf(ke, qe, kq);
        }
      }
      kk2 = row_group_sum(kk2, 8);
      qq2 = row_group_sum(qq2, 8);
      kq = row_group_sum(kq, 8);
      if (tt < nt && sub == 0) {
        const float k_inv = PLAIN ? 1.f : 1.0f / sqrtf(kk2 + 1e-6f), q_inv = PLAIN ? q_scale : q_scale / sqrtf(qq2 + 1e-6f);
        sc_l[6 * tt + 2] = k_inv;
        sc_l[6 * tt + 3] = q_inv;
        sc_l[6 * tt + 4] = kq * k_inv * q_inv;  // k^ . q^
      }
    }
    __syncthreads();
    {  // every thread scales the elements that it put there
      int tt = tt_first, d = d_first;
#pragma unroll
      for (int u = 0; u < kPreKQ; ++u) {
        const int dd = d < dk ? d : d - dk;
        if (tt < nt) (d < dk ? k_l : q_l)[tt * dkp + dd + dd / 16 * 4] *= sc_l[6 * tt + (d < dk ? 2 : 3)];
        tt += tt_step;
        d += d_step;
        if (d >= two_dk) { d -= two_dk; ++tt; }
      }
    }
    __syncthreads();
    // One token: S <- decay S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.  The read-out follows from the
    // decayed state and u, o = (decay S)^T q + u (k . q), so both products with the state are taken in one walk
    // over the lane's rows and summed over the column's lanes together, and the state's update is no part of
    // the chain that o waits for.  A token's operands are read from LDS while the token before is worked on.
    struct Operands {
      float kk[kDeltaRows], qq[kDeltaRows], dd[CH ? kDeltaRows : 1], v, beta, decay, kq;
    };
    auto read = [&](Operands& x, int tt_raw) {
      const int tt = tt_raw < kDeltaTile ? tt_raw : kDeltaTile - 1;
      const float* kt = k_l + tt * dkp + i0 + i0 / 16 * 4;  // (i0 is a multiple of 16: a lane's rows have no padding between them)
      const float* qt = q_l + tt * dkp + i0 + i0 / 16 * 4;
      if (CH) {
        const float* gt = g_l + tt * dkp + i0 + i0 / 16 * 4;
#pragma unroll
        for (int r = 0; r < kDeltaRows; ++r) x.dd[r] = i0 + r < dk ? gt[r] : 0.f;
      }
      if (VEC) {  // dk is a multiple of 4: four channels a read
#pragma unroll
        for (int r = 0; r < kDeltaRows; r += 4) {
          const bool in = i0 + r < dk;
          const float4 k4 = in ? *reinterpret_cast<const float4*>(kt + r) : float4{0.f, 0.f, 0.f, 0.f};
          const float4 q4 = in ? *reinterpret_cast<const float4*>(qt + r) : float4{0.f, 0.f, 0.f, 0.f};
          x.kk[r] = k4.x; x.kk[r + 1] = k4.y; x.kk[r + 2] = k4.z; x.kk[r + 3] = k4.w;
          x.qq[r] = q4.x; x.qq[r + 1] = q4.y; x.qq[r + 2] = q4.z; x.qq[r + 3] = q4.w;
        }
      } else {
#pragma unroll
        for (int r = 0; r < kDeltaRows; ++r) {
          x.kk[r] = i0 + r < dk ? kt[r] : 0.f;
          x.qq[r] = i0 + r < dk ? qt[r] : 0.f;
        }
      }
      x.v = v_l[tt * kDeltaCols + (j_loc < kDeltaCols ? j_loc : 0)];
      x.beta = sc_l[6 * tt];
      x.decay = sc_l[6 * tt + 1];
      x.kq = sc_l[6 * tt + 4];
    };
    auto token = [&](const Operands& x, int tt) {
      float kv[4] = {0.f, 0.f, 0.f, 0.f}, sq[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = 0; r < kDeltaRows; ++r) {
        S[r] = (CH ? x.dd[r] : x.decay) * S[r];
        kv[r % 4] = fmaf(S[r], x.kk[r], kv[r % 4]);
        sq[r % 4] = fmaf(S[r], x.qq[r], sq[r % 4]);
      }
      float kv_all = (kv[0] + kv[1]) + (kv[2] + kv[3]), sq_all = (sq[0] + sq[1]) + (sq[2] + sq[3]);
      if (lpc >= 2) { kv_all += dpp_xor1(kv_all); sq_all += dpp_xor1(sq_all); }
      if (lpc >= 4) { kv_all += dpp_xor2(kv_all); sq_all += dpp_xor2(sq_all); }
      if (lpc >= 8) { kv_all += dpp_half_mirror(kv_all); sq_all += dpp_half_mirror(sq_all); }
      if (lpc >= 16) { kv_all += dpp_mirror(kv_all); sq_all += dpp_mirror(sq_all); }
      const float u = PLAIN ? x.v : x.beta * (x.v - kv_all);
      if (live && part == 0) o_l[tt * kDeltaCols + j_loc] = fmaf(u, x.kq, sq_all);
#pragma unroll
      for (int r = 0; r < kDeltaRows; ++r) S[r] = fmaf(x.kk[r], u, S[r]);
    };
    Operands xa, xb;
    read(xa, 0);
#pragma unroll 1
    for (int tt = 0; tt < nt; tt += 2) {
      read(xb, tt + 1);
      token(xa, tt);
      if (tt + 1 < nt) {
        read(xa, tt + 2);
        token(xb, tt + 1);
      }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < nt * kDeltaCols; e += n_threads) {
      const int tt = e / kDeltaCols, d = e % kDeltaCols;
      if (d < v_cols) o_raw[((size_t)(t0 + tt) * H + h) * dv + cg * kDeltaCols + d] = o_l[tt * kDeltaCols + d];
    }
  }
  if (live) {
    if (VEC) {
#pragma unroll
      for (int r = 0; r < kDeltaRows; r += 4)
        if (i0 + r < dk) *reinterpret_cast<float4*>(st + i0 + r) = float4{S[r], S[r + 1], S[r + 2], S[r + 3]};
    } else {
#pragma unroll
      for (int r = 0; r < kDeltaRows; ++r)
        if (i0 + r < dk) st[i0 + r] = S[r];
    }
  }
}

// The same recurrence for a step in which every request brings one token (decode): no tiles, nothing fetched
// ahead, few registers, so that many of these short blocks share a CU.  Every sum is taken in the order in which
// gated_delta_kernel takes it (the norms by eight lanes over every eighth channel, the products with the state by
// four chains a lane and then the column's lanes), so a token's result has the same bits from either kernel.
template <typename T, bool VEC, int kDeltaRows, int RULE>
__global__ void __launch_bounds__(512)
gated_delta_step_kernel(const T* __restrict__ qkv, int qkv_stride, const T* __restrict__ proj, int proj_stride, int b_off,
                        int a_off, const float* __restrict__ A_log, const float* __restrict__ dt_bias,
                        float* __restrict__ state, long long state_stride, const int32_t* __restrict__ qo_indptr,
                        const int32_t* __restrict__ slot_ids, float* __restrict__ o_raw, int H, int G, int dk, int dv,
                        int lpc, int col_groups, const float* __restrict__ a_ch, int a_stride, float plain_rate) {
  constexpr bool CH = RULE >= 1, PLAIN = RULE == 2;
  constexpr int kCols = 32;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int dkp = dk + dk / 16 * 4;
  float* k_l = lds;
  float* q_l = lds + dkp;
  const int row = blockIdx.y;
  const int h = blockIdx.x / col_groups, cg = blockIdx.x % col_groups;
  const int g = h / (H / G);
  const size_t t = (size_t)qo_indptr[row];
  const int j_loc = threadIdx.x / lpc, part = threadIdx.x % lpc;
  const int j_raw = cg * kCols + j_loc;
  const bool live = j_loc < kCols && j_raw < dv;
  const int j = j_raw < dv ? j_raw : dv - 1;
  const int i0 = part * kDeltaRows;
  const T* tok = qkv + t * qkv_stride;
  for (int d = threadIdx.x; d < 2 * dk; d += blockDim.x) {
    const int dd = d < dk ? d : d - dk;
    (d < dk ? k_l : q_l)[dd + dd / 16 * 4] = to_f32(tok[d < dk ? G * dk + g * dk + dd : g * dk + dd]);
  }
  float* g_l = lds + 2 * dkp;  // (CH) the token's decays, once for all columns of the block
  if (CH) {
    const float rate = PLAIN ? 0.f : -expf(A_log[h]);
    for (int d = threadIdx.x; d < dk; d += blockDim.x) {
      const float pre = a_ch[t * a_stride + h * dk + d] + dt_bias[h * dk + d];
      g_l[d + d / 16 * 4] = PLAIN ? expf(plain_rate * log_sigmoid_f(pre)) : expf(rate * softplus_f(pre));
    }
  }
  float* st = state + (long long)slot_ids[row] * state_stride + ((size_t)h * dv + j) * dk;
  float S[kDeltaRows];
  if (VEC) {
#pragma unroll
    for (int r = 0; r < kDeltaRows; r += 4) {
      const float4 s4 = i0 + r < dk ? *reinterpret_cast<const float4*>(st + i0 + r) : float4{0.f, 0.f, 0.f, 0.f};
      S[r] = s4.x; S[r + 1] = s4.y; S[r + 2] = s4.z; S[r + 3] = s4.w;
    }
  } else {
#pragma unroll
    for (int r = 0; r < kDeltaRows; ++r) S[r] = i0 + r < dk ? st[i0 + r] : 0.f;
  }
  const float v = to_f32(tok[2 * G * dk + h * dv + j]);
  const float pb = PLAIN ? 0.f : to_f32(proj[t * proj_stride + b_off + h]), pa = CH ? 0.f : to_f32(proj[t * proj_stride + a_off + h]);
  const float neg_rate = PLAIN ? 0.f : -expf(A_log[h]), bias = CH ? 0.f : dt_bias[h];
  __syncthreads();
  const int sub = threadIdx.x % 8;
  float kk2 = 0.f, qq2 = 0.f, kq = 0.f;
  for (int d = sub; d < dk; d += 8) {
    const float ke = k_l[d + d / 16 * 4], qe = q_l[d + d / 16 * 4];
    kk2 = fmaf(ke, ke, kk2);
    qq2 = fmaf(qe, qe, qq2);
    kq = fmaf(ke, qe, kq);
  }
  kk2 = row_group_sum(kk2, 8);
  qq2 = row_group_sum(qq2, 8);
  kq = row_group_sum(kq, 8);
  const float k_inv = PLAIN ? 1.f : 1.0f / sqrtf(kk2 + 1e-6f);
  const float q_inv = PLAIN ? 1.0f / sqrtf((float)dk) : (1.0f / sqrtf((float)dk)) / sqrtf(qq2 + 1e-6f);
  const float kq_hat = kq * k_inv * q_inv;
  const float beta = sigmoid_f(pb), decay = CH ? 0.f : expf(neg_rate * softplus_f(pa + bias));
  float kv[4] = {0.f, 0.f, 0.f, 0.f}, sq[4] = {0.f, 0.f, 0.f, 0.f};
  float kk[kDeltaRows];
#pragma unroll
  for (int r = 0; r < kDeltaRows; ++r) {
    const int i = i0 + r;
    const bool in = i < dk;
    kk[r] = in ? k_l[i + i / 16 * 4] * k_inv : 0.f;
    const float qq = in ? q_l[i + i / 16 * 4] * q_inv : 0.f;
    float dec = decay;
    if (CH) dec = in ? g_l[i + i / 16 * 4] : 0.f;
    S[r] = dec * S[r];
    kv[r % 4] = fmaf(S[r], kk[r], kv[r % 4]);
    sq[r % 4] = fmaf(S[r], qq, sq[r % 4]);
  }
  const float kv_all = row_group_sum((kv[0] + kv[1]) + (kv[2] + kv[3]), lpc);
  const float sq_all = row_group_sum((sq[0] + sq[1]) + (sq[2] + sq[3]), lpc);
  const float u = PLAIN ? v : beta * (v - kv_all);
  if (live && part == 0) o_raw[(t * H + h) * dv + j] = fmaf(u, kq_hat, sq_all);
#pragma unroll
  for (int r = 0; r < kDeltaRows; ++r) S[r] = fmaf(kk[r], u, S[r]);
  if (live) {
    if (VEC) {
#pragma unroll
      for (int r = 0; r < kDeltaRows; r += 4)
        if (i0 + r < dk) *reinterpret_cast<float4*>(st + i0 + r) = float4{S[r], S[r + 1], S[r + 2], S[r + 3]};
    } else {
#pragma unroll
      for (int r = 0; r < kDeltaRows; ++r)
        if (i0 + r < dk) st[i0 + r] = S[r];
    }
  }
}

// out[t, h, :] = T(o / sqrt(mean(o^2) + eps) * norm_w * act(gate[t, h, :])): one wave a (token, head).  act is silu
// or (SIGMOID) the logistic function; the weight is one vector for all heads (w_stride 0) or a vector a head (dv).
template <typename T, bool SIGMOID>
__global__ void __launch_bounds__(kHeadWaves* kWave)
delta_output_kernel(const float* __restrict__ o_raw, const T* __restrict__ proj, int proj_stride, int gate_off,
                    const float* __restrict__ norm_w, int w_stride, float eps, T* __restrict__ out, int H, int dv,
                    const float* __restrict__ den) {
  const int t = blockIdx.x;
  const int h = blockIdx.y * kHeadWaves + threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  if (h >= H) return;
  const float* o = o_raw + ((size_t)t * H + h) * dv;
  // (den: every element of the head is first divided by the head's own number)
  const float pre = den ? 1.0f / den[(size_t)t * H + h] : 1.0f;
  float ss = 0.f;
  for (int d = lane; d < dv; d += kWave) ss = fmaf(o[d] * pre, o[d] * pre, ss);
  ss = wave_sum(ss);
  const float inv = pre / sqrtf(ss / (float)dv + eps);
  const T* gp = proj + (size_t)t * proj_stride + gate_off + (size_t)h * dv;
  T* op = out + ((size_t)t * H + h) * dv;
  const float* wp = norm_w + (size_t)h * w_stride;
  for (int d = lane; d < dv; d += kWave) {
    const float gate = to_f32(gp[d]);
    op[d] = from_f32<T>(o[d] * inv * wp[d] * (SIGMOID ? sigmoid_f(gate) : silu_f(gate)));
  }
}

// The same for rows of o_raw in units of 65535 tokens (a grid's first dimension).
template <typename T>
int launch_head_output(const float* o_raw, const T* gate, int gate_stride, int gate_off, const float* norm_w, int w_stride,
                       float eps, T* out, int n_tokens, int H, int dv, bool sigmoid, hipStream_t stream,
                       const float* den = nullptr) {
  for (int t0 = 0; t0 < n_tokens; t0 += 65535) {
    const int nt = n_tokens - t0 < 65535 ? n_tokens - t0 : 65535;
    const dim3 ogrid(nt, (H + kHeadWaves - 1) / kHeadWaves);
    const float* src = o_raw + (size_t)t0 * H * dv;
    if (sigmoid)
      delta_output_kernel<T, true><<<ogrid, kHeadWaves * kWave, 0, stream>>>(src, gate + (size_t)t0 * gate_stride, gate_stride, gate_off,
                                                                             norm_w, w_stride, eps, out + (size_t)t0 * H * dv, H, dv,
                                                                             den ? den + (size_t)t0 * H : nullptr);
    else
      delta_output_kernel<T, false><<<ogrid, kHeadWaves * kWave, 0, stream>>>(src, gate + (size_t)t0 * gate_stride, gate_stride, gate_off,
                                                                              norm_w, w_stride, eps, out + (size_t)t0 * H * dv, H, dv,
                                                                             den ? den + (size_t)t0 * H : nullptr);
  }
  return tl_check_launch("head_output");
}

}  // namespace

// ============================================================================= C interface
TL_EXPORT int tl_embed_scaled(const int32_t* tokens, const void* table, float* out, int n_tokens, int hidden, float scale,
                              int dtype, hipStream_t stream) {
  TL_REQUIRE(n_tokens >= 0 && hidden > 0, "embed_scaled: bad sizes n_tokens=%d hidden=%d", n_tokens, hidden);
  if (n_tokens == 0) return TL_OK;
  if (dtype == TL_F32)
    embed_scaled_kernel<float><<<n_tokens, 256, 0, stream>>>(tokens, (const float*)table, out, hidden, scale);
  else if (dtype == TL_BF16)
    embed_scaled_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>(tokens, (const bf16_t*)table, out, hidden, scale);
  else
    return tl_fail(TL_ERR_ARG, "embed_scaled: unknown dtype %d", dtype);
  return tl_check_launch("embed_scaled");
}

// x, h_out: [.., hidden] of stream_dtype; d0, d1, y of dtype; w, b 32-bit.  n output rows.
TL_EXPORT int tl_layernorm(const void* x, const void* d0, const void* d1, float mult, const int32_t* rows, const float* w,
                           const float* b, void* h_out, void* y, int n, int hidden, float eps, int stream_dtype, int dtype,
                           hipStream_t stream) {
  TL_REQUIRE(n >= 0 && hidden > 0, "layernorm: bad sizes n=%d hidden=%d", n, hidden);
  TL_REQUIRE(d1 == nullptr || d0 != nullptr, "layernorm: a second term without a first");
  if ((size_t)hidden * sizeof(float) + 1024 > (size_t)tl_device_facts().lds_bytes)
    return tl_fail(TL_ERR_UNSUPPORTED, "layernorm: rows of %d elements do not fit the LDS", hidden);
  if (n == 0) return TL_OK;
  if (stream_dtype == TL_F32 && dtype == TL_F32)
    return layernorm_launch<float, float>(x, d0, d1, mult, rows, w, b, h_out, y, n, hidden, eps, stream);
  if (stream_dtype == TL_F32 && dtype == TL_BF16)
    return layernorm_launch<float, bf16_t>(x, d0, d1, mult, rows, w, b, h_out, y, n, hidden, eps, stream);
  if (stream_dtype == TL_BF16 && dtype == TL_BF16)
    return layernorm_launch<bf16_t, bf16_t>(x, d0, d1, mult, rows, w, b, h_out, y, n, hidden, eps, stream);
  return tl_fail(TL_ERR_ARG, "layernorm: stream dtype %d with dtype %d", stream_dtype, dtype);
}

TL_EXPORT int tl_gelu_mul(const void* gate_up, void* out, int n, int inter, int dtype, hipStream_t stream) {
  TL_REQUIRE(n >= 0 && inter > 0, "gelu_mul: bad sizes n=%d inter=%d", n, inter);
  if (n == 0) return TL_OK;
  if (dtype == TL_F32) return gelu_mul_launch((const float*)gate_up, (float*)out, n, inter, stream);
  if (dtype == TL_BF16) return gelu_mul_launch((const bf16_t*)gate_up, (bf16_t*)out, n, inter, stream);
  return tl_fail(TL_ERR_ARG, "gelu_mul: unknown dtype %d", dtype);
}

TL_EXPORT int tl_rope_norm_kv_write(void* qkv, int n_tokens, int n_q, int n_kv, int dk, int dv, const float* cos_sin, int rot,
                                    int pairing, float norm_eps, void* k_pages, void* v_pages, const int32_t* slot_mapping,
                                    int page_size, int dtype, hipStream_t stream) {
  TL_REQUIRE(n_tokens >= 0 && n_q > 0 && n_kv >= 0 && dk > 0 && dv > 0, "rope_norm: bad sizes");
  TL_REQUIRE(dk <= kHeadChan * kWave && dv <= kHeadChan * kWave, "rope_norm: heads of %d and %d channels, at most %d", dk, dv, kHeadChan * kWave);
  TL_REQUIRE(rot >= 0 && rot <= dk && rot % 2 == 0, "rope_norm: %d rotated channels of %d (even, at most the head)", rot, dk);
  TL_REQUIRE(pairing == 0 || pairing == 1, "rope_norm: pairing must be 0 (interleaved) or 1 (half split)");
  TL_REQUIRE(rot == 0 || cos_sin != nullptr, "rope_norm: rotation without a table of cosines and sines");
  TL_REQUIRE(k_pages == nullptr || (v_pages != nullptr && slot_mapping != nullptr && page_size > 0), "rope_norm: pages without slots");
  if (n_tokens == 0) return TL_OK;
  const int row = (n_q + n_kv) * dk + n_kv * dv;
  const int per_block = kHeadWaves * kHeadsPerWave;
  const dim3 grid(n_tokens, (n_q + 2 * n_kv + per_block - 1) / per_block);
  if (dtype == TL_F32)
    rope_norm_kv_write_kernel<float><<<grid, kHeadWaves * kWave, 0, stream>>>(
        (float*)qkv, row, n_q, n_kv, dk, dv, (const float2*)cos_sin, rot, pairing, norm_eps, (float*)k_pages, (float*)v_pages,
        slot_mapping, page_size);
  else if (dtype == TL_BF16)
    rope_norm_kv_write_kernel<bf16_t><<<grid, kHeadWaves * kWave, 0, stream>>>(
        (bf16_t*)qkv, row, n_q, n_kv, dk, dv, (const float2*)cos_sin, rot, pairing, norm_eps, (bf16_t*)k_pages, (bf16_t*)v_pages,
        slot_mapping, page_size);
  else
    return tl_fail(TL_ERR_ARG, "rope_norm: unknown dtype %d", dtype);
  return tl_check_launch("rope_norm_kv_write");
}

// The convolution of every token of the step and then the requests' new histories (two launches).
TL_EXPORT int tl_causal_conv(const void* x, int x_stride, const float* taps, const float* bias, float* state,
                             long long state_stride, const int32_t* token_seq, const int32_t* qo_indptr,
                             const int32_t* slot_ids, void* out, int out_stride, int n_tokens, int n_seqs, int C, int K,
                             int act, int dtype, hipStream_t stream) {
  TL_REQUIRE(n_tokens >= 0 && n_seqs >= 0 && C > 0 && K >= 1 && K <= 64, "causal_conv: bad sizes C=%d K=%d", C, K);
  TL_REQUIRE(n_tokens <= 65535 * 32 && n_seqs <= 65535, "causal_conv: too many tokens or requests for one launch");
  TL_REQUIRE(act == 0 || act == 1, "causal_conv: act must be 0 (none) or 1 (silu)");
  if (n_tokens == 0) return TL_OK;
  if (dtype != TL_F32 && dtype != TL_BF16) return tl_fail(TL_ERR_ARG, "causal_conv: unknown dtype %d", dtype);
  const int cblocks = (C + 255) / 256;
  const int elt = dtype == TL_F32 ? 4 : 2, vec = 16 / elt;
  const bool wide = C % vec == 0 && x_stride % vec == 0 && out_stride % vec == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)out % 16) == 0;
  const int vblocks = (C / (wide ? vec : 1) + 255) / 256;
  if (n_tokens == n_seqs) {  // one token a request: convolution and history in one launch
    const dim3 grid(vblocks, n_seqs);
#define TL_CONV_STEP(T, V)                                                                                            \
  conv_step_kernel<T, V><<<grid, 256, 0, stream>>>((const T*)x, x_stride, taps, bias, state, state_stride, qo_indptr, \
                                                   slot_ids, (T*)out, out_stride, C, K, act)
    if (dtype == TL_F32) {
      if (wide) TL_CONV_STEP(float, 4);
      else TL_CONV_STEP(float, 1);
    } else {
      if (wide) TL_CONV_STEP(bf16_t, 8);
      else TL_CONV_STEP(bf16_t, 1);
    }
#undef TL_CONV_STEP
    return tl_check_launch("conv_step");
  }
  for (int t0 = 0; t0 < n_tokens; t0 += 65535) {
    const int nt = n_tokens - t0 < 65535 ? n_tokens - t0 : 65535;
    const dim3 grid(vblocks, nt);
#define TL_CONV(T, V)                                                                                                  \
  causal_conv_kernel<T, V><<<grid, 256, 0, stream>>>((const T*)x, x_stride, taps, bias, state, state_stride, token_seq, \
                                                     qo_indptr, slot_ids, (T*)out, out_stride, C, K, act, t0)
    if (dtype == TL_F32) {
      if (wide) TL_CONV(float, 4);
      else TL_CONV(float, 1);
    } else {
      if (wide) TL_CONV(bf16_t, 8);
      else TL_CONV(bf16_t, 1);
    }
#undef TL_CONV
  }
  int rc = tl_check_launch("causal_conv");
  if (rc != TL_OK || K == 1 || n_seqs == 0) return rc;
  const dim3 hgrid(cblocks, n_seqs);
  if (dtype == TL_F32)
    conv_history_kernel<float><<<hgrid, 256, 0, stream>>>((const float*)x, x_stride, state, state_stride, qo_indptr, slot_ids, C, K);
  else
    conv_history_kernel<bf16_t><<<hgrid, 256, 0, stream>>>((const bf16_t*)x, x_stride, state, state_stride, qo_indptr, slot_ids, C, K);
  return tl_check_launch("conv_history");
}

namespace {
template <typename T, typename DT>
int scan_launch(const void* x, const void* dt_pre, const void* bc, int bc_stride, int b_off, int c_off, const void* z,
                int z_stride, const float* dt_bias, const float* A, const float* D, float* state, long long state_stride,
                const int32_t* qo_indptr, const int32_t* slot_ids, void* out, int n_seqs, int inner, int N,
                const int32_t* segs, const int32_t* row_seg, int n_segs, float* ws, float* seg_dt, hipStream_t stream) {
  // states a lane holds and lanes a channel: up to 32 states one lane, then 2, 4, 8 lanes of 32
  int nb = N <= 8 ? 8 : N <= 16 ? 16 : 32;
  int lpc = 1;
  while (nb * lpc < N) lpc *= 2;
  const int per_block = kScanThreads / lpc;
  const int cblocks = (inner + per_block - 1) / per_block;
  const size_t lds = (size_t)kScanTile * 2 * N * sizeof(float);
#define TL_SCAN(NB, MODE, ROWS, STATE, STRIDE)                                                                          \
  selective_scan_kernel<T, DT, NB, MODE><<<dim3(cblocks, ROWS), kScanThreads, lds, stream>>>(                           \
      (const T*)x, (const DT*)dt_pre, (const T*)bc, bc_stride, b_off, c_off, (const T*)z, z_stride, dt_bias, A, D, STATE, \
      STRIDE, qo_indptr, slot_ids, (T*)out, inner, N, lpc, segs, seg_dt)
#define TL_SCAN_NB(MODE, ROWS, STATE, STRIDE)               \
  do {                                                      \
    if (nb == 8) TL_SCAN(8, MODE, ROWS, STATE, STRIDE);     \
    else if (nb == 16) TL_SCAN(16, MODE, ROWS, STATE, STRIDE); \
    else TL_SCAN(32, MODE, ROWS, STATE, STRIDE);            \
  } while (0)
  if (segs == nullptr) {
    TL_SCAN_NB(0, n_seqs, state, state_stride);
    return tl_check_launch("selective_scan");
  }
  const long long per = (long long)inner * N;
  TL_SCAN_NB(1, n_segs, ws, per);
  int rc = tl_check_launch("selective_scan (segments)");
  if (rc != TL_OK) return rc;
  scan_carry_kernel<<<dim3((unsigned)((per + 255) / 256), n_seqs), 256, 0, stream>>>(ws, seg_dt, A, state, state_stride, row_seg,
                                                                                 slot_ids, inner, N);
  rc = tl_check_launch("selective_scan (carry)");
  if (rc != TL_OK) return rc;
  TL_SCAN_NB(2, n_segs, ws, per);
#undef TL_SCAN_NB
#undef TL_SCAN
  return tl_check_launch("selective_scan (emit)");
}
}  // namespace

// x, out: [n_tokens, inner] of dtype; dt_pre: [n_tokens, inner] of dt_dtype (32-bit, or dtype); bc and z: see the
// kernel; state: the requests' rows, S[c][n] at state + slot * state_stride + c * N + n.  With segs (first and last
// token of n_segs segments, every request's in order) and row_seg (n_seqs + 1: the first segment of every request)
// the segments run side by side; ws: n_segs * inner * N floats, seg_dt: n_segs * inner floats.
TL_EXPORT int tl_selective_scan(const void* x, const void* dt_pre, int dt_dtype, const void* bc, int bc_stride, int b_off,
                                int c_off, const void* z, int z_stride, const float* dt_bias, const float* A, const float* D,
                                float* state, long long state_stride, const int32_t* qo_indptr, const int32_t* slot_ids,
                                void* out, int n_seqs, int inner, int N, int dtype, const int32_t* segs,
                                const int32_t* row_seg, int n_segs, float* ws, float* seg_dt, hipStream_t stream) {
  TL_REQUIRE(n_seqs >= 0 && inner > 0 && N > 0, "selective_scan: bad sizes");
  TL_REQUIRE(N <= 256, "selective_scan: %d states a channel, at most 256", N);
  TL_REQUIRE(n_seqs <= 65535 && n_segs <= 65535, "selective_scan: at most 65535 requests and segments a step");
  TL_REQUIRE(segs == nullptr || (row_seg != nullptr && ws != nullptr && seg_dt != nullptr && n_segs > 0),
             "selective_scan: segments without their workspace");
  if (n_seqs == 0) return TL_OK;
#define TL_SCAN_ARGS x, dt_pre, bc, bc_stride, b_off, c_off, z, z_stride, dt_bias, A, D, state, state_stride, qo_indptr, slot_ids, \
                     out, n_seqs, inner, N, segs, row_seg, n_segs, ws, seg_dt, stream
  if (dtype == TL_F32 && dt_dtype == TL_F32) return scan_launch<float, float>(TL_SCAN_ARGS);
  if (dtype == TL_BF16 && dt_dtype == TL_F32) return scan_launch<bf16_t, float>(TL_SCAN_ARGS);
  if (dtype == TL_BF16 && dt_dtype == TL_BF16) return scan_launch<bf16_t, bf16_t>(TL_SCAN_ARGS);
#undef TL_SCAN_ARGS
  return tl_fail(TL_ERR_ARG, "selective_scan: dtype %d with step sizes of dtype %d", dtype, dt_dtype);
}

// qkv, proj, out as the kernels describe; state: S^T of head h at state + slot * state_stride + h * dv * dk;
// o_raw: workspace of n_tokens * H * dv floats.  gate: the matrix whose H * dv columns from gate_off hold the output
// gate (proj itself, or a tensor of its own); gate_sigmoid: the gate's activation is the logistic function, not silu.
// a_ch (or null): 32-bit pre-activations of a decay per key channel, [n_tokens, a_stride] with H * dk columns; then
// dt_bias has H * dk entries.
TL_EXPORT int tl_gated_delta(const void* qkv, int qkv_stride, const void* proj, int proj_stride, int gate_off, int b_off,
                             int a_off, const float* A_log, const float* dt_bias, const float* norm_w, float eps, float* state,
                             long long state_stride, const int32_t* qo_indptr, const int32_t* slot_ids, void* out, int n_tokens,
                             int n_seqs, int H, int G, int dk, int dv, float* o_raw, int dtype, const void* gate, int gate_stride,
                             int gate_sigmoid, const float* a_ch, int a_stride, float plain_rate, hipStream_t stream) {
  TL_REQUIRE(n_seqs >= 0 && n_tokens >= 0 && H > 0 && G > 0 && dk > 0 && dv > 0, "gated_delta: bad sizes");
  TL_REQUIRE(H % G == 0, "gated_delta: %d heads are not a multiple of %d key heads", H, G);
  if (dk > 256) return tl_fail(TL_ERR_UNSUPPORTED, "gated_delta: keys of %d channels, at most 256", dk);
  TL_REQUIRE(n_seqs <= 65535 && n_tokens <= 0x7fffffff / 4, "gated_delta: too many requests or tokens a step");
  TL_REQUIRE(o_raw != nullptr && gate != nullptr, "gated_delta: no workspace or no gate");
  TL_REQUIRE(a_ch == nullptr || a_stride >= H * dk, "gated_delta: rows of %d decays, %d needed", a_stride, H * dk);
  if (n_seqs == 0 || n_tokens == 0) return TL_OK;
  if (dtype != TL_F32 && dtype != TL_BF16) return tl_fail(TL_ERR_ARG, "gated_delta: unknown dtype %d", dtype);
  const int rows = dk <= 128 ? 8 : 16;
  int lpc = 1;
  while (rows * lpc < dk) lpc *= 2;  // at most 16: a column's lanes lie in one row of 16 lanes
  // columns a block: 16 while that leaves fewer than two blocks a CU, else 32 (a step of single tokens: always 32)
  const bool single = n_tokens == n_seqs;
  const bool ch = a_ch != nullptr;
  const bool plain = plain_rate > 0.f;
  TL_REQUIRE(!plain || ch, "gated_delta: the plain rule has a decay per key channel");
  TL_REQUIRE(plain || (A_log != nullptr && proj != nullptr), "gated_delta: no A_log or no projections");
  const int cols = !single && (long long)n_seqs * H * ((dv + 15) / 16) < 2LL * tl_device_facts().compute_units ? 16 : 32;
  const int threads = (cols * lpc + kWave - 1) / kWave * kWave;
  const int col_groups = (dv + cols - 1) / cols;
  const int dkp = dk + dk / 16 * 4;
  const size_t lds = ((size_t)kDeltaTile * (2 * dkp + 2 * cols + 6 + (ch ? dkp : 0))) * sizeof(float);
  const dim3 grid(H * col_groups, n_seqs);
#define TL_DELTA_R(T, VEC, R, C, CH)                                                                                   \
  gated_delta_kernel<T, VEC, R, C, CH><<<grid, threads, lds, stream>>>(                                                \
      (const T*)qkv, qkv_stride, (const T*)proj, proj_stride, b_off, a_off, A_log, dt_bias, state, state_stride,       \
      qo_indptr, slot_ids, o_raw, H, G, dk, dv, lpc, col_groups, a_ch, a_stride, plain_rate)
#define TL_DELTA(T, VEC, CH)                                      \
  do {                                                            \
    if (rows == 8 && cols == 16) TL_DELTA_R(T, VEC, 8, 16, CH);   \
    else if (rows == 8) TL_DELTA_R(T, VEC, 8, 32, CH);            \
    else if (cols == 16) TL_DELTA_R(T, VEC, 16, 16, CH);          \
    else TL_DELTA_R(T, VEC, 16, 32, CH);                          \
  } while (0)
  // four rows a load where every lane's rows start at a multiple of 16 bytes, in LDS and in the state
  const bool vec = dk % 4 == 0 && ((uintptr_t)state % 16) == 0 && state_stride % 4 == 0;
#define TL_DELTA_STEP(T, VEC, CH)                                                                                      \
  do {                                                                                                                 \
    const size_t step_lds = (CH ? 3 : 2) * (size_t)dkp * sizeof(float);                                               \
    if (rows == 8)                                                                                                     \
      gated_delta_step_kernel<T, VEC, 8, CH><<<grid, threads, step_lds, stream>>>(                                     \
          (const T*)qkv, qkv_stride, (const T*)proj, proj_stride, b_off, a_off, A_log, dt_bias, state, state_stride,   \
          qo_indptr, slot_ids, o_raw, H, G, dk, dv, lpc, col_groups, a_ch, a_stride, plain_rate);                      \
    else                                                                                                               \
      gated_delta_step_kernel<T, VEC, 16, CH><<<grid, threads, step_lds, stream>>>(                                    \
          (const T*)qkv, qkv_stride, (const T*)proj, proj_stride, b_off, a_off, A_log, dt_bias, state, state_stride,   \
          qo_indptr, slot_ids, o_raw, H, G, dk, dv, lpc, col_groups, a_ch, a_stride, plain_rate);                      \
  } while (0)
#define TL_DELTA_ANY(T, VEC, CH)          \
  do {                                    \
    if (single) TL_DELTA_STEP(T, VEC, CH); \
    else TL_DELTA(T, VEC, CH);            \
  } while (0)
#define TL_DELTA_T(T)                            \
  do {                                           \
    if (vec && plain) TL_DELTA_ANY(T, true, 2);  \
    else if (plain) TL_DELTA_ANY(T, false, 2);   \
    else if (vec && ch) TL_DELTA_ANY(T, true, 1);  \
    else if (vec) TL_DELTA_ANY(T, true, 0);      \
    else if (ch) TL_DELTA_ANY(T, false, 1);      \
    else TL_DELTA_ANY(T, false, 0);              \
  } while (0)
  if (dtype == TL_F32) TL_DELTA_T(float);
  else TL_DELTA_T(bf16_t);
#undef TL_DELTA_T
#undef TL_DELTA_ANY
#undef TL_DELTA_STEP
#undef TL_DELTA
#undef TL_DELTA_R
  int rc = tl_check_launch("gated_delta");
  if (rc != TL_OK) return rc;
  if (dtype == TL_F32)
    return launch_head_output<float>(o_raw, (const float*)gate, gate_stride, gate_off, norm_w, 0, eps, (float*)out, n_tokens, H, dv,
                                     gate_sigmoid != 0, stream);
  return launch_head_output<bf16_t>(o_raw, (const bf16_t*)gate, gate_stride, gate_off, norm_w, 0, eps, (bf16_t*)out, n_tokens, H, dv,
                                    gate_sigmoid != 0, stream);
}


// ============================================================================= matrix memory (mLSTM)
// Per request and head h, in 32-bit: a matrix C [dk][dv], a vector n [dk] and a running maximum m (all zero at the
// start).  For every token, with q already times dk^-1/2, the log input gate i = cap tanh((i~ + b_i) / cap) and the
// log forget gate f = logsigmoid(cap tanh((f~ + b_f) / cap)):
//   m' = max(f + m, i);  keep = exp(f + m - m');  take = exp(i - m')
//   C <- keep C + take k v^T;  n <- keep n + take k;  o = C^T q / (max(|n . q|, exp(-m')) + 1e-6)
// n is the matrix's column dv (its "value" is 1), so the state of a head is [dv + 1][dk], column by column, and
// behind all heads' columns lies m, once for every column (the blocks that share a head each keep their own).
// A block takes kMemCols columns of one (request, head); lpc neighbouring lanes share a column, each holding R rows.
// The tokens come in tiles of kDeltaTile: the next tile's raw q, k, v and gates travel into registers while this one
// is worked on; one wave walks the tile's maxima (a chain of additions and comparisons, no exponentials on it)
// and then takes the exponentials side by side; the keys go to LDS times `take`, so a token costs a lane three
// operations a row.  The numerators go to o_raw [n, H, dv], the denominators to den [n, H].
namespace {
constexpr int kMemCols = 32;


template <typename T, bool VEC, int R>
__global__ void __launch_bounds__(512)
matrix_memory_kernel(const T* __restrict__ proj, int stride, int q_off, int k_off, int v_off, int i_off, int f_off,
                     const float* __restrict__ i_bias, const float* __restrict__ f_bias, float cap,
                     float* __restrict__ state, long long state_stride, const int32_t* __restrict__ qo_indptr,
                     const int32_t* __restrict__ slot_ids, float* __restrict__ o_raw, float* __restrict__ den, int H, int dk,
                     int dv, int lpc, int col_groups) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int dkp = dk + dk / 16 * 4;
  float* k_l = lds;
  float* q_l = k_l + kDeltaTile * dkp;
  float* v_l = q_l + kDeltaTile * dkp;
  float* o_l = v_l + kDeltaTile * kMemCols;
  float* sc_l = o_l + kDeltaTile * kMemCols;  // [kDeltaTile][4]: keep, take, exp(-m'); then the maximum that enters the next tile
  const int W = dv + 1;
  const int row = blockIdx.y;
  const int h = blockIdx.x / col_groups, cg = blockIdx.x % col_groups;
  const int start = qo_indptr[row], end = qo_indptr[row + 1];
  const int n_threads = blockDim.x;
  const int j_loc = threadIdx.x / lpc, part = threadIdx.x % lpc;
  const int j_raw = cg * kMemCols + j_loc;
  const bool live = j_loc < kMemCols && j_raw < W;
  const int j = j_raw < W ? j_raw : W - 1;
  const bool norm_col = j == dv;
  const int i0 = part * R;
  float* slot = state + (long long)slot_ids[row] * state_stride;
  float* st = slot + ((size_t)h * W + j) * dk;
  float* m_at = slot + (size_t)H * W * dk + (size_t)h * W + j;
  float S[R];
  if (VEC) {
#pragma unroll
    for (int r = 0; r < R; r += 4) {
      const float4 s4 = i0 + r < dk ? *reinterpret_cast<const float4*>(st + i0 + r) : float4{0.f, 0.f, 0.f, 0.f};
      S[r] = s4.x; S[r + 1] = s4.y; S[r + 2] = s4.z; S[r + 3] = s4.w;
    }
  } else {
#pragma unroll
    for (int r = 0; r < R; ++r) S[r] = i0 + r < dk ? st[i0 + r] : 0.f;
  }
  if (threadIdx.x == 0) sc_l[4 * kDeltaTile] = *m_at;  // (thread 0 holds a live column: cg * kMemCols < W)
  const float q_scale = 1.0f / sqrtf((float)dk);
  const float bi = i_bias[h], bf = f_bias[h];
  const int v_cols = min(kMemCols, W - cg * kMemCols);  // (the normaliser's column included)
  const int v_col = v_off + h * dv + cg * kMemCols;

  const int two_dk = 2 * dk;
  const int tt_first = threadIdx.x / two_dk, d_first = threadIdx.x % two_dk;
  const int tt_step = n_threads / two_dk, d_step = n_threads % two_dk;
  constexpr int kPreKQ = R, kPreV = 8;
  T pre_kq[kPreKQ], pre_v[kPreV], pre_i = from_f32<T>(0.f), pre_f = from_f32<T>(0.f);
  auto fetch = [&](int t0) {
    const int nt = min(kDeltaTile, end - t0);
    if (threadIdx.x < nt) {
      const T* pr = proj + (size_t)(t0 + threadIdx.x) * stride;
      pre_i = pr[i_off + h];
      pre_f = pr[f_off + h];
    }
    int tt = tt_first, d = d_first;
#pragma unroll
    for (int u = 0; u < kPreKQ; ++u) {
      if (tt < nt) pre_kq[u] = proj[(size_t)(t0 + tt) * stride + (d < dk ? k_off + h * dk + d : q_off + h * dk + d - dk)];
      tt += tt_step;
      d += d_step;
      if (d >= two_dk) { d -= two_dk; ++tt; }
    }
#pragma unroll
    for (int u = 0; u < kPreV; ++u) {
      const int e = threadIdx.x + u * n_threads;
      const int tt = e / kMemCols, d = e % kMemCols;
      if (tt < nt && d < v_cols && cg * kMemCols + d < dv) pre_v[u] = proj[(size_t)(t0 + tt) * stride + v_col + d];
    }
  };
  if (start < end) fetch(start);
  for (int t0 = start; t0 < end; t0 += kDeltaTile) {
    const int nt = min(kDeltaTile, end - t0);
    __syncthreads();  // the tile before has been read to its end
    if (threadIdx.x < kWave) {
      // the gates of the tile's tokens, a lane a token; then the maxima, every lane walking the same chain
      const int lane = threadIdx.x;
      float gi = 0.f, gf = 0.f;
      if (lane < nt) {
        gi = cap * tanhf((to_f32(pre_i) + bi) / cap);
        gf = log_sigmoid_f(cap * tanhf((to_f32(pre_f) + bf) / cap));
      }
      float m = sc_l[4 * kDeltaTile], m_before = 0.f, m_mine = 0.f;
      for (int tt = 0; tt < nt; ++tt) {
        const float ft = __shfl(gf, tt, kWave), it = __shfl(gi, tt, kWave);
        const float m_new = fmaxf(ft + m, it);
        if (lane == tt) { m_before = m; m_mine = m_new; }
        m = m_new;
      }
      if (lane < nt) {
        sc_l[4 * lane] = expf(gf + m_before - m_mine);
        sc_l[4 * lane + 1] = expf(gi - m_mine);
        sc_l[4 * lane + 2] = expf(-m_mine);
      }
      if (lane == 0) sc_l[4 * kDeltaTile] = m;
    }
    __syncthreads();
    {
      int tt = tt_first, d = d_first;
#pragma unroll
      for (int u = 0; u < kPreKQ; ++u) {
        const int dd = d < dk ? d : d - dk;
        if (tt < nt) (d < dk ? k_l : q_l)[tt * dkp + dd + dd / 16 * 4] = to_f32(pre_kq[u]) * (d < dk ? sc_l[4 * tt + 1] : q_scale);
        tt += tt_step;
        d += d_step;
        if (d >= two_dk) { d -= two_dk; ++tt; }
      }
    }
#pragma unroll
    for (int u = 0; u < kPreV; ++u) {
      const int e = threadIdx.x + u * n_threads;
      const int tt = e / kMemCols, d = e % kMemCols;
      if (tt < nt && d < v_cols) v_l[tt * kMemCols + d] = cg * kMemCols + d < dv ? to_f32(pre_v[u]) : 1.0f;
    }
    if (t0 + kDeltaTile < end) fetch(t0 + kDeltaTile);  // on its way while this tile is worked on
    __syncthreads();
    struct Operands {
      float kk[R], qq[R], v, keep, floor;
    };
    auto read = [&](Operands& x, int tt_raw) {
      const int tt = tt_raw < kDeltaTile ? tt_raw : kDeltaTile - 1;
      const float* kt = k_l + tt * dkp + i0 + i0 / 16 * 4;
      const float* qt = q_l + tt * dkp + i0 + i0 / 16 * 4;
      if (VEC) {
#pragma unroll
        for (int r = 0; r < R; r += 4) {
          const bool in = i0 + r < dk;
          const float4 k4 = in ? *reinterpret_cast<const float4*>(kt + r) : float4{0.f, 0.f, 0.f, 0.f};
          const float4 q4 = in ? *reinterpret_cast<const float4*>(qt + r) : float4{0.f, 0.f, 0.f, 0.f};
          x.kk[r] = k4.x; x.kk[r + 1] = k4.y; x.kk[r + 2] = k4.z; x.kk[r + 3] = k4.w;
          x.qq[r] = q4.x; x.qq[r + 1] = q4.y; x.qq[r + 2] = q4.z; x.qq[r + 3] = q4.w;
        }
      } else {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          x.kk[r] = i0 + r < dk ? kt[r] : 0.f;
          x.qq[r] = i0 + r < dk ? qt[r] : 0.f;
        }
      }
      x.v = v_l[tt * kMemCols + (j_loc < kMemCols ? j_loc : 0)];
      x.keep = sc_l[4 * tt];
      x.floor = sc_l[4 * tt + 2];
    };
    auto token = [&](const Operands& x, int tt) {
      float sq[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = 0; r < R; ++r) {
        S[r] = fmaf(x.kk[r], x.v, x.keep * S[r]);
        sq[r % 4] = fmaf(S[r], x.qq[r], sq[r % 4]);
      }
      const float sq_all = row_group_sum((sq[0] + sq[1]) + (sq[2] + sq[3]), lpc);
      if (live && part == 0) o_l[tt * kMemCols + j_loc] = norm_col ? fmaxf(fabsf(sq_all), x.floor) + 1e-6f : sq_all;
    };
    Operands xa, xb;
    read(xa, 0);
#pragma unroll 1
    for (int tt = 0; tt < nt; tt += 2) {
      read(xb, tt + 1);
      token(xa, tt);
      if (tt + 1 < nt) {
        read(xa, tt + 2);
        token(xb, tt + 1);
      }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < nt * kMemCols; e += n_threads) {
      const int tt = e / kMemCols, d = e % kMemCols;
      if (d < v_cols) {
        const int col = cg * kMemCols + d;
        if (col < dv) o_raw[((size_t)(t0 + tt) * H + h) * dv + col] = o_l[e];
        else den[(size_t)(t0 + tt) * H + h] = o_l[e];
      }
    }
  }
  __syncthreads();
  if (live) {
    if (VEC) {
#pragma unroll
      for (int r = 0; r < R; r += 4)
        if (i0 + r < dk) *reinterpret_cast<float4*>(st + i0 + r) = float4{S[r], S[r + 1], S[r + 2], S[r + 3]};
    } else {
#pragma unroll
      for (int r = 0; r < R; ++r)
        if (i0 + r < dk) st[i0 + r] = S[r];
    }
    if (part == 0) *m_at = sc_l[4 * kDeltaTile];
  }
}

// The same cell for a step in which every request brings one token (decode): no tiles, nothing fetched ahead, every
// thread works the gates out for itself.  Every product and sum is taken as matrix_memory_kernel takes it, so a token's
// result has the same bits from either kernel.
template <typename T, bool VEC, int R>
__global__ void __launch_bounds__(512)
matrix_memory_step_kernel(const T* __restrict__ proj, int stride, int q_off, int k_off, int v_off, int i_off, int f_off,
                          const float* __restrict__ i_bias, const float* __restrict__ f_bias, float cap,
                          float* __restrict__ state, long long state_stride, const int32_t* __restrict__ qo_indptr,
                          const int32_t* __restrict__ slot_ids, float* __restrict__ o_raw, float* __restrict__ den, int H,
                          int dk, int dv, int lpc, int col_groups) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int dkp = dk + dk / 16 * 4;
  float* k_l = lds;
  float* q_l = lds + dkp;
  const int W = dv + 1;
  const int row = blockIdx.y;
  const int h = blockIdx.x / col_groups, cg = blockIdx.x % col_groups;
  const size_t t = (size_t)qo_indptr[row];
  const int j_loc = threadIdx.x / lpc, part = threadIdx.x % lpc;
  const int j_raw = cg * kMemCols + j_loc;
  const bool live = j_loc < kMemCols && j_raw < W;
  const int j = j_raw < W ? j_raw : W - 1;
  const bool norm_col = j == dv;
  const int i0 = part * R;
  float* slot = state + (long long)slot_ids[row] * state_stride;
  float* st = slot + ((size_t)h * W + j) * dk;
  float* m_at = slot + (size_t)H * W * dk + (size_t)h * W + j;
  const T* tok = proj + t * stride;
  const float m = *m_at;
  const float gi = cap * tanhf((to_f32(tok[i_off + h]) + i_bias[h]) / cap);
  const float gf = log_sigmoid_f(cap * tanhf((to_f32(tok[f_off + h]) + f_bias[h]) / cap));
  const float m_new = fmaxf(gf + m, gi);
  const float keep = expf(gf + m - m_new), take = expf(gi - m_new), floor = expf(-m_new);
  const float q_scale = 1.0f / sqrtf((float)dk);
  for (int d = threadIdx.x; d < 2 * dk; d += blockDim.x) {
    const int dd = d < dk ? d : d - dk;
    (d < dk ? k_l : q_l)[dd + dd / 16 * 4] = to_f32(tok[d < dk ? k_off + h * dk + dd : q_off + h * dk + dd]) * (d < dk ? take : q_scale);
  }
  float S[R];
  if (VEC) {
#pragma unroll
    for (int r = 0; r < R; r += 4) {
      const float4 s4 = i0 + r < dk ? *reinterpret_cast<const float4*>(st + i0 + r) : float4{0.f, 0.f, 0.f, 0.f};
      S[r] = s4.x; S[r + 1] = s4.y; S[r + 2] = s4.z; S[r + 3] = s4.w;
    }
  } else {
#pragma unroll
    for (int r = 0; r < R; ++r) S[r] = i0 + r < dk ? st[i0 + r] : 0.f;
  }
  const float v = norm_col ? 1.0f : to_f32(tok[v_off + h * dv + j]);
  __syncthreads();
  float sq[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = i0 + r;
    const bool in = i < dk;
    const float kk = in ? k_l[i + i / 16 * 4] : 0.f;
    const float qq = in ? q_l[i + i / 16 * 4] : 0.f;
    S[r] = fmaf(kk, v, keep * S[r]);
    sq[r % 4] = fmaf(S[r], qq, sq[r % 4]);
  }
  const float sq_all = row_group_sum((sq[0] + sq[1]) + (sq[2] + sq[3]), lpc);
  if (live && part == 0) {
    if (norm_col) den[t * H + h] = fmaxf(fabsf(sq_all), floor) + 1e-6f;
    else o_raw[(t * H + h) * dv + j] = sq_all;
  }
  if (live) {
    if (VEC) {
#pragma unroll
      for (int r = 0; r < R; r += 4)
        if (i0 + r < dk) *reinterpret_cast<float4*>(st + i0 + r) = float4{S[r], S[r + 1], S[r + 2], S[r + 3]};
    } else {
#pragma unroll
      for (int r = 0; r < R; ++r)
        if (i0 + r < dk) st[i0 + r] = S[r];
    }
    if (part == 0) *m_at = m_new;
  }
}
}  // namespace

// proj [n_tokens, stride]: the columns of q (H * dk from q_off), k, v (H * dv) and of the two gates' pre-activations
// (H each) of one matrix.  state: per slot H * (dv + 1) * dk + H * (dv + 1) floats.  gate [n_tokens, gate_stride]:
// the output gate's H * dv columns from gate_off.  norm_w: H * dv floats.  o_raw, den: workspaces of n_tokens * H * dv
// and n_tokens * H floats.  out [n_tokens, H * dv] = T(o / rms(o) * norm_w * sigmoid(gate)).
TL_EXPORT int tl_matrix_memory(const void* proj, int stride, int q_off, int k_off, int v_off, int i_off, int f_off,
                               const float* i_bias, const float* f_bias, float cap, const void* gate, int gate_stride,
                               int gate_off, const float* norm_w, float eps, float* state, long long state_stride,
                               const int32_t* qo_indptr, const int32_t* slot_ids, void* out, int n_tokens, int n_seqs, int H,
                               int dk, int dv, float* o_raw, float* den, int dtype, hipStream_t stream) {
  TL_REQUIRE(n_seqs >= 0 && n_tokens >= 0 && H > 0 && dk > 0 && dv > 0 && cap > 0.f, "matrix_memory: bad sizes");
  if (dk > 256) return tl_fail(TL_ERR_UNSUPPORTED, "matrix_memory: keys of %d channels, at most 256", dk);
  TL_REQUIRE(n_seqs <= 65535 && n_tokens <= 0x7fffffff / 4, "matrix_memory: too many requests or tokens a step");
  TL_REQUIRE(o_raw != nullptr && den != nullptr && gate != nullptr, "matrix_memory: no workspace or no gate");
  if (n_seqs == 0 || n_tokens == 0) return TL_OK;
  if (dtype != TL_F32 && dtype != TL_BF16) return tl_fail(TL_ERR_ARG, "matrix_memory: unknown dtype %d", dtype);
  const int rows = dk <= 128 ? 8 : 16;
  int lpc = 1;
  while (rows * lpc < dk) lpc *= 2;
  const int threads = (kMemCols * lpc + kWave - 1) / kWave * kWave;
  const int col_groups = (dv + 1 + kMemCols - 1) / kMemCols;
  const int dkp = dk + dk / 16 * 4;
  const size_t lds = ((size_t)kDeltaTile * (2 * dkp + 2 * kMemCols + 4) + 4) * sizeof(float);
  const dim3 grid(H * col_groups, n_seqs);
  const bool vec = dk % 4 == 0 && ((uintptr_t)state % 16) == 0 && state_stride % 4 == 0;
  const bool single = n_tokens == n_seqs;
  const size_t step_lds = 2 * (size_t)dkp * sizeof(float);
#define TL_MEM(T, VEC, R)                                                                                               \
  do {                                                                                                                  \
    if (single)                                                                                                         \
      matrix_memory_step_kernel<T, VEC, R><<<grid, threads, step_lds, stream>>>(                                        \
          (const T*)proj, stride, q_off, k_off, v_off, i_off, f_off, i_bias, f_bias, cap, state, state_stride, qo_indptr, \
          slot_ids, o_raw, den, H, dk, dv, lpc, col_groups);                                                            \
    else                                                                                                                \
      matrix_memory_kernel<T, VEC, R><<<grid, threads, lds, stream>>>(                                                  \
          (const T*)proj, stride, q_off, k_off, v_off, i_off, f_off, i_bias, f_bias, cap, state, state_stride, qo_indptr, \
          slot_ids, o_raw, den, H, dk, dv, lpc, col_groups);                                                            \
  } while (0)
#define TL_MEM_T(T)                                  \
  do {                                               \
    if (vec && rows == 8) TL_MEM(T, true, 8);        \
    else if (vec) TL_MEM(T, true, 16);               \
    else if (rows == 8) TL_MEM(T, false, 8);         \
    else TL_MEM(T, false, 16);                       \
  } while (0)
  if (dtype == TL_F32) TL_MEM_T(float);
  else TL_MEM_T(bf16_t);
#undef TL_MEM_T
#undef TL_MEM
  int rc = tl_check_launch("matrix_memory");
  if (rc != TL_OK) return rc;
  if (dtype == TL_F32)
    return launch_head_output<float>(o_raw, (const float*)gate, gate_stride, gate_off, norm_w, dv, eps, (float*)out, n_tokens, H, dv,
                                     true, stream, den);
  return launch_head_output<bf16_t>(o_raw, (const bf16_t*)gate, gate_stride, gate_off, norm_w, dv, eps, (bf16_t*)out, n_tokens, H, dv,
                                    true, stream, den);
}
