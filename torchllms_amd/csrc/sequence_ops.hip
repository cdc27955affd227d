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
template <typename T>
__global__ void gelu_mul_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int n, int inter) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= inter) return;
  for (int r = blockIdx.y; r < n; r += gridDim.y) {
    const T* gp = gate_up + (size_t)r * 2 * inter + c;
    out[(size_t)r * inter + c] = from_f32<T>(gelu_tanh_f(to_f32(gp[0])) * to_f32(gp[inter]));
  }
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

template <typename T>
__global__ void __launch_bounds__(kHeadWaves* kWave)
rope_norm_kv_write_kernel(T* qkv, int row, int n_q, int n_kv, int dk, int dv, const float2* __restrict__ cos_sin,
                          int rot, int pairing, float norm_eps, T* __restrict__ k_pages, T* __restrict__ v_pages,
                          const int32_t* __restrict__ slot_mapping, int page_size) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int unit = blockIdx.y * kHeadWaves + wave;
  if (unit >= n_q + 2 * n_kv) return;
  T* base = qkv + (size_t)t * row;
  const int slot = slot_mapping ? slot_mapping[t] : -1;
  const bool store = k_pages != nullptr && slot >= 0;
  const size_t page = store ? slot / page_size : 0;
  const int off = store ? slot % page_size : 0;
  if (unit >= n_q + n_kv) {  // a value head: copied
    if (!store || v_pages == nullptr) return;
    const int kh = unit - n_q - n_kv;
    const T* src = base + (size_t)(n_q + n_kv) * dk + (size_t)kh * dv;
    T* dst = v_pages + ((page * n_kv + kh) * page_size + off) * dv;
    for (int d = lane; d < dv; d += kWave) dst[d] = src[d];
    return;
  }
  T* head = base + (size_t)unit * dk;
  const int rh = rot / 2;
  float val[kHeadChan];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < kHeadChan; ++c) {
    const int d = lane + c * kWave;
    val[c] = 0.f;
    if (d < dk) {
      const float a = to_f32(head[d]);
      float v = a;
      if (d < rot) {
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
      val[c] = v;
      ss += v * v;
    }
  }
  ss = wave_sum(ss);  // (every load of the head lies before this exchange, every store behind it)
  const float inv = norm_eps > 0.f ? 1.0f / sqrtf(ss / (float)dk + norm_eps) : 1.0f;
  const bool is_q = unit < n_q;
  T* dst = head;
  if (!is_q && store) dst = k_pages + ((page * n_kv + (unit - n_q)) * page_size + off) * dk;
  if (!is_q && k_pages != nullptr && !store) return;  // a token without a slot keeps nothing
#pragma unroll
  for (int c = 0; c < kHeadChan; ++c) {
    const int d = lane + c * kWave;
    if (d < dk) dst[d] = from_f32<T>(val[c] * inv);
  }
}

// ----------------------------------------------------------------------------- short causal convolution
// x: element (t, c) at x + t * x_stride + c, c < C (a slice of a projection's output).  Tokens of a
// request are consecutive (qo_indptr); the request's K - 1 inputs before them are its history, 32-bit,
// hist[k][c] at state + slot * state_stride + k * C + c, oldest first, zero for a new request.
//   out[t, c] = act(bias[c] + sum_j taps[c][j] * in(t - (K - 1 - j))),  j ascending, 32-bit
// act 0: none, 1: silu.  The history is brought up to date by a second kernel, after every token has read it.
template <typename T>
__global__ void __launch_bounds__(256)
causal_conv_kernel(const T* __restrict__ x, int x_stride, const float* __restrict__ taps, const float* __restrict__ bias,
                   const float* __restrict__ state, long long state_stride, const int32_t* __restrict__ token_seq,
                   const int32_t* __restrict__ qo_indptr, const int32_t* __restrict__ slot_ids, T* __restrict__ out,
                   int out_stride, int C, int K, int act, int t0) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int t = t0 + blockIdx.y;
  const int row = token_seq[t];
  const int start = qo_indptr[row];
  const int i = t - start;
  const float* hist = state + (long long)slot_ids[row] * state_stride;
  float acc = bias ? bias[c] : 0.f;
  for (int j = 0; j < K; ++j) {
    const int src = i - (K - 1 - j);
    const float v = src >= 0 ? to_f32(x[(size_t)(start + src) * x_stride + c]) : hist[(size_t)(K - 1 + src) * C + c];
    acc = fmaf(taps[(size_t)c * K + j], v, acc);
  }
  out[(size_t)t * out_stride + c] = from_f32<T>(act == 1 ? silu_f(acc) : acc);
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

template <typename T, typename DT, int NB>
__global__ void __launch_bounds__(kScanThreads)
selective_scan_kernel(const T* __restrict__ x, const DT* __restrict__ dt_pre, const T* __restrict__ bc, int bc_stride,
                      int b_off, int c_off, const T* __restrict__ z, int z_stride, const float* __restrict__ dt_bias,
                      const float* __restrict__ A, const float* __restrict__ D, float* __restrict__ state,
                      long long state_stride, const int32_t* __restrict__ qo_indptr, const int32_t* __restrict__ slot_ids,
                      T* __restrict__ out, int inner, int N, int lpc) {
  extern __shared__ float bc_lds[];  // [kScanTile][2 * N]
  const int row = blockIdx.y;
  const int start = qo_indptr[row], end = qo_indptr[row + 1];
  const int per_block = kScanThreads / lpc;
  const int c_raw = blockIdx.x * per_block + threadIdx.x / lpc;
  const int part = threadIdx.x % lpc;
  const bool live = c_raw < inner;
  const int c = live ? c_raw : inner - 1;
  const int n0 = part * NB;
  float* st = state + (long long)slot_ids[row] * state_stride + (size_t)c * N;
  float s[NB], a[NB];
#pragma unroll
  for (int n = 0; n < NB; ++n) {
    const bool in = n0 + n < N;
    s[n] = in ? st[n0 + n] : 0.f;
    a[n] = in ? A[(size_t)c * N + n0 + n] : 0.f;
  }
  const float bias = dt_bias[c], dd = D[c];
  for (int t0 = start; t0 < end; t0 += kScanTile) {
    const int nt = min(kScanTile, end - t0);
    __syncthreads();  // everybody has finished with the tile before
    for (int idx = threadIdx.x; idx < nt * 2 * N; idx += kScanThreads) {
      const int tt = idx / (2 * N), e = idx % (2 * N);
      const T* src = bc + (size_t)(t0 + tt) * bc_stride;
      bc_lds[idx] = to_f32(e < N ? src[b_off + e] : src[c_off + e - N]);
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const size_t t = (size_t)(t0 + tt);
      const float xv = to_f32(x[t * inner + c]);
      const float dt = softplus_f(to_f32(dt_pre[t * inner + c]) + bias);
      const float zv = to_f32(z[t * z_stride + c]);
      const float dx = dt * xv;
      const float* Bt = bc_lds + tt * 2 * N + n0;
      const float* Ct = Bt + N;
      float y = 0.f;
#pragma unroll
      for (int n = 0; n < NB; ++n) {
        if (n0 + n < N) {
          s[n] = fmaf(expf(dt * a[n]), s[n], dx * Bt[n]);
          y = fmaf(s[n], Ct[n], y);
        }
      }
      y = group_sum(y, lpc);
      y = fmaf(dd, xv, y);
      if (live && part == 0) out[t * inner + c] = from_f32<T>(y * silu_f(zv));
    }
  }
  if (live) {
#pragma unroll
    for (int n = 0; n < NB; ++n)
      if (n0 + n < N) st[n0 + n] = s[n];
  }
}

// ----------------------------------------------------------------------------- gated delta rule
// Per request and head h (key/query head g = h / (H / G)), state S [dk][dv] in 32-bit, kept transposed in
// state[slot][h][j][i] (column j of S is contiguous).  For every token, in order:
//   k^ = k / sqrt(sum k^2 + 1e-6);  q^ = q / sqrt(sum q^2 + 1e-6) * dk^-1/2
//   beta = sigmoid(b);  decay = exp(-exp(A_log[h]) * softplus(a + dt_bias[h]))
//   S <- decay * S;  u = beta * (v - S^T k^);  S <- S + k^ u^T;  o = S^T q^
//   out[t, h, :] = T(o / sqrt(mean(o^2) + eps) * norm_w * silu(gate[t, h, :]))
// qkv: the convolved and activated q | k | v channels, [n_tokens, qkv_stride]; proj: the layer's input
// projection, of which gate (H * dv columns from gate_off), b and a (H columns each) are read.
// A block is one (request, head); lpc neighbouring lanes share column j, each holding RB rows of it.
constexpr int kDeltaTile = 8;

template <typename T, int RB>
__global__ void __launch_bounds__(1024)
gated_delta_kernel(const T* __restrict__ qkv, int qkv_stride, const T* __restrict__ proj, int proj_stride, int gate_off,
                   int b_off, int a_off, const float* __restrict__ A_log, const float* __restrict__ dt_bias,
                   const float* __restrict__ norm_w, float eps, float* __restrict__ state, long long state_stride,
                   const int32_t* __restrict__ qo_indptr, const int32_t* __restrict__ slot_ids, T* __restrict__ out,
                   int H, int G, int dk, int dv, int lpc) {
  extern __shared__ float lds[];
  // per token of the tile: k^ [dk], q^ [dk], v [dv], o [dv], then beta and decay
  float* k_l = lds;
  float* q_l = k_l + kDeltaTile * dk;
  float* v_l = q_l + kDeltaTile * dk;
  float* o_l = v_l + kDeltaTile * dv;
  float* bd_l = o_l + kDeltaTile * dv;  // [kDeltaTile][2]
  const int row = blockIdx.y, h = blockIdx.x;
  const int g = h / (H / G);
  const int start = qo_indptr[row], end = qo_indptr[row + 1];
  const int n_threads = blockDim.x, n_waves = n_threads / kWave;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int j_raw = threadIdx.x / lpc, part = threadIdx.x % lpc;
  const bool live = j_raw < dv;
  const int j = live ? j_raw : dv - 1;
  const int i0 = part * RB;
  float* st = state + (long long)slot_ids[row] * state_stride + ((size_t)h * dv + j) * dk;
  float S[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) S[r] = i0 + r < dk ? st[i0 + r] : 0.f;
  const float neg_rate = -expf(A_log[h]), bias = dt_bias[h];
  const float q_scale = 1.0f / sqrtf((float)dk);
  const int q_col = g * dk, k_col = G * dk + g * dk, v_col = 2 * G * dk + h * dv;
  for (int t0 = start; t0 < end; t0 += kDeltaTile) {
    const int nt = min(kDeltaTile, end - t0);
    __syncthreads();  // the tile before has been written out
    // unit keys and queries: one wave per (token, which)
    for (int item = wave; item < 2 * nt; item += n_waves) {
      const int tt = item / 2, which = item % 2;  // 0: k, 1: q
      const T* src = qkv + (size_t)(t0 + tt) * qkv_stride + (which ? q_col : k_col);
      float ss = 0.f;
      for (int d = lane; d < dk; d += kWave) {
        const float v = to_f32(src[d]);
        ss += v * v;
      }
      ss = wave_sum(ss);
      const float inv = (which ? q_scale : 1.0f) / sqrtf(ss + 1e-6f);
      float* dst = (which ? q_l : k_l) + tt * dk;
      for (int d = lane; d < dk; d += kWave) dst[d] = to_f32(src[d]) * inv;
    }
    for (int idx = threadIdx.x; idx < nt * dv; idx += n_threads) {
      const int tt = idx / dv, d = idx % dv;
      v_l[idx] = to_f32(qkv[(size_t)(t0 + tt) * qkv_stride + v_col + d]);
    }
    if (threadIdx.x < nt) {
      const T* pr = proj + (size_t)(t0 + threadIdx.x) * proj_stride;
      bd_l[2 * threadIdx.x] = sigmoid_f(to_f32(pr[b_off + h]));
      bd_l[2 * threadIdx.x + 1] = expf(neg_rate * softplus_f(to_f32(pr[a_off + h]) + bias));
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float beta = bd_l[2 * tt], decay = bd_l[2 * tt + 1];
      const float* kt = k_l + tt * dk + i0;
      const float* qt = q_l + tt * dk + i0;
      float kv = 0.f;
#pragma unroll
      for (int r = 0; r < RB; ++r) {
        if (i0 + r < dk) {
          S[r] = decay * S[r];
          kv = fmaf(S[r], kt[r], kv);
        }
      }
      kv = group_sum(kv, lpc);
      const float u = beta * (v_l[tt * dv + j] - kv);
      float o = 0.f;
#pragma unroll
      for (int r = 0; r < RB; ++r) {
        if (i0 + r < dk) {
          S[r] = fmaf(kt[r], u, S[r]);
          o = fmaf(S[r], qt[r], o);
        }
      }
      o = group_sum(o, lpc);
      if (live && part == 0) o_l[tt * dv + j] = o;
    }
    __syncthreads();
    // per-head RMS norm of the outputs, the norm's weight and the gate: one wave per token
    for (int tt = wave; tt < nt; tt += n_waves) {
      float ss = 0.f;
      for (int d = lane; d < dv; d += kWave) ss += o_l[tt * dv + d] * o_l[tt * dv + d];
      ss = wave_sum(ss);
      const float inv = 1.0f / sqrtf(ss / (float)dv + eps);
      const T* gp = proj + (size_t)(t0 + tt) * proj_stride + gate_off + (size_t)h * dv;
      T* op = out + ((size_t)(t0 + tt) * H + h) * dv;
      for (int d = lane; d < dv; d += kWave)
        op[d] = from_f32<T>(o_l[tt * dv + d] * inv * norm_w[d] * silu_f(to_f32(gp[d])));
    }
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < RB; ++r)
      if (i0 + r < dk) st[i0 + r] = S[r];
  }
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
  const dim3 grid((inter + 255) / 256, n < 65535 ? n : 65535);
  if (dtype == TL_F32)
    gelu_mul_kernel<float><<<grid, 256, 0, stream>>>((const float*)gate_up, (float*)out, n, inter);
  else if (dtype == TL_BF16)
    gelu_mul_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)gate_up, (bf16_t*)out, n, inter);
  else
    return tl_fail(TL_ERR_ARG, "gelu_mul: unknown dtype %d", dtype);
  return tl_check_launch("gelu_mul");
}

TL_EXPORT int tl_rope_norm_kv_write(void* qkv, int n_tokens, int n_q, int n_kv, int dk, int dv, const float* cos_sin, int rot,
                                    int pairing, float norm_eps, void* k_pages, void* v_pages, const int32_t* slot_mapping,
                                    int page_size, int dtype, hipStream_t stream) {
  TL_REQUIRE(n_tokens >= 0 && n_q > 0 && n_kv >= 0 && dk > 0 && dv > 0, "rope_norm: bad sizes");
  TL_REQUIRE(dk <= kHeadChan * kWave, "rope_norm: heads of %d channels, at most %d", dk, kHeadChan * kWave);
  TL_REQUIRE(rot >= 0 && rot <= dk && rot % 2 == 0, "rope_norm: %d rotated channels of %d (even, at most the head)", rot, dk);
  TL_REQUIRE(pairing == 0 || pairing == 1, "rope_norm: pairing must be 0 (interleaved) or 1 (half split)");
  TL_REQUIRE(rot == 0 || cos_sin != nullptr, "rope_norm: rotation without a table of cosines and sines");
  TL_REQUIRE(k_pages == nullptr || (v_pages != nullptr && slot_mapping != nullptr && page_size > 0), "rope_norm: pages without slots");
  if (n_tokens == 0) return TL_OK;
  const int row = (n_q + n_kv) * dk + n_kv * dv;
  const dim3 grid(n_tokens, (n_q + 2 * n_kv + kHeadWaves - 1) / kHeadWaves);
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
  for (int t0 = 0; t0 < n_tokens; t0 += 65535) {
    const int nt = n_tokens - t0 < 65535 ? n_tokens - t0 : 65535;
    const dim3 grid(cblocks, nt);
    if (dtype == TL_F32)
      causal_conv_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, x_stride, taps, bias, state, state_stride,
                                                          token_seq, qo_indptr, slot_ids, (float*)out, out_stride, C, K,
                                                          act, t0);
    else
      causal_conv_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, x_stride, taps, bias, state, state_stride,
                                                           token_seq, qo_indptr, slot_ids, (bf16_t*)out, out_stride, C, K,
                                                           act, t0);
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
                const int32_t* qo_indptr, const int32_t* slot_ids, void* out, int n_seqs, int inner, int N, hipStream_t stream) {
  // states a lane holds and lanes a channel: up to 32 states one lane, then 2, 4, 8 lanes of 32
  int nb = N <= 8 ? 8 : N <= 16 ? 16 : 32;
  int lpc = 1;
  while (nb * lpc < N) lpc *= 2;
  const int per_block = kScanThreads / lpc;
  const dim3 grid((inner + per_block - 1) / per_block, n_seqs);
  const size_t lds = (size_t)kScanTile * 2 * N * sizeof(float);
#define TL_SCAN(NB)                                                                                                     \
  selective_scan_kernel<T, DT, NB><<<grid, kScanThreads, lds, stream>>>(                                                \
      (const T*)x, (const DT*)dt_pre, (const T*)bc, bc_stride, b_off, c_off, (const T*)z, z_stride, dt_bias, A, D, state, \
      state_stride, qo_indptr, slot_ids, (T*)out, inner, N, lpc)
  if (nb == 8) TL_SCAN(8);
  else if (nb == 16) TL_SCAN(16);
  else TL_SCAN(32);
#undef TL_SCAN
  return tl_check_launch("selective_scan");
}
}  // namespace

// x, out: [n_tokens, inner] of dtype; dt_pre: [n_tokens, inner] of dt_dtype (32-bit, or dtype); bc and z: see the
// kernel; state: the requests' rows, S[c][n] at state + slot * state_stride + c * N + n.
TL_EXPORT int tl_selective_scan(const void* x, const void* dt_pre, int dt_dtype, const void* bc, int bc_stride, int b_off,
                                int c_off, const void* z, int z_stride, const float* dt_bias, const float* A, const float* D,
                                float* state, long long state_stride, const int32_t* qo_indptr, const int32_t* slot_ids,
                                void* out, int n_seqs, int inner, int N, int dtype, hipStream_t stream) {
  TL_REQUIRE(n_seqs >= 0 && inner > 0 && N > 0, "selective_scan: bad sizes");
  TL_REQUIRE(N <= 256, "selective_scan: %d states a channel, at most 256", N);
  TL_REQUIRE(n_seqs <= 65535, "selective_scan: at most 65535 requests a step");
  if (n_seqs == 0) return TL_OK;
  if (dtype == TL_F32 && dt_dtype == TL_F32)
    return scan_launch<float, float>(x, dt_pre, bc, bc_stride, b_off, c_off, z, z_stride, dt_bias, A, D, state, state_stride,
                                     qo_indptr, slot_ids, out, n_seqs, inner, N, stream);
  if (dtype == TL_BF16 && dt_dtype == TL_F32)
    return scan_launch<bf16_t, float>(x, dt_pre, bc, bc_stride, b_off, c_off, z, z_stride, dt_bias, A, D, state, state_stride,
                                      qo_indptr, slot_ids, out, n_seqs, inner, N, stream);
  if (dtype == TL_BF16 && dt_dtype == TL_BF16)
    return scan_launch<bf16_t, bf16_t>(x, dt_pre, bc, bc_stride, b_off, c_off, z, z_stride, dt_bias, A, D, state, state_stride,
                                       qo_indptr, slot_ids, out, n_seqs, inner, N, stream);
  return tl_fail(TL_ERR_ARG, "selective_scan: dtype %d with step sizes of dtype %d", dtype, dt_dtype);
}

// qkv, proj, out as the kernel describes; state: S^T of head h at state + slot * state_stride + h * dv * dk.
TL_EXPORT int tl_gated_delta(const void* qkv, int qkv_stride, const void* proj, int proj_stride, int gate_off, int b_off,
                             int a_off, const float* A_log, const float* dt_bias, const float* norm_w, float eps, float* state,
                             long long state_stride, const int32_t* qo_indptr, const int32_t* slot_ids, void* out, int n_seqs,
                             int H, int G, int dk, int dv, int dtype, hipStream_t stream) {
  TL_REQUIRE(n_seqs >= 0 && H > 0 && G > 0 && dk > 0 && dv > 0, "gated_delta: bad sizes");
  TL_REQUIRE(H % G == 0, "gated_delta: %d heads are not a multiple of %d key heads", H, G);
  TL_REQUIRE(dk <= 1024 && dv <= 1024, "gated_delta: head sizes %d and %d, at most 1024", dk, dv);
  TL_REQUIRE(n_seqs <= 65535, "gated_delta: at most 65535 requests a step");
  if (n_seqs == 0) return TL_OK;
  // rows of a column that a lane holds (16, 32 or 64) and lanes a column, so that a block has at most 1024 threads
  int rb = 16, lpc = 1;
  for (;;) {
    lpc = 1;
    while (rb * lpc < dk) lpc *= 2;
    if (lpc <= kWave && (size_t)dv * lpc <= 1024) break;
    if (rb == 64) return tl_fail(TL_ERR_UNSUPPORTED, "gated_delta: heads of %d by %d do not fit a block", dk, dv);
    rb *= 2;
  }
  int threads = (dv * lpc + kWave - 1) / kWave * kWave;
  const size_t lds = ((size_t)kDeltaTile * (2 * dk + 2 * dv + 2)) * sizeof(float);
  if (lds + 1024 > (size_t)tl_device_facts().lds_bytes)
    return tl_fail(TL_ERR_UNSUPPORTED, "gated_delta: heads of %d by %d do not fit the LDS", dk, dv);
  const dim3 grid(H, n_seqs);
#define TL_DELTA(T, RB)                                                                                                  \
  do {                                                                                                                   \
    if (lds > 48 * 1024) {                                                                                               \
      hipError_t e = hipFuncSetAttribute((const void*)gated_delta_kernel<T, RB>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
      if (e != hipSuccess) return tl_fail(TL_ERR_HIP, "gated_delta: %s", hipGetErrorString(e));                          \
    }                                                                                                                    \
    gated_delta_kernel<T, RB><<<grid, threads, lds, stream>>>((const T*)qkv, qkv_stride, (const T*)proj, proj_stride, gate_off, \
                                                              b_off, a_off, A_log, dt_bias, norm_w, eps, state, state_stride, \
                                                              qo_indptr, slot_ids, (T*)out, H, G, dk, dv, lpc);          \
  } while (0)
#define TL_DELTA_RB(T)              \
  do {                              \
    if (rb == 16) TL_DELTA(T, 16);  \
    else if (rb == 32) TL_DELTA(T, 32); \
    else TL_DELTA(T, 64);           \
  } while (0)
  if (dtype == TL_F32) TL_DELTA_RB(float);
  else if (dtype == TL_BF16) TL_DELTA_RB(bf16_t);
  else return tl_fail(TL_ERR_ARG, "gated_delta: unknown dtype %d", dtype);
#undef TL_DELTA_RB
#undef TL_DELTA
  return tl_check_launch("gated_delta");
}
