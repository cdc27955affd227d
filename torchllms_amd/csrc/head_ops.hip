// Kernels of layers whose branches are normed on their way into a 32-bit residual stream, and of attention
// layers that prepare their heads before the scores: a weighted RMS norm per query and key head, rotation of
// a part of the head, a query factor that grows with the logarithm of the position, values mixed with those
// of an earlier layer, gates on the heads' outputs, queries and outputs of attention through a latent, and a
// cap on the logits.  Statistics, factors, gates and the stream are 32-bit; every result is rounded once.
#include "common.h"

namespace {

__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }

// ----------------------------------------------------------------------------- heads before the scores
// rows: [n_tokens, row_stride], a row = Hq query heads of dk | Hkv key heads of dk | Hkv value heads of dv |
// whatever follows (left alone).  One wave a head:
//   every head first takes its bias (bias given: one entry per column of the heads, q | k | v);
//   query and key heads: the first norm_dims channels become x / sqrt(mean(x^2) + eps) * w (w given; q_w for
//     queries, k_w for keys), the channels rot_off .. rot_off + rot - 1 are rotated by the step's table of
//     cosines and sines (pairing 0: (2i, 2i+1); 1: (i, i + rot/2)), queries are multiplied by
//     1 + temp_coef * ln(floor((p + 1) / temp_every) + 1) at position p (temp_coef 0: not);
//   value heads: v <- (1 - lam) v + lam v_first (v_first given), written back in place.
// Queries go back in place; keys and values go to their pages [page][Hkv][P][dk] and [..][dv] at
// slot_mapping[t] (keys in place too when there are no pages).
constexpr int kPrepWaves = 4;
constexpr int kPrepMaxChan = 16;  // channels a lane holds at most: heads of up to 1,024

template <typename T>
struct PrepArgs {
  T* rows;
  int row_stride, n_q, n_kv, dk, dv;
  const T* bias;
  const float* q_w;
  const float* k_w;
  int norm_dims;
  float eps;
  const float2* cos_sin;
  int rot_off, rot, pairing;
  const int32_t* positions;
  float temp_coef;
  int temp_every;
  const T* v_first;
  int v_first_stride;
  const float* lam;
  T* k_pages;
  T* v_pages;
  const int32_t* slot_mapping;
  int page_size;
};

// kPrepChan: channels a lane holds (the widest head of the launch over 64, rounded up to a power of two).  kPrepTok:
// consecutive tokens a wave takes for its head, all their loads asked for before anything is computed: a wave has
// a few hundred bytes of one (token, head) to fetch, and with one token a wave the bytes in flight on the whole GPU
// are what bounds the kernel.
template <typename T, int kPrepChan, int kPrepTok>
__global__ void __launch_bounds__(kPrepWaves* kWave) head_prepare_kernel(const PrepArgs<T> a, int n_tokens) {
#pragma clang fp contract(off)  // the same operations in every instantiation: a head's result does not depend on the launch's form
  __shared__ float turned[kPrepWaves][kPrepChan * kWave];
  const int t0 = blockIdx.x * kPrepTok;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int unit = blockIdx.y * kPrepWaves + wave;
  const int n_units = a.n_q + a.n_kv + (a.dv > 0 ? a.n_kv : 0);
  const bool live = unit < n_units;
  const bool is_q = live && unit < a.n_q;
  const bool is_k = live && !is_q && unit < a.n_q + a.n_kv;
  const bool is_v = live && !is_q && !is_k;
  const int width = is_v ? a.dv : a.dk;
  const int g = unit - a.n_q - a.n_kv;  // the kv head of a value unit
  // where the unit's head starts in a row (an idle wave shadows the first head and stores nothing)
  const size_t head_at = is_v ? (size_t)(a.n_q + a.n_kv) * a.dk + (size_t)g * a.dv : (size_t)(live ? unit : 0) * a.dk;
  const float* w = is_q ? a.q_w : (is_k ? a.k_w : nullptr);
  const bool mixes = is_v && a.v_first != nullptr;
  // every load is made whatever the head's width (a channel past the end is the head's first once more, and not
  // used), and nothing looks at a loaded value before all are asked for: a select right behind a load makes the
  // wave wait for each load in turn
  T raw[kPrepTok][kPrepChan], first[kPrepTok][kPrepChan], raw_bias[kPrepChan];
  float wv[kPrepChan];
  int slot[kPrepTok], pos[kPrepTok];
#pragma unroll
  for (int j = 0; j < kPrepTok; ++j) {
    const int t = t0 + j < n_tokens ? t0 + j : n_tokens - 1;  // (tokens past the end: the last once more, not stored)
    const T* head = a.rows + (size_t)t * a.row_stride + head_at;
    slot[j] = a.slot_mapping ? a.slot_mapping[t] : -1;
    pos[j] = a.temp_coef != 0.f ? a.positions[t] : 0;
#pragma unroll
    for (int c = 0; c < kPrepChan; ++c) {
      const int d = lane + c * kWave;
      raw[j][c] = head[d < width ? d : 0];
      if (mixes) first[j][c] = a.v_first[(size_t)t * a.v_first_stride + (size_t)g * a.dv + (d < width ? d : 0)];  // (uniform)
    }
  }
#pragma unroll
  for (int c = 0; c < kPrepChan; ++c) {
    const int d = lane + c * kWave;
    if (a.bias) raw_bias[c] = a.bias[head_at + (d < width ? d : 0)];  // (uniform)
    if (w) wv[c] = w[d < a.norm_dims ? d : 0];                        // (uniform)
  }
#pragma unroll
  for (int j = 0; j < kPrepTok; ++j) {
    const int t = t0 + j;
    const bool there = live && t < n_tokens;
    T* head = a.rows + (size_t)(t < n_tokens ? t : n_tokens - 1) * a.row_stride + head_at;
    float val[kPrepChan];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < kPrepChan; ++c) {
      const int d = lane + c * kWave;
      val[c] = (live && d < width) ? to_f32(raw[j][c]) : 0.f;
      // (the sum is rounded to the rows' type, as a projection with a bias would have stored it)
      if (a.bias && live && d < width) val[c] = to_f32(from_f32<T>(val[c] + to_f32(raw_bias[c])));
      if (d < a.norm_dims) ss += val[c] * val[c];
    }
    if (w != nullptr) {  // (uniform per wave)
      ss = wave_sum(ss);
      const float inv = 1.0f / sqrtf(ss / (float)a.norm_dims + a.eps);
#pragma unroll
      for (int c = 0; c < kPrepChan; ++c) {
        const int d = lane + c * kWave;
        if (d < a.norm_dims) val[c] = val[c] * inv * wv[c];
      }
    }
    // rotation: every lane needs its partner's channel as it is after the norm
    if (a.rot > 0) {  // (uniform over the block)
      if (j > 0) __syncthreads();  // everybody has read the token before
#pragma unroll
      for (int c = 0; c < kPrepChan; ++c) turned[wave][lane + c * kWave] = val[c];
      __syncthreads();
      if (is_q || is_k) {
        const int rh = a.rot / 2;
        const size_t row = (size_t)(t < n_tokens ? t : n_tokens - 1) * rh;
#pragma unroll
        for (int c = 0; c < kPrepChan; ++c) {
          const int d = lane + c * kWave;
          const int r = d - a.rot_off;
          if (d < width && r >= 0 && r < a.rot) {
            int i, partner;
            bool one;
            if (a.pairing == 0) {
              i = r / 2; one = (r % 2) == 0; partner = one ? d + 1 : d - 1;
            } else {
              one = r < rh; i = one ? r : r - rh; partner = one ? d + rh : d - rh;
            }
            const float o = turned[wave][partner];
            const float2 cs = a.cos_sin[row + i];
            val[c] = one ? val[c] * cs.x - o * cs.y : val[c] * cs.x + o * cs.y;
          }
        }
      }
    }
    if (!there) continue;
    const bool store = a.k_pages != nullptr && slot[j] >= 0;
    const size_t page = store ? slot[j] / a.page_size : 0;
    const int off = store ? slot[j] % a.page_size : 0;
    if (is_q) {
      float f = 1.0f;
      if (a.temp_coef != 0.f) f = 1.0f + a.temp_coef * logf((float)((pos[j] + 1) / a.temp_every + 1));
#pragma unroll
      for (int c = 0; c < kPrepChan; ++c) {
        const int d = lane + c * kWave;
        if (d < width) head[d] = from_f32<T>(val[c] * f);
      }
      continue;
    }
    if (is_k) {
      if (a.k_pages != nullptr && !store) continue;  // a token without a slot keeps nothing
      T* dst = store ? a.k_pages + ((page * a.n_kv + (unit - a.n_q)) * a.page_size + off) * a.dk : head;
#pragma unroll
      for (int c = 0; c < kPrepChan; ++c) {
        const int d = lane + c * kWave;
        if (d < width) dst[d] = from_f32<T>(val[c]);
      }
      continue;
    }
    // a value head
    if (mixes) {
      const float lam = a.lam[0];
#pragma unroll
      for (int c = 0; c < kPrepChan; ++c) {
        const int d = lane + c * kWave;
        if (d < width) val[c] = (1.0f - lam) * val[c] + lam * to_f32(first[j][c]);
      }
    }
    if (mixes || a.bias != nullptr) {  // (what changed goes back: later layers may read these values)
#pragma unroll
      for (int c = 0; c < kPrepChan; ++c) {
        const int d = lane + c * kWave;
        if (d < width) head[d] = from_f32<T>(val[c]);
      }
    }
    if (store && a.v_pages != nullptr) {
      T* dst = a.v_pages + ((page * a.n_kv + g) * a.page_size + off) * a.dv;
#pragma unroll
      for (int c = 0; c < kPrepChan; ++c) {
        const int d = lane + c * kWave;
        if (d < width) dst[d] = from_f32<T>(val[c]);
      }
    }
  }
}

// ----------------------------------------------------------------------------- a normed branch into the stream
// stream[r, :] += y[r, :] / sqrt(mean(y[r, :]^2) + eps) * w   (32-bit), and rows[r, :] = T(stream[r, :]) for the
// next reader (rows may be null).  A block a row; the statistics in a fixed order.
constexpr int kRowThreads = 256;
constexpr int kRowHeldMost = 32;  // elements a thread holds at most in the form that reads everything at once: rows of up to 8,192

// The same for rows that the block's registers hold: the branch, the stream and the weight are all asked for before
// anything waits, so a row costs one trip to memory and not three (a step of few rows is nothing but that wait).
// The sums are those of the kernel below, in the same order.
template <typename T, int kRowHeld>
__global__ void __launch_bounds__(kRowThreads)
branch_norm_add_held_kernel(float* __restrict__ stream, const T* __restrict__ y, const float* __restrict__ w,
                            T* __restrict__ rows, int hidden, float eps) {
#pragma clang fp contract(off)  // operation for operation the kernel below: no multiply-add is fused in one and not the other
  __shared__ float scratch[kRowThreads / kWave];
  const size_t r = blockIdx.x;
  const T* yr = y + r * hidden;
  float* sr = stream + r * hidden;
  // every load is made whatever the row's width (an element past the end is the row's first once more, and not
  // used): a select right behind a load makes the wave wait for each load in turn
  T yraw[kRowHeld];
  float sv[kRowHeld], wv[kRowHeld];
#pragma unroll
  for (int c = 0; c < kRowHeld; ++c) {
    const int i = threadIdx.x + c * kRowThreads;
    const int at = i < hidden ? i : 0;
    yraw[c] = yr[at];
    sv[c] = sr[at];
    wv[c] = w[at];
  }
  float yv[kRowHeld];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < kRowHeld; ++c) {
    yv[c] = threadIdx.x + c * kRowThreads < hidden ? to_f32(yraw[c]) : 0.f;
    ss += yv[c] * yv[c];
  }
  ss = block_sum<kRowThreads / kWave>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)hidden + eps);
#pragma unroll
  for (int c = 0; c < kRowHeld; ++c) {
    const int i = threadIdx.x + c * kRowThreads;
    if (i < hidden) {
      const float h = sv[c] + yv[c] * inv * wv[c];
      sr[i] = h;
      if (rows) rows[r * hidden + i] = from_f32<T>(h);
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(kRowThreads)
branch_norm_add_kernel(float* __restrict__ stream, const T* __restrict__ y, const float* __restrict__ w,
                       T* __restrict__ rows, int hidden, float eps) {
#pragma clang fp contract(off)
  __shared__ float scratch[kRowThreads / kWave];
  const size_t r = blockIdx.x;
  const T* yr = y + r * hidden;
  float* sr = stream + r * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += kRowThreads) {
    const float v = to_f32(yr[i]);
    ss += v * v;
  }
  ss = block_sum<kRowThreads / kWave>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)hidden + eps);
  for (int i = threadIdx.x; i < hidden; i += kRowThreads) {
    const float h = sr[i] + to_f32(yr[i]) * inv * w[i];
    sr[i] = h;
    if (rows) rows[r * hidden + i] = from_f32<T>(h);
  }
}

// y[r, :] = T(x[s, :] / sqrt(mean(x[s, :]^2) + eps) * w) over `width` columns, s = rows ? rows[r] : r; x and y
// are addressed with row strides of their own, so either may be some columns of a wider matrix.
template <typename XT, typename T>
__global__ void __launch_bounds__(kRowThreads)
rmsnorm_columns_kernel(const XT* __restrict__ x, int x_stride, const int32_t* __restrict__ rows,
                       const float* __restrict__ w, T* __restrict__ y, int y_stride, int width, float eps) {
#pragma clang fp contract(off)
  __shared__ float scratch[kRowThreads / kWave];
  const size_t r = blockIdx.x;
  const size_t s = rows ? (size_t)rows[r] : r;
  const XT* xr = x + s * x_stride;
  // eight loads are asked for together, whatever the width (an element past the end is the first once more, and
  // not used); the sums keep the order of one element after the other
  constexpr int U = 8;
  float ss = 0.f;
  for (int i0 = threadIdx.x; i0 < width; i0 += U * kRowThreads) {
    XT raw[U];
#pragma unroll
    for (int u = 0; u < U; ++u) raw[u] = xr[i0 + u * kRowThreads < width ? i0 + u * kRowThreads : 0];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const float v = i0 + u * kRowThreads < width ? to_f32(raw[u]) : 0.f;
      ss += v * v;
    }
  }
  ss = block_sum<kRowThreads / kWave>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  for (int i0 = threadIdx.x; i0 < width; i0 += U * kRowThreads) {
    XT raw[U];
    float wv[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int at = i0 + u * kRowThreads < width ? i0 + u * kRowThreads : 0;
      raw[u] = xr[at];
      wv[u] = w[at];
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (i0 + u * kRowThreads < width) y[r * y_stride + i0 + u * kRowThreads] = from_f32<T>(to_f32(raw[u]) * inv * wv[u]);
  }
}

// ----------------------------------------------------------------------------- gates, packing, cap
// x[t, c] *= sigmoid(g[t, c / per]) for c < width: per = 1 gates channel by channel, per = the head size gates
// head by head.
template <typename T>
__global__ void sigmoid_gate_kernel(T* __restrict__ x, int x_stride, const T* __restrict__ g, int g_stride, int n,
                                    int width, int per) {
  const size_t total = (size_t)n * width;
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / width;
    const int c = (int)(idx % width);
    T* p = x + t * x_stride + c;
    *p = from_f32<T>(to_f32(*p) * sigmoid_f(to_f32(g[t * g_stride + c / per])));
  }
}

// The same for bfloat16 rows whose eight-element pieces are aligned: a thread takes 16 bytes of x (and of the gates,
// channel by channel; head by head the eight channels share one gate).
__global__ void sigmoid_gate_wide_kernel(bf16_t* __restrict__ x, int x_stride, const bf16_t* __restrict__ g, int g_stride,
                                         int n, int width, int per) {
  const int pieces = width / 8;
  const size_t total = (size_t)n * pieces;
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / pieces;
    const int c = (int)(idx % pieces) * 8;
    uint4* p = reinterpret_cast<uint4*>(x + t * x_stride + c);
    uint4 xv = *p;
    float gates[8];
    if (per == 1) {
      const uint4 gv = *reinterpret_cast<const uint4*>(g + t * g_stride + c);
      const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        gates[2 * e] = sigmoid_f(__uint_as_float(gw[e] << 16));
        gates[2 * e + 1] = sigmoid_f(__uint_as_float(gw[e] & 0xffff0000u));
      }
    } else {
      const float one = sigmoid_f(to_f32(g[t * g_stride + c / per]));
#pragma unroll
      for (int e = 0; e < 8; ++e) gates[e] = one;
    }
    uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const bf16_t lo = from_f32<bf16_t>(__uint_as_float(xw[e] << 16) * gates[2 * e]);
      const bf16_t hi = from_f32<bf16_t>(__uint_as_float(xw[e] & 0xffff0000u) * gates[2 * e + 1]);
      xw[e] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
    }
    *p = uint4{xw[0], xw[1], xw[2], xw[3]};
  }
}

// out[t, h, :] = a[h, t, 0 .. na) | b[t, h * b_head + b_off .. + nb): the two parts of a query against a latent.
template <typename T>
__global__ void pack_heads_kernel(const T* __restrict__ a, int na, const T* __restrict__ b, int b_stride, int b_head,
                                  int b_off, int nb, T* __restrict__ out, int n, int heads) {
  const int t = blockIdx.x, h = blockIdx.y;
  const T* ar = a + ((size_t)h * n + t) * na;
  const T* br = b + (size_t)t * b_stride + (size_t)h * b_head + b_off;
  T* o = out + ((size_t)t * heads + h) * (na + nb);
  for (int i = threadIdx.x; i < na; i += blockDim.x) o[i] = ar[i];
  for (int i = threadIdx.x; i < nb; i += blockDim.x) o[na + i] = br[i];
}

// out[t, h * d + j] = a[h, t, j] * sigmoid(g[t * g_stride + h])   (g null: no gate)
template <typename T>
__global__ void unpack_heads_gate_kernel(const T* __restrict__ a, T* __restrict__ out, const T* __restrict__ g,
                                         int g_stride, int n, int heads, int d) {
  const int t = blockIdx.x, h = blockIdx.y;
  const float f = g ? sigmoid_f(to_f32(g[(size_t)t * g_stride + h])) : 1.0f;
  const T* ar = a + ((size_t)h * n + t) * d;
  T* o = out + ((size_t)t * heads + h) * d;
  for (int i = threadIdx.x; i < d; i += blockDim.x) o[i] = from_f32<T>(to_f32(ar[i]) * f);
}

__global__ void softcap_kernel(float* __restrict__ z, size_t total, float cap) {
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x)
    z[idx] = cap * tanhf(z[idx] / cap);
}

int elementwise_blocks(size_t total) {
  const size_t want = (total + 255) / 256;
  return (int)(want < 1 ? 1 : (want > 65535 ? 65535 : want));
}

}  // namespace

TL_EXPORT int tl_head_prepare(void* rows, int row_stride, int n_tokens, int n_q, int n_kv, int dk, int dv, const void* bias,
                              const float* q_w, const float* k_w, int norm_dims, float eps, const float* cos_sin,
                              int rot_off, int rot, int pairing, const int32_t* positions, float temp_coef,
                              int temp_every, const void* v_first, int v_first_stride, const float* lam,
                              void* k_pages, void* v_pages, const int32_t* slot_mapping, int page_size, int dtype,
                              hipStream_t stream) {
  TL_REQUIRE(n_tokens >= 0 && n_q >= 0 && n_kv >= 0 && n_q + n_kv > 0 && dk > 0 && dv >= 0, "head_prepare: bad sizes");
  TL_REQUIRE(dk <= kPrepMaxChan * kWave && dv <= kPrepMaxChan * kWave, "head_prepare: heads of %d and %d channels, at most %d", dk, dv,
             kPrepMaxChan * kWave);
  TL_REQUIRE(row_stride >= (n_q + n_kv) * dk + n_kv * dv, "head_prepare: rows of %d elements do not hold the heads", row_stride);
  TL_REQUIRE(norm_dims >= 0 && norm_dims <= dk, "head_prepare: a norm over %d of %d channels", norm_dims, dk);
  TL_REQUIRE((q_w == nullptr && k_w == nullptr) || norm_dims > 0, "head_prepare: norm weights without channels to norm");
  TL_REQUIRE(rot >= 0 && rot % 2 == 0 && rot_off >= 0 && rot_off + rot <= dk, "head_prepare: %d rotated channels from %d of %d", rot, rot_off, dk);
  TL_REQUIRE(pairing == 0 || pairing == 1, "head_prepare: pairing must be 0 (interleaved) or 1 (half split)");
  TL_REQUIRE(rot == 0 || cos_sin != nullptr, "head_prepare: rotation without a table of cosines and sines");
  TL_REQUIRE(temp_coef == 0.f || (positions != nullptr && temp_every > 0), "head_prepare: a query factor needs positions and a positive step");
  TL_REQUIRE(v_first == nullptr || (lam != nullptr && dv > 0 && v_first_stride >= n_kv * dv), "head_prepare: mixed values need their factor and rows of the values' width");
  TL_REQUIRE(k_pages == nullptr || (slot_mapping != nullptr && page_size > 0 && (dv == 0 || v_pages != nullptr)), "head_prepare: pages without slots");
  if (n_tokens == 0) return TL_OK;
  const int units = n_q + n_kv + (dv > 0 ? n_kv : 0);
  const int widest = dk > dv ? dk : dv;
  // four tokens a wave while a lane holds few channels and the launch still has blocks for every CU several times over
  const bool four = widest <= 4 * kWave && (long long)n_tokens * units >= 64LL * tl_device_facts().compute_units;
  const int tok = four ? 4 : 1;
  const dim3 grid((n_tokens + tok - 1) / tok, (units + kPrepWaves - 1) / kPrepWaves);
#define TL_PREP_LAUNCH(T, CH, TOK) head_prepare_kernel<T, CH, TOK><<<grid, kPrepWaves * kWave, 0, stream>>>(a, n_tokens)
#define TL_PREP(T)                                                                                                   \
  do {                                                                                                               \
    PrepArgs<T> a{(T*)rows, row_stride, n_q, n_kv, dk, dv, (const T*)bias, q_w, k_w, (q_w || k_w) ? norm_dims : 0, eps, \
                  (const float2*)cos_sin, rot_off, rot, pairing, positions, temp_coef, temp_every, (const T*)v_first, \
                  v_first_stride, lam, (T*)k_pages, (T*)v_pages, slot_mapping, page_size};                           \
    if (widest <= kWave) { if (four) TL_PREP_LAUNCH(T, 1, 4); else TL_PREP_LAUNCH(T, 1, 1); }                        \
    else if (widest <= 2 * kWave) { if (four) TL_PREP_LAUNCH(T, 2, 4); else TL_PREP_LAUNCH(T, 2, 1); }               \
    else if (widest <= 4 * kWave) { if (four) TL_PREP_LAUNCH(T, 4, 4); else TL_PREP_LAUNCH(T, 4, 1); }               \
    else if (widest <= 8 * kWave) TL_PREP_LAUNCH(T, 8, 1);                                                           \
    else TL_PREP_LAUNCH(T, kPrepMaxChan, 1);                                                                         \
  } while (0)
  if (dtype == TL_F32) TL_PREP(float);
  else if (dtype == TL_BF16) TL_PREP(bf16_t);
  else return tl_fail(TL_ERR_ARG, "head_prepare: unknown dtype %d", dtype);
#undef TL_PREP_LAUNCH
#undef TL_PREP
  return tl_check_launch("head_prepare");
}

TL_EXPORT int tl_branch_norm_add(float* stream_rows, const void* y, const float* w, void* rows, int n, int hidden, float eps,
                                 int dtype, hipStream_t stream) {
  TL_REQUIRE(n >= 0 && hidden > 0, "branch_norm_add: bad sizes");
  if (n == 0) return TL_OK;
  // few rows: a launch is as long as a row's trips to memory, so everything is fetched at once; many rows hide
  // the trips behind each other and do better with few registers
  const bool held = hidden <= kRowHeldMost * kRowThreads && n <= 2 * tl_device_facts().compute_units;
#define TL_BRANCH(T)                                                                                                              \
  do {                                                                                                                            \
    if (!held) branch_norm_add_kernel<T><<<n, kRowThreads, 0, stream>>>(stream_rows, (const T*)y, w, (T*)rows, hidden, eps);      \
    else if (hidden <= 2 * kRowThreads) branch_norm_add_held_kernel<T, 2><<<n, kRowThreads, 0, stream>>>(stream_rows, (const T*)y, w, (T*)rows, hidden, eps);   \
    else if (hidden <= 8 * kRowThreads) branch_norm_add_held_kernel<T, 8><<<n, kRowThreads, 0, stream>>>(stream_rows, (const T*)y, w, (T*)rows, hidden, eps);   \
    else if (hidden <= 16 * kRowThreads) branch_norm_add_held_kernel<T, 16><<<n, kRowThreads, 0, stream>>>(stream_rows, (const T*)y, w, (T*)rows, hidden, eps); \
    else branch_norm_add_held_kernel<T, kRowHeldMost><<<n, kRowThreads, 0, stream>>>(stream_rows, (const T*)y, w, (T*)rows, hidden, eps);                     \
  } while (0)
  if (dtype == TL_F32) TL_BRANCH(float);
  else if (dtype == TL_BF16) TL_BRANCH(bf16_t);
  else return tl_fail(TL_ERR_ARG, "branch_norm_add: unknown dtype %d", dtype);
#undef TL_BRANCH
  return tl_check_launch("branch_norm_add");
}

TL_EXPORT int tl_rmsnorm_columns(const void* x, int x_stride, int x_dtype, const int32_t* rows, const float* w, void* y,
                                 int y_stride, int y_dtype, int n, int width, float eps, hipStream_t stream) {
  TL_REQUIRE(n >= 0 && width > 0 && x_stride >= width && y_stride >= width, "rmsnorm_columns: bad sizes");
  if (n == 0) return TL_OK;
#define TL_NORM(XT, T) rmsnorm_columns_kernel<XT, T><<<n, kRowThreads, 0, stream>>>((const XT*)x, x_stride, rows, w, (T*)y, y_stride, width, eps)
  if (x_dtype == TL_F32 && y_dtype == TL_F32) TL_NORM(float, float);
  else if (x_dtype == TL_F32 && y_dtype == TL_BF16) TL_NORM(float, bf16_t);
  else if (x_dtype == TL_BF16 && y_dtype == TL_BF16) TL_NORM(bf16_t, bf16_t);
  else return tl_fail(TL_ERR_ARG, "rmsnorm_columns: input dtype %d with output dtype %d", x_dtype, y_dtype);
#undef TL_NORM
  return tl_check_launch("rmsnorm_columns");
}

TL_EXPORT int tl_sigmoid_gate(void* x, int x_stride, const void* g, int g_stride, int n, int width, int per, int dtype,
                              hipStream_t stream) {
  TL_REQUIRE(n >= 0 && width > 0 && per > 0 && x_stride >= width, "sigmoid_gate: bad sizes");
  if (n == 0) return TL_OK;
  const int blocks = elementwise_blocks((size_t)n * width);
  if (dtype == TL_F32) sigmoid_gate_kernel<float><<<blocks, 256, 0, stream>>>((float*)x, x_stride, (const float*)g, g_stride, n, width, per);
  else if (dtype == TL_BF16) {
    const bool wide = width % 8 == 0 && x_stride % 8 == 0 && ((uintptr_t)x % 16) == 0 &&
                      (per == 1 ? (g_stride % 8 == 0 && ((uintptr_t)g % 16) == 0) : per % 8 == 0);
    if (wide) sigmoid_gate_wide_kernel<<<elementwise_blocks((size_t)n * (width / 8)), 256, 0, stream>>>((bf16_t*)x, x_stride, (const bf16_t*)g, g_stride, n, width, per);
    else sigmoid_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)x, x_stride, (const bf16_t*)g, g_stride, n, width, per);
  } else {
    return tl_fail(TL_ERR_ARG, "sigmoid_gate: unknown dtype %d", dtype);
  }
  return tl_check_launch("sigmoid_gate");
}

TL_EXPORT int tl_pack_heads(const void* a, int na, const void* b, int b_stride, int b_head, int b_off, int nb, void* out, int n,
                            int heads, int dtype, hipStream_t stream) {
  TL_REQUIRE(n >= 0 && heads > 0 && heads <= 65535 && na >= 0 && nb >= 0 && na + nb > 0, "pack_heads: bad sizes");
  if (n == 0) return TL_OK;
  const dim3 grid(n, heads);
  if (dtype == TL_F32) pack_heads_kernel<float><<<grid, 128, 0, stream>>>((const float*)a, na, (const float*)b, b_stride, b_head, b_off, nb, (float*)out, n, heads);
  else if (dtype == TL_BF16) pack_heads_kernel<bf16_t><<<grid, 128, 0, stream>>>((const bf16_t*)a, na, (const bf16_t*)b, b_stride, b_head, b_off, nb, (bf16_t*)out, n, heads);
  else return tl_fail(TL_ERR_ARG, "pack_heads: unknown dtype %d", dtype);
  return tl_check_launch("pack_heads");
}

TL_EXPORT int tl_unpack_heads_gate(const void* a, void* out, const void* g, int g_stride, int n, int heads, int d, int dtype,
                                   hipStream_t stream) {
  TL_REQUIRE(n >= 0 && heads > 0 && heads <= 65535 && d > 0, "unpack_heads_gate: bad sizes");
  if (n == 0) return TL_OK;
  const dim3 grid(n, heads);
  if (dtype == TL_F32) unpack_heads_gate_kernel<float><<<grid, 128, 0, stream>>>((const float*)a, (float*)out, (const float*)g, g_stride, n, heads, d);
  else if (dtype == TL_BF16) unpack_heads_gate_kernel<bf16_t><<<grid, 128, 0, stream>>>((const bf16_t*)a, (bf16_t*)out, (const bf16_t*)g, g_stride, n, heads, d);
  else return tl_fail(TL_ERR_ARG, "unpack_heads_gate: unknown dtype %d", dtype);
  return tl_check_launch("unpack_heads_gate");
}

TL_EXPORT int tl_softcap(float* z, long long total, float cap, hipStream_t stream) {
  TL_REQUIRE(total >= 0 && cap > 0.f, "softcap: bad sizes or a cap that is not positive");
  if (total == 0) return TL_OK;
  softcap_kernel<<<elementwise_blocks((size_t)total), 256, 0, stream>>>(z, (size_t)total, cap);
  return tl_check_launch("softcap");
}
