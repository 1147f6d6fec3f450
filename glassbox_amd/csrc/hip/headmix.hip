// What stands around the attention of two mixers and around sublayers whose *output* is normed:
//
//   time_conv      h = x + conv(x): a short causal convolution over time on every channel of the 32-bit residual,
//                  conv(x)[t, c] = sum_j w[j, c] x[t - taps + 1 + j, c] (the weights a row a tap), zeros before the request's first token.  The last
//                  taps - 1 rows of x of each request live in its state slot, [taps - 1, channels] float32 (index i is the
//                  position `first position of the step` - (taps - 1) + i).
//   norm_slices    RMS norms with a weight over one or two runs of columns of a row (the latents of queries and of
//                  keys/values, which one stacked product leaves side by side).
//   latent_heads   heads for attention through latents: a query head is [dim as projected | rot_dim rotated], a key
//                  head [dim of the head's own up-projection | rot_dim rotated, one part shared by all heads], a value
//                  head vdim columns; rotation in half-split pairs (i, i + rot / 2) of the first `rot` of the rot_dim
//                  columns by the step's cos/sin table; every head filled up with zeros to hd columns; cache write.
//   diff_heads     heads for differential attention: a query head h holds two maps [q1 | q2] of dim columns and so does
//                  a key head; each map is divided by its root mean square, times a weight of dim numbers, and the query
//                  maps times the row's temperature 1 + coef ln(floor((p + 1) / every) + 1).  The two maps become two
//                  query heads of 2 dim columns, [q1 | 0] and [0 | q2], over ONE key head [k1 | k2]: q . k is then the
//                  map's own score, both maps read the same values, and grouped-query attention does the rest.
//   diff_combine   o = a1 - lambda a2 for every head, divided by its root mean square over vdim, times a constant.
//   gate_heads     out = heads * sigmoid(gate), the heads' zero columns dropped.
//   poly_norm      a N(z) + b N(z^2) + c N(z^3) + e over a row, N(v) = v / sqrt(mean(v^2) + eps).
//   norm_add       x += g * y / sqrt(mean(y^2) + eps), g one number; optionally the new x rounded to the activations' type.
//
// All arithmetic is 32-bit; a value is rounded once, when it is stored in the activations' type.
#include "common.h"

using namespace gb;

GB_DEFINE_LAST_ERROR

namespace {

constexpr int kMaxTaps = 8;

// A 16-byte word of a row: 8 bfloat16 or 4 floats.  The kernels with `Word` in their parameters take rows whose runs of
// columns begin and end at such words (the entry points check that and fall back to one element a thread otherwise).
template <typename T> struct Word;
template <> struct Word<bf16> {
  static constexpr int N = 8;
  typedef bf16x8 V;
};
template <> struct Word<float> {
  static constexpr int N = 4;
  typedef f32x4 V;
};
template <typename T> __device__ __forceinline__ void load_word(const T* p, float (&f)[Word<T>::N]) {
  const typename Word<T>::V v = *reinterpret_cast<const typename Word<T>::V*>(p);
#pragma unroll
  for (int e = 0; e < Word<T>::N; ++e) f[e] = to_f(v[e]);
}
template <typename T> __device__ __forceinline__ typename Word<T>::V make_word(const float (&f)[Word<T>::N]) {
  typename Word<T>::V v;
#pragma unroll
  for (int e = 0; e < Word<T>::N; ++e) v[e] = from_f<T>(f[e]);
  return v;
}
template <typename T> __device__ __forceinline__ void store_word(T* p, const float (&f)[Word<T>::N]) {
  *reinterpret_cast<typename Word<T>::V*>(p) = make_word<T>(f);
}
// four values of the 32-bit residual, rounded to the activations' type
__device__ __forceinline__ void store4(float* p, const f32x4& v) { *reinterpret_cast<f32x4*>(p) = v; }
__device__ __forceinline__ void store4(bf16* p, const f32x4& v) {
  bf16x4 o;
#pragma unroll
  for (int e = 0; e < 4; ++e) o[e] = (bf16)v[e];
  *reinterpret_cast<bf16x4*>(p) = o;
}
inline bool words16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// Three sums over a block of up to 1024 threads at once; `scratch` holds 48 floats.  Every thread adds the waves' sums in
// the same order.
__device__ __forceinline__ void block_sum3(float& a, float& b, float& c, float* scratch) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int waves = (blockDim.x + kWave - 1) / kWave;
  a = wave_sum(a), b = wave_sum(b), c = wave_sum(c);
  if (lane == 0) scratch[wave * 3] = a, scratch[wave * 3 + 1] = b, scratch[wave * 3 + 2] = c;
  __syncthreads();
  a = b = c = 0.f;
  for (int w = 0; w < waves; ++w) a += scratch[w * 3], b += scratch[w * 3 + 1], c += scratch[w * 3 + 2];
}

// ------------------------------------------------------------------------------------------------ time_conv
// A thread a (token, channel).  single: every request of the step brings one row, and the thread moves its channel of the
// slot on by one itself.
template <typename T>
__global__ void time_conv_kernel(const float* __restrict__ x, int ldx, const float* __restrict__ w, int taps,
                                 float* __restrict__ state, const int32_t* __restrict__ tok_seq,
                                 const int32_t* __restrict__ q_start, const int32_t* __restrict__ pos0,
                                 const int32_t* __restrict__ state_slots, T* __restrict__ out, int ldo, long long count, int d,
                                 int single) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= count) return;
  const int t = (int)(idx / d), c = (int)(idx % d);
  const float cur = x[(size_t)t * ldx + c];
  if (taps <= 0) {
    out[(size_t)t * ldo + c] = from_f<T>(cur);
    return;
  }
  const int K = taps - 1;
  const int seq = tok_seq[t], off = t - q_start[seq], first_pos = pos0[seq];
  float* st = K > 0 ? state + (size_t)state_slots[seq] * K * d + c : nullptr;
  float acc = 0.f;
  float old[kMaxTaps - 1];
  if (single) {
#pragma unroll
    for (int i = 0; i < kMaxTaps - 1; ++i) old[i] = i < K ? st[(size_t)i * d] : 0.f;
  }
  for (int j = 0; j < taps; ++j) {
    const int back = K - j;   // how many tokens before this one
    float v = 0.f;
    if (back == 0) {
      v = cur;
    } else if (off >= back) {
      v = x[(size_t)(t - back) * ldx + c];
    } else if (first_pos + off - back >= 0) {
      v = st[(size_t)(off + j) * d];   // index (position - back) - first_pos + K
    }
    acc = fmaf(w[(size_t)j * d + c], v, acc);
  }
  out[(size_t)t * ldo + c] = from_f<T>(cur + acc);
  if (single) {
#pragma unroll
    for (int i = 0; i < kMaxTaps - 1; ++i)
      if (i < K) st[(size_t)i * d] = i + 1 < K ? old[i + 1 < kMaxTaps - 1 ? i + 1 : 0] : cur;
  }
}

// Four channels a thread, a workgroup inside one token (whose request's tables it reads once): d and the row strides are
// multiples of 4.
template <typename T>
__global__ __launch_bounds__(256) void time_conv4_kernel(const float* __restrict__ x, int ldx, const float* __restrict__ w,
                                                         int taps, float* __restrict__ state,
                                                         const int32_t* __restrict__ tok_seq,
                                                         const int32_t* __restrict__ q_start, const int32_t* __restrict__ pos0,
                                                         const int32_t* __restrict__ state_slots, T* __restrict__ out, int ldo,
                                                         int d, int single) {
  const int t = blockIdx.x, c = (blockIdx.y * 256 + threadIdx.x) * 4;
  if (c >= d) return;
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  const f32x4 cur = *reinterpret_cast<const f32x4*>(x + (size_t)t * ldx + c);
  if (taps <= 0) {
    store4(out + (size_t)t * ldo + c, cur);
    return;
  }
  const int K = taps - 1;
  // the rows before this one and the weights are asked for before the request's tables say which of the rows count:
  // the loads of a token are then all on their way together
  f32x4 rows[kMaxTaps - 1];
  f32x4 wv[kMaxTaps];
#pragma unroll
  for (int j = 0; j < kMaxTaps - 1; ++j) {
    const int back = K - j;
    rows[j] = (j < K && !single && t - back >= 0) ? *reinterpret_cast<const f32x4*>(x + (size_t)(t - back) * ldx + c) : zero;
  }
#pragma unroll
  for (int j = 0; j < kMaxTaps; ++j) wv[j] = j < taps ? *reinterpret_cast<const f32x4*>(w + (size_t)j * d + c) : zero;
  const int seq = tok_seq[t], off = t - q_start[seq], first_pos = pos0[seq];
  float* st = K > 0 ? state + (size_t)state_slots[seq] * K * d + c : nullptr;
  f32x4 old[kMaxTaps - 1];
  if (single) {
#pragma unroll
    for (int i = 0; i < kMaxTaps - 1; ++i)
      if (i < K) old[i] = *reinterpret_cast<const f32x4*>(st + (size_t)i * d);
  }
  f32x4 acc = zero;
#pragma unroll
  for (int j = 0; j < kMaxTaps; ++j) {
    if (j >= taps) break;
    const int back = K - j;   // how many tokens before this one
    f32x4 v = zero;
    if (back == 0) {
      v = cur;
    } else if (off >= back) {
      v = rows[j < kMaxTaps - 1 ? j : 0];
    } else if (first_pos + off - back >= 0) {
      // index (position - back) - first_pos + K of the slot; a step of single tokens has off = 0 and the slot in hand
      v = single ? old[j < kMaxTaps - 1 ? j : 0] : *reinterpret_cast<const f32x4*>(st + (size_t)(off + j) * d);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] = fmaf(wv[j][e], v[e], acc[e]);
  }
  store4(out + (size_t)t * ldo + c, cur + acc);
  if (single) {
#pragma unroll
    for (int i = 0; i < kMaxTaps - 1; ++i)
      if (i < K) *reinterpret_cast<f32x4*>(st + (size_t)i * d) = i + 1 < K ? old[i + 1 < kMaxTaps - 1 ? i + 1 : 0] : cur;
  }
}

// Steps with portions: four channels and four tokens in a row a thread, so that a row of x is read for four tokens'
// sums and not for one (taps + 3 rows where four tokens alone would read 4 taps).  The tokens may be of different
// requests; each looks up its own.
constexpr int kConvTokens = 4;
template <typename T>
__global__ __launch_bounds__(256) void time_conv4x4_kernel(const float* __restrict__ x, int ldx, const float* __restrict__ w,
                                                           int taps, const float* __restrict__ state,
                                                           const int32_t* __restrict__ tok_seq,
                                                           const int32_t* __restrict__ q_start,
                                                           const int32_t* __restrict__ pos0,
                                                           const int32_t* __restrict__ state_slots, T* __restrict__ out,
                                                           int ldo, int n, int d) {
  const int t0 = blockIdx.x * kConvTokens, c = (blockIdx.y * 256 + threadIdx.x) * 4;
  if (c >= d) return;
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  const int K = taps - 1;
  // rows[k] is the row of token t0 - K + k: what the four tokens' taps can reach of the step's rows; tap j of token
  // t0 + i reads rows[i + j]
  f32x4 rows[kMaxTaps - 1 + kConvTokens], cur[kConvTokens], wv[kMaxTaps];
#pragma unroll
  for (int k = 0; k < kMaxTaps - 1 + kConvTokens; ++k) {
    const int t = t0 - K + k;
    rows[k] = (k < K + kConvTokens && t >= 0 && t < n) ? *reinterpret_cast<const f32x4*>(x + (size_t)t * ldx + c) : zero;
  }
#pragma unroll
  for (int i = 0; i < kConvTokens; ++i)
    cur[i] = t0 + i < n ? *reinterpret_cast<const f32x4*>(x + (size_t)(t0 + i) * ldx + c) : zero;
#pragma unroll
  for (int j = 0; j < kMaxTaps; ++j) wv[j] = j < taps ? *reinterpret_cast<const f32x4*>(w + (size_t)j * d + c) : zero;
#pragma unroll
  for (int i = 0; i < kConvTokens; ++i) {
    const int t = t0 + i;
    if (t >= n) break;
    const int seq = tok_seq[t], off = t - q_start[seq], first_pos = pos0[seq];
    const float* st = K > 0 ? state + (size_t)state_slots[seq] * K * d + c : nullptr;
    f32x4 acc = zero;   // the taps in their order, then x: the sums of the kernel that takes a token a thread
#pragma unroll
    for (int j = 0; j < kMaxTaps; ++j) {
      if (j >= taps) break;
      const int back = K - j;
      f32x4 v = zero;
      if (back == 0) {
        v = cur[i];
      } else if (off >= back) {
        v = rows[i + j];
      } else if (first_pos + off - back >= 0) {
        v = *reinterpret_cast<const f32x4*>(st + (size_t)(off + j) * d);   // index position - first_pos + K of the slot
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] = fmaf(wv[j][e], v[e], acc[e]);
    }
    store4(out + (size_t)t * ldo + c, cur[i] + acc);
  }
}

// ------------------------------------------------------------------------------------------------ norm_slices
struct Slice {
  int col, d, ldo;
  const float* gamma;
  void* out;
};

template <typename T>
__global__ __launch_bounds__(256) void norm_slices_kernel(const T* __restrict__ in, int ld, Slice s0, Slice s1, float eps) {
  __shared__ float scratch[17];
  const Slice s = blockIdx.y == 0 ? s0 : s1;
  const T* row = in + (size_t)blockIdx.x * ld + s.col;
  float ss = 0.f;
  for (int c = threadIdx.x; c < s.d; c += blockDim.x) {
    const float v = to_f(row[c]);
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)s.d + eps);
  T* o = (T*)s.out + (size_t)blockIdx.x * s.ldo;
  for (int c = threadIdx.x; c < s.d; c += blockDim.x) o[c] = from_f<T>(to_f(row[c]) * r * s.gamma[c]);
}

// A wave a (row, slice), the slice in registers: runs of whole words, at most 4 words a lane.
template <typename T>
__global__ __launch_bounds__(256) void norm_slices_words_kernel(const T* __restrict__ in, int ld, int n, Slice s0, Slice s1,
                                                                float eps) {
  constexpr int N = Word<T>::N;
  const Slice s = blockIdx.y == 0 ? s0 : s1;
  const int r = blockIdx.x * 4 + threadIdx.x / kWave, lane = threadIdx.x % kWave;
  if (r >= n) return;
  const T* row = in + (size_t)r * ld + s.col;
  float v[4][N];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = (lane + i * kWave) * N;
    if (c < s.d) {
      load_word(row + c, v[i]);
#pragma unroll
      for (int e = 0; e < N; ++e) ss = fmaf(v[i][e], v[i][e], ss);
    }
  }
  ss = wave_sum(ss);
  const float scale = 1.0f / sqrtf(ss / (float)s.d + eps);
  T* o = (T*)s.out + (size_t)r * s.ldo;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = (lane + i * kWave) * N;
    if (c < s.d) {
#pragma unroll
      for (int e = 0; e < N; ++e) v[i][e] = v[i][e] * scale * s.gamma[c + e];
      store_word(o + c, v[i]);
    }
  }
}

// ------------------------------------------------------------------------------------------------ cache write
template <typename T>
__device__ __forceinline__ void store_key(T* k_pages, int slot, int page_size, int nkv, int kvh, int hd, int c, T v) {
  T* kb = k_pages + ((size_t)(slot / page_size) * nkv + kvh) * (size_t)page_size * hd;
  kb[key_offset(slot % page_size, c, page_size, key_piece(hd))] = v;
}
template <typename T>
__device__ __forceinline__ void store_value(T* v_pages, int slot, int page_size, int nkv, int kvh, int hd, int c, T v) {
  T* vb = v_pages + ((size_t)(slot / page_size) * nkv + kvh) * (size_t)page_size * hd;
  vb[(size_t)c * page_size + slot % page_size] = v;
}

// ------------------------------------------------------------------------------------------------ latent_heads
// A thread a (token, head, column): query heads, key heads, value heads, H of each.
template <typename T>
__global__ void latent_heads_kernel(const T* __restrict__ q, int ldq, const T* __restrict__ kv, int ldkv,
                                    const T* __restrict__ krot, int ldr, const float* __restrict__ cosv,
                                    const float* __restrict__ sinv, int rot, T* __restrict__ out, int ldo, int hd,
                                    const int32_t* __restrict__ slots, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                    int page_size, long long count, int H, int dim, int rdim, int vdim) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= count) return;
  const int c = (int)(idx % hd);
  const int u = (int)((idx / hd) % (3 * H));
  const int t = (int)(idx / ((long long)hd * 3 * H));
  float v = 0.f;
  if (u < 2 * H) {
    const bool is_q = u < H;
    const int h = is_q ? u : u - H;
    if (c < dim) {
      v = is_q ? to_f(q[(size_t)t * ldq + (size_t)h * (dim + rdim) + c]) : to_f(kv[(size_t)t * ldkv + (size_t)h * dim + c]);
    } else if (c < dim + rdim) {
      const T* src = is_q ? q + (size_t)t * ldq + (size_t)h * (dim + rdim) + dim : krot + (size_t)t * ldr;
      const int r = c - dim, half = rot / 2;
      if (r < rot) {
        const int i = r < half ? r : r - half;
        const float a = to_f(src[i]), b = to_f(src[i + half]);
        const float cs = cosv[(size_t)t * half + i], sn = sinv[(size_t)t * half + i];
        v = r < half ? a * cs - b * sn : b * cs + a * sn;
      } else {
        v = to_f(src[r]);
      }
    }
  } else if (c < vdim) {
    v = to_f(kv[(size_t)t * ldkv + (size_t)H * dim + (size_t)(u - 2 * H) * vdim + c]);
  }
  const T r = from_f<T>(v);
  out[(size_t)t * ldo + (size_t)u * hd + c] = r;
  if (slots && u >= H) {
    const int slot = slots[t];
    if (slot >= 0) {
      if (u < 2 * H) store_key(k_pages, slot, page_size, H, u - H, hd, c, r);
      else store_value(v_pages, slot, page_size, H, u - 2 * H, hd, c, r);
    }
  }
}

// A word of a head a thread: dim, rot_dim, rot / 2, vdim, hd and the row strides are whole words, so a word lies in one
// run of a head (as projected, first or second halves of the rotated pairs, unrotated, zeros).
template <typename T>
__device__ __forceinline__ void store_key_word(T* k_pages, int slot, int page_size, int nkv, int kvh, int hd, int c,
                                               const typename Word<T>::V& v) {
  T* kb = k_pages + ((size_t)(slot / page_size) * nkv + kvh) * (size_t)page_size * hd;
  *reinterpret_cast<typename Word<T>::V*>(kb + key_offset(slot % page_size, c, page_size, 8)) = v;   // inside a piece of 8
}
template <typename T>
__device__ __forceinline__ void store_value_word(T* v_pages, int slot, int page_size, int nkv, int kvh, int hd, int c,
                                                 const typename Word<T>::V& v) {
  T* vb = v_pages + ((size_t)(slot / page_size) * nkv + kvh) * (size_t)page_size * hd + slot % page_size;
#pragma unroll
  for (int e = 0; e < Word<T>::N; ++e) vb[(size_t)(c + e) * page_size] = v[e];
}

template <typename T>
__global__ void latent_heads_words_kernel(const T* __restrict__ q, int ldq, const T* __restrict__ kv, int ldkv,
                                          const T* __restrict__ krot, int ldr, const float* __restrict__ cosv,
                                          const float* __restrict__ sinv, int rot, T* __restrict__ out, int ldo, int hd,
                                          const int32_t* __restrict__ slots, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                          int page_size, long long count, int H, int dim, int rdim, int vdim) {
  constexpr int N = Word<T>::N;
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= count) return;
  const int per = hd / N;
  const int c = (int)(idx % per) * N;
  const int u = (int)((idx / per) % (3 * H));
  const int t = (int)(idx / ((long long)per * 3 * H));
  float v[N];
#pragma unroll
  for (int e = 0; e < N; ++e) v[e] = 0.f;
  if (u < 2 * H) {
    const bool is_q = u < H;
    const int h = is_q ? u : u - H;
    if (c < dim) {
      load_word(is_q ? q + (size_t)t * ldq + (size_t)h * (dim + rdim) + c : kv + (size_t)t * ldkv + (size_t)h * dim + c, v);
    } else if (c < dim + rdim) {
      const T* src = is_q ? q + (size_t)t * ldq + (size_t)h * (dim + rdim) + dim : krot + (size_t)t * ldr;
      const int r = c - dim, half = rot / 2;
      if (r < rot) {
        const int i = r < half ? r : r - half;
        float a[N], b[N];
        load_word(src + i, a);
        load_word(src + i + half, b);
        const float* cs = cosv + (size_t)t * half + i;
        const float* sn = sinv + (size_t)t * half + i;
#pragma unroll
        for (int e = 0; e < N; ++e) v[e] = r < half ? a[e] * cs[e] - b[e] * sn[e] : b[e] * cs[e] + a[e] * sn[e];
      } else {
        load_word(src + r, v);
      }
    }
  } else if (c < vdim) {
    load_word(kv + (size_t)t * ldkv + (size_t)H * dim + (size_t)(u - 2 * H) * vdim + c, v);
  }
  const typename Word<T>::V w = make_word<T>(v);
  *reinterpret_cast<typename Word<T>::V*>(out + (size_t)t * ldo + (size_t)u * hd + c) = w;
  if (slots && u >= H) {
    const int slot = slots[t];
    if (slot >= 0) {
      if (u < 2 * H) store_key_word<T>(k_pages, slot, page_size, H, u - H, hd, c, w);
      else store_value_word<T>(v_pages, slot, page_size, H, u - 2 * H, hd, c, w);
    }
  }
}

// ------------------------------------------------------------------------------------------------ diff_heads
// Sixteen lanes a (token, unit); the units of a token: 2 H query maps, 2 G key maps, G value heads.
constexpr int kLanes = 16;

template <typename T>
__global__ __launch_bounds__(4 * kWave) void diff_heads_kernel(
    const T* __restrict__ proj, int ld, const float* __restrict__ wq, const float* __restrict__ wk, float eps, float coef,
    int every, const int32_t* __restrict__ positions, T* __restrict__ out, int ldo, int hd, const int32_t* __restrict__ slots,
    T* __restrict__ k_pages, T* __restrict__ v_pages, int page_size, long long units, int H, int G, int dim, int vdim) {
  const int li = threadIdx.x % kLanes;
  const long long unit = ((long long)blockIdx.x * blockDim.x + threadIdx.x) / kLanes;
  const bool live = unit < units;
  const int per = 2 * H + 3 * G;
  const int t = live ? (int)(unit / per) : 0, u = live ? (int)(unit % per) : 0;
  const bool is_q = u < 2 * H, is_k = !is_q && u < 2 * H + 2 * G;
  // where the unit's numbers lie in the row, and which head and columns of the result they fill
  int src, head, col0, width, upto;
  if (is_q) {
    src = u * dim, head = u, col0 = (u % 2) * dim, width = dim, upto = hd;          // [q1 | 0] or [0 | q2]: all columns
  } else if (is_k) {
    const int j = u - 2 * H;
    src = 2 * H * dim + j * dim, head = 2 * H + j / 2, col0 = (j % 2) * dim, width = dim;
    upto = j % 2 ? hd : dim;                                                        // the second map fills up with zeros
  } else {
    const int g = u - 2 * H - 2 * G;
    src = (2 * H + 2 * G) * dim + g * vdim, head = 2 * H + G + g, col0 = 0, width = vdim, upto = hd;
  }
  const T* row = proj + (size_t)t * ld + src;
  float ss = 0.f;
  if (live && (is_q || is_k))
    for (int c = li; c < width; c += kLanes) {
      const float v = to_f(row[c]);
      ss = fmaf(v, v, ss);
    }
#pragma unroll
  for (int o = kLanes / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, kWave);
  if (!live) return;
  float s = 1.f;
  if (is_q || is_k) s = 1.0f / sqrtf(ss / (float)dim + eps);
  if (is_q && every > 0) s *= 1.0f + coef * logf((float)((positions[t] + 1) / every) + 1.0f);
  const float* gamma = is_q ? wq : is_k ? wk : nullptr;
  const int slot = (!is_q && slots) ? slots[t] : -1;
  T* orow = out + (size_t)t * ldo + (size_t)head * hd;
  const int first = (is_k && col0 > 0) ? col0 : 0;   // a key head's first map is written by its own unit
  for (int c = first + li; c < upto; c += kLanes) {
    float v = 0.f;
    if (c >= col0 && c < col0 + width) v = to_f(row[c - col0]) * s * (gamma ? gamma[c - col0] : 1.0f);
    const T r = from_f<T>(v);
    orow[c] = r;
    if (slot >= 0) {
      if (is_k) store_key(k_pages, slot, page_size, G, head - 2 * H, hd, c, r);
      else store_value(v_pages, slot, page_size, G, head - 2 * H - G, hd, c, r);
    }
  }
}

// The same in words: LANES lanes a (token, unit), a lane a word at a time; dim, vdim, hd and the row strides are whole words.
template <typename T, int LANES>
__global__ __launch_bounds__(4 * kWave) void diff_heads_words_kernel(
    const T* __restrict__ proj, int ld, const float* __restrict__ wq, const float* __restrict__ wk, float eps, float coef,
    int every, const int32_t* __restrict__ positions, T* __restrict__ out, int ldo, int hd, const int32_t* __restrict__ slots,
    T* __restrict__ k_pages, T* __restrict__ v_pages, int page_size, long long units, int H, int G, int dim, int vdim) {
  constexpr int N = Word<T>::N;
  const int li = threadIdx.x % LANES;
  const long long unit = ((long long)blockIdx.x * blockDim.x + threadIdx.x) / LANES;
  const bool live = unit < units;
  const int per = 2 * H + 3 * G;
  const int t = live ? (int)(unit / per) : 0, u = live ? (int)(unit % per) : 0;
  const bool is_q = u < 2 * H, is_k = !is_q && u < 2 * H + 2 * G;
  int src, head, col0, width, upto;
  if (is_q) {
    src = u * dim, head = u, col0 = (u % 2) * dim, width = dim, upto = hd;
  } else if (is_k) {
    const int j = u - 2 * H;
    src = 2 * H * dim + j * dim, head = 2 * H + j / 2, col0 = (j % 2) * dim, width = dim;
    upto = j % 2 ? hd : dim;
  } else {
    const int g = u - 2 * H - 2 * G;
    src = (2 * H + 2 * G) * dim + g * vdim, head = 2 * H + G + g, col0 = 0, width = vdim, upto = hd;
  }
  const T* row = proj + (size_t)t * ld + src;
  float ss = 0.f;
  if (live && (is_q || is_k))
    for (int c = li * N; c < width; c += LANES * N) {
      float v[N];
      load_word(row + c, v);
#pragma unroll
      for (int e = 0; e < N; ++e) ss = fmaf(v[e], v[e], ss);
    }
#pragma unroll
  for (int o = LANES / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, kWave);
  if (!live) return;
  float s = 1.f;
  if (is_q || is_k) s = 1.0f / sqrtf(ss / (float)dim + eps);
  if (is_q && every > 0) s *= 1.0f + coef * logf((float)((positions[t] + 1) / every) + 1.0f);
  const float* gamma = is_q ? wq : is_k ? wk : nullptr;
  const int slot = (!is_q && slots) ? slots[t] : -1;
  T* orow = out + (size_t)t * ldo + (size_t)head * hd;
  const int first = (is_k && col0 > 0) ? col0 : 0;
  for (int c = first + li * N; c < upto; c += LANES * N) {
    float v[N];
#pragma unroll
    for (int e = 0; e < N; ++e) v[e] = 0.f;
    if (c >= col0 && c < col0 + width) {
      load_word(row + c - col0, v);
#pragma unroll
      for (int e = 0; e < N; ++e) v[e] = v[e] * s * (gamma ? gamma[c - col0 + e] : 1.0f);
    }
    const typename Word<T>::V w = make_word<T>(v);
    *reinterpret_cast<typename Word<T>::V*>(orow + c) = w;
    if (slot >= 0) {
      if (is_k) store_key_word<T>(k_pages, slot, page_size, G, head - 2 * H, hd, c, w);
      else store_value_word<T>(v_pages, slot, page_size, G, head - 2 * H - G, hd, c, w);
    }
  }
}

// ------------------------------------------------------------------------------------------------ diff_combine
// Sixteen lanes a (token, head): att holds 2 H heads of hd columns, the maps of head h in heads 2 h and 2 h + 1.
template <typename AT, typename T>
__global__ __launch_bounds__(4 * kWave) void diff_combine_kernel(const AT* __restrict__ att, int lda, int hd,
                                                                 const float* __restrict__ lambda, float mult, float eps,
                                                                 T* __restrict__ out, int ldo, long long units, int H,
                                                                 int vdim) {
  const int li = threadIdx.x % kLanes;
  const long long unit = ((long long)blockIdx.x * blockDim.x + threadIdx.x) / kLanes;
  const bool live = unit < units;
  const int t = live ? (int)(unit / H) : 0, h = live ? (int)(unit % H) : 0;
  const AT* a1 = att + (size_t)t * lda + (size_t)(2 * h) * hd;
  const AT* a2 = a1 + hd;
  const float lam = lambda[0];
  float ss = 0.f;
  if (live)
    for (int c = li; c < vdim; c += kLanes) {
      const float o = to_f(a1[c]) - lam * to_f(a2[c]);
      ss = fmaf(o, o, ss);
    }
#pragma unroll
  for (int o = kLanes / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, kWave);
  if (!live) return;
  const float s = mult / sqrtf(ss / (float)vdim + eps);
  T* orow = out + (size_t)t * ldo + (size_t)h * vdim;
  for (int c = li; c < vdim; c += kLanes) orow[c] = from_f<T>((to_f(a1[c]) - lam * to_f(a2[c])) * s);
}

// ------------------------------------------------------------------------------------------------ gate_heads
template <typename T>
__global__ void gate_heads_kernel(const T* __restrict__ att, int lda, int hd, const T* __restrict__ gate, int ldg,
                                  T* __restrict__ out, int ldo, long long count, int H, int vdim) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= count) return;
  const int c = (int)(idx % vdim);
  const int h = (int)((idx / vdim) % H);
  const int t = (int)(idx / ((long long)vdim * H));
  const float g = to_f(gate[(size_t)t * ldg + (size_t)h * vdim + c]);
  const float a = to_f(att[(size_t)t * lda + (size_t)h * hd + c]);
  out[(size_t)t * ldo + (size_t)h * vdim + c] = from_f<T>(a / (1.0f + expf(-g)));
}

// A word of a head a thread (vdim, hd and the row strides are whole words).
template <typename T>
__global__ void gate_heads_words_kernel(const T* __restrict__ att, int lda, int hd, const T* __restrict__ gate, int ldg,
                                        T* __restrict__ out, int ldo, long long count, int H, int vdim) {
  constexpr int N = Word<T>::N;
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= count) return;
  const int per = vdim / N;
  const int c = (int)(idx % per) * N;
  const int h = (int)((idx / per) % H);
  const int t = (int)(idx / ((long long)per * H));
  float g[N], a[N];
  load_word(gate + (size_t)t * ldg + (size_t)h * vdim + c, g);
  load_word(att + (size_t)t * lda + (size_t)h * hd + c, a);
#pragma unroll
  for (int e = 0; e < N; ++e) a[e] = a[e] / (1.0f + expf(-g[e]));
  store_word(out + (size_t)t * ldo + (size_t)h * vdim + c, a);
}

// ------------------------------------------------------------------------------------------------ poly_norm
template <typename T>
__global__ __launch_bounds__(256) void poly_norm_kernel(const T* __restrict__ z, int ldz, const float* __restrict__ coef,
                                                        float eps, T* __restrict__ out, int ldo, int d) {
  __shared__ float scratch[17];
  const T* row = z + (size_t)blockIdx.x * ldz;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  for (int c = threadIdx.x; c < d; c += blockDim.x) {
    const float v = to_f(row[c]), v2 = v * v;
    s2 += v2;
    s4 = fmaf(v2, v2, s4);
    s6 = fmaf(v2 * v2, v2, s6);
  }
  s2 = block_sum(s2, scratch);
  s4 = block_sum(s4, scratch);
  s6 = block_sum(s6, scratch);
  const float r1 = coef[0] / sqrtf(s2 / (float)d + eps), r2 = coef[1] / sqrtf(s4 / (float)d + eps),
              r3 = coef[2] / sqrtf(s6 / (float)d + eps), e = coef[3];
  T* o = out + (size_t)blockIdx.x * ldo;
  for (int c = threadIdx.x; c < d; c += blockDim.x) {
    const float v = to_f(row[c]);
    o[c] = from_f<T>(v * r1 + v * v * r2 + v * v * v * r3 + e);
  }
}

// The row stays in registers between the pass that sums its powers and the pass that writes it: WORDS words a thread,
// d at most THREADS * WORDS words of whole words.
template <typename T, int THREADS, int WORDS>
__global__ __launch_bounds__(THREADS) void poly_norm_rows_kernel(const T* __restrict__ z, int ldz, const float* __restrict__ coef,
                                                                 float eps, T* __restrict__ out, int ldo, int d) {
  constexpr int N = Word<T>::N;
  __shared__ float scratch[48];
  const T* row = z + (size_t)blockIdx.x * ldz;
  float v[WORDS][N];
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
#pragma unroll
  for (int i = 0; i < WORDS; ++i) {
    const int c = (threadIdx.x + i * THREADS) * N;
    if (c < d) {
      load_word(row + c, v[i]);
#pragma unroll
      for (int e = 0; e < N; ++e) {
        const float v2 = v[i][e] * v[i][e];
        s2 += v2;
        s4 = fmaf(v2, v2, s4);
        s6 = fmaf(v2 * v2, v2, s6);
      }
    }
  }
  block_sum3(s2, s4, s6, scratch);
  const float r1 = coef[0] / sqrtf(s2 / (float)d + eps), r2 = coef[1] / sqrtf(s4 / (float)d + eps),
              r3 = coef[2] / sqrtf(s6 / (float)d + eps), e0 = coef[3];
  T* o = out + (size_t)blockIdx.x * ldo;
#pragma unroll
  for (int i = 0; i < WORDS; ++i) {
    const int c = (threadIdx.x + i * THREADS) * N;
    if (c < d) {
#pragma unroll
      for (int e = 0; e < N; ++e) {
        const float x = v[i][e];
        v[i][e] = x * r1 + x * x * r2 + x * x * x * r3 + e0;
      }
      store_word(o + c, v[i]);
    }
  }
}

// ------------------------------------------------------------------------------------------------ norm_add
template <typename T>
__global__ __launch_bounds__(256) void norm_add_kernel(float* __restrict__ x, const float* __restrict__ y,
                                                       const float* __restrict__ g, float eps, T* __restrict__ rounded, int d) {
  __shared__ float scratch[17];
  const float* yr = y + (size_t)blockIdx.x * d;
  float* xr = x + (size_t)blockIdx.x * d;
  float ss = 0.f;
  for (int c = threadIdx.x; c < d; c += blockDim.x) ss = fmaf(yr[c], yr[c], ss);
  ss = block_sum(ss, scratch);
  const float r = g[0] / sqrtf(ss / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += blockDim.x) {
    const float v = fmaf(yr[c], r, xr[c]);
    xr[c] = v;
    if (rounded) rounded[(size_t)blockIdx.x * d + c] = from_f<T>(v);
  }
}

// The same with the row of y in registers (d a multiple of 4, at most THREADS * WORDS * 4).  y may lie in `slices` pieces
// that are to be added, slice_stride floats apart (what the workgroups of a product that divides k leave): they are added
// in their order.  With `conv_w` (a step of single tokens) the row that `rounded` receives is not the new x but what the
// next mixer reads of it, x + conv(x), with the request's slot moved on as time_conv does.
template <typename T, int THREADS, int WORDS>
__global__ __launch_bounds__(THREADS) void norm_add_rows_kernel(float* __restrict__ x, const float* __restrict__ y, int slices,
                                                                long long slice_stride, const float* __restrict__ g, float eps,
                                                                T* __restrict__ rounded, int d, const float* __restrict__ conv_w,
                                                                int taps, float* __restrict__ state,
                                                                const int32_t* __restrict__ tok_seq,
                                                                const int32_t* __restrict__ pos0,
                                                                const int32_t* __restrict__ state_slots) {
  __shared__ float scratch[17];
  const int t = blockIdx.x;
  const float* yr = y + (size_t)t * d;
  float* xr = x + (size_t)t * d;
  f32x4 v[WORDS];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < WORDS; ++i) {
    const int c = (threadIdx.x + i * THREADS) * 4;
    if (c < d) {
      f32x4 sum = *reinterpret_cast<const f32x4*>(yr + c);
      for (int z = 1; z < slices; ++z) sum += *reinterpret_cast<const f32x4*>(yr + (size_t)z * slice_stride + c);
      v[i] = sum;
      ss += sum[0] * sum[0] + sum[1] * sum[1] + sum[2] * sum[2] + sum[3] * sum[3];
    }
  }
  ss = block_sum(ss, scratch);
  const float r = g[0] / sqrtf(ss / (float)d + eps);
  const int K = taps - 1;
  int seq = 0, pos = 0;
  if (conv_w) seq = tok_seq[t], pos = pos0[seq];
  float* st = conv_w && K > 0 ? state + (size_t)state_slots[seq] * K * d : nullptr;
#pragma unroll
  for (int i = 0; i < WORDS; ++i) {
    const int c = (threadIdx.x + i * THREADS) * 4;
    if (c < d) {
      const f32x4 old = *reinterpret_cast<const f32x4*>(xr + c);
      f32x4 nx;
#pragma unroll
      for (int e = 0; e < 4; ++e) nx[e] = fmaf(v[i][e], r, old[e]);
      *reinterpret_cast<f32x4*>(xr + c) = nx;
      if (conv_w) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        for (int j = 0; j < taps; ++j) {
          f32x4 in = nx;
          if (j < K) {   // index j of the slot is the row of position pos - (K - j); it moves to index j - 1
            in = *reinterpret_cast<const f32x4*>(st + (size_t)j * d + c);
            if (j > 0) *reinterpret_cast<f32x4*>(st + (size_t)(j - 1) * d + c) = in;
            if (pos - (K - j) < 0) in = f32x4{0.f, 0.f, 0.f, 0.f};   // before the request's first token
          }
          const f32x4 wj = *reinterpret_cast<const f32x4*>(conv_w + (size_t)j * d + c);
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[e] = fmaf(wj[e], in[e], acc[e]);
        }
        if (K > 0) *reinterpret_cast<f32x4*>(st + (size_t)(K - 1) * d + c) = nx;
        store4(rounded + (size_t)t * d + c, nx + acc);
      } else if (rounded) {
        store4(rounded + (size_t)t * d + c, nx);
      }
    }
  }
}

inline bool grid_fits(long long count, int per_block) { return (count + per_block - 1) / per_block < (1ll << 31); }

}  // namespace

#define GB_BY_DTYPE(dtype, what, CALL)              \
  if (dtype == kF32) {                              \
    typedef float TT;                               \
    CALL;                                           \
  } else if (dtype == kBF16) {                      \
    typedef bf16 TT;                                \
    CALL;                                           \
  } else {                                          \
    return fail(what ": unknown dtype %d", dtype);  \
  }

// x [n, ldx] float32, w [taps, d] float32 (taps 0: none, out = x rounded), state [slots, taps - 1, d] float32,
// out [n, ldo] of `dtype`.  single: every request brings one row and its slot is moved on here; otherwise the caller moves
// the slots after this call, before x changes.
extern "C" int gb_time_conv(const float* x, int ldx, const float* w, int taps, float* state, const int32_t* tok_seq,
                            const int32_t* q_start, const int32_t* pos0, const int32_t* state_slots, void* out, int dtype,
                            int ldo, int n, int d, int single, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && d > 0 && ldx >= d && ldo >= d, "time_conv: bad sizes n=%d d=%d", n, d);
  GB_REQUIRE(taps >= 0 && taps <= kMaxTaps, "time_conv: %d taps (at most %d)", taps, kMaxTaps);
  GB_REQUIRE(taps == 0 || (w && tok_seq && q_start && pos0 && state_slots && (taps == 1 || state)),
             "time_conv: weights, the step's tables and the state are needed");
  if (n == 0) return 0;
  const long long count = (long long)n * d;
  GB_REQUIRE(grid_fits(count, 256), "time_conv: too many elements");
  if (d % 4 == 0 && ldx % 4 == 0 && ldo % 4 == 0 && words16(x) && words16(out) && words16(state) && words16(w) && (d + 1023) / 1024 < 65536) {
    if (taps >= 1 && !single && n >= 256) {
      const dim3 grid44((unsigned)((n + kConvTokens - 1) / kConvTokens), (unsigned)((d + 1023) / 1024));
      GB_BY_DTYPE(dtype, "time_conv",
                  hipLaunchKernelGGL(time_conv4x4_kernel<TT>, grid44, dim3(256), 0, stream, x, ldx, w, taps, state, tok_seq,
                                     q_start, pos0, state_slots, (TT*)out, ldo, n, d))
      return launched("time_conv");
    }
    const dim3 grid4((unsigned)n, (unsigned)((d + 1023) / 1024));
    GB_BY_DTYPE(dtype, "time_conv",
                hipLaunchKernelGGL(time_conv4_kernel<TT>, grid4, dim3(256), 0, stream, x, ldx, w, taps, state, tok_seq, q_start,
                                   pos0, state_slots, (TT*)out, ldo, d, single))
    return launched("time_conv");
  }
  const dim3 grid((unsigned)((count + 255) / 256));
  GB_BY_DTYPE(dtype, "time_conv",
              hipLaunchKernelGGL(time_conv_kernel<TT>, grid, dim3(256), 0, stream, x, ldx, w, taps, state, tok_seq, q_start,
                                 pos0, state_slots, (TT*)out, ldo, count, d, single))
  return launched("time_conv");
}

// in [n, ld] of `dtype`; slice s: columns col_s .. col_s + d_s, weight gamma_s float32 [d_s], result out_s [n, ldo_s].
// d1 = 0: one slice.
extern "C" int gb_norm_slices(const void* in, int dtype, int ld, int n, float eps, int col0, int d0, const float* gamma0,
                              void* out0, int ldo0, int col1, int d1, const float* gamma1, void* out1, int ldo1,
                              hipStream_t stream) {
  GB_REQUIRE(n >= 0 && d0 > 0 && d1 >= 0 && col0 >= 0 && col0 + d0 <= ld && ldo0 >= d0 && gamma0 && out0,
             "norm_slices: bad first slice (%d columns from %d of %d)", d0, col0, ld);
  GB_REQUIRE(d1 == 0 || (col1 >= 0 && col1 + d1 <= ld && ldo1 >= d1 && gamma1 && out1),
             "norm_slices: bad second slice (%d columns from %d of %d)", d1, col1, ld);
  GB_REQUIRE(n <= 0x7fffffff, "norm_slices: too many rows");
  if (n == 0) return 0;
  const Slice s0{col0, d0, ldo0, gamma0, out0}, s1{col1, d1, ldo1, gamma1, out1};
  const int wn = dtype == kBF16 ? 8 : 4;
  auto in_words = [&](const Slice& s) {
    return s.d == 0 || (s.col % wn == 0 && s.d % wn == 0 && s.d <= 4 * kWave * wn && s.ldo % wn == 0 && words16(s.out));
  };
  if (ld % wn == 0 && words16(in) && in_words(s0) && in_words(s1)) {
    const dim3 gridw((unsigned)((n + 3) / 4), d1 > 0 ? 2u : 1u);
    GB_BY_DTYPE(dtype, "norm_slices",
                hipLaunchKernelGGL(norm_slices_words_kernel<TT>, gridw, dim3(256), 0, stream, (const TT*)in, ld, n, s0, s1, eps))
    return launched("norm_slices");
  }
  const dim3 grid((unsigned)n, d1 > 0 ? 2u : 1u);
  GB_BY_DTYPE(dtype, "norm_slices",
              hipLaunchKernelGGL(norm_slices_kernel<TT>, grid, dim3(256), 0, stream, (const TT*)in, ld, s0, s1, eps))
  return launched("norm_slices");
}

// q [n, ldq]: H heads of dim + rdim; kv [n, ldkv]: H key parts of dim, then H value heads of vdim; krot [n, ldr]: the
// shared rdim columns; cos/sin [n, rot / 2] float32; out [n, ldo]: 3 H heads of hd columns; slots (or nullptr) the cache
// rows of the tokens in pages of H heads of hd.
extern "C" int gb_latent_heads(const void* q, int ldq, const void* kv, int ldkv, const void* krot, int ldr, int dtype,
                               const float* cosv, const float* sinv, int rot, void* out, int ldo, int hd,
                               const int32_t* slots, void* k_pages, void* v_pages, int page_size, int n, int H, int dim,
                               int rdim, int vdim, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && H > 0 && dim > 0 && rdim >= 0 && vdim > 0 && hd >= dim + rdim && hd >= vdim,
             "latent_heads: bad sizes heads=%d dim=%d rot_dim=%d vdim=%d head columns=%d", H, dim, rdim, vdim, hd);
  GB_REQUIRE(ldq >= H * (dim + rdim) && ldkv >= H * (dim + vdim) && ldr >= rdim && ldo >= 3 * H * hd,
             "latent_heads: rows shorter than their heads");
  GB_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= rdim && (rot == 0 || (cosv && sinv)), "latent_heads: %d rotated columns of %d",
             rot, rdim);
  GB_REQUIRE(!slots || (k_pages && v_pages && page_size > 0), "latent_heads: cache rows without pages");
  if (n == 0) return 0;
  const long long count = (long long)n * 3 * H * hd;
  GB_REQUIRE(grid_fits(count, 256), "latent_heads: too many elements");
  const int wn = dtype == kBF16 ? 8 : 4;
  // hd a multiple of 8: the pages hold keys in pieces of 8 (key_piece), and a word lies inside one
  if (dim % wn == 0 && rdim % wn == 0 && vdim % wn == 0 && hd % 8 == 0 && (rot / 2) % wn == 0 && ldq % wn == 0 &&
      ldkv % wn == 0 && ldr % wn == 0 && ldo % wn == 0 && words16(q) && words16(kv) && words16(krot) && words16(out) &&
      words16(k_pages)) {
    const dim3 gridw((unsigned)((count / wn + 255) / 256));
    GB_BY_DTYPE(dtype, "latent_heads",
                hipLaunchKernelGGL(latent_heads_words_kernel<TT>, gridw, dim3(256), 0, stream, (const TT*)q, ldq, (const TT*)kv,
                                   ldkv, (const TT*)krot, ldr, cosv, sinv, rot, (TT*)out, ldo, hd, slots, (TT*)k_pages,
                                   (TT*)v_pages, page_size, count / wn, H, dim, rdim, vdim))
    return launched("latent_heads");
  }
  const dim3 grid((unsigned)((count + 255) / 256));
  GB_BY_DTYPE(dtype, "latent_heads",
              hipLaunchKernelGGL(latent_heads_kernel<TT>, grid, dim3(256), 0, stream, (const TT*)q, ldq, (const TT*)kv, ldkv,
                                 (const TT*)krot, ldr, cosv, sinv, rot, (TT*)out, ldo, hd, slots, (TT*)k_pages, (TT*)v_pages,
                                 page_size, count, H, dim, rdim, vdim))
  return launched("latent_heads");
}

// proj [n, ld]: H query heads of 2 dim, G key heads of 2 dim, G value heads of vdim; out [n, ldo]: 2 H query heads, G key
// heads, G value heads, all of hd >= max(2 dim, vdim) columns; every: 0 for no temperature.
extern "C" int gb_diff_heads(const void* proj, int dtype, int ld, const float* wq, const float* wk, float eps, float coef,
                             int every, const int32_t* positions, void* out, int ldo, int hd, const int32_t* slots,
                             void* k_pages, void* v_pages, int page_size, int n, int H, int G, int dim, int vdim,
                             hipStream_t stream) {
  GB_REQUIRE(n >= 0 && H > 0 && G > 0 && dim > 0 && vdim > 0 && hd >= 2 * dim && hd >= vdim,
             "diff_heads: bad sizes heads=%d kv heads=%d dim=%d vdim=%d head columns=%d", H, G, dim, vdim, hd);
  GB_REQUIRE(ld >= (2 * H + 2 * G) * dim + G * vdim && ldo >= (2 * H + 2 * G) * hd, "diff_heads: rows shorter than their heads");
  GB_REQUIRE(wq && wk && every >= 0 && (every == 0 || positions), "diff_heads: weights and positions are needed");
  GB_REQUIRE(!slots || (k_pages && v_pages && page_size > 0), "diff_heads: cache rows without pages");
  if (n == 0) return 0;
  const long long units = (long long)n * (2 * H + 3 * G);
  GB_REQUIRE(grid_fits(units * kLanes, 256), "diff_heads: too many heads");
  const int wn = dtype == kBF16 ? 8 : 4;
  if (dim % wn == 0 && vdim % wn == 0 && hd % 8 == 0 && ld % wn == 0 && ldo % wn == 0 && words16(proj) && words16(out) &&
      words16(k_pages)) {
    if (hd / wn <= 8) {
      const dim3 gridw((unsigned)((units * 8 + 255) / 256));
      GB_BY_DTYPE(dtype, "diff_heads",
                  hipLaunchKernelGGL((diff_heads_words_kernel<TT, 8>), gridw, dim3(256), 0, stream, (const TT*)proj, ld, wq, wk,
                                     eps, coef, every, positions, (TT*)out, ldo, hd, slots, (TT*)k_pages, (TT*)v_pages,
                                     page_size, units, H, G, dim, vdim))
    } else {
      const dim3 gridw((unsigned)((units * 16 + 255) / 256));
      GB_BY_DTYPE(dtype, "diff_heads",
                  hipLaunchKernelGGL((diff_heads_words_kernel<TT, 16>), gridw, dim3(256), 0, stream, (const TT*)proj, ld, wq, wk,
                                     eps, coef, every, positions, (TT*)out, ldo, hd, slots, (TT*)k_pages, (TT*)v_pages,
                                     page_size, units, H, G, dim, vdim))
    }
    return launched("diff_heads");
  }
  const dim3 grid((unsigned)((units * kLanes + 255) / 256));
  GB_BY_DTYPE(dtype, "diff_heads",
              hipLaunchKernelGGL(diff_heads_kernel<TT>, grid, dim3(256), 0, stream, (const TT*)proj, ld, wq, wk, eps, coef,
                                 every, positions, (TT*)out, ldo, hd, slots, (TT*)k_pages, (TT*)v_pages, page_size, units, H, G,
                                 dim, vdim))
  return launched("diff_heads");
}

// att [n, lda]: 2 H heads of hd columns, of the result's type or float32; lambda: one float32 on the device;
// out [n, ldo]: H heads of vdim.
extern "C" int gb_diff_combine(const void* att, int att_dtype, int lda, int hd, const float* lambda, float mult, float eps,
                               void* out, int dtype, int ldo, int n, int H, int vdim, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && H > 0 && vdim > 0 && hd >= vdim && lda >= 2 * H * hd && ldo >= H * vdim && lambda,
             "diff_combine: bad sizes heads=%d vdim=%d head columns=%d", H, vdim, hd);
  GB_REQUIRE(att_dtype == dtype || att_dtype == kF32, "diff_combine: the heads are of the result's type or float32");
  if (n == 0) return 0;
  const long long units = (long long)n * H;
  GB_REQUIRE(grid_fits(units * kLanes, 256), "diff_combine: too many heads");
  const dim3 grid((unsigned)((units * kLanes + 255) / 256));
  if (att_dtype == kF32 && dtype == kBF16) {
    hipLaunchKernelGGL((diff_combine_kernel<float, bf16>), grid, dim3(256), 0, stream, (const float*)att, lda, hd, lambda, mult,
                       eps, (bf16*)out, ldo, units, H, vdim);
    return launched("diff_combine");
  }
  GB_BY_DTYPE(dtype, "diff_combine",
              hipLaunchKernelGGL((diff_combine_kernel<TT, TT>), grid, dim3(256), 0, stream, (const TT*)att, lda, hd, lambda, mult,
                                 eps, (TT*)out, ldo, units, H, vdim))
  return launched("diff_combine");
}

// att [n, lda]: H heads of hd columns; gate [n, ldg]: H * vdim columns; out [n, ldo]: H heads of vdim.
extern "C" int gb_gate_heads(const void* att, int lda, int hd, const void* gate, int ldg, int dtype, void* out, int ldo, int n,
                             int H, int vdim, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && H > 0 && vdim > 0 && hd >= vdim && lda >= H * hd && ldg >= H * vdim && ldo >= H * vdim,
             "gate_heads: bad sizes heads=%d vdim=%d head columns=%d", H, vdim, hd);
  if (n == 0) return 0;
  const long long count = (long long)n * H * vdim;
  GB_REQUIRE(grid_fits(count, 256), "gate_heads: too many elements");
  const int wn = dtype == kBF16 ? 8 : 4;
  if (vdim % wn == 0 && hd % wn == 0 && lda % wn == 0 && ldg % wn == 0 && ldo % wn == 0 && words16(att) && words16(gate) &&
      words16(out)) {
    const dim3 gridw((unsigned)((count / wn + 255) / 256));
    GB_BY_DTYPE(dtype, "gate_heads",
                hipLaunchKernelGGL(gate_heads_words_kernel<TT>, gridw, dim3(256), 0, stream, (const TT*)att, lda, hd,
                                   (const TT*)gate, ldg, (TT*)out, ldo, count / wn, H, vdim))
    return launched("gate_heads");
  }
  const dim3 grid((unsigned)((count + 255) / 256));
  GB_BY_DTYPE(dtype, "gate_heads",
              hipLaunchKernelGGL(gate_heads_kernel<TT>, grid, dim3(256), 0, stream, (const TT*)att, lda, hd, (const TT*)gate,
                                 ldg, (TT*)out, ldo, count, H, vdim))
  return launched("gate_heads");
}

// z [n, ldz], out [n, ldo] of `dtype`; coef: float32 a, b, c, e on the device.
extern "C" int gb_poly_norm(const void* z, int ldz, const float* coef, float eps, void* out, int ldo, int dtype, int n, int d,
                            hipStream_t stream) {
  GB_REQUIRE(n >= 0 && n <= 0x7fffffff && d > 0 && ldz >= d && ldo >= d && coef, "poly_norm: bad sizes n=%d d=%d", n, d);
  if (n == 0) return 0;
  const int wn = dtype == kBF16 ? 8 : 4;
  if (d % wn == 0 && ldz % wn == 0 && ldo % wn == 0 && words16(z) && words16(out) && d <= 2048 * wn) {
    // few rows: four times the threads a row, so that a row's loads are on their way together
    if (n < 512) {
      GB_BY_DTYPE(dtype, "poly_norm",
                  hipLaunchKernelGGL((poly_norm_rows_kernel<TT, 1024, 2>), dim3((unsigned)n), dim3(1024), 0, stream,
                                     (const TT*)z, ldz, coef, eps, (TT*)out, ldo, d))
    } else {
      GB_BY_DTYPE(dtype, "poly_norm",
                  hipLaunchKernelGGL((poly_norm_rows_kernel<TT, 256, 8>), dim3((unsigned)n), dim3(256), 0, stream,
                                     (const TT*)z, ldz, coef, eps, (TT*)out, ldo, d))
    }
    return launched("poly_norm");
  }
  GB_BY_DTYPE(dtype, "poly_norm",
              hipLaunchKernelGGL(poly_norm_kernel<TT>, dim3((unsigned)n), dim3(256), 0, stream, (const TT*)z, ldz, coef, eps,
                                 (TT*)out, ldo, d))
  return launched("poly_norm");
}

// x, y [n, d] float32, g one float32 on the device; rounded (or nullptr) [n, d] of `dtype` receives the new x.
// slices > 1: y is the sum of that many [n, d] pieces, slice_stride floats apart.  conv_w (float32 [taps, d]; a step in
// which every request brings one row): rounded receives x + conv(x) of the new x, and the requests' slots in
// state [slots, taps - 1, d] are moved on by this row.
extern "C" int gb_norm_add(float* x, const float* y, int slices, long long slice_stride, const float* g, float eps,
                           void* rounded, int dtype, int n, int d, const float* conv_w, int taps, float* state,
                           const int32_t* tok_seq, const int32_t* pos0, const int32_t* state_slots, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && n <= 0x7fffffff && d > 0 && x && y && g, "norm_add: bad sizes n=%d d=%d", n, d);
  GB_REQUIRE(slices >= 1 && (slices == 1 || slice_stride >= (long long)n * d), "norm_add: %d slices", slices);
  GB_REQUIRE(!conv_w || (rounded && taps >= 1 && taps <= kMaxTaps && tok_seq && pos0 && state_slots && (taps == 1 || state)),
             "norm_add: the convolution needs a result, weights of at most %d taps, the step's tables and the state", kMaxTaps);
  if (n == 0) return 0;
  const bool words = d % 4 == 0 && d <= 8192 && words16(x) && words16(y) && words16(rounded) && words16(state) && words16(conv_w) &&
                     slice_stride % 4 == 0;
  GB_REQUIRE(words || (slices == 1 && !conv_w), "norm_add: slices and the convolution take rows of at most 8192 columns, a multiple of 4");
  if (words) {
    if (n < 512) {
      GB_BY_DTYPE(dtype, "norm_add",
                  hipLaunchKernelGGL((norm_add_rows_kernel<TT, 1024, 2>), dim3((unsigned)n), dim3(1024), 0, stream, x, y, slices,
                                     slice_stride, g, eps, (TT*)rounded, d, conv_w, taps, state, tok_seq, pos0, state_slots))
    } else {
      GB_BY_DTYPE(dtype, "norm_add",
                  hipLaunchKernelGGL((norm_add_rows_kernel<TT, 256, 8>), dim3((unsigned)n), dim3(256), 0, stream, x, y, slices,
                                     slice_stride, g, eps, (TT*)rounded, d, conv_w, taps, state, tok_seq, pos0, state_slots))
    }
    return launched("norm_add");
  }
  GB_BY_DTYPE(dtype, "norm_add",
              hipLaunchKernelGGL(norm_add_kernel<TT>, dim3((unsigned)n), dim3(256), 0, stream, x, y, g, eps, (TT*)rounded, d))
  return launched("norm_add");
}

GB_TAPED(gb_time_conv)
GB_TAPED(gb_norm_slices)
GB_TAPED(gb_latent_heads)
GB_TAPED(gb_diff_heads)
GB_TAPED(gb_diff_combine)
GB_TAPED(gb_gate_heads)
GB_TAPED(gb_poly_norm)
GB_TAPED(gb_norm_add)
