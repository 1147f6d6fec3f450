// Kernels of layers whose norms are bounded, statistic-free maps, and of attention mixers whose query and key heads
// are prepared in one pass (bias, short convolution over time, RMS norm over the whole projection or head by head,
// rotation of a part of each head in either pairing) and whose heads are gated before the output product.
//
//   tanh_norm:      out = tanh(alpha x) * w + b                         (alpha one number; no mean, no variance)
//   tanh_norm_add:  x += tanh(alpha y) * w + b, and, where the norm that reads x next is of the same kind,
//                   h = tanh(alpha' x) * w' + b' in the same pass
//   qk_heads:       a token's query, key and value heads as attention reads them, from its stacked projections
//   conv_state:     the last taps - 1 projections of each request, kept for the step that follows
//   gate_rows:      heads times sigmoid(gate), one gate a head or one a channel
//
// All arithmetic is 32-bit; a result is rounded once, when it is stored.
#include "common.h"

using namespace gb;

GB_DEFINE_LAST_ERROR

namespace {

constexpr int kMaxTaps = 8;

template <typename O>
__global__ __launch_bounds__(256) void tanh_norm_kernel(const float* __restrict__ x, int ldx, const int32_t* __restrict__ rows,
                                                        const float* __restrict__ alpha, const float* __restrict__ w,
                                                        const float* __restrict__ b, O* __restrict__ out, int ldo,
                                                        long long count, int d) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= count) return;
  const long long r = idx / d;
  const int c = (int)(idx % d);
  const long long src = rows ? rows[r] : r;
  const float v = x[src * ldx + c];
  out[r * ldo + c] = from_f<O>(fmaf(tanhf(alpha[0] * v), w[c], b[c]));
}

template <typename O>
__global__ __launch_bounds__(256) void tanh_norm_add_kernel(float* __restrict__ x, const float* __restrict__ y, int slices,
                                                            long long slice_stride, const float* __restrict__ alpha,
                                                            const float* __restrict__ w, const float* __restrict__ b,
                                                            const float* __restrict__ alpha2, const float* __restrict__ w2,
                                                            const float* __restrict__ b2, O* __restrict__ h, long long count,
                                                            int d) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= count) return;
  const int c = (int)(idx % d);
  float v = y[idx];
  for (int s = 1; s < slices; ++s) v += y[idx + s * slice_stride];
  const float r = x[idx] + fmaf(tanhf(alpha[0] * v), w[c], b[c]);
  x[idx] = r;
  if (h) h[idx] = from_f<O>(fmaf(tanhf(alpha2[0] * r), w2[c], b2[c]));
}

// Four columns a thread (rows of whole 16-byte words): the forms that steps of many rows take.
__device__ __forceinline__ void store4(float* p, const f32x4& v) { *reinterpret_cast<f32x4*>(p) = v; }
__device__ __forceinline__ void store4(bf16* p, const f32x4& v) {
  bf16x4 o;
#pragma unroll
  for (int e = 0; e < 4; ++e) o[e] = (bf16)v[e];
  *reinterpret_cast<bf16x4*>(p) = o;
}

template <typename O>
__global__ __launch_bounds__(256) void tanh_norm_words_kernel(const float* __restrict__ x, int ldx, const int32_t* __restrict__ rows,
                                                              const float* __restrict__ alpha, const float* __restrict__ w,
                                                              const float* __restrict__ b, O* __restrict__ out, int ldo,
                                                              long long count, int words) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= count) return;
  const long long r = idx / words;
  const int c = (int)(idx % words) * 4;
  const long long src = rows ? rows[r] : r;
  const f32x4 v = *reinterpret_cast<const f32x4*>(x + src * ldx + c);
  const f32x4 ww = *reinterpret_cast<const f32x4*>(w + c), bb = *reinterpret_cast<const f32x4*>(b + c);
  const float a = alpha[0];
  f32x4 o;
#pragma unroll
  for (int e = 0; e < 4; ++e) o[e] = fmaf(tanhf(a * v[e]), ww[e], bb[e]);
  store4(out + r * ldo + c, o);
}

template <typename O>
__global__ __launch_bounds__(256) void tanh_norm_add_words_kernel(float* __restrict__ x, const float* __restrict__ y, int slices,
                                                                  long long slice_stride, const float* __restrict__ alpha,
                                                                  const float* __restrict__ w, const float* __restrict__ b,
                                                                  const float* __restrict__ alpha2, const float* __restrict__ w2,
                                                                  const float* __restrict__ b2, O* __restrict__ h, long long count,
                                                                  int words) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= count) return;
  const int c = (int)(idx % words) * 4;
  const long long at = idx * 4;
  f32x4 v = *reinterpret_cast<const f32x4*>(y + at);
  for (int s = 1; s < slices; ++s) v += *reinterpret_cast<const f32x4*>(y + at + s * slice_stride);
  const f32x4 ww = *reinterpret_cast<const f32x4*>(w + c), bb = *reinterpret_cast<const f32x4*>(b + c);
  f32x4 r = *reinterpret_cast<const f32x4*>(x + at);
  const float a = alpha[0];
#pragma unroll
  for (int e = 0; e < 4; ++e) r[e] += fmaf(tanhf(a * v[e]), ww[e], bb[e]);
  *reinterpret_cast<f32x4*>(x + at) = r;
  if (h) {
    const f32x4 w2v = *reinterpret_cast<const f32x4*>(w2 + c), b2v = *reinterpret_cast<const f32x4*>(b2 + c);
    const float a2 = alpha2[0];
    f32x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = fmaf(tanhf(a2 * r[e]), w2v[e], b2v[e]);
    store4(h + at, o);
  }
}

// One workgroup a (token, query or key head).  A row of `proj` holds nh query heads and nkv key heads of dk channels, then
// (unless the values are the keys) nkv value heads of dv, then whatever else the product made (gates), which is not read
// here.  A key head's workgroup also makes the value head of its number.
//   1. bias, and with taps > 0 the convolution (wconv a row a tap, [taps, channels]) over the request's earlier rows of
//      this step and its state slot ([taps - 1, channels] float32, index i = the position `first position of the step` -
//      (taps - 1) + i);
//   2. tied values: the key channels as they stand now are the value heads (dv = dk);
//   3. RMS norm: joint = over all query channels at once (and all key channels), weights [nh dk] and [nkv dk]: the
//      sums of squares come from `sums` ([n, 2], made by row_squares_kernel for steps of many rows), or every
//      workgroup adds up the squares of all channels of its kind for itself (no convolution then); else head by head
//      over dk, weights [dk] that all heads share;
//   4. the first `rot` channels of every query and key head turn by the step's angles (cos, sin [n, rot / 2], times
//      mag): neighbours = channel 2i with 2i + 1, else channel i with i + rot / 2;
//   5. heads of hd >= max(dk, dv) columns in `out`, zeros beyond their channels; with `slots` keys and values also go
//      to their pages.
// `single` (every request brings one row): the thread that reads a channel's slot also moves it on by one.
template <typename T>
__global__ void qk_heads_kernel(
    const T* __restrict__ proj, int ld, const float* __restrict__ bias, const float* __restrict__ wconv, int taps,
    float* __restrict__ state, const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ pos0, const int32_t* __restrict__ state_slots, int single, const float* __restrict__ wq,
    const float* __restrict__ wk, float eps, int joint, const float* __restrict__ cosv, const float* __restrict__ sinv, int rot,
    float mag, int neighbours, int tied, T* __restrict__ out, int ldo, int hd, const int32_t* __restrict__ slots,
    T* __restrict__ k_pages, T* __restrict__ v_pages, int page_size, int nh, int nkv, int dk, int dv,
    const float* __restrict__ sums) {
  extern __shared__ float lds[];
  const int qd = nh * dk, kd = nkv * dk, channels = qd + kd, heads = nh + nkv;
  float* vals = lds;              // [dk]: the head's channels after step 1
  float* scratch = vals + dk;     // [17]
  const int t = blockIdx.x / heads, u = blockIdx.x % heads, tid = threadIdx.x, step = blockDim.x;
  const bool is_q = u < nh;
  const int ch0 = u * dk;         // (query heads, then key heads, lie side by side in a row)
  const T* row = proj + (size_t)t * ld;
  const int K = taps > 0 ? taps - 1 : 0;
  int off = 0, first_pos = 0;
  float* st = nullptr;
  if (taps > 0) {
    const int seq = single ? t : tok_seq[t];      // (every request one row: row t is request t's)
    off = single ? 0 : t - q_start[seq];
    first_pos = pos0[seq];
    if (K > 0) st = state + (size_t)state_slots[seq] * K * channels;
  }
  float ss = 0.f;
  for (int c = tid; c < dk; c += step) {
    const int ch = ch0 + c;
    const float b = bias ? bias[ch] : 0.f;
    float v;
    if (taps == 0) {
      v = to_f(row[ch]) + b;
    } else {
      float old[kMaxTaps - 1];
#pragma unroll
      for (int i = 0; i < kMaxTaps - 1; ++i) old[i] = (i < K && (single || i >= off)) ? st[(size_t)i * channels + ch] : 0.f;
      v = 0.f;
#pragma unroll
      for (int jt = 0; jt < kMaxTaps; ++jt) {
        if (jt >= taps) break;
        const int back = K - jt;   // how many tokens before this one
        float x = 0.f;
        if (off >= back) {
          x = to_f(proj[(size_t)(t - back) * ld + ch]) + b;
        } else if (first_pos + off - back >= 0) {
#pragma unroll
          for (int i = 0; i < kMaxTaps - 1; ++i)
            if (i == off + jt) x = old[i];
        }
        v = fmaf(wconv[(size_t)jt * channels + ch], x, v);
      }
      if (single && K > 0) {
#pragma unroll
        for (int i = 0; i < kMaxTaps - 1; ++i)
          if (i < K) st[(size_t)i * channels + ch] = i + 1 < K ? old[i + 1 < kMaxTaps - 1 ? i + 1 : 0] : to_f(row[ch]) + b;
      }
    }
    vals[c] = v;
    ss = fmaf(v, v, ss);
  }
  float inv;
  if (joint && sums) {
    __syncthreads();   // (vals are written)
    inv = 1.0f / sqrtf(sums[2 * (size_t)t + (is_q ? 0 : 1)] / (float)(is_q ? qd : kd) + eps);
  } else if (joint) {   // the squares of every channel of the kind, in one order for all of the kind's workgroups
    const int first = is_q ? 0 : qd, count = is_q ? qd : kd;
    float all = 0.f;
    for (int c = tid; c < count; c += step) {
      const float v = to_f(row[first + c]) + (bias ? bias[first + c] : 0.f);
      all = fmaf(v, v, all);
    }
    inv = 1.0f / sqrtf(block_sum(all, scratch) / (float)count + eps);
  } else {
    inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)dk + eps);
  }   // (the barriers inside also order the writes of vals before the reads below)
  const int slot = slots ? slots[t] : -1;
  const int piece = key_piece(hd);
  const int half = rot / 2;
  const float* wn = is_q ? wq : wk;
  const int wbase = joint ? (is_q ? u : u - nh) * dk : 0;
  T* orow = out + (size_t)t * ldo + (size_t)u * hd;
  T* kb = (slot >= 0 && !is_q) ? k_pages + ((size_t)(slot / page_size) * nkv + (u - nh)) * (size_t)page_size * hd : nullptr;
  for (int c = tid; c < hd; c += step) {
    float r = 0.f;
    if (c < dk) {
      r = vals[c] * inv * (wn ? wn[wbase + c] : 1.f);
      if (c < rot) {
        const int pc = neighbours ? (c ^ 1) : (c < half ? c + half : c - half);
        const int i = neighbours ? c / 2 : (c < half ? c : c - half);
        const bool lead = neighbours ? !(c & 1) : c < half;
        const float p = vals[pc] * inv * (wn ? wn[wbase + pc] : 1.f);
        const float cs = cosv[(size_t)t * half + i] * mag, sn = sinv[(size_t)t * half + i] * mag;
        r = lead ? r * cs - p * sn : r * cs + p * sn;
      }
    }
    const T o = from_f<T>(r);
    orow[c] = o;
    if (kb) kb[key_offset(slot % page_size, c, page_size, piece)] = o;
  }
  if (is_q) return;
  const int g = u - nh;
  T* vrow = out + (size_t)t * ldo + (size_t)(heads + g) * hd;
  T* vb = slot >= 0 ? v_pages + ((size_t)(slot / page_size) * nkv + g) * (size_t)page_size * hd : nullptr;
  for (int c = tid; c < hd; c += step) {
    float r = 0.f;
    if (c < dv) r = tied ? vals[c] : to_f(row[channels + g * dv + c]) + (bias ? bias[channels + g * dv + c] : 0.f);
    const T o = from_f<T>(r);
    vrow[c] = o;
    if (vb) vb[(size_t)c * page_size + slot % page_size] = o;
  }
}

__device__ __forceinline__ void load8f(const float* __restrict__ p, float (&x)[8]) {   // p at a 16-byte word
  const f32x4 lo = *reinterpret_cast<const f32x4*>(p), hi = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
  for (int e = 0; e < 4; ++e) x[e] = lo[e], x[4 + e] = hi[e];
}

// The same for bfloat16 heads made of whole groups of eight channels: a lane takes eight neighbouring channels of a
// (token, head) as one 16-byte word, `lanes` lanes a head (a power of two that covers hd / 8; the lanes beyond the
// head's words idle), so a wave takes several heads and a head's sum of squares and rotation partners are a few
// moves between lanes away.  With halves that pair up, rot / 2 is a multiple of 8 (a partner's word is another
// lane's word); with one norm over a row, `sums` holds the rows' sums of squares.
__global__ __launch_bounds__(256) void qk_heads_words_kernel(
    const bf16* __restrict__ proj, int ld, const float* __restrict__ bias, const float* __restrict__ wconv, int taps,
    float* __restrict__ state, const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ pos0, const int32_t* __restrict__ state_slots, int single, const float* __restrict__ wq,
    const float* __restrict__ wk, float eps, int joint, const float* __restrict__ cosv, const float* __restrict__ sinv, int rot,
    float mag, int neighbours, int tied, bf16* __restrict__ out, int ldo, int hd, const int32_t* __restrict__ slots,
    bf16* __restrict__ k_pages, bf16* __restrict__ v_pages, int page_size, int nh, int nkv, int dk, int dv,
    const float* __restrict__ sums, int lanes, long long units) {
  const int qd = nh * dk, kd = nkv * dk, channels = qd + kd, heads = nh + nkv;
  const long long gl = (long long)blockIdx.x * 256 + threadIdx.x;
  const long long unit = gl / lanes;
  const int li = (int)(gl % lanes), lane = threadIdx.x % kWave;
  const bool live = unit < units;
  const int t = live ? (int)(unit / heads) : 0, u = live ? (int)(unit % heads) : 0;
  const bool is_q = u < nh;
  const int c0 = li * 8, ch = u * dk + c0;
  const bool has = live && c0 < dk;
  const bf16* row = proj + (size_t)t * ld;
  float b[8], v[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) b[e] = 0.f, v[e] = 0.f;
  if (has && bias) load8f(bias + ch, b);
  if (has && taps == 0) {
    const bf16x8 x = *reinterpret_cast<const bf16x8*>(row + ch);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (float)x[e] + b[e];
  } else if (has) {
    // (every request one row: row t is request t's)
    const int K = taps - 1, seq = single ? t : tok_seq[t], off = single ? 0 : t - q_start[seq], first_pos = pos0[seq];
    float* st = K > 0 ? state + (size_t)state_slots[seq] * K * channels + ch : nullptr;
    for (int jt = 0; jt < taps; ++jt) {
      const int back = K - jt;   // how many tokens before this one
      float x[8];
      if (off >= back) {
        const bf16x8 w8 = *reinterpret_cast<const bf16x8*>(proj + (size_t)(t - back) * ld + ch);
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = (float)w8[e] + b[e];
      } else if (first_pos + off - back >= 0) {
        load8f(st + (size_t)(off + jt) * channels, x);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = 0.f;
      }
      float wt[8];
      load8f(wconv + (size_t)jt * channels + ch, wt);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = fmaf(wt[e], x[e], v[e]);
    }
    if (single && K > 0) {   // the slot moves on by one: entry i takes entry i + 1, the last one this row's projections
      for (int i = 0; i + 1 < K; ++i) {
        float* sp = st + (size_t)i * channels;
        const f32x4 lo = *reinterpret_cast<const f32x4*>(sp + channels), hi = *reinterpret_cast<const f32x4*>(sp + channels + 4);
        *reinterpret_cast<f32x4*>(sp) = lo;
        *reinterpret_cast<f32x4*>(sp + 4) = hi;
      }
      const bf16x8 x = *reinterpret_cast<const bf16x8*>(row + ch);
      f32x4 lo, hi;
#pragma unroll
      for (int e = 0; e < 4; ++e) lo[e] = (float)x[e] + b[e], hi[e] = (float)x[4 + e] + b[4 + e];
      float* sp = st + (size_t)(K - 1) * channels;
      *reinterpret_cast<f32x4*>(sp) = lo;
      *reinterpret_cast<f32x4*>(sp + 4) = hi;
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) ss = fmaf(v[e], v[e], ss);
  for (int o = lanes / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, kWave);
  const float inv = joint ? 1.0f / sqrtf(sums[2 * (size_t)t + (is_q ? 0 : 1)] / (float)(is_q ? qd : kd) + eps)
                          : 1.0f / sqrtf(ss / (float)dk + eps);
  const float* wn = is_q ? wq : wk;
  const int wbase = (joint ? (is_q ? u : u - nh) * dk : 0) + c0;
  float r[8], g8[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) g8[e] = 1.f;
  if (has && wn) load8f(wn + wbase, g8);
#pragma unroll
  for (int e = 0; e < 8; ++e) r[e] = has ? v[e] * inv * g8[e] : 0.f;
  const int half = rot / 2;
  if (rot > 0 && neighbours) {
#pragma unroll
    for (int e = 0; e < 8; e += 2) {
      if (has && c0 + e < rot) {
        const float cs = cosv[(size_t)t * half + (c0 + e) / 2] * mag, sn = sinv[(size_t)t * half + (c0 + e) / 2] * mag;
        const float a = r[e], p = r[e + 1];
        r[e] = a * cs - p * sn;
        r[e + 1] = p * cs + a * sn;
      }
    }
  } else if (rot > 0) {   // the word's partner is the word half a rotation away: another lane's
    const bool lead = c0 < half, turns = c0 < rot;
    const int partner = lane + (lead ? half / 8 : -(half / 8));
    float p[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) p[e] = __shfl(r[e], turns ? partner : lane, kWave);
    if (has && turns) {
      const int i0 = lead ? c0 : c0 - half;   // (half is a multiple of 8: the angles of a word are two words)
      float c8[8], s8[8];
      load8f(cosv + (size_t)t * half + i0, c8);
      load8f(sinv + (size_t)t * half + i0, s8);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float cs = c8[e] * mag, sn = s8[e] * mag;
        r[e] = lead ? r[e] * cs - p[e] * sn : r[e] * cs + p[e] * sn;
      }
    }
  }
  if (!live || c0 >= hd) return;
  const int slot = slots ? slots[t] : -1;
  bf16x8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = (bf16)r[e];
  *reinterpret_cast<bf16x8*>(out + (size_t)t * ldo + (size_t)u * hd + c0) = o;
  if (is_q) return;
  const int g = u - nh;
  if (slot >= 0) {   // (hd is a multiple of 8: a key's pieces are words of eight)
    bf16* kb = k_pages + ((size_t)(slot / page_size) * nkv + g) * (size_t)page_size * hd;
    *reinterpret_cast<bf16x8*>(kb + ((size_t)(c0 / 8) * page_size + slot % page_size) * 8) = o;
  }
  bf16x8 val;
  if (c0 < dv) {
    if (tied) {
#pragma unroll
      for (int e = 0; e < 8; ++e) val[e] = (bf16)v[e];
    } else {
      const bf16x8 x = *reinterpret_cast<const bf16x8*>(row + channels + g * dv + c0);
#pragma unroll
      for (int e = 0; e < 8; ++e) val[e] = (bf16)((float)x[e] + (bias ? bias[channels + g * dv + c0 + e] : 0.f));
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) val[e] = (bf16)0.f;
  }
  *reinterpret_cast<bf16x8*>(out + (size_t)t * ldo + (size_t)(heads + g) * hd + c0) = val;
  if (slot >= 0) {
    bf16* vb = v_pages + ((size_t)(slot / page_size) * nkv + g) * (size_t)page_size * hd + slot % page_size;
#pragma unroll
    for (int e = 0; e < 8; ++e) vb[(size_t)(c0 + e) * page_size] = val[e];
  }
}

// sums[t] = (sum of squares of the query channels, of the key channels) of row t, bias added; a workgroup a row.
template <typename T>
__global__ __launch_bounds__(256) void row_squares_kernel(const T* __restrict__ proj, int ld, const float* __restrict__ bias, int qd,
                                                          int kd, float* __restrict__ sums) {
  __shared__ float scratch[17];
  const int t = blockIdx.x;
  const T* row = proj + (size_t)t * ld;
  float sq = 0.f, sk = 0.f;
  if (std::is_same<T, bf16>::value && qd % 8 == 0 && kd % 8 == 0 && ld % 8 == 0 && (uintptr_t)proj % 16 == 0 && (uintptr_t)bias % 16 == 0) {
    for (int c = threadIdx.x * 8; c < qd + kd; c += 256 * 8) {   // a word of eight channels a thread
      const bf16x8 x = *reinterpret_cast<const bf16x8*>(reinterpret_cast<const bf16*>(row) + c);
      float b[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) b[e] = 0.f;
      if (bias) load8f(bias + c, b);
      float part = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float v = (float)x[e] + b[e];
        part = fmaf(v, v, part);
      }
      if (c < qd) sq += part; else sk += part;
    }
  } else {
    for (int c = threadIdx.x; c < qd + kd; c += 256) {
      const float v = to_f(row[c]) + (bias ? bias[c] : 0.f);
      if (c < qd) sq = fmaf(v, v, sq); else sk = fmaf(v, v, sk);
    }
  }
  sq = block_sum(sq, scratch);
  sk = block_sum(sk, scratch);
  if (threadIdx.x == 0) {
    sums[2 * (size_t)t] = sq;
    sums[2 * (size_t)t + 1] = sk;
  }
}

// After a step with portions: slot index i of a request becomes the projection at position `end of the step` - K + i,
// from the step's rows where it lies among them, else from the slot as it was (K = taps - 1).  A thread a (request,
// channel) walks i upwards, so it reads every old entry before it writes over it.
template <typename T>
__global__ __launch_bounds__(256) void conv_state_kernel(const T* __restrict__ proj, int ld, const float* __restrict__ bias,
                                                         float* __restrict__ state, const int32_t* __restrict__ q_start,
                                                         const int32_t* __restrict__ q_len,
                                                         const int32_t* __restrict__ state_slots, int n_seqs, int channels,
                                                         int K) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long long)n_seqs * channels) return;
  const int s = (int)(idx / channels), ch = (int)(idx % channels);
  const int start = q_start[s], len = q_len[s];
  float* st = state + (size_t)state_slots[s] * K * channels;
  for (int i = 0; i < K; ++i) {
    const int r = len - K + i;   // row of the step's portion that holds the position, if not negative
    float v;
    if (r >= 0) v = to_f(proj[(size_t)(start + r) * ld + ch]) + (bias ? bias[ch] : 0.f);
    else v = st[(size_t)(i + len) * channels + ch];
    st[(size_t)i * channels + ch] = v;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gate_rows_kernel(const T* __restrict__ att, int lda, int hd, const T* __restrict__ gate,
                                                        int ldg, int per_head, T* __restrict__ out, int ldo, long long count,
                                                        int nh, int dv) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= count) return;
  const int cols = nh * dv;
  const long long t = idx / cols;
  const int j = (int)(idx % cols), h = j / dv, c = j % dv;
  const float g = to_f(gate[t * ldg + (per_head ? h : j)]);
  out[t * ldo + j] = from_f<T>(to_f(att[t * lda + (size_t)h * hd + c]) / (1.0f + expf(-g)));
}

// Eight channels a thread: bfloat16 heads whose rows and heads begin at 16-byte words.
__global__ __launch_bounds__(256) void gate_rows_words_kernel(const bf16* __restrict__ att, int lda, int hd, const bf16* __restrict__ gate,
                                                              int ldg, int per_head, bf16* __restrict__ out, int ldo, long long count,
                                                              int nh, int dv) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= count) return;
  const int words = nh * dv / 8;
  const long long t = idx / words;
  const int j = (int)(idx % words) * 8, h = j / dv, c = j % dv;
  const bf16x8 a = *reinterpret_cast<const bf16x8*>(att + t * lda + (size_t)h * hd + c);
  bf16x8 o;
  if (per_head) {
    const float g = 1.0f / (1.0f + expf(-(float)gate[t * ldg + h]));
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (bf16)((float)a[e] * g);
  } else {
    const bf16x8 g = *reinterpret_cast<const bf16x8*>(gate + t * ldg + j);
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (bf16)((float)a[e] / (1.0f + expf(-(float)g[e])));
  }
  *reinterpret_cast<bf16x8*>(out + t * ldo + j) = o;
}

inline bool grid_fits(long long count) { return (count + 255) / 256 < (1ll << 31); }
inline bool words16(const void* p) { return (uintptr_t)p % 16 == 0; }

}  // namespace

extern "C" int gb_tanh_norm(const float* x, int ldx, const int32_t* rows, const float* alpha, const float* w, const float* b,
                            void* out, int out_dtype, int ldo, int n, int d, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && d > 0 && ldx >= d && ldo >= d, "tanh_norm: bad sizes n=%d d=%d (strides %d, %d)", n, d, ldx, ldo);
  GB_REQUIRE(alpha && w && b, "tanh_norm: the norm's number, weight and bias are needed");
  if (n == 0) return 0;
  const long long count = (long long)n * d;
  GB_REQUIRE(grid_fits(count), "tanh_norm: too many elements");
  if (d % 4 == 0 && ldx % 4 == 0 && ldo % 4 == 0 && words16(x) && words16(out) && words16(w) && words16(b) &&
      (out_dtype == kF32 || out_dtype == kBF16)) {
    const dim3 wgrid((unsigned)((count / 4 + 255) / 256));
    if (out_dtype == kF32)
      hipLaunchKernelGGL(tanh_norm_words_kernel<float>, wgrid, dim3(256), 0, stream, x, ldx, rows, alpha, w, b, (float*)out, ldo, count / 4, d / 4);
    else
      hipLaunchKernelGGL(tanh_norm_words_kernel<bf16>, wgrid, dim3(256), 0, stream, x, ldx, rows, alpha, w, b, (bf16*)out, ldo, count / 4, d / 4);
    return launched("tanh_norm");
  }
  const dim3 grid((unsigned)((count + 255) / 256));
  if (out_dtype == kF32)
    hipLaunchKernelGGL(tanh_norm_kernel<float>, grid, dim3(256), 0, stream, x, ldx, rows, alpha, w, b, (float*)out, ldo, count, d);
  else if (out_dtype == kBF16)
    hipLaunchKernelGGL(tanh_norm_kernel<bf16>, grid, dim3(256), 0, stream, x, ldx, rows, alpha, w, b, (bf16*)out, ldo, count, d);
  else
    return fail("tanh_norm: unknown dtype %d", out_dtype);
  return launched("tanh_norm");
}

// x [n, d] += norm(y); y [slices][n, d] (slice_stride floats apart) is added up in the slices' order first.  With h:
// h [n, d] = norm2(new x) in h_dtype.
extern "C" int gb_tanh_norm_add(float* x, const float* y, int slices, long long slice_stride, const float* alpha, const float* w,
                                const float* b, const float* alpha2, const float* w2, const float* b2, void* h, int h_dtype,
                                int n, int d, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && d > 0 && slices >= 1, "tanh_norm_add: bad sizes n=%d d=%d slices=%d", n, d, slices);
  GB_REQUIRE(alpha && w && b && (!h || (alpha2 && w2 && b2)), "tanh_norm_add: a norm's number, weight and bias are needed");
  if (n == 0) return 0;
  const long long count = (long long)n * d;
  GB_REQUIRE(grid_fits(count), "tanh_norm_add: too many elements");
  GB_REQUIRE(slices == 1 || slice_stride >= count, "tanh_norm_add: slices %lld floats apart hold %lld", slice_stride, count);
  if (d % 4 == 0 && (slices == 1 || slice_stride % 4 == 0) && words16(x) && words16(y) && words16(w) && words16(b) &&
      (!h || (words16(h) && words16(w2) && words16(b2))) && (h_dtype == kF32 || h_dtype == kBF16)) {
    const dim3 wgrid((unsigned)((count / 4 + 255) / 256));
    if (h_dtype == kF32)
      hipLaunchKernelGGL(tanh_norm_add_words_kernel<float>, wgrid, dim3(256), 0, stream, x, y, slices, slice_stride, alpha, w, b, alpha2,
                         w2, b2, (float*)h, count / 4, d / 4);
    else
      hipLaunchKernelGGL(tanh_norm_add_words_kernel<bf16>, wgrid, dim3(256), 0, stream, x, y, slices, slice_stride, alpha, w, b, alpha2,
                         w2, b2, (bf16*)h, count / 4, d / 4);
    return launched("tanh_norm_add");
  }
  const dim3 grid((unsigned)((count + 255) / 256));
  if (h_dtype == kF32)
    hipLaunchKernelGGL(tanh_norm_add_kernel<float>, grid, dim3(256), 0, stream, x, y, slices, slice_stride, alpha, w, b, alpha2, w2,
                       b2, (float*)h, count, d);
  else if (h_dtype == kBF16)
    hipLaunchKernelGGL(tanh_norm_add_kernel<bf16>, grid, dim3(256), 0, stream, x, y, slices, slice_stride, alpha, w, b, alpha2, w2,
                       b2, (bf16*)h, count, d);
  else
    return fail("tanh_norm_add: unknown dtype %d", h_dtype);
  return launched("tanh_norm_add");
}

// flags: 1 = every request brings one row (the slots are moved on here), 2 = one norm over all query (key) channels,
// 4 = neighbouring channels pair up, 8 = the values are the keys; the bits from 256 on are the taps.
// sums: with flag 2, 2 n floats of scratch for the rows' sums of squares (made here, in a pass of its own), or null:
// every workgroup then adds up its row for itself, which steps of few rows do.
extern "C" int gb_qk_heads(const void* proj, int dtype, int ld, const float* bias, const float* wconv, float* sums, float* state,
                           const int32_t* tok_seq, const int32_t* q_start, const int32_t* pos0, const int32_t* state_slots,
                           int flags, const float* wq, const float* wk, float eps, const float* cosv, const float* sinv, int rot,
                           float mag, void* out, int ldo, int hd, const int32_t* slots, void* k_pages, void* v_pages,
                           int page_size, int n, int nh, int nkv, int dk, int dv, hipStream_t stream) {
  const int single = flags & 1, joint = (flags >> 1) & 1, neighbours = (flags >> 2) & 1, tied = (flags >> 3) & 1, taps = flags >> 8;
  GB_REQUIRE(n >= 0 && nh > 0 && nkv > 0 && dk > 0 && dv > 0 && hd >= dk && hd >= dv, "qk_heads: bad sizes nh=%d nkv=%d dk=%d dv=%d hd=%d", nh, nkv, dk, dv, hd);
  GB_REQUIRE(!tied || dv == dk, "qk_heads: values that are the keys have the keys' size (dk=%d, dv=%d)", dk, dv);
  const int channels = (nh + nkv) * dk;
  GB_REQUIRE(ld >= channels + (tied ? 0 : nkv * dv) && ldo >= (nh + 2 * nkv) * hd, "qk_heads: rows shorter than the heads");
  GB_REQUIRE(taps >= 0 && taps <= kMaxTaps, "qk_heads: %d taps (at most %d)", taps, kMaxTaps);
  GB_REQUIRE(taps == 0 || (wconv && tok_seq && q_start && pos0 && (taps == 1 || (state && state_slots))),
             "qk_heads: a convolution needs its weights, the step's requests and their state");
  GB_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= dk && (rot == 0 || (cosv && sinv)), "qk_heads: %d rotated channels of %d", rot, dk);
  GB_REQUIRE(!slots || (k_pages && v_pages && page_size > 0), "qk_heads: cache rows without pages");
  GB_REQUIRE(!(joint && taps > 0), "qk_heads: one norm over all channels behind a convolution is not served");
  GB_REQUIRE((long long)n * (nh + nkv) < (1ll << 31), "qk_heads: too many (token, head) pairs");
  const size_t lds = sizeof(float) * ((size_t)dk + 17);
  const int most = hd > dk ? hd : dk;
  const int threads = most <= 64 ? 64 : most <= 128 ? 128 : 256;
  if (n == 0) return 0;
  if (!joint) sums = nullptr;
  if (sums) {
    if (dtype == kF32)
      hipLaunchKernelGGL(row_squares_kernel<float>, dim3((unsigned)n), dim3(256), 0, stream, (const float*)proj, ld, bias, nh * dk, nkv * dk, sums);
    else if (dtype == kBF16)
      hipLaunchKernelGGL(row_squares_kernel<bf16>, dim3((unsigned)n), dim3(256), 0, stream, (const bf16*)proj, ld, bias, nh * dk, nkv * dk, sums);
  }
  const int half = rot / 2;
  if (dtype == kBF16 && dk % 8 == 0 && dv % 8 == 0 && hd % 8 == 0 && ld % 8 == 0 && ldo % 8 == 0 && (uintptr_t)proj % 16 == 0 &&
      (uintptr_t)out % 16 == 0 && (neighbours || rot == 0 || half % 8 == 0) && (!joint || sums) && hd <= 256 &&
      (!state || (uintptr_t)state % 16 == 0) && (!slots || (uintptr_t)k_pages % 16 == 0) && (uintptr_t)bias % 16 == 0 &&
      (uintptr_t)wconv % 16 == 0 && (uintptr_t)wq % 16 == 0 && (uintptr_t)wk % 16 == 0 && (uintptr_t)cosv % 16 == 0 &&
      (uintptr_t)sinv % 16 == 0) {
    int lanes = 1;
    while (lanes * 8 < hd) lanes *= 2;
    const long long units = (long long)n * (nh + nkv), threads_all = units * lanes;
    hipLaunchKernelGGL(qk_heads_words_kernel, dim3((unsigned)((threads_all + 255) / 256)), dim3(256), 0, stream, (const bf16*)proj, ld, bias,
                       wconv, taps, state, tok_seq, q_start, pos0, state_slots, single, wq, wk, eps, joint, cosv, sinv, rot, mag, neighbours,
                       tied, (bf16*)out, ldo, hd, slots, (bf16*)k_pages, (bf16*)v_pages, page_size, nh, nkv, dk, dv, sums, lanes, units);
    return launched("qk_heads");
  }
  if (dtype == kF32)
    hipLaunchKernelGGL(qk_heads_kernel<float>, dim3((unsigned)(n * (nh + nkv))), dim3(threads), lds, stream, (const float*)proj, ld, bias, wconv, taps,
                       state, tok_seq, q_start, pos0, state_slots, single, wq, wk, eps, joint, cosv, sinv, rot, mag, neighbours, tied,
                       (float*)out, ldo, hd, slots, (float*)k_pages, (float*)v_pages, page_size, nh, nkv, dk, dv, sums);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(qk_heads_kernel<bf16>, dim3((unsigned)(n * (nh + nkv))), dim3(threads), lds, stream, (const bf16*)proj, ld, bias, wconv, taps,
                       state, tok_seq, q_start, pos0, state_slots, single, wq, wk, eps, joint, cosv, sinv, rot, mag, neighbours, tied,
                       (bf16*)out, ldo, hd, slots, (bf16*)k_pages, (bf16*)v_pages, page_size, nh, nkv, dk, dv, sums);
  else
    return fail("qk_heads: unknown dtype %d", dtype);
  return launched("qk_heads");
}

extern "C" int gb_qk_conv_state(const void* proj, int dtype, int ld, const float* bias, float* state, const int32_t* q_start,
                                const int32_t* q_len, const int32_t* state_slots, int n_seqs, int channels, int taps,
                                hipStream_t stream) {
  GB_REQUIRE(n_seqs >= 0 && channels > 0 && ld >= channels && taps >= 2 && taps <= kMaxTaps, "qk_conv_state: bad sizes");
  if (n_seqs == 0) return 0;
  const long long count = (long long)n_seqs * channels;
  GB_REQUIRE(grid_fits(count), "qk_conv_state: too many elements");
  const dim3 grid((unsigned)((count + 255) / 256));
  if (dtype == kF32)
    hipLaunchKernelGGL(conv_state_kernel<float>, grid, dim3(256), 0, stream, (const float*)proj, ld, bias, state, q_start, q_len,
                       state_slots, n_seqs, channels, taps - 1);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(conv_state_kernel<bf16>, grid, dim3(256), 0, stream, (const bf16*)proj, ld, bias, state, q_start, q_len,
                       state_slots, n_seqs, channels, taps - 1);
  else
    return fail("qk_conv_state: unknown dtype %d", dtype);
  return launched("qk_conv_state");
}

extern "C" int gb_gate_rows(const void* att, int lda, int hd, const void* gate, int ldg, int per_head, int dtype, void* out,
                            int ldo, int n, int nh, int dv, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && nh > 0 && dv > 0 && hd >= dv && lda >= nh * hd && ldo >= nh * dv && ldg >= (per_head ? nh : nh * dv),
             "gate_rows: bad sizes nh=%d dv=%d hd=%d (strides %d, %d, %d)", nh, dv, hd, lda, ldg, ldo);
  if (n == 0) return 0;
  const long long count = (long long)n * nh * dv;
  GB_REQUIRE(grid_fits(count), "gate_rows: too many elements");
  if (dtype == kBF16 && dv % 8 == 0 && hd % 8 == 0 && lda % 8 == 0 && ldo % 8 == 0 && (per_head || ldg % 8 == 0) && words16(att) &&
      words16(out) && (per_head || words16(gate))) {
    hipLaunchKernelGGL(gate_rows_words_kernel, dim3((unsigned)((count / 8 + 255) / 256)), dim3(256), 0, stream, (const bf16*)att, lda, hd,
                       (const bf16*)gate, ldg, per_head, (bf16*)out, ldo, count / 8, nh, dv);
    return launched("gate_rows");
  }
  const dim3 grid((unsigned)((count + 255) / 256));
  if (dtype == kF32)
    hipLaunchKernelGGL(gate_rows_kernel<float>, grid, dim3(256), 0, stream, (const float*)att, lda, hd, (const float*)gate, ldg,
                       per_head, (float*)out, ldo, count, nh, dv);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(gate_rows_kernel<bf16>, grid, dim3(256), 0, stream, (const bf16*)att, lda, hd, (const bf16*)gate, ldg,
                       per_head, (bf16*)out, ldo, count, nh, dv);
  else
    return fail("gate_rows: unknown dtype %d", dtype);
  return launched("gate_rows");
}

GB_TAPED(gb_tanh_norm)
GB_TAPED(gb_tanh_norm_add)
GB_TAPED(gb_qk_heads)
GB_TAPED(gb_qk_conv_state)
GB_TAPED(gb_gate_rows)
