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

// One workgroup a token.  A row of `proj` holds nh query heads and nkv key heads of dk channels, then (unless the values
// are the keys) nkv value heads of dv, then whatever else the product made (gates), which is not read here.
//   1. bias, and with taps > 0 the convolution over the request's earlier rows of this step and its state slot
//      ([taps - 1, channels] float32, index i = the position `first position of the step` - (taps - 1) + i);
//   2. tied values: the key channels as they stand now are the value heads (dv = dk);
//   3. RMS norm: joint = over all query channels at once (and all key channels), weights [nh dk] and [nkv dk];
//      else head by head over dk, weights [dk] that all heads share;
//   4. the first `rot` channels of every query and key head turn by the step's angles (cos, sin [n, rot / 2], times
//      mag): neighbours = channel 2i with 2i + 1, else channel i with i + rot / 2;
//   5. heads of hd >= max(dk, dv) columns in `out`, zeros beyond their channels; with `slots` keys and values also go
//      to their pages.
// `single` (every request brings one row): the thread that reads a channel's slot also moves it on by one.
template <typename T>
__global__ __launch_bounds__(256) void qk_heads_kernel(
    const T* __restrict__ proj, int ld, const float* __restrict__ bias, const float* __restrict__ wconv, int taps,
    float* __restrict__ state, const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ pos0, const int32_t* __restrict__ state_slots, int single, const float* __restrict__ wq,
    const float* __restrict__ wk, float eps, int joint, const float* __restrict__ cosv, const float* __restrict__ sinv, int rot,
    float mag, int neighbours, int tied, T* __restrict__ out, int ldo, int hd, const int32_t* __restrict__ slots,
    T* __restrict__ k_pages, T* __restrict__ v_pages, int page_size, int nh, int nkv, int dk, int dv) {
  extern __shared__ float lds[];
  const int qd = nh * dk, kd = nkv * dk, channels = qd + kd, heads = nh + nkv;
  float* vals = lds;                  // [channels]: q then k, after step 1
  float* inv = vals + channels;       // [heads]: 1 / rms of each head (joint: the same for all heads of a kind)
  float* scratch = inv + heads;       // [17]
  const int t = blockIdx.x, tid = threadIdx.x;
  const T* row = proj + (size_t)t * ld;
  const int K = taps > 0 ? taps - 1 : 0;
  int off = 0, first_pos = 0;
  float* st = nullptr;
  if (taps > 0) {
    const int seq = tok_seq[t];
    off = t - q_start[seq];
    first_pos = pos0[seq];
    if (K > 0) st = state + (size_t)state_slots[seq] * K * channels;
  }
  float sq = 0.f, sk = 0.f;
  for (int ch = tid; ch < channels; ch += 256) {
    float v;
    if (taps == 0) {
      v = to_f(row[ch]) + (bias ? bias[ch] : 0.f);
    } else {
      float old[kMaxTaps - 1];
#pragma unroll
      for (int i = 0; i < kMaxTaps - 1; ++i) old[i] = (i < K && (single || i >= off)) ? st[(size_t)i * channels + ch] : 0.f;
      v = 0.f;
#pragma unroll
      for (int jt = 0; jt < kMaxTaps; ++jt) {
        if (jt >= taps) break;
        const int back = K - jt;   // how many tokens before this one
        float u = 0.f;
        if (off >= back) {
          u = to_f(proj[(size_t)(t - back) * ld + ch]) + (bias ? bias[ch] : 0.f);
        } else if (first_pos + off - back >= 0) {
#pragma unroll
          for (int i = 0; i < kMaxTaps - 1; ++i)
            if (i == off + jt) u = old[i];
        }
        v = fmaf(wconv[(size_t)ch * taps + jt], u, v);
      }
      if (single && K > 0) {
#pragma unroll
        for (int i = 0; i < kMaxTaps - 1; ++i)
          if (i < K) st[(size_t)i * channels + ch] = i + 1 < K ? old[i + 1 < kMaxTaps - 1 ? i + 1 : 0] : to_f(row[ch]) + (bias ? bias[ch] : 0.f);
      }
    }
    vals[ch] = v;
    if (ch < qd) sq = fmaf(v, v, sq); else sk = fmaf(v, v, sk);
  }
  if (joint) {
    sq = block_sum(sq, scratch);
    sk = block_sum(sk, scratch);   // (the barriers inside also order the writes of vals before the reads below)
    const float rq = 1.0f / sqrtf(sq / (float)qd + eps), rk = 1.0f / sqrtf(sk / (float)kd + eps);
    for (int u = tid; u < heads; u += 256) inv[u] = u < nh ? rq : rk;
  } else {
    __syncthreads();
    const int lane = tid % kWave, wave = tid / kWave;
    for (int u = wave; u < heads; u += 4) {
      float s = 0.f;
      for (int c = lane; c < dk; c += kWave) {
        const float v = vals[u * dk + c];
        s = fmaf(v, v, s);
      }
      s = wave_sum(s);
      if (lane == 0) inv[u] = 1.0f / sqrtf(s / (float)dk + eps);
    }
  }
  __syncthreads();
  const int slot = slots ? slots[t] : -1;
  const int piece = key_piece(hd);
  const int half = rot / 2;
  T* orow = out + (size_t)t * ldo;
  for (int idx = tid; idx < heads * hd; idx += 256) {
    const int u = idx / hd, c = idx % hd;
    float r = 0.f;
    if (c < dk) {
      const bool is_q = u < nh;
      const float* wn = is_q ? wq : wk;
      const int wbase = joint ? (is_q ? u : u - nh) * dk : 0;
      const float s = inv[u];
      r = vals[u * dk + c] * s * (wn ? wn[wbase + c] : 1.f);
      if (c < rot) {
        const int pc = neighbours ? (c ^ 1) : (c < half ? c + half : c - half);
        const int i = neighbours ? c / 2 : (c < half ? c : c - half);
        const bool first = neighbours ? !(c & 1) : c < half;
        const float p = vals[u * dk + pc] * s * (wn ? wn[wbase + pc] : 1.f);
        const float cs = cosv[(size_t)t * half + i] * mag, sn = sinv[(size_t)t * half + i] * mag;
        r = first ? r * cs - p * sn : r * cs + p * sn;
      }
    }
    const T o = from_f<T>(r);
    orow[idx] = o;
    if (slot >= 0 && u >= nh) {
      T* kb = k_pages + ((size_t)(slot / page_size) * nkv + (u - nh)) * (size_t)page_size * hd;
      kb[key_offset(slot % page_size, c, page_size, piece)] = o;
    }
  }
  for (int idx = tid; idx < nkv * hd; idx += 256) {
    const int g = idx / hd, c = idx % hd;
    float r = 0.f;
    if (c < dv) r = tied ? vals[qd + g * dk + c] : to_f(row[channels + g * dv + c]) + (bias ? bias[channels + g * dv + c] : 0.f);
    const T o = from_f<T>(r);
    orow[(size_t)heads * hd + idx] = o;
    if (slot >= 0) {
      T* vb = v_pages + ((size_t)(slot / page_size) * nkv + g) * (size_t)page_size * hd;
      vb[(size_t)c * page_size + slot % page_size] = o;
    }
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

inline bool grid_fits(long long count) { return (count + 255) / 256 < (1ll << 31); }

}  // namespace

extern "C" int gb_tanh_norm(const float* x, int ldx, const int32_t* rows, const float* alpha, const float* w, const float* b,
                            void* out, int out_dtype, int ldo, int n, int d, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && d > 0 && ldx >= d && ldo >= d, "tanh_norm: bad sizes n=%d d=%d (strides %d, %d)", n, d, ldx, ldo);
  GB_REQUIRE(alpha && w && b, "tanh_norm: the norm's number, weight and bias are needed");
  if (n == 0) return 0;
  const long long count = (long long)n * d;
  GB_REQUIRE(grid_fits(count), "tanh_norm: too many elements");
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
// 4 = neighbouring channels pair up, 8 = the values are the keys.
extern "C" int gb_qk_heads(const void* proj, int dtype, int ld, const float* bias, const float* wconv, int taps, float* state,
                           const int32_t* tok_seq, const int32_t* q_start, const int32_t* pos0, const int32_t* state_slots,
                           int flags, const float* wq, const float* wk, float eps, const float* cosv, const float* sinv, int rot,
                           float mag, void* out, int ldo, int hd, const int32_t* slots, void* k_pages, void* v_pages,
                           int page_size, int n, int nh, int nkv, int dk, int dv, hipStream_t stream) {
  const int single = flags & 1, joint = (flags >> 1) & 1, neighbours = (flags >> 2) & 1, tied = (flags >> 3) & 1;
  GB_REQUIRE(n >= 0 && nh > 0 && nkv > 0 && dk > 0 && dv > 0 && hd >= dk && hd >= dv, "qk_heads: bad sizes nh=%d nkv=%d dk=%d dv=%d hd=%d", nh, nkv, dk, dv, hd);
  GB_REQUIRE(!tied || dv == dk, "qk_heads: values that are the keys have the keys' size (dk=%d, dv=%d)", dk, dv);
  const int channels = (nh + nkv) * dk;
  GB_REQUIRE(ld >= channels + (tied ? 0 : nkv * dv) && ldo >= (nh + 2 * nkv) * hd, "qk_heads: rows shorter than the heads");
  GB_REQUIRE(taps >= 0 && taps <= kMaxTaps, "qk_heads: %d taps (at most %d)", taps, kMaxTaps);
  GB_REQUIRE(taps == 0 || (wconv && tok_seq && q_start && pos0 && (taps == 1 || (state && state_slots))),
             "qk_heads: a convolution needs its weights, the step's requests and their state");
  GB_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= dk && (rot == 0 || (cosv && sinv)), "qk_heads: %d rotated channels of %d", rot, dk);
  GB_REQUIRE(!slots || (k_pages && v_pages && page_size > 0), "qk_heads: cache rows without pages");
  const size_t lds = sizeof(float) * ((size_t)channels + nh + nkv + 17);
  GB_REQUIRE(lds <= 64 * 1024, "qk_heads: %d query and key channels a token are more than a workgroup stages", channels);
  if (n == 0) return 0;
  if (dtype == kF32)
    hipLaunchKernelGGL(qk_heads_kernel<float>, dim3((unsigned)n), dim3(256), lds, stream, (const float*)proj, ld, bias, wconv, taps,
                       state, tok_seq, q_start, pos0, state_slots, single, wq, wk, eps, joint, cosv, sinv, rot, mag, neighbours, tied,
                       (float*)out, ldo, hd, slots, (float*)k_pages, (float*)v_pages, page_size, nh, nkv, dk, dv);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(qk_heads_kernel<bf16>, dim3((unsigned)n), dim3(256), lds, stream, (const bf16*)proj, ld, bias, wconv, taps,
                       state, tok_seq, q_start, pos0, state_slots, single, wq, wk, eps, joint, cosv, sinv, rot, mag, neighbours, tied,
                       (bf16*)out, ldo, hd, slots, (bf16*)k_pages, (bf16*)v_pages, page_size, nh, nkv, dk, dv);
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
