// Routing of tokens to experts, and the experts' gated units.
//
//   s = sigmoid(z)                          z [n, E] the router's logits, 32-bit
//   chosen: the `top` experts with the largest s + correction (of equal ones the lower index)
//   weight of a chosen expert: s / (sum of the chosen s + 1e-20) * scale
//
// Other routers are the same kernel with other arguments: scores by softmax over all experts instead of the sigmoid;
// weights that are the scores as they stand (times scale), not divided by their sum; experts in `groups` equal runs
// of neighbours, of which only the `keep` runs with the largest pick score (s + correction) of any of their experts can
// be chosen; a shared expert that counts fully (weight 1) instead of through a gate of its own.
//
// `route` leaves the result in two forms: the chosen experts and their weights a token ([n, top]), and a row of E
// weights a token with zeros for the experts not chosen (with `shared`, one more column: sigmoid of z's column E, the
// gate of an expert that every token uses).  `gated_units` turns the stacked gate and up projections of all experts
// into act = silu(gate) * up * weight, so that one product with the experts' down matrices side by side adds up
// sum_e a_e y_e over the token's experts (an expert not chosen contributes exact zeros).
//
// With many tokens a step, the experts run on the rows that chose them alone.  `sort` puts the (token, choice) entries
// in the order of their experts (entries of an expert in the order of the tokens): rows[r] is the token behind sorted
// row r, pos[t * top + k] the sorted row of token t's k-th choice, and `map` cuts the sorted rows into row tiles that
// lie in one expert each (three numbers a tile: expert, first row, end of the expert's rows; the tiles past the last one
// carry expert -1).  The products then go tile by tile with the tile's expert's matrices, and `combine` adds up, for
// each token, its chosen experts' output rows times their weights in the order of the choices, and the shared
// expert's row times its gate.
#include "common.h"

using namespace gb;

GB_DEFINE_LAST_ERROR

namespace {

constexpr int kPerLane = 8;   // experts a lane: up to 512 experts
constexpr int kMaxTop = 16;

// shared: 0 none, 1 a gate sigmoid(z[E]), 2 weight 1.  softmax: scores over all experts (else sigmoid of each).
// renorm: weights divided by the sum of the chosen scores.  groups > 0: see above.
__global__ __launch_bounds__(4 * kWave) void route_kernel(const float* __restrict__ z, int ldz, int E,
                                                        const float* __restrict__ correction, int top, float scale,
                                                        int shared, int softmax, int renorm, int groups, int keep,
                                                        float* __restrict__ combine, int32_t* __restrict__ ids,
                                                        float* __restrict__ wts, int n) {
  __shared__ float pick[4][kPerLane * kWave];   // a wave's pick scores, for the groups' maxima
  __shared__ float best_of[4][kWave];           // a group's best pick score, then 1 if the group is kept
  const int wave = threadIdx.x / kWave;
  const int t = blockIdx.x * 4 + wave, lane = threadIdx.x % kWave;
  if (t >= n) return;   // (a wave as a whole: no barrier below, a wave's lanes run together)
  const float* row = z + (size_t)t * ldz;
  float s[kPerLane], c[kPerLane];
  float top_z = -INFINITY, denom = 0.f;
  if (softmax) {
#pragma unroll
    for (int j = 0; j < kPerLane; ++j)
      if (lane + j * kWave < E) top_z = fmaxf(top_z, row[lane + j * kWave]);
    top_z = wave_max(top_z);
#pragma unroll
    for (int j = 0; j < kPerLane; ++j)
      if (lane + j * kWave < E) denom += expf(row[lane + j * kWave] - top_z);
    denom = wave_sum(denom);
  }
#pragma unroll
  for (int j = 0; j < kPerLane; ++j) {
    const int e = lane + j * kWave;
    s[j] = 0.f;
    c[j] = -INFINITY;
    if (e < E) {
      s[j] = softmax ? expf(row[e] - top_z) / denom : 1.0f / (1.0f + expf(-row[e]));
      c[j] = s[j] + (correction ? correction[e] : 0.f);
    }
  }
  if (groups > 0) {
    const int size = E / groups;
#pragma unroll
    for (int j = 0; j < kPerLane; ++j)
      if (lane + j * kWave < E) pick[wave][lane + j * kWave] = c[j];
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    float mine = -INFINITY;   // lane g: group g's best
    if (lane < groups)
      for (int i = 0; i < size; ++i) mine = fmaxf(mine, pick[wave][lane * size + i]);
    best_of[wave][lane] = mine;
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    int ahead = 0;            // groups that go before this one: a larger best, or the same and a lower number
    if (lane < groups)
      for (int g = 0; g < groups; ++g) {
        const float o = best_of[wave][g];
        ahead += (o > mine || (o == mine && g < lane)) ? 1 : 0;
      }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    best_of[wave][lane] = (lane < groups && ahead < keep) ? 1.f : 0.f;
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
#pragma unroll
    for (int j = 0; j < kPerLane; ++j) {
      const int e = lane + j * kWave;
      if (e < E && best_of[wave][e / size] == 0.f) c[j] = -INFINITY;
    }
  }
  int chosen[kMaxTop];
  float cs[kMaxTop];
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < kMaxTop; ++k) {
    chosen[k] = -1;
    cs[k] = 0.f;
    if (k >= top) continue;
    float best = -INFINITY;
    int be = 0x7fffffff;
    float bs = 0.f;
#pragma unroll
    for (int j = 0; j < kPerLane; ++j) {
      const int e = lane + j * kWave;
      if (e < E && (c[j] > best || (c[j] == best && e < be))) {
        best = c[j];
        be = e;
        bs = s[j];
      }
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, kWave), os = __shfl_xor(bs, off, kWave);
      const int oe = __shfl_xor(be, off, kWave);
      if (ob > best || (ob == best && oe < be)) {
        best = ob;
        be = oe;
        bs = os;
      }
    }
    chosen[k] = be;
    cs[k] = bs;
    sum += bs;
#pragma unroll
    for (int j = 0; j < kPerLane; ++j)
      if (lane + j * kWave == be) c[j] = -INFINITY;   // taken
  }
  const float inv = renorm ? scale / (sum + 1e-20f) : scale;
  const int cols = E + (shared ? 1 : 0);
#pragma unroll
  for (int j = 0; j < kPerLane; ++j) {
    const int e = lane + j * kWave;
    if (e >= E) continue;
    float w = 0.f;
#pragma unroll
    for (int k = 0; k < kMaxTop; ++k)
      if (k < top && chosen[k] == e) w = cs[k] * inv;
    combine[(size_t)t * cols + e] = w;
  }
  if (shared && lane == 0) combine[(size_t)t * cols + E] = shared == 2 ? 1.0f : 1.0f / (1.0f + expf(-row[E]));
#pragma unroll
  for (int k = 0; k < kMaxTop; ++k)
    if (k < top && lane == k % kWave) {
      ids[(size_t)t * top + k] = chosen[k];
      wts[(size_t)t * top + k] = cs[k] * inv;
    }
}

// act[t, j] = silu(g) * u * combine[t, expert of column j]: columns e * ff .. (e + 1) * ff - 1 are expert e's, the
// columns from E * ff on the shared expert's (weight in column E of combine).  Rows of `gu`: the experts' gate columns,
// the experts' up columns, then the shared expert's gate columns and its up columns.
template <typename I, typename O>
__global__ void gated_units_kernel(const I* __restrict__ gu, int ld, const float* __restrict__ combine, int cols, O* __restrict__ act,
                                   long long count, int inter, int E, int ff) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= count) return;
  const long long t = idx / inter;
  const int j = (int)(idx % inter);
  const int routed = E * ff;
  const int e = j < routed ? j / ff : E;
  const float w = combine[(size_t)t * cols + e];
  float y = 0.f;
  if (w != 0.f) {
    const I* row = gu + (size_t)t * ld;
    const int at = j < routed ? j : 2 * routed + (j - routed), up = j < routed ? routed : inter - routed;
    const float g = to_f(row[at]), u = to_f(row[at + up]);
    y = g / (1.0f + expf(-g)) * u * w;
  }
  act[idx] = from_f<O>(y);
}

// act[t, j] = relu(z[t, j])^2 * combine[t, expert of column j] for units without a gate half: columns
// e * ff .. (e + 1) * ff - 1 are expert e's, those from E * ff on the shared expert's.  Without `combine` every weight is 1.
template <typename I, typename O>
__global__ void relu2_units_kernel(const I* __restrict__ z, int ld, const float* __restrict__ combine, int cols, O* __restrict__ act,
                                   int lda, long long count, int inter, int E, int ff) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= count) return;
  const long long t = idx / inter;
  const int j = (int)(idx % inter);
  const float w = combine ? combine[(size_t)t * cols + (j < E * ff ? j / ff : E)] : 1.f;
  float y = 0.f;
  if (w != 0.f) {
    const float v = fmaxf(to_f(z[(size_t)t * ld + j]), 0.f);
    y = v * v * w;
  }
  act[(size_t)t * lda + j] = from_f<O>(y);
}

// The same, eight columns a thread (rows of whole 16-byte words, experts of whole groups of eight columns).
template <typename I>
__global__ void relu2_units_words_kernel(const I* __restrict__ z, int ld, const float* __restrict__ combine, int cols, bf16* __restrict__ act,
                                         int lda, long long count, int inter, int E, int ff) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= count) return;
  const int words = inter / 8;
  const long long t = idx / words;
  const int j = (int)(idx % words) * 8;
  const float w = combine ? combine[(size_t)t * cols + (j < E * ff ? j / ff : E)] : 1.f;
  bf16x8 o;
  if (w != 0.f) {
    float v[8];
    if constexpr (std::is_same<I, float>::value) {
      const f32x4 a = *reinterpret_cast<const f32x4*>(z + (size_t)t * ld + j), b = *reinterpret_cast<const f32x4*>(z + (size_t)t * ld + j + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = a[e], v[4 + e] = b[e];
    } else {
      const bf16x8 a = *reinterpret_cast<const bf16x8*>(z + (size_t)t * ld + j);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = (float)a[e];
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float r = fmaxf(v[e], 0.f);
      o[e] = (bf16)(r * r * w);
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (bf16)0.f;
  }
  *reinterpret_cast<bf16x8*>(act + (size_t)t * lda + j) = o;
}

// counts[e]: how many of the n * top entries chose expert e.  One workgroup an expert.
__global__ __launch_bounds__(256) void count_kernel(const int32_t* __restrict__ ids, int entries, int32_t* __restrict__ counts) {
  __shared__ int part[4];
  const int e = blockIdx.x;
  int mine = 0;
  for (int i = threadIdx.x; i < entries; i += 256) mine += ids[i] == e;
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) mine += __shfl_xor(mine, off, kWave);
  if (threadIdx.x % kWave == 0) part[threadIdx.x / kWave] = mine;
  __syncthreads();
  if (threadIdx.x == 0) counts[e] = part[0] + part[1] + part[2] + part[3];
}

// Workgroup e places expert e's entries behind those of the experts before it, in the order of the entries, and writes
// its row tiles; the last workgroup also marks the tiles that are left over.
__global__ __launch_bounds__(256) void place_kernel(const int32_t* __restrict__ ids, int entries, int top, int E,
                                                    const int32_t* __restrict__ counts, int tile_rows, int tiles,
                                                    int32_t* __restrict__ rows, int32_t* __restrict__ pos,
                                                    int32_t* __restrict__ map) {
  __shared__ int part[4];
  __shared__ int first_row, first_tile, all_tiles;
  const int e = blockIdx.x, lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  if (threadIdx.x == 0) {
    int r = 0, t = 0, all = 0;
    for (int o = 0; o < E; ++o) {
      if (o == e) {
        first_row = r;
        first_tile = t;
      }
      r += counts[o];
      t += (counts[o] + tile_rows - 1) / tile_rows;
    }
    all = t;
    all_tiles = all;
  }
  __syncthreads();
  const int base = first_row, mine = counts[e];
  int placed = 0;
  for (int i0 = 0; i0 < entries; i0 += 256) {
    const int i = i0 + threadIdx.x;
    const bool hit = i < entries && ids[i] == e;
    const unsigned long long votes = __ballot(hit);
    const int before = __popcll(votes & ((1ull << lane) - 1ull));
    __syncthreads();   // the last round's sums have been read
    if (lane == 0) part[wave] = __popcll(votes);
    __syncthreads();
    int ahead = 0;
    for (int v = 0; v < wave; ++v) ahead += part[v];
    if (hit) {
      const int r = base + placed + ahead + before;
      rows[r] = i / top;
      pos[i] = r;
    }
    placed += part[0] + part[1] + part[2] + part[3];
  }
  const int my_tiles = (mine + tile_rows - 1) / tile_rows;
  for (int j = threadIdx.x; j < my_tiles; j += 256) {
    int32_t* t = map + 3 * (size_t)(first_tile + j);
    t[0] = e;
    t[1] = base + j * tile_rows;
    t[2] = base + mine;
  }
  if (e == E - 1)
    for (int j = all_tiles + threadIdx.x; j < tiles; j += 256) {
      int32_t* t = map + 3 * (size_t)j;
      t[0] = -1;
      t[1] = 0;
      t[2] = 0;
    }
}

// out[t] (+)= sum over k of wts[t, k] * y[pos[t, k]]  +  gates[t * ldg] * y_shared[t]; four columns a thread.
__global__ __launch_bounds__(256) void combine_kernel(const float* __restrict__ y, int ldy, const int32_t* __restrict__ pos,
                                                      const float* __restrict__ wts, int top, const float* __restrict__ ysh,
                                                      int ldsh, const float* __restrict__ gates, int ldg, float* __restrict__ out,
                                                      int ldo, int accumulate, int n, int quads, int y_rows) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long long)n * quads) return;
  const int t = (int)(idx / quads), c = (int)(idx % quads) * 4;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int k = 0; k < top; ++k) {
    const float w = wts[(size_t)t * top + k];
    // an entry whose expert is none (a row of logits that are no numbers) was never placed: any row will do for it
    const int r = min(max(pos[(size_t)t * top + k], 0), y_rows - 1);
    const float4 v = *reinterpret_cast<const float4*>(y + (size_t)r * ldy + c);
    acc.x += w * v.x;
    acc.y += w * v.y;
    acc.z += w * v.z;
    acc.w += w * v.w;
  }
  if (ysh) {
    const float g = gates[(size_t)t * ldg];
    const float4 v = *reinterpret_cast<const float4*>(ysh + (size_t)t * ldsh + c);
    acc.x += g * v.x;
    acc.y += g * v.y;
    acc.z += g * v.z;
    acc.w += g * v.w;
  }
  float4* o = reinterpret_cast<float4*>(out + (size_t)t * ldo + c);
  if (accumulate) {
    const float4 old = *o;
    acc.x += old.x;
    acc.y += old.y;
    acc.z += old.z;
    acc.w += old.w;
  }
  *o = acc;
}

}  // namespace

extern "C" int gb_moe_route_by(const float* z, int ldz, int n, int E, const float* correction, int top, float scale, int shared,
                               int softmax, int renorm, int groups, int keep, float* combine, int32_t* ids, float* wts,
                               hipStream_t stream) {
  GB_REQUIRE(n >= 0 && E > 0 && E <= kPerLane * kWave, "moe_route: %d experts (at most %d)", E, kPerLane * kWave);
  GB_REQUIRE(top > 0 && top <= kMaxTop && top <= E, "moe_route: %d chosen experts of %d (at most %d)", top, E, kMaxTop);
  GB_REQUIRE(shared >= 0 && shared <= 2 && ldz >= E + (shared == 1 ? 1 : 0), "moe_route: rows of %d logits for %d experts", ldz, E);
  GB_REQUIRE(groups >= 0 && (groups == 0 || (groups <= kWave && E % groups == 0 && keep >= 1 && keep <= groups &&
                                             keep * (E / groups) >= top)),
             "moe_route: %d groups of %d experts, %d kept, %d experts a token", groups, E, keep, top);
  if (n == 0) return 0;
  hipLaunchKernelGGL(route_kernel, dim3((unsigned)((n + 3) / 4)), dim3(4 * kWave), 0, stream, z, ldz, E, correction, top, scale,
                     shared, softmax, renorm, groups, keep, combine, ids, wts, n);
  return launched("moe_route");
}

extern "C" int gb_moe_route(const float* z, int ldz, int n, int E, const float* correction, int top, float scale, int shared,
                            float* combine, int32_t* ids, float* wts, hipStream_t stream) {
  return gb_moe_route_by(z, ldz, n, E, correction, top, scale, shared ? 1 : 0, 0, 1, 0, 0, combine, ids, wts, stream);
}

extern "C" int gb_moe_relu2_units(const void* z, int in_dtype, int ld, const float* combine, int cols, void* act, int out_dtype,
                                  int lda, int n, int inter, int E, int ff, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && inter > 0 && ld >= inter && lda >= inter && E >= 0 && ff > 0 && E * ff <= inter &&
                 (!combine || cols >= E + (E * ff < inter ? 1 : 0)),
             "moe_relu2_units: bad sizes n=%d inter=%d experts=%d of %d cols=%d", n, inter, E, ff, cols);
  if (n == 0) return 0;
  const long long count = (long long)n * inter;
  GB_REQUIRE((count + 255) / 256 < (1ll << 31), "moe_relu2_units: too many elements");
  if (out_dtype == kBF16 && inter % 8 == 0 && ff % 8 == 0 && ld % 8 == 0 && lda % 8 == 0 && (uintptr_t)z % 16 == 0 && (uintptr_t)act % 16 == 0) {
    const dim3 wgrid((unsigned)((count / 8 + 255) / 256));
    if (in_dtype == kF32)
      hipLaunchKernelGGL(relu2_units_words_kernel<float>, wgrid, dim3(256), 0, stream, (const float*)z, ld, combine, cols, (bf16*)act, lda, count / 8, inter, E, ff);
    else
      hipLaunchKernelGGL(relu2_units_words_kernel<bf16>, wgrid, dim3(256), 0, stream, (const bf16*)z, ld, combine, cols, (bf16*)act, lda, count / 8, inter, E, ff);
    return launched("moe_relu2_units");
  }
  const dim3 grid((unsigned)((count + 255) / 256));
  if (in_dtype == kF32 && out_dtype == kF32)
    hipLaunchKernelGGL((relu2_units_kernel<float, float>), grid, dim3(256), 0, stream, (const float*)z, ld, combine, cols, (float*)act, lda, count, inter, E, ff);
  else if (in_dtype == kF32 && out_dtype == kBF16)
    hipLaunchKernelGGL((relu2_units_kernel<float, bf16>), grid, dim3(256), 0, stream, (const float*)z, ld, combine, cols, (bf16*)act, lda, count, inter, E, ff);
  else if (in_dtype == kBF16 && out_dtype == kBF16)
    hipLaunchKernelGGL((relu2_units_kernel<bf16, bf16>), grid, dim3(256), 0, stream, (const bf16*)z, ld, combine, cols, (bf16*)act, lda, count, inter, E, ff);
  else
    return fail("moe_relu2_units: no kernel for operand type %d and result type %d", in_dtype, out_dtype);
  return launched("moe_relu2_units");
}

extern "C" int gb_moe_gated_units(const void* gu, int in_dtype, int ld, const float* combine, int cols, void* act, int out_dtype,
                                  int n, int inter, int E, int ff, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && inter > 0 && ld >= 2 * inter && E >= 0 && ff > 0 && E * ff <= inter && cols >= E + (E * ff < inter ? 1 : 0),
             "moe_gated_units: bad sizes n=%d inter=%d experts=%d of %d cols=%d", n, inter, E, ff, cols);
  if (n == 0) return 0;
  const long long count = (long long)n * inter;
  GB_REQUIRE((count + 255) / 256 < (1ll << 31), "moe_gated_units: too many elements");
  const dim3 grid((unsigned)((count + 255) / 256));
  if (in_dtype == kF32 && out_dtype == kF32)
    hipLaunchKernelGGL((gated_units_kernel<float, float>), grid, dim3(256), 0, stream, (const float*)gu, ld, combine, cols, (float*)act, count, inter, E, ff);
  else if (in_dtype == kF32 && out_dtype == kBF16)
    hipLaunchKernelGGL((gated_units_kernel<float, bf16>), grid, dim3(256), 0, stream, (const float*)gu, ld, combine, cols, (bf16*)act, count, inter, E, ff);
  else if (in_dtype == kBF16 && out_dtype == kBF16)
    hipLaunchKernelGGL((gated_units_kernel<bf16, bf16>), grid, dim3(256), 0, stream, (const bf16*)gu, ld, combine, cols, (bf16*)act, count, inter, E, ff);
  else
    return fail("moe_gated_units: no kernel for operand type %d and result type %d", in_dtype, out_dtype);
  return launched("moe_gated_units");
}

// Row tiles that `sort` may need for n * top entries over E experts: every expert's last tile may be short.
extern "C" int gb_moe_sort_tiles(int entries, int E, int tile_rows) { return entries / tile_rows + E; }

extern "C" int gb_moe_sort(const int32_t* ids, int n, int top, int E, int tile_rows, int tiles, int32_t* counts, int32_t* rows,
                           int32_t* pos, int32_t* map, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && top > 0 && E > 0 && tile_rows > 0 && (long long)n * top < (1ll << 31), "moe_sort: bad sizes n=%d top=%d experts=%d", n, top, E);
  GB_REQUIRE(tiles >= gb_moe_sort_tiles(n * top, E, tile_rows), "moe_sort: %d row tiles, %d may be needed", tiles,
             gb_moe_sort_tiles(n * top, E, tile_rows));
  if (n == 0) return 0;
  hipLaunchKernelGGL(count_kernel, dim3(E), dim3(256), 0, stream, ids, n * top, counts);
  hipLaunchKernelGGL(place_kernel, dim3(E), dim3(256), 0, stream, ids, n * top, top, E, counts, tile_rows, tiles, rows, pos, map);
  return launched("moe_sort");
}

extern "C" int gb_moe_combine(const float* y, int ldy, const int32_t* pos, const float* wts, int top, const float* ysh, int ldsh,
                              const float* gates, int ldg, float* out, int ldo, int accumulate, int n, int d, int y_rows, hipStream_t stream) {
  GB_REQUIRE(y_rows >= (long long)n * top, "moe_combine: y holds %d rows for %d tokens of %d choices", y_rows, n, top);
  GB_REQUIRE(n >= 0 && d > 0 && d % 4 == 0 && ldy % 4 == 0 && ldo % 4 == 0 && (!ysh || (ldsh % 4 == 0 && gates)) && ldy >= d && ldo >= d,
             "moe_combine: rows of %d columns (strides %d, %d, %d) must be whole groups of four", d, ldy, ldsh, ldo);
  GB_REQUIRE(((uintptr_t)y % 16 == 0) && ((uintptr_t)out % 16 == 0) && ((uintptr_t)ysh % 16 == 0), "moe_combine: rows must be 16-byte aligned");
  if (n == 0) return 0;
  const long long count = (long long)n * (d / 4);
  GB_REQUIRE((count + 255) / 256 < (1ll << 31), "moe_combine: too many elements");
  hipLaunchKernelGGL(combine_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, y, ldy, pos, wts, top, ysh, ldsh,
                     gates, ldg, out, ldo, accumulate, n, d / 4, y_rows);
  return launched("moe_combine");
}

GB_TAPED(gb_moe_sort)
GB_TAPED(gb_moe_combine)
GB_TAPED(gb_moe_route)
GB_TAPED(gb_moe_route_by)
GB_TAPED(gb_moe_relu2_units)
GB_TAPED(gb_moe_gated_units)
