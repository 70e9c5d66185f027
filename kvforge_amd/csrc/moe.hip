// Routed experts: the router's choice per token, and the row-wise steps around the experts'
// matrix products.  Router arithmetic is fp32 throughout.
#include "common.h"

namespace {
constexpr int MAX_PER_LANE = 8;   // router outputs per lane: up to 512 of them
constexpr int MAX_TOP = 16;

// A wave per token.  s = softmax(z) over all R router outputs; the `top` outputs with the
// largest s + correction are chosen (the lowest index among equals), and weighted by their s
// alone, divided by the sum of the chosen s (+ 1e-20).  sel [N, top], wgt [N, top].
__global__ __launch_bounds__(KVF_WAVE) void moe_topk_kernel(const float* __restrict__ z, int z_stride,
                                                            const float* __restrict__ correction,
                                                            int* __restrict__ sel, float* __restrict__ wgt,
                                                            int R, int top) {
  const int n = blockIdx.x, lane = threadIdx.x;
  const float* zr = z + static_cast<size_t>(n) * z_stride;
  float s[MAX_PER_LANE], c[MAX_PER_LANE];
  float mx = -INFINITY;
#pragma unroll
  for (int j = 0; j < MAX_PER_LANE; ++j) {
    const int e = lane + KVF_WAVE * j;
    s[j] = e < R ? zr[e] : -INFINITY;
    mx = fmaxf(mx, s[j]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < MAX_PER_LANE; ++j) {
    const int e = lane + KVF_WAVE * j;
    s[j] = e < R ? expf(s[j] - mx) : 0.f;
    sum += s[j];
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int j = 0; j < MAX_PER_LANE; ++j) {
    const int e = lane + KVF_WAVE * j;
    s[j] = s[j] / sum;
    c[j] = e < R ? s[j] + correction[e] : -INFINITY;
  }
  float picked_s = 0.f, total = 0.f;   // lane k keeps the k-th choice
  int picked_e = -1;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < MAX_PER_LANE; ++j) {
      const int e = lane + KVF_WAVE * j;
      if (c[j] > best) {   // a lane's own candidates come in rising index: '>' keeps the lowest
        best = c[j];
        at = e;
      }
    }
    const float wbest = wave_max(best);
    int cand = best == wbest ? at : 0x7fffffff;
#pragma unroll
    for (int o = KVF_WAVE / 2; o > 0; o >>= 1) cand = min(cand, __shfl_xor(cand, o, KVF_WAVE));
    // the owner hands over its probability and retires the choice
    float sv = 0.f;
#pragma unroll
    for (int j = 0; j < MAX_PER_LANE; ++j) {
      if (lane + KVF_WAVE * j == cand) {
        sv = s[j];
        c[j] = -INFINITY;
      }
    }
    sv = wave_sum(sv);   // one lane holds it, the others zero
    total += sv;
    if (lane == k) {
      picked_s = sv;
      picked_e = cand;
    }
  }
  if (lane < top) {
    sel[static_cast<size_t>(n) * top + lane] = picked_e;
    wgt[static_cast<size_t>(n) * top + lane] = picked_s / (total + 1e-20f);
  }
}

__device__ __forceinline__ float silu(float g) { return g / (1.f + expf(-g)); }

// Every expert's gate/up pair for every token is there (one product over all experts, columns
// 2 (e ff + j) and 2 (e ff + j) + 1): act[n, e ff + j] = weight(n, e) * silu(gate) * up where the
// token chose expert e, and an exact zero elsewhere, so that one product with the experts' down
// matrices side by side along K is the weighted sum over the chosen experts.
template <typename T>
__global__ void moe_dense_act_kernel(const T* __restrict__ gu, const int* __restrict__ sel,
                                     const float* __restrict__ wgt, T* __restrict__ act, int E, int ff,
                                     int top, long total) {
  const long i = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long cols = static_cast<long>(E) * ff;
  const long n = i / cols;
  const int col = static_cast<int>(i - n * cols), e = col / ff;
  float w = 0.f;
  bool chosen = false;
  for (int k = 0; k < top; ++k)
    if (sel[n * top + k] == e) {
      w = wgt[n * top + k];
      chosen = true;
    }
  float y = 0.f;
  if (chosen) {
    const float g = Elem<T>::load(gu + 2 * i), u = Elem<T>::load(gu + 2 * i + 1);
    y = w * (silu(g) * u);
  }
  Elem<T>::store(act + i, y);
}

// x[n, :] += (sum of the weights of the token's choices at or beyond `first`) * h[n, :]: router
// outputs that stand for "pass the input on".  x fp32, h of type T.
template <typename T>
__global__ __launch_bounds__(256) void moe_identity_kernel(float* __restrict__ x, const T* __restrict__ h,
                                                           const int* __restrict__ sel,
                                                           const float* __restrict__ wgt, int width,
                                                           int top, int first) {
  const int n = blockIdx.x;
  float w = 0.f;
  for (int k = 0; k < top; ++k)
    if (sel[static_cast<size_t>(n) * top + k] >= first) w += wgt[static_cast<size_t>(n) * top + k];
  if (w == 0.f) return;
  float* xr = x + static_cast<size_t>(n) * width;
  const T* hr = h + static_cast<size_t>(n) * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) xr[i] = fmaf(w, Elem<T>::load(hr + i), xr[i]);
}

// ---------------------------------------------------------------------------------------------
// The experts' products over only the rows that chose them (bf16, matrix cores).
//
// moe_plan: the (token, choice) pairs are grouped by expert: where[pair] is the pair's place in
// that order (-1 for a choice that names no expert), order[place] the pair; every expert's rows
// are cut into tiles of tile_rows: tiles[t] = (expert, first place, rows).  One workgroup; the order of
// an expert's rows among themselves is whatever the atomics give, which no result depends on
// (a row's products do not depend on its neighbours).
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
constexpr int PLAN_MAX_EXPERTS = 512;
constexpr int PREFETCH_SETS = 3;   // sets of operand registers in flight in the grouped products

__global__ __launch_bounds__(1024) void moe_plan_kernel(const int* __restrict__ sel, int pairs, int E,
                                                        int* __restrict__ where, int* __restrict__ order,
                                                        int* __restrict__ tiles, int* __restrict__ num_tiles,
                                                        int max_tiles, int tile_rows) {
  __shared__ int cnt[PLAN_MAX_EXPERTS], off[PLAN_MAX_EXPERTS];
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int p = tid; p < pairs; p += blockDim.x) {
    const int e = sel[p];
    where[p] = (e >= 0 && e < E) ? atomicAdd(&cnt[e], 1) : -1;
  }
  __syncthreads();
  if (tid == 0) {
    int o = 0, nt = 0;
    for (int e = 0; e < E; ++e) {
      off[e] = o;
      const int c = cnt[e];
      for (int r0 = 0; r0 < c && nt < max_tiles; r0 += tile_rows) {
        tiles[3 * nt] = e;
        tiles[3 * nt + 1] = o + r0;
        tiles[3 * nt + 2] = min(tile_rows, c - r0);
        ++nt;
      }
      o += c;
    }
    *num_tiles = nt;
  }
  __syncthreads();
  for (int p = tid; p < pairs; p += blockDim.x) {
    const int e = sel[p];
    if (e >= 0 && e < E) {
      const int pos = off[e] + where[p];
      where[p] = pos;
      order[pos] = p;
    }
  }
}

// v_mfma_f32_16x16x32_bf16 computes D[i][j] += sum_k A[i][k] B[j][k]; lane 16 c + r gives row r,
// elements 8c..8c+7 of the step's 32 of either operand, and holds D[4 (l / 16) + v][l % 16].
// A is a tile of the weight (1 KB in lane order, as ``StreamedWeight`` keeps it), B the tile's 16
// rows: a lane ends with four neighbouring output columns of one row.
//
// moe_up: act[place, :] = silu(gate) * up for the tile's rows with their expert's matrices; the
// weight holds every expert's gate and up rows interleaved (gate_j, up_j neighbours), so a lane's
// four columns are two whole pairs.  Grid (column blocks, tiles); a wave takes GW groups of 16
// weight rows.
template <int RT, int GW>
__global__ __launch_bounds__(256) void moe_up_kernel(const bf16_t* __restrict__ x, int ldx, int K,
                                                     const uint4* __restrict__ wt, int S,
                                                     const int* __restrict__ order,
                                                     const int* __restrict__ tiles,
                                                     const int* __restrict__ num_tiles, int top, int ff,
                                                     bf16_t* __restrict__ act) {
  const int tile = blockIdx.y;
  if (tile >= *num_tiles) return;
  const int e = tiles[3 * tile], row0 = tiles[3 * tile + 1], rows = tiles[3 * tile + 2];
  const int lane = threadIdx.x % KVF_WAVE, wave = threadIdx.x / KVF_WAVE;
  const int j = lane % 16, c = lane / 16;
  const int groups = ff / 8;   // groups of 16 interleaved rows per expert
  const int g_first = (blockIdx.x * 4 + wave) * GW;
  if (g_first >= groups) return;
  // a tile holds RT sub-tiles of 16 rows; a weight fragment is loaded once for all of them
  const bf16_t* xr[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r)
    xr[r] = 16 * r + j < rows ? x + static_cast<size_t>(order[row0 + 16 * r + j] / top) * ldx + 8 * c : nullptr;
  f32x4 acc[RT][GW];
#pragma unroll
  for (int r = 0; r < RT; ++r)
#pragma unroll
    for (int g = 0; g < GW; ++g) acc[r][g] = f32x4{0.f, 0.f, 0.f, 0.f};
  const uint4* wbase = wt + (static_cast<size_t>(e) * groups + g_first) * S * KVF_WAVE + lane;
  const int s_full = K / 32;   // steps whose 32 elements all lie inside a row
  // the fragments of a step are asked for NB - 1 steps ahead of the matrix instructions that use
  // them: NB sets of registers take turns
  constexpr int NB = PREFETCH_SETS;
  bf16x8 xb[NB][RT], wb[NB][GW];
  auto load = [&](int s, bf16x8 (&xs)[RT], bf16x8 (&ws)[GW]) {
#pragma unroll
    for (int r = 0; r < RT; ++r) {
      uint4 xf = make_uint4(0u, 0u, 0u, 0u);
      if (xr[r] && (s < s_full || 32 * s + 8 * c + 8 <= K)) xf = *reinterpret_cast<const uint4*>(xr[r] + 32 * s);
      xs[r] = __builtin_bit_cast(bf16x8, xf);
    }
#pragma unroll
    for (int g = 0; g < GW; ++g)   // ff is a multiple of 32, so the groups come in whole fours
      ws[g] = __builtin_bit_cast(bf16x8, wbase[(static_cast<size_t>(g) * S + s) * KVF_WAVE]);
  };
  auto mma = [&](const bf16x8 (&xs)[RT], const bf16x8 (&ws)[GW]) {
#pragma unroll
    for (int g = 0; g < GW; ++g)
#pragma unroll
      for (int r = 0; r < RT; ++r) acc[r][g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ws[g], xs[r], acc[r][g], 0, 0, 0);
  };
#pragma unroll
  for (int i = 0; i < NB - 1; ++i)
    if (i < S) load(i, xb[i], wb[i]);
  for (int s = 0; s < S; s += NB) {
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      if (s + i < S) {
        if (s + i + NB - 1 < S) load(s + i + NB - 1, xb[(i + NB - 1) % NB], wb[(i + NB - 1) % NB]);
        mma(xb[i], wb[i]);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    if (16 * r + j >= rows) continue;
    bf16_t* out = act + static_cast<size_t>(row0 + 16 * r + j) * ff;
#pragma unroll
    for (int g = 0; g < GW; ++g) {
      if (g_first + g >= groups) continue;
      const int col = (g_first + g) * 8 + 2 * c;
      const float y0 = silu(acc[r][g][0]) * acc[r][g][1], y1 = silu(acc[r][g][2]) * acc[r][g][3];
      *reinterpret_cast<uint32_t*>(out + col) =
          static_cast<uint32_t>(f32_to_bf16(y0)) | (static_cast<uint32_t>(f32_to_bf16(y1)) << 16);
    }
  }
}

// moe_down: y[place, :] = act[place, :] W_down[expert]^T (bf16, not yet weighted).  The weight
// holds the experts' down matrices side by side along K: expert e owns the steps e ff/32 ...
template <int RT, int GW>
__global__ __launch_bounds__(256) void moe_down_kernel(const bf16_t* __restrict__ act, int ff,
                                                       const uint4* __restrict__ wt, int S_all,
                                                       const int* __restrict__ tiles,
                                                       const int* __restrict__ num_tiles,
                                                       bf16_t* __restrict__ y, int hidden) {
  const int tile = blockIdx.y;
  if (tile >= *num_tiles) return;
  const int e = tiles[3 * tile], row0 = tiles[3 * tile + 1], rows = tiles[3 * tile + 2];
  const int lane = threadIdx.x % KVF_WAVE, wave = threadIdx.x / KVF_WAVE;
  const int j = lane % 16, c = lane / 16;
  const int groups = (hidden + 15) / 16;
  const int g_first = (blockIdx.x * 4 + wave) * GW;
  if (g_first >= groups) return;
  const bf16_t* ar[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r)
    ar[r] = 16 * r + j < rows ? act + static_cast<size_t>(row0 + 16 * r + j) * ff + 8 * c : nullptr;
  f32x4 acc[RT][GW];
#pragma unroll
  for (int r = 0; r < RT; ++r)
#pragma unroll
    for (int g = 0; g < GW; ++g) acc[r][g] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int S = ff / 32;
  const uint4* wbase = wt + (static_cast<size_t>(g_first) * S_all + static_cast<size_t>(e) * S) * KVF_WAVE + lane;
  int goff[GW];
#pragma unroll
  for (int g = 0; g < GW; ++g) goff[g] = min(g, groups - 1 - g_first);
  constexpr int NB = PREFETCH_SETS;
  bf16x8 xb[NB][RT], wb[NB][GW];
  auto load = [&](int s, bf16x8 (&xs)[RT], bf16x8 (&ws)[GW]) {
#pragma unroll
    for (int r = 0; r < RT; ++r) {
      uint4 af = make_uint4(0u, 0u, 0u, 0u);
      if (ar[r]) af = *reinterpret_cast<const uint4*>(ar[r] + 32 * s);
      xs[r] = __builtin_bit_cast(bf16x8, af);
    }
#pragma unroll
    for (int g = 0; g < GW; ++g)   // a group past the last is read as the last and not stored
      ws[g] = __builtin_bit_cast(bf16x8, wbase[(static_cast<size_t>(goff[g]) * S_all + s) * KVF_WAVE]);
  };
  auto mma = [&](const bf16x8 (&xs)[RT], const bf16x8 (&ws)[GW]) {
#pragma unroll
    for (int g = 0; g < GW; ++g)
#pragma unroll
      for (int r = 0; r < RT; ++r) acc[r][g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ws[g], xs[r], acc[r][g], 0, 0, 0);
  };
#pragma unroll
  for (int i = 0; i < NB - 1; ++i)
    if (i < S) load(i, xb[i], wb[i]);
  for (int s = 0; s < S; s += NB) {
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      if (s + i < S) {
        if (s + i + NB - 1 < S) load(s + i + NB - 1, xb[(i + NB - 1) % NB], wb[(i + NB - 1) % NB]);
        mma(xb[i], wb[i]);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    if (16 * r + j >= rows) continue;
    bf16_t* out = y + static_cast<size_t>(row0 + 16 * r + j) * hidden;
#pragma unroll
    for (int g = 0; g < GW; ++g) {
      if (g_first + g >= groups) continue;
      const int col = (g_first + g) * 16 + 4 * c;
#pragma unroll
      for (int v = 0; v < 4; ++v)
        if (col + v < hidden) out[col + v].bits = f32_to_bf16(acc[r][g][v]);
    }
  }
}

// x[n, :] += sum over the token's choices, in their order, of weight * (the expert's row of y, or
// the token's own input h for a choice that names no expert): fp32 sums into the fp32 stream.
// A thread takes eight neighbouring elements (hidden is a multiple of 8 here): per choice one
// 16-byte load, the choice itself being the same for the whole workgroup.
__device__ __forceinline__ void load8_any(const bf16_t* p, float (&v)[8]) { load8(p, v); }
__device__ __forceinline__ void load8_any(const float* p, float (&v)[8]) { load8(p, v); }

template <typename T>
__global__ __launch_bounds__(256) void moe_combine_kernel(float* __restrict__ x, const bf16_t* __restrict__ y,
                                                          const T* __restrict__ h, const int* __restrict__ sel,
                                                          const float* __restrict__ wgt,
                                                          const int* __restrict__ where, int hidden, int top,
                                                          int E) {
  const int n = blockIdx.x;
  float* xr = x + static_cast<size_t>(n) * hidden;
  const T* hr = h + static_cast<size_t>(n) * hidden;
  for (int i = 8 * threadIdx.x; i < hidden; i += 8 * blockDim.x) {
    float sum[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int k = 0; k < top; ++k) {
      const int p = n * top + k, e = sel[p];
      const float w = wgt[p];
      float v[8];
      if (e >= E) load8_any(hr + i, v);
      else if (e >= 0) load8(y + static_cast<size_t>(where[p]) * hidden + i, v);
      else continue;
#pragma unroll
      for (int u = 0; u < 8; ++u) sum[u] = fmaf(w, v[u], sum[u]);
    }
    float4 a = *reinterpret_cast<const float4*>(xr + i), b = *reinterpret_cast<const float4*>(xr + i + 4);
    a.x += sum[0]; a.y += sum[1]; a.z += sum[2]; a.w += sum[3];
    b.x += sum[4]; b.y += sum[5]; b.z += sum[6]; b.w += sum[7];
    *reinterpret_cast<float4*>(xr + i) = a;
    *reinterpret_cast<float4*>(xr + i + 4) = b;
  }
}
// A choice that a table makes: token id t uses the experts table[t, 0 .. top-1] (a row's entries
// differ), each with weight 1 / top.  An id outside the table, or an entry that names no expert,
// gives the pair (expert 0, weight 0): such a token adds nothing.
__global__ void moe_table_kernel(const int* __restrict__ tokens, const int* __restrict__ table, int* __restrict__ sel,
                                 float* __restrict__ wgt, int n, int vocab, int top, int E) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n * top) return;
  const int t = tokens[i / top];
  const int e = t >= 0 && t < vocab ? table[static_cast<size_t>(t) * top + i % top] : -1;
  const bool ok = e >= 0 && e < E;
  sel[i] = ok ? e : 0;
  wgt[i] = ok ? 1.f / static_cast<float>(top) : 0.f;
}
}  // namespace

KVF_EXPORT int kvf_moe_topk(const float* z, int z_stride, const float* correction, int* sel, float* wgt,
                            int n, int R, int top, hipStream_t s) {
  if (n <= 0) return 0;
  if (R <= 0 || R > MAX_PER_LANE * KVF_WAVE || top <= 0 || top > MAX_TOP || top > R)
    return static_cast<int>(hipErrorInvalidValue);
  hipLaunchKernelGGL(moe_topk_kernel, dim3(n), dim3(KVF_WAVE), 0, s, z, z_stride, correction, sel, wgt, R, top);
  return kvf_last_error();
}

KVF_EXPORT int kvf_moe_table(const int* tokens, const int* table, int* sel, float* wgt, int n, int vocab, int top,
                             int E, hipStream_t s) {
  if (n <= 0) return 0;
  if (vocab <= 0 || top <= 0 || top > MAX_TOP || E <= 0) return static_cast<int>(hipErrorInvalidValue);
  hipLaunchKernelGGL(moe_table_kernel, dim3((n * top + 255) / 256), dim3(256), 0, s, tokens, table, sel, wgt, n,
                     vocab, top, E);
  return kvf_last_error();
}

KVF_EXPORT int kvf_moe_dense_act(int dtype, const void* gu, const int* sel, const float* wgt, void* act,
                                 int n, int E, int ff, int top, hipStream_t s) {
  const long total = static_cast<long>(n) * E * ff;
  if (total <= 0) return 0;
  const dim3 grid(static_cast<unsigned>((total + 255) / 256));
  if (dtype == 0)
    hipLaunchKernelGGL(moe_dense_act_kernel<float>, grid, dim3(256), 0, s, static_cast<const float*>(gu), sel,
                       wgt, static_cast<float*>(act), E, ff, top, total);
  else if (dtype == 1)
    hipLaunchKernelGGL(moe_dense_act_kernel<bf16_t>, grid, dim3(256), 0, s, static_cast<const bf16_t*>(gu), sel,
                       wgt, static_cast<bf16_t*>(act), E, ff, top, total);
  else
    return static_cast<int>(hipErrorInvalidValue);
  return kvf_last_error();
}

KVF_EXPORT int kvf_moe_identity(int dtype, float* x, const void* h, const int* sel, const float* wgt, int n,
                                int width, int top, int first, hipStream_t s) {
  if (n <= 0) return 0;
  if (dtype == 0)
    hipLaunchKernelGGL(moe_identity_kernel<float>, dim3(n), dim3(256), 0, s, x, static_cast<const float*>(h),
                       sel, wgt, width, top, first);
  else if (dtype == 1)
    hipLaunchKernelGGL(moe_identity_kernel<bf16_t>, dim3(n), dim3(256), 0, s, x, static_cast<const bf16_t*>(h),
                       sel, wgt, width, top, first);
  else
    return static_cast<int>(hipErrorInvalidValue);
  return kvf_last_error();
}

// The routed experts of a bf16 step without the rows that did not choose them.  x [n, K] (row
// stride ldx), w_gate_up / w_down: the tiled forms of [E 2 ff, K] (gate and up rows interleaved)
// and [K, E ff]; sel / wgt [n, top]; scratch: where, order [n top], tiles [3 max_tiles],
// num_tiles [1], act [n top, ff], y [n top, K].  Needs K % 8 == 0 and ff % 32 == 0.
KVF_EXPORT int kvf_moe_grouped(const void* x, int ldx, const void* h, int n, int K, int E, int ff, int top,
                               const void* w_gate_up, const void* w_down, const int* sel, const float* wgt,
                               int* where, int* order, int* tiles, int* num_tiles, int max_tiles, void* act,
                               void* y, float* residual, hipStream_t s) {
  if (n <= 0) return 0;
  const int pairs = n * top;
  // many rows: tiles of 64 rows (four sub-tiles share every weight fragment); few: tiles of 16
  const bool many = pairs >= 1024;
  const int tile_rows = many ? 64 : 16;
  if (E <= 0 || E > PLAN_MAX_EXPERTS || K % 8 != 0 || ff % 32 != 0 || ldx % 8 != 0 || max_tiles > 65535 ||
      max_tiles < (pairs + 15) / 16 + E)
    return static_cast<int>(hipErrorInvalidValue);
  hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), 0, s, sel, pairs, E, where, order, tiles, num_tiles,
                     max_tiles, tile_rows);
  const int S = (K + 31) / 32, up_groups = ff / 8, down_groups = (K + 15) / 16;
  const int gw = many ? 4 : 1;
  const int grid_tiles = many ? (pairs + 63) / 64 + E : max_tiles;
  const dim3 up_grid((up_groups + 4 * gw - 1) / (4 * gw), grid_tiles), down_grid((down_groups + 4 * gw - 1) / (4 * gw), grid_tiles);
  const bf16_t* xb = static_cast<const bf16_t*>(x);
  if (many) {
    hipLaunchKernelGGL((moe_up_kernel<4, 4>), up_grid, dim3(256), 0, s, xb, ldx, K, static_cast<const uint4*>(w_gate_up), S,
                       order, tiles, num_tiles, top, ff, static_cast<bf16_t*>(act));
    hipLaunchKernelGGL((moe_down_kernel<4, 4>), down_grid, dim3(256), 0, s, static_cast<const bf16_t*>(act), ff,
                       static_cast<const uint4*>(w_down), E * (ff / 32), tiles, num_tiles, static_cast<bf16_t*>(y), K);
  } else {
    hipLaunchKernelGGL((moe_up_kernel<1, 1>), up_grid, dim3(256), 0, s, xb, ldx, K, static_cast<const uint4*>(w_gate_up), S,
                       order, tiles, num_tiles, top, ff, static_cast<bf16_t*>(act));
    hipLaunchKernelGGL((moe_down_kernel<1, 1>), down_grid, dim3(256), 0, s, static_cast<const bf16_t*>(act), ff,
                       static_cast<const uint4*>(w_down), E * (ff / 32), tiles, num_tiles, static_cast<bf16_t*>(y), K);
  }
  hipLaunchKernelGGL(moe_combine_kernel<bf16_t>, dim3(n), dim3(256), 0, s, residual, static_cast<const bf16_t*>(y),
                     static_cast<const bf16_t*>(h), sel, wgt, where, K, top, E);
  return kvf_last_error();
}
