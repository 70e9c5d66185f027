// Row-wise kernels of the decoder: embedding gather, RMS norm, SwiGLU gate, rotary + cache write.
// The residual stream is fp32 in every mode; T is the activation / weight element type.
#include "common.h"

// ----------------------------------------------------------------------------- embedding
// out[n, :] = table[ids[n], :] widened to fp32, times `scale` (an fp32 multiply; 1 changes
// nothing).  An id outside [0, vocab) writes zeros.
template <typename T>
__global__ void embed_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                             float* __restrict__ out, int h, int vocab, float scale) {
  const int n = blockIdx.x;
  const int id = ids[n];
  float* o = out + static_cast<size_t>(n) * h;
  if (id < 0 || id >= vocab) {
    for (int i = threadIdx.x; i < h; i += blockDim.x) o[i] = 0.f;
    return;
  }
  const T* row = table + static_cast<size_t>(id) * h;
  for (int i = threadIdx.x; i < h; i += blockDim.x) o[i] = Elem<T>::load(row + i) * scale;
}

template <typename T>
static int embed_launch(const int* ids, const void* table, float* out, int n, int h, int vocab,
                        float scale, hipStream_t s) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL(embed_kernel<T>, dim3(n), dim3(256), 0, s, ids, static_cast<const T*>(table),
                     out, h, vocab, scale);
  return kvf_last_error();
}
KVF_EXPORT int kvf_embed_f32(const int* ids, const void* t, float* o, int n, int h, int v, float scale,
                             hipStream_t s) { return embed_launch<float>(ids, t, o, n, h, v, scale, s); }
KVF_EXPORT int kvf_embed_bf16(const int* ids, const void* t, float* o, int n, int h, int v, float scale,
                              hipStream_t s) { return embed_launch<bf16_t>(ids, t, o, n, h, v, scale, s); }

// ----------------------------------------------------------------------------- RMS norm
// y = x * rsqrt(mean(x^2) + eps) * w, all in fp32, rounded once to T on store.
// x is the fp32 residual stream; `rows` (may be null) gathers input rows; w is fp32 or T, or
// null when the weight has been folded into the matrix that consumes y.
// `delta` (may be null, [x_rows, h] of T) is a sum still owed to the stream: the norm is taken of
// x + delta, and without `rows` the sum is also written back to x, which saves the pass of an
// add kernel of its own.
__device__ __forceinline__ float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4(const bf16_t* p) {
  const uint2 r = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u),
                     __uint_as_float(r.y << 16), __uint_as_float(r.y & 0xffff0000u));
}
__device__ __forceinline__ void store4(float* p, const float4& v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void store4(bf16_t* p, const float4& v) {
  uint2 r;
  r.x = static_cast<uint32_t>(f32_to_bf16(v.x)) | (static_cast<uint32_t>(f32_to_bf16(v.y)) << 16);
  r.y = static_cast<uint32_t>(f32_to_bf16(v.z)) | (static_cast<uint32_t>(f32_to_bf16(v.w)) << 16);
  *reinterpret_cast<uint2*>(p) = r;
}

constexpr int NORM_KEEP = 4;  // float4s a thread keeps in registers between the two passes

template <typename T, typename W, typename D>
__global__ void rmsnorm_kernel(float* __restrict__ x, const int* __restrict__ rows,
                               const D* __restrict__ delta, const W* __restrict__ w, float eps,
                               T* __restrict__ out, int h, int x_rows, int aligned) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  int src = rows ? rows[m] : m;
  T* o = out + static_cast<size_t>(m) * h;
  if (src < 0 || src >= x_rows) {
    for (int i = threadIdx.x; i < h; i += blockDim.x) Elem<T>::store(o + i, 0.f);
    return;
  }
  float* xr = x + static_cast<size_t>(src) * h;
  const D* dr = delta ? delta + static_cast<size_t>(src) * h : nullptr;
  const bool write_back = dr && !rows;
  float ss = 0.f;
  if (aligned && h <= static_cast<int>(blockDim.x) * 4 * NORM_KEEP) {
    // the row stays in registers: one read of x (and delta), one write of y (and x)
    float4 v[NORM_KEEP];
#pragma unroll
    for (int k = 0; k < NORM_KEEP; ++k) {
      const int i = (k * blockDim.x + threadIdx.x) * 4;
      v[k] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (i < h) {
        v[k] = load4(xr + i);
        if (dr) {
          const float4 d = load4(dr + i);
          v[k].x += d.x; v[k].y += d.y; v[k].z += d.z; v[k].w += d.w;
          if (write_back) store4(xr + i, v[k]);
        }
        ss += v[k].x * v[k].x + v[k].y * v[k].y + v[k].z * v[k].z + v[k].w * v[k].w;
      }
    }
    ss = block_sum(ss, scratch);
    const float r = rsqrtf(ss / static_cast<float>(h) + eps);
#pragma unroll
    for (int k = 0; k < NORM_KEEP; ++k) {
      const int i = (k * blockDim.x + threadIdx.x) * 4;
      if (i < h) {
        float4 y = make_float4(v[k].x * r, v[k].y * r, v[k].z * r, v[k].w * r);
        if (w) {
          const float4 g = load4(w + i);
          y.x *= g.x; y.y *= g.y; y.z *= g.z; y.w *= g.w;
        }
        store4(o + i, y);
      }
    }
    return;
  }
  for (int i = threadIdx.x; i < h; i += blockDim.x) {
    float v = xr[i];
    if (dr) {
      v += Elem<D>::load(dr + i);
      if (write_back) xr[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float r = rsqrtf(ss / static_cast<float>(h) + eps);
  for (int i = threadIdx.x; i < h; i += blockDim.x) {
    float v = xr[i];  // already the sum where it was written back (by this same thread)
    if (dr && !write_back) v += Elem<D>::load(dr + i);
    Elem<T>::store(o + i, w ? v * r * Elem<W>::load(w + i) : v * r);
  }
}

template <typename T, typename D>
static int rmsnorm_launch(float* x, const int* rows, const void* delta, const void* w, int w_is_f32,
                          float eps, void* out, int m, int h, int x_rows, hipStream_t s) {
  if (m <= 0) return 0;
  const int threads = h >= 1024 ? 256 : (h >= 256 ? 128 : 64);
  auto at = [](const void* p, size_t a) { return reinterpret_cast<uintptr_t>(p) % a == 0; };
  const int aligned = h % 4 == 0 && at(x, 16) && at(out, 4 * sizeof(T)) && at(delta, 4 * sizeof(D)) &&
                      at(w, w_is_f32 ? 16 : 4 * sizeof(T));
  if (w_is_f32)
    hipLaunchKernelGGL((rmsnorm_kernel<T, float, D>), dim3(m), dim3(threads), 0, s, x, rows,
                       static_cast<const D*>(delta), static_cast<const float*>(w), eps,
                       static_cast<T*>(out), h, x_rows, aligned);
  else
    hipLaunchKernelGGL((rmsnorm_kernel<T, T, D>), dim3(m), dim3(threads), 0, s, x, rows,
                       static_cast<const D*>(delta), static_cast<const T*>(w), eps,
                       static_cast<T*>(out), h, x_rows, aligned);
  return kvf_last_error();
}
// delta (may be null): a sum still owed to x, in the type of `out` or (delta_f32) in fp32
KVF_EXPORT int kvf_rmsnorm_f32(float* x, const int* rows, const void* delta, int delta_f32, const void* w,
                               int wf, float eps, void* out, int m, int h, int xr, hipStream_t s) {
  (void)delta_f32;
  return rmsnorm_launch<float, float>(x, rows, delta, w, wf, eps, out, m, h, xr, s);
}
KVF_EXPORT int kvf_rmsnorm_bf16(float* x, const int* rows, const void* delta, int delta_f32, const void* w,
                                int wf, float eps, void* out, int m, int h, int xr, hipStream_t s) {
  if (delta_f32) return rmsnorm_launch<bf16_t, float>(x, rows, delta, w, wf, eps, out, m, h, xr, s);
  return rmsnorm_launch<bf16_t, bf16_t>(x, rows, delta, w, wf, eps, out, m, h, xr, s);
}

// Two norms of the same row in one pass: y1 = v r w1 and y2 = v r w2 with v = x (+ delta, which is
// then written back to x) and r = rsqrt(mean(v^2) + eps): for a block whose two sublayers each
// have a norm of their own over the same stream.  Weights are fp32.
template <typename T, typename D>
__global__ void rmsnorm_pair_kernel(float* __restrict__ x, const D* __restrict__ delta,
                                    const float* __restrict__ w1, const float* __restrict__ w2, float eps,
                                    T* __restrict__ out1, T* __restrict__ out2, int h) {
  __shared__ float scratch[16];
  const size_t m = blockIdx.x;
  float* xr = x + m * h;
  const D* dr = delta ? delta + m * h : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < h; i += blockDim.x) {
    float v = xr[i];
    if (dr) {
      v += Elem<D>::load(dr + i);
      xr[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float r = rsqrtf(ss / static_cast<float>(h) + eps);
  for (int i = threadIdx.x; i < h; i += blockDim.x) {
    const float v = xr[i] * r;   // the sum where it was written back (by this same thread)
    Elem<T>::store(out1 + m * h + i, v * w1[i]);
    Elem<T>::store(out2 + m * h + i, v * w2[i]);
  }
}
template <typename T, typename D>
static int rmsnorm_pair_launch(float* x, const void* delta, const float* w1, const float* w2, float eps, void* o1,
                               void* o2, int m, int h, hipStream_t s) {
  if (m <= 0) return 0;
  const int threads = h >= 1024 ? 256 : (h >= 256 ? 128 : 64);
  hipLaunchKernelGGL((rmsnorm_pair_kernel<T, D>), dim3(m), dim3(threads), 0, s, x, static_cast<const D*>(delta), w1, w2,
                     eps, static_cast<T*>(o1), static_cast<T*>(o2), h);
  return kvf_last_error();
}
KVF_EXPORT int kvf_rmsnorm_pair_f32(float* x, const void* delta, int delta_f32, const float* w1, const float* w2,
                                    float eps, void* o1, void* o2, int m, int h, hipStream_t s) {
  (void)delta_f32;
  return rmsnorm_pair_launch<float, float>(x, delta, w1, w2, eps, o1, o2, m, h, s);
}
KVF_EXPORT int kvf_rmsnorm_pair_bf16(float* x, const void* delta, int delta_f32, const float* w1, const float* w2,
                                     float eps, void* o1, void* o2, int m, int h, hipStream_t s) {
  if (delta_f32) return rmsnorm_pair_launch<bf16_t, float>(x, delta, w1, w2, eps, o1, o2, m, h, s);
  return rmsnorm_pair_launch<bf16_t, bf16_t>(x, delta, w1, w2, eps, o1, o2, m, h, s);
}

// ----------------------------------------------------------------------------- residual sum
// x[m] += delta[m] in fp32 (x is the residual stream, delta a product in T).
template <typename T>
__global__ void add_rows_kernel(float* __restrict__ x, const T* __restrict__ delta, size_t total) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < total) x[i] += Elem<T>::load(delta + i);
}
template <typename T>
static int add_rows_launch(float* x, const void* delta, int m, int h, hipStream_t s) {
  const size_t total = static_cast<size_t>(m) * h;
  if (total == 0) return 0;
  hipLaunchKernelGGL(add_rows_kernel<T>, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, s,
                     x, static_cast<const T*>(delta), total);
  return kvf_last_error();
}
KVF_EXPORT int kvf_add_rows_f32(float* x, const void* d, int m, int h, hipStream_t s) {
  return add_rows_launch<float>(x, d, m, h, s);
}
KVF_EXPORT int kvf_add_rows_bf16(float* x, const void* d, int m, int h, hipStream_t s) {
  return add_rows_launch<bf16_t>(x, d, m, h, s);
}

// ----------------------------------------------------------------------------- SwiGLU gate
// out[m, i] = silu(gate) * up with silu(x) = x / (1 + exp(-x)), in fp32.  The input row holds
// gate and up side by side: gate at 2i and up at 2i + 1 (`paired` != 0, the layout the fused
// gate/up matrix produces) or gate at i and up at I + i.
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter,
                                size_t total, int paired) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t m = idx / inter;
  const int i = static_cast<int>(idx - m * inter);
  const T* row = gu + m * 2 * static_cast<size_t>(inter);
  const float g = Elem<T>::load(paired ? row + 2 * i : row + i);
  const float u = Elem<T>::load(paired ? row + 2 * i + 1 : row + inter + i);
  Elem<T>::store(out + idx, g / (1.f + expf(-g)) * u);
}
// bf16, paired: a thread takes four neighbouring (gate, up) pairs (16 bytes in, 8 bytes out)
__global__ void silu_mul_pairs4_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out,
                                       size_t quads) {
  const size_t q = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (q >= quads) return;
  float v[8];
  load8(gu + q * 8, v);
  uint2 packed;
  uint32_t h[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) h[i] = f32_to_bf16(v[2 * i] / (1.f + __expf(-v[2 * i])) * v[2 * i + 1]);
  packed.x = h[0] | (h[1] << 16);
  packed.y = h[2] | (h[3] << 16);
  *reinterpret_cast<uint2*>(out + q * 4) = packed;
}

template <typename T>
static int silu_mul_launch(const void* gu, void* out, int m, int inter, int paired,
                           hipStream_t s) {
  const size_t total = static_cast<size_t>(m) * inter;
  if (total == 0) return 0;
  if (sizeof(T) == 2 && paired && inter % 4 == 0 && reinterpret_cast<uintptr_t>(gu) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(out) % 8 == 0) {
    const size_t quads = total / 4;
    hipLaunchKernelGGL(silu_mul_pairs4_kernel, dim3(static_cast<unsigned>((quads + 255) / 256)), dim3(256),
                       0, s, static_cast<const bf16_t*>(gu), static_cast<bf16_t*>(out), quads);
    return kvf_last_error();
  }
  const unsigned blocks = static_cast<unsigned>((total + 255) / 256);
  hipLaunchKernelGGL(silu_mul_kernel<T>, dim3(blocks), dim3(256), 0, s,
                     static_cast<const T*>(gu), static_cast<T*>(out), inter, total, paired);
  return kvf_last_error();
}
KVF_EXPORT int kvf_silu_mul_f32(const void* gu, void* out, int m, int inter, int paired,
                                hipStream_t s) {
  return silu_mul_launch<float>(gu, out, m, inter, paired, s);
}
KVF_EXPORT int kvf_silu_mul_bf16(const void* gu, void* out, int m, int inter, int paired,
                                 hipStream_t s) {
  return silu_mul_launch<bf16_t>(gu, out, m, inter, paired, s);
}

// ----------------------------------------------------------------------------- rotary + cache write
// qkv: [N, (H + 2*KV) * d] rows of q heads, then k heads, then v heads.
// A rotary pair is two neighbouring elements (2i, 2i + 1) of a head: the projection matrices
// are stored with their rows permuted so that what the checkpoint's layout calls elements i and
// i + rot/2 land there (a dot product of q and k does not care about the order, and v and the
// output projection are not permuted).  For token n at position p (cos/sin tables
// [table_len, rot/2] fp32) and i < rot/2:
//   x'[2i] = x[2i]*cos[i] - x[2i+1]*sin[i];   x'[2i+1] = x[2i+1]*cos[i] + x[2i]*sin[i]
// elements at or beyond `rot` are copied.  q is rotated in place.
// Rotated k and v go to the pages: page = block_table[seq_of_token[n], p / block_size];
// a negative page (padding, or a page already given back) or p outside the table skips the write.
// K pages are [num_blocks, KV, block_size, d]; V pages are transposed, [num_blocks, KV, d,
// block_size], so that the keys of one element lie side by side (what the P*V product of the
// matrix cores contracts over).  With write_kv == 0 only q is rotated.
struct RopeArgs {
  int H, KV, d, rot, table_len, block_size, table_stride, num_blocks, write_kv, n_seqs;
  int row_len;  // elements from one token's row to the next: (H + 2 KV) d, or more when the
                // product that made the rows has further columns behind q, k and v
};

template <typename T>
__global__ void rope_kvwrite_kernel(T* __restrict__ qkv, const int* __restrict__ positions,
                                    const int* __restrict__ seq_of_token,
                                    const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                    const int* __restrict__ block_table, T* __restrict__ k_pages,
                                    T* __restrict__ v_pages, RopeArgs a) {
  const int n = blockIdx.x;
  const int p = positions[n];
  const int half = a.rot / 2;
  T* row = qkv + static_cast<size_t>(n) * a.row_len;
  const bool pos_ok = p >= 0 && p < a.table_len;
  const float* cs = cos_t + static_cast<size_t>(pos_ok ? p : 0) * half;
  const float* sn = sin_t + static_cast<size_t>(pos_ok ? p : 0) * half;

  int page = -1, off = 0;
  if (a.write_kv && pos_ok) {
    const int seq = seq_of_token[n];
    const int blk = p / a.block_size;
    if (seq >= 0 && seq < a.n_seqs && blk < a.table_stride) {
      page = block_table[static_cast<size_t>(seq) * a.table_stride + blk];
      if (page >= a.num_blocks) page = -1;
      off = p - blk * a.block_size;
    }
  }
  // q heads: rotate in place (pairs are owned by one thread, so no hazard)
  const int q_pairs = a.H * half;
  for (int t = threadIdx.x; t < q_pairs; t += blockDim.x) {
    const int hh = t / half, i = t - hh * half;
    T* x = row + hh * a.d;
    const float x1 = Elem<T>::load(x + 2 * i), x2 = Elem<T>::load(x + 2 * i + 1);
    const float c = pos_ok ? cs[i] : 1.f, s = pos_ok ? sn[i] : 0.f;
    Elem<T>::store(x + 2 * i, x1 * c - x2 * s);
    Elem<T>::store(x + 2 * i + 1, x2 * c + x1 * s);
  }
  if (page < 0) return;
  // k heads: rotate, write to the page; the unrotated tail is copied
  const int k_pairs = a.KV * half;
  for (int t = threadIdx.x; t < k_pairs; t += blockDim.x) {
    const int hh = t / half, i = t - hh * half;
    const T* x = row + (a.H + hh) * a.d;
    T* dst = k_pages + ((static_cast<size_t>(page) * a.KV + hh) * a.block_size + off) * a.d;
    const float x1 = Elem<T>::load(x + 2 * i), x2 = Elem<T>::load(x + 2 * i + 1);
    Elem<T>::store(dst + 2 * i, x1 * cs[i] - x2 * sn[i]);
    Elem<T>::store(dst + 2 * i + 1, x2 * cs[i] + x1 * sn[i]);
  }
  const int tail = a.d - a.rot;
  for (int t = threadIdx.x; t < a.KV * tail; t += blockDim.x) {
    const int hh = t / tail, i = a.rot + (t - hh * tail);
    T* dst = k_pages + ((static_cast<size_t>(page) * a.KV + hh) * a.block_size + off) * a.d;
    dst[i] = row[(a.H + hh) * a.d + i];
  }
  for (int t = threadIdx.x; t < a.KV * a.d; t += blockDim.x) {
    const int hh = t / a.d, i = t - hh * a.d;
    v_pages[((static_cast<size_t>(page) * a.KV + hh) * a.d + i) * a.block_size + off] =
        row[(a.H + a.KV + hh) * a.d + i];
  }
}

// The same work for a tile of 16 tokens per workgroup with 8 elements per lane and access
// (d and the rotary width multiples of 8).  V is stored transposed, so a token's elements lie
// block_size apart; where the tile's 16 tokens fill consecutive places of one page (a prompt
// read from a page boundary) the tile is turned in LDS and each (head, element) row of 16
// tokens is stored in one piece.  Other tiles store V element by element.
constexpr int ROPE_TILE = 16;

__device__ __forceinline__ void store8(float* p, const float (&v)[8]) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ void store8(bf16_t* p, const float (&v)[8]) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    w[i] = static_cast<uint32_t>(f32_to_bf16(v[2 * i])) | (static_cast<uint32_t>(f32_to_bf16(v[2 * i + 1])) << 16);
  *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
}

template <typename T>
__global__ __launch_bounds__(256) void rope_kvwrite_tile_kernel(
    T* __restrict__ qkv, const int* __restrict__ positions, const int* __restrict__ seq_of_token,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ block_table, T* __restrict__ k_pages, T* __restrict__ v_pages, int n,
    int turn_v, RopeArgs a) {
  extern __shared__ __align__(16) unsigned char tile_raw[];  // [ROPE_TILE][V columns of this share] of T, if turn_v
  __shared__ int s_pos[ROPE_TILE], s_page[ROPE_TILE], s_off[ROPE_TILE], s_run;
  const int n0 = blockIdx.x * ROPE_TILE;
  const int cnt = min(ROPE_TILE, n - n0);
  const int half = a.rot / 2;
  if (threadIdx.x < ROPE_TILE) {
    const int t = threadIdx.x;
    int p = -1, page = -1, off = 0;
    if (t < cnt) {
      p = positions[n0 + t];
      if (p < 0 || p >= a.table_len) p = -1;
      if (p >= 0 && a.write_kv) {
        const int seq = seq_of_token[n0 + t];
        const int blk = p / a.block_size;
        if (seq >= 0 && seq < a.n_seqs && blk < a.table_stride) {
          page = block_table[static_cast<size_t>(seq) * a.table_stride + blk];
          if (page >= a.num_blocks) page = -1;
          off = p - blk * a.block_size;
        }
      }
    }
    s_pos[t] = p;
    s_page[t] = page;
    s_off[t] = off;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    bool run = turn_v && cnt == ROPE_TILE && s_page[0] >= 0 && s_off[0] % 8 == 0 &&
               a.block_size % 8 == 0 && s_off[0] + ROPE_TILE <= a.block_size;
    for (int t = 1; t < ROPE_TILE; ++t) run = run && s_page[t] == s_page[0] && s_off[t] == s_off[0] + t;
    s_run = run;
  }
  __syncthreads();
  // blockIdx.y names a share of the row: of its q and k vectors, and of its V columns
  const int row_len = a.row_len;
  const int qk_vecs = (a.H + a.KV) * a.d / 8;
  const int qk_share = (qk_vecs + gridDim.y - 1) / gridDim.y;
  const int qk_begin = blockIdx.y * qk_share;
  const int qk_mine = max(0, min(qk_share, qk_vecs - qk_begin));
  for (int item = threadIdx.x; item < cnt * qk_mine; item += blockDim.x) {
    const int t = item / qk_mine, e = (qk_begin + item - t * qk_mine) * 8;
    const int head = e / a.d, i0 = e - head * a.d;
    const bool is_k = head >= a.H;
    const int p = s_pos[t], page = s_page[t];
    // a query that is not rotated stays as it is; a key without a page is not stored
    if (is_k ? page < 0 : (p < 0 || i0 >= a.rot)) continue;
    T* src = qkv + static_cast<size_t>(n0 + t) * row_len + e;
    float x[8];
    load8(src, x);
    if (p >= 0 && i0 < a.rot) {
      const float4 c = *reinterpret_cast<const float4*>(cos_t + static_cast<size_t>(p) * half + i0 / 2);
      const float4 sn = *reinterpret_cast<const float4*>(sin_t + static_cast<size_t>(p) * half + i0 / 2);
      const float cs[4] = {c.x, c.y, c.z, c.w}, ss[4] = {sn.x, sn.y, sn.z, sn.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float x1 = x[2 * i], x2 = x[2 * i + 1];
        x[2 * i] = x1 * cs[i] - x2 * ss[i];
        x[2 * i + 1] = x2 * cs[i] + x1 * ss[i];
      }
    }
    T* dst = is_k ? k_pages + ((static_cast<size_t>(page) * a.KV + (head - a.H)) * a.block_size + s_off[t]) * a.d + i0
                  : src;
    store8(dst, x);
  }
  if (!a.write_kv) return;
  const int v0 = (a.H + a.KV) * a.d, v_len = a.KV * a.d;
  const int v_share = (v_len / 8 + gridDim.y - 1) / gridDim.y * 8;  // columns, whole vectors
  const int v_begin = blockIdx.y * v_share;
  const int v_mine = max(0, min(v_share, v_len - v_begin));
  if (s_run) {
    T* tile = reinterpret_cast<T*>(tile_raw);  // [ROPE_TILE][v_share]
    const int v_vecs = v_mine / 8;
    for (int item = threadIdx.x; item < ROPE_TILE * v_vecs; item += blockDim.x) {
      const int t = item / v_vecs, e = (item - t * v_vecs) * 8;
      const T* src = qkv + static_cast<size_t>(n0 + t) * row_len + v0 + v_begin + e;
      constexpr int Q = sizeof(T) * 8 / 16;  // 16-byte pieces of eight elements
#pragma unroll
      for (int q = 0; q < Q; ++q)
        reinterpret_cast<uint4*>(tile + t * v_share + e)[q] = reinterpret_cast<const uint4*>(src)[q];
    }
    __syncthreads();
    const int page = s_page[0], off0 = s_off[0];
    for (int c = threadIdx.x; c < v_mine; c += blockDim.x) {  // v_begin + c = head * d + element
      __align__(16) T vals[ROPE_TILE];
#pragma unroll
      for (int t = 0; t < ROPE_TILE; ++t) vals[t] = tile[t * v_share + c];
      T* dst = v_pages + (static_cast<size_t>(page) * v_len + v_begin + c) * a.block_size + off0;
      constexpr int Q = sizeof(T) * ROPE_TILE / 16;
#pragma unroll
      for (int q = 0; q < Q; ++q) reinterpret_cast<uint4*>(dst)[q] = reinterpret_cast<const uint4*>(vals)[q];
    }
  } else {
    for (int item = threadIdx.x; item < cnt * v_mine; item += blockDim.x) {
      const int t = item / v_mine, c = v_begin + item - t * v_mine;
      const int page = s_page[t];
      if (page < 0) continue;
      v_pages[(static_cast<size_t>(page) * v_len + c) * a.block_size + s_off[t]] =
          qkv[static_cast<size_t>(n0 + t) * row_len + v0 + c];
    }
  }
}

template <typename T>
static int rope_launch(void* qkv, const int* positions, const int* seq_of_token, const float* cos_t,
                       const float* sin_t, const int* block_table, void* k_pages, void* v_pages,
                       int n, RopeArgs a, hipStream_t s) {
  if (n <= 0) return 0;
  if (a.d % 8 == 0 && a.rot % 8 == 0 && a.row_len % 8 == 0) {
    // few tiles: several workgroups share a tile's row, so that the chip has work
    const int tiles = (n + ROPE_TILE - 1) / ROPE_TILE;
    int shares = tiles >= 512 ? 1 : (512 + tiles - 1) / tiles;
    if (shares > 8) shares = 8;
    const int v_share = (a.KV * a.d / 8 + shares - 1) / shares * 8;
    // the tile of V rows turned in LDS; without room for it V goes element by element
    const size_t lds = static_cast<size_t>(ROPE_TILE) * v_share * sizeof(T);
    const int turn_v = lds <= 48 * 1024;
    hipLaunchKernelGGL(rope_kvwrite_tile_kernel<T>, dim3(tiles, shares), dim3(256), turn_v ? lds : 0, s,
                       static_cast<T*>(qkv), positions, seq_of_token, cos_t, sin_t, block_table,
                       static_cast<T*>(k_pages), static_cast<T*>(v_pages), n, turn_v, a);
    return kvf_last_error();
  }
  hipLaunchKernelGGL(rope_kvwrite_kernel<T>, dim3(n), dim3(128), 0, s, static_cast<T*>(qkv),
                     positions, seq_of_token, cos_t, sin_t, block_table, static_cast<T*>(k_pages),
                     static_cast<T*>(v_pages), a);
  return kvf_last_error();
}
#define ROPE_ARGS_DECL                                                                           \
  void *qkv, const int *positions, const int *seq_of_token, const float *cos_t,                 \
      const float *sin_t, const int *block_table, void *k_pages, void *v_pages, int n, int H,   \
      int KV, int d, int rot, int table_len, int block_size, int table_stride, int num_blocks,  \
      int write_kv, int n_seqs, int row_len, hipStream_t s
#define ROPE_ARGS_PACK                                                                           \
  RopeArgs { H, KV, d, rot, table_len, block_size, table_stride, num_blocks, write_kv, n_seqs, row_len }
KVF_EXPORT int kvf_rope_kvwrite_f32(ROPE_ARGS_DECL) {
  return rope_launch<float>(qkv, positions, seq_of_token, cos_t, sin_t, block_table, k_pages,
                            v_pages, n, ROPE_ARGS_PACK, s);
}
KVF_EXPORT int kvf_rope_kvwrite_bf16(ROPE_ARGS_DECL) {
  return rope_launch<bf16_t>(qkv, positions, seq_of_token, cos_t, sin_t, block_table, k_pages,
                             v_pages, n, ROPE_ARGS_PACK, s);
}

// The same with a norm per head in front of the rotation: every q head and every k head is
// divided by the root mean square of its first `dk` elements (eps inside the root) and
// multiplied by a weight vector of dk numbers that all q heads (qw) or all k heads (kw) share,
// all in fp32 from the projected row; then rotated and stored as above, one rounding.  Elements
// dk..d-1 of a head (padding of the kernels' head size) are zero and stay zero.  A workgroup
// takes a token, its waves take the heads in turn; a lane holds the pairs lane and lane + 64.
template <typename T>
__global__ __launch_bounds__(256) void qknorm_rope_kvwrite_kernel(
    T* __restrict__ qkv, const int* __restrict__ positions, const int* __restrict__ seq_of_token,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ block_table, T* __restrict__ k_pages, T* __restrict__ v_pages,
    const float* __restrict__ qw, const float* __restrict__ kw, int dk, float eps, float qt_coef,
    int qt_every, RopeArgs a) {
  const int n = blockIdx.x;
  const int p = positions[n];
  const int half = a.rot / 2;
  T* row = qkv + static_cast<size_t>(n) * a.row_len;
  const bool pos_ok = p >= 0 && p < a.table_len;
  // query temperature: q heads are stretched by 1 + coef * ln(floor((p + 1) / every) + 1)
  const float q_temp = qt_every > 0 && p >= 0
                           ? 1.f + qt_coef * logf(static_cast<float>((p + 1) / qt_every) + 1.f)
                           : 1.f;
  const float* cs = cos_t ? cos_t + static_cast<size_t>(pos_ok ? p : 0) * half : nullptr;
  const float* sn = sin_t ? sin_t + static_cast<size_t>(pos_ok ? p : 0) * half : nullptr;
  int page = -1, off = 0;
  if (a.write_kv && pos_ok) {
    const int seq = seq_of_token[n];
    const int blk = p / a.block_size;
    if (seq >= 0 && seq < a.n_seqs && blk < a.table_stride) {
      page = block_table[static_cast<size_t>(seq) * a.table_stride + blk];
      if (page >= a.num_blocks) page = -1;
      off = p - blk * a.block_size;
    }
  }
  const int lane = threadIdx.x % KVF_WAVE, wave = threadIdx.x / KVF_WAVE, waves = blockDim.x / KVF_WAVE;
  const int heads = a.H + (a.write_kv ? a.KV : 0);
  // blockIdx.y names a share of the token's heads (and of its V elements): few tokens still fill the chip
  for (int hh = blockIdx.y * waves + wave; hh < heads; hh += gridDim.y * waves) {
    const bool is_k = hh >= a.H;
    if (is_k && page < 0) continue;
    T* x = row + hh * a.d;
    const float* w = is_k ? kw : qw;
    float u[2], v[2], ss = 0.f;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int e = 2 * (lane + KVF_WAVE * j);
      u[j] = e < dk ? Elem<T>::load(x + e) : 0.f;
      v[j] = e + 1 < dk ? Elem<T>::load(x + e + 1) : 0.f;
      ss = fmaf(u[j], u[j], fmaf(v[j], v[j], ss));
    }
    const float r = (is_k ? 1.f : q_temp) / sqrtf(wave_sum(ss) / static_cast<float>(dk) + eps);
    T* dst = is_k ? k_pages + ((static_cast<size_t>(page) * a.KV + (hh - a.H)) * a.block_size + off) * a.d : x;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int i = lane + KVF_WAVE * j, e = 2 * i;
      if (e >= a.d) continue;
      float y0 = e < dk ? u[j] * r * w[e] : 0.f;
      float y1 = e + 1 < dk ? v[j] * r * w[e + 1] : 0.f;
      if (e < a.rot && pos_ok && cs) {
        const float c = cs[i], sv = sn[i];
        const float t0 = y0 * c - y1 * sv, t1 = y1 * c + y0 * sv;
        y0 = t0;
        y1 = t1;
      }
      Elem<T>::store(dst + e, y0);
      if (e + 1 < a.d) Elem<T>::store(dst + e + 1, y1);
    }
  }
  if (page < 0) return;
  for (int t = blockIdx.y * blockDim.x + threadIdx.x; t < a.KV * a.d; t += gridDim.y * blockDim.x) {
    const int hh = t / a.d, i = t - hh * a.d;
    v_pages[((static_cast<size_t>(page) * a.KV + hh) * a.d + i) * a.block_size + off] =
        row[(a.H + a.KV + hh) * a.d + i];
  }
}

template <typename T>
static int qknorm_rope_launch(void* qkv, const int* positions, const int* seq_of_token, const float* cos_t,
                              const float* sin_t, const int* block_table, void* k_pages, void* v_pages,
                              const float* qw, const float* kw, int dk, float eps, float qt_coef,
                              int qt_every, int n, RopeArgs a, hipStream_t s) {
  if (n <= 0) return 0;
  if (a.d > 4 * KVF_WAVE || dk > a.d || dk <= 0 || a.rot > dk || a.rot % 2 || !qw || (a.write_kv && !kw))
    return static_cast<int>(hipErrorInvalidValue);
  // a wave a head where the tokens alone do not fill the chip; four heads a wave for many tokens
  const int heads = a.H + (a.write_kv ? a.KV : 0);
  int shares = n >= 1024 ? 1 : (heads + 3) / 4;
  if (shares > 64) shares = 64;
  hipLaunchKernelGGL(qknorm_rope_kvwrite_kernel<T>, dim3(n, shares), dim3(256), 0, s, static_cast<T*>(qkv), positions,
                     seq_of_token, cos_t, sin_t, block_table, static_cast<T*>(k_pages),
                     static_cast<T*>(v_pages), qw, kw, dk, eps, qt_coef, qt_every, a);
  return kvf_last_error();
}
#define QKNORM_ARGS_DECL                                                                         \
  void *qkv, const int *positions, const int *seq_of_token, const float *cos_t,                 \
      const float *sin_t, const int *block_table, void *k_pages, void *v_pages, const float *qw, \
      const float *kw, int dk, float eps, float qt_coef, int qt_every, int n, int H, int KV,    \
      int d, int rot, int table_len,                                                             \
      int block_size, int table_stride, int num_blocks, int write_kv, int n_seqs, int row_len,   \
      hipStream_t s
KVF_EXPORT int kvf_qknorm_rope_kvwrite_f32(QKNORM_ARGS_DECL) {
  return qknorm_rope_launch<float>(qkv, positions, seq_of_token, cos_t, sin_t, block_table, k_pages,
                                   v_pages, qw, kw, dk, eps, qt_coef, qt_every, n, ROPE_ARGS_PACK, s);
}
KVF_EXPORT int kvf_qknorm_rope_kvwrite_bf16(QKNORM_ARGS_DECL) {
  return qknorm_rope_launch<bf16_t>(qkv, positions, seq_of_token, cos_t, sin_t, block_table, k_pages,
                                    v_pages, qw, kw, dk, eps, qt_coef, qt_every, n, ROPE_ARGS_PACK, s);
}

// ----------------------------------------------------------------------------- soft cap
// x = cap * tanh(x * scale / cap) over fp32 values (logits), in place; cap 0: x = x * scale.
__global__ void softcap_kernel(float* __restrict__ x, long total, float cap, float scale) {
  const long i = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const float v = x[i] * scale;
  x[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
}
KVF_EXPORT int kvf_softcap(float* x, long total, float cap, float scale, hipStream_t s) {
  if (total <= 0) return 0;
  if (!(cap >= 0.f)) return static_cast<int>(hipErrorInvalidValue);
  hipLaunchKernelGGL(softcap_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, s, x,
                     total, cap, scale);
  return kvf_last_error();
}

// ----------------------------------------------------------------------------- learned positions
// x[n, :] += table[positions[n], :] in fp32 (an absolute position encoding on the embedding
// output).  A position outside the table adds nothing.
template <typename T>
__global__ void add_positions_kernel(float* __restrict__ x, const T* __restrict__ table,
                                     const int* __restrict__ positions, int h, int table_len) {
  const int n = blockIdx.x;
  const int p = positions[n];
  if (p < 0 || p >= table_len) return;
  float* o = x + static_cast<size_t>(n) * h;
  const T* row = table + static_cast<size_t>(p) * h;
  for (int i = threadIdx.x; i < h; i += blockDim.x) o[i] += Elem<T>::load(row + i);
}
template <typename T>
static int add_positions_launch(float* x, const void* table, const int* positions, int n, int h,
                                int table_len, hipStream_t s) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL(add_positions_kernel<T>, dim3(n), dim3(256), 0, s, x, static_cast<const T*>(table),
                     positions, h, table_len);
  return kvf_last_error();
}
KVF_EXPORT int kvf_add_positions_f32(float* x, const void* t, const int* p, int n, int h, int len,
                                     hipStream_t s) { return add_positions_launch<float>(x, t, p, n, h, len, s); }
KVF_EXPORT int kvf_add_positions_bf16(float* x, const void* t, const int* p, int n, int h, int len,
                                      hipStream_t s) { return add_positions_launch<bf16_t>(x, t, p, n, h, len, s); }

// ----------------------------------------------------------------------------- norm + token shift
// For token t of the flat batch, with y(r) = x[r] * rsqrt(mean(x[r]^2) + eps) * w (all fp32):
//   plain[t]   = y(t)
//   shifted[t] = y(t) + (prev - y(t)) * mu,   prev = the y of the token before t in its sequence:
//     zeros at position 0; y(t - 1) where t - 1 belongs to the same query run (computed again
//     here, with the same order of sums, so that it is the number the other workgroup stores);
//     state[slot of the sequence] for the first token of a run that continues a sequence.
// The workgroup of a run's first token is also the one that leaves the y of the run's *last*
// token in the sequence's state slot, after it has read the slot: no other workgroup touches
// that slot, so reading and writing it need no order between workgroups.  A sequence without a
// slot (negative: the padding of a captured batch) has no state.
constexpr int SHIFT_THREADS = 512, SHIFT_KEEP = 8;  // rows up to 4,096 elements live in registers

template <typename T>
__global__ __launch_bounds__(SHIFT_THREADS) void norm_shift_kernel(
    const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ mu,
    float* __restrict__ state, const int* __restrict__ slot_ids, const int* __restrict__ seq_of_token,
    const int* __restrict__ cu_q, const int* __restrict__ positions, T* __restrict__ plain,
    T* __restrict__ shifted, float eps, int h, int n_seqs, int n_slots, int n_tokens) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  int seq = seq_of_token[t];
  if (seq < 0 || seq >= n_seqs) seq = -1;
  const int q_first = seq >= 0 ? cu_q[seq] : t;
  int q_last = seq >= 0 ? cu_q[seq + 1] - 1 : t;
  if (q_last < t || q_last >= n_tokens) q_last = t;
  const bool first = t == q_first;
  const int pos = positions[t];
  int slot = seq >= 0 ? slot_ids[seq] : -1;
  if (slot >= n_slots) slot = -1;
  const float* xr = x + static_cast<size_t>(t) * h;
  const float inv_h = 1.f / static_cast<float>(h);
  // where the predecessor comes from: 0 nothing, 1 the row before, 2 the state slot
  const int from = pos <= 0 ? 0 : (!first ? 1 : (slot >= 0 ? 2 : 0));
  const float* xp = xr - h;
  const float* st = slot >= 0 ? state + static_cast<size_t>(slot) * h : nullptr;
  const bool save = first && slot >= 0;
  const float* xl = x + static_cast<size_t>(q_last) * h;   // the row whose y goes to the slot

  // Everything a thread needs of its first SHIFT_KEEP elements is asked for before the first
  // reduction, so that the loads' latencies overlap; elements past them are read where used.
  float xv[SHIFT_KEEP], pv[SHIFT_KEEP], lv[SHIFT_KEEP], wv[SHIFT_KEEP], mv[SHIFT_KEEP];
  float ss = 0.f, sp = 0.f, sl = 0.f;
#pragma unroll
  for (int k = 0; k < SHIFT_KEEP; ++k) {
    const int i = threadIdx.x + k * SHIFT_THREADS;
    const bool in = i < h;
    xv[k] = in ? xr[i] : 0.f;
    pv[k] = !in ? 0.f : (from == 1 ? xp[i] : (from == 2 ? st[i] : 0.f));
    lv[k] = in && save && q_last != t ? xl[i] : 0.f;
    wv[k] = in ? w[i] : 0.f;
    mv[k] = in ? mu[i] : 0.f;
  }
#pragma unroll
  for (int k = 0; k < SHIFT_KEEP; ++k) {
    ss = fmaf(xv[k], xv[k], ss);
    if (from == 1) sp = fmaf(pv[k], pv[k], sp);
    sl = fmaf(lv[k], lv[k], sl);
  }
  for (int i = threadIdx.x + SHIFT_KEEP * SHIFT_THREADS; i < h; i += SHIFT_THREADS) {
    ss = fmaf(xr[i], xr[i], ss);
    if (from == 1) sp = fmaf(xp[i], xp[i], sp);
    if (save && q_last != t) sl = fmaf(xl[i], xl[i], sl);
  }
  // the same order of sums for a row whichever workgroup norms it: a thread's elements in
  // turn, then the block's tree
  const float r = rsqrtf(block_sum(ss, scratch) * inv_h + eps);
  const float rp = from == 1 ? rsqrtf(block_sum(sp, scratch) * inv_h + eps) : 1.f;
  const float rl = save && q_last != t ? rsqrtf(block_sum(sl, scratch) * inv_h + eps) : r;

  T* po = plain + static_cast<size_t>(t) * h;
  T* so = shifted + static_cast<size_t>(t) * h;
  float* sw = save ? state + static_cast<size_t>(slot) * h : nullptr;
#pragma unroll
  for (int k = 0; k < SHIFT_KEEP; ++k) {
    const int i = threadIdx.x + k * SHIFT_THREADS;
    if (i >= h) break;
    const float y = xv[k] * r * wv[k];
    const float prev = from == 1 ? pv[k] * rp * wv[k] : pv[k];
    Elem<T>::store(po + i, y);
    Elem<T>::store(so + i, fmaf(prev - y, mv[k], y));
    // this thread has read the slot's element that it writes
    if (save) sw[i] = q_last == t ? y : lv[k] * rl * wv[k];
  }
  for (int i = threadIdx.x + SHIFT_KEEP * SHIFT_THREADS; i < h; i += SHIFT_THREADS) {
    const float y = xr[i] * r * w[i];
    const float prev = from == 1 ? xp[i] * rp * w[i] : (from == 2 ? st[i] : 0.f);
    Elem<T>::store(po + i, y);
    Elem<T>::store(so + i, fmaf(prev - y, mu[i], y));
    if (save) sw[i] = q_last == t ? y : xl[i] * rl * w[i];
  }
}
template <typename T>
static int norm_shift_launch(const float* x, const float* w, const float* mu, float* state,
                             const int* slot_ids, const int* seq_of_token, const int* cu_q,
                             const int* positions, void* plain, void* shifted, float eps, int n, int h,
                             int n_seqs, int n_slots, hipStream_t s) {
  if (n <= 0) return 0;
  // one block size for every call: the order of a row's sum of squares must not depend on the batch
  hipLaunchKernelGGL(norm_shift_kernel<T>, dim3(n), dim3(SHIFT_THREADS), 0, s, x, w, mu, state, slot_ids,
                     seq_of_token, cu_q, positions, static_cast<T*>(plain), static_cast<T*>(shifted), eps,
                     h, n_seqs, n_slots, n);
  return kvf_last_error();
}
#define NORM_SHIFT_DECL                                                                          \
  const float *x, const float *w, const float *mu, float *state, const int *slot_ids,           \
      const int *seq_of_token, const int *cu_q, const int *positions, void *plain, void *shifted, \
      float eps, int n, int h, int n_seqs, int n_slots, hipStream_t s
KVF_EXPORT int kvf_norm_shift_f32(NORM_SHIFT_DECL) {
  return norm_shift_launch<float>(x, w, mu, state, slot_ids, seq_of_token, cu_q, positions, plain,
                                  shifted, eps, n, h, n_seqs, n_slots, s);
}
KVF_EXPORT int kvf_norm_shift_bf16(NORM_SHIFT_DECL) {
  return norm_shift_launch<bf16_t>(x, w, mu, state, slot_ids, seq_of_token, cu_q, positions, plain,
                                   shifted, eps, n, h, n_seqs, n_slots, s);
}

// ----------------------------------------------------------------------------- gated activations
// out[m, i] = act(gate_i + bg[i]) * (up_i + bu[i]) in fp32; the input row holds gate at 2i and
// up at 2i + 1 (`paired`) or gate at i and up at I + i.  act: 0 silu, 1 the tanh form of gelu.
// The biases are fp32 vectors and may be null.
__device__ __forceinline__ float gelu_tanh_f(float z) {
  const float u = 0.7978845608028654f * (z + 0.044715f * z * z * z);
  return 0.5f * z * (1.f + tanhf(u));
}
__device__ __forceinline__ float act_f(int act, float z) {
  return act == 1 ? gelu_tanh_f(z) : z / (1.f + expf(-z));
}
template <typename T>
__global__ void gated_act_kernel(const T* __restrict__ gu, const float* __restrict__ bg,
                                 const float* __restrict__ bu, T* __restrict__ out, int inter,
                                 size_t total, int paired, int act) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t m = idx / inter;
  const int i = static_cast<int>(idx - m * inter);
  const T* row = gu + m * 2 * static_cast<size_t>(inter);
  float g = Elem<T>::load(paired ? row + 2 * i : row + i);
  float u = Elem<T>::load(paired ? row + 2 * i + 1 : row + inter + i);
  if (bg) g += bg[i];
  if (bu) u += bu[i];
  Elem<T>::store(out + idx, act_f(act, g) * u);
}
// bf16, paired: a thread takes four neighbouring (gate, up) pairs (16 bytes in, 8 bytes out)
// (the grid's x runs along a row, its y over the rows, so that no index is divided)
__global__ void gated_act_pairs4_kernel(const bf16_t* __restrict__ gu, const float* __restrict__ bg,
                                        const float* __restrict__ bu, bf16_t* __restrict__ out,
                                        int inter, int rows, int act) {
  const int i0 = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i0 >= inter) return;
  float4 b_g = make_float4(0.f, 0.f, 0.f, 0.f), b_u = b_g;
  if (bg) b_g = *reinterpret_cast<const float4*>(bg + i0);
  if (bu) b_u = *reinterpret_cast<const float4*>(bu + i0);
  const float gb[4] = {b_g.x, b_g.y, b_g.z, b_g.w}, ub[4] = {b_u.x, b_u.y, b_u.z, b_u.w};
  for (int m = blockIdx.y; m < rows; m += gridDim.y) {
  float v[8];
  load8(gu + (static_cast<size_t>(m) * inter + i0) * 2, v);
  uint32_t hh[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float g = v[2 * i] + gb[i], u = v[2 * i + 1] + ub[i];
    float a;
    if (act == 1) {
      // tanh(t) = 1 - 2 / (1 + exp(2 t)); exp overflows to +inf for large t, which gives 1
      const float t = 0.7978845608028654f * (g + 0.044715f * g * g * g);
      a = 0.5f * g * (2.f - 2.f / (1.f + __expf(2.f * t)));
    } else {
      a = g / (1.f + __expf(-g));
    }
    hh[i] = f32_to_bf16(a * u);
  }
  uint2 packed;
  packed.x = hh[0] | (hh[1] << 16);
  packed.y = hh[2] | (hh[3] << 16);
  *reinterpret_cast<uint2*>(out + static_cast<size_t>(m) * inter + i0) = packed;
  }
}

template <typename T>
static int gated_act_launch(const void* gu, const float* bg, const float* bu, void* out, int m,
                            int inter, int paired, int act, hipStream_t s) {
  const size_t total = static_cast<size_t>(m) * inter;
  if (total == 0) return 0;
  auto at16 = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  if (sizeof(T) == 2 && paired && inter % 4 == 0 && at16(gu) && reinterpret_cast<uintptr_t>(out) % 8 == 0 &&
      at16(bg) && at16(bu)) {
    const int threads = inter / 4 >= 256 ? 256 : 64;
    const dim3 grid((inter / 4 + threads - 1) / threads, m < 65535 ? m : 65535);
    hipLaunchKernelGGL(gated_act_pairs4_kernel, grid, dim3(threads), 0, s, static_cast<const bf16_t*>(gu), bg,
                       bu, static_cast<bf16_t*>(out), inter, m, act);
    return kvf_last_error();
  }
  hipLaunchKernelGGL(gated_act_kernel<T>, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, s,
                     static_cast<const T*>(gu), bg, bu, static_cast<T*>(out), inter, total, paired, act);
  return kvf_last_error();
}
KVF_EXPORT int kvf_gated_act_f32(const void* gu, const float* bg, const float* bu, void* out, int m,
                                 int inter, int paired, int act, hipStream_t s) {
  return gated_act_launch<float>(gu, bg, bu, out, m, inter, paired, act, s);
}
KVF_EXPORT int kvf_gated_act_bf16(const void* gu, const float* bg, const float* bu, void* out, int m,
                                  int inter, int paired, int act, hipStream_t s) {
  return gated_act_launch<bf16_t>(gu, bg, bu, out, m, inter, paired, act, s);
}

// ----------------------------------------------------------------------------- sigmoid gate
// y[m, c] *= sigmoid(g[m, c]) for c < cols; rows of y and g are y_stride / g_stride apart.
template <typename T>
__global__ void sigmoid_gate_kernel(T* __restrict__ y, const T* __restrict__ g, int cols, int y_stride,
                                    int g_stride, size_t total) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t m = idx / cols;
  const int c = static_cast<int>(idx - m * cols);
  T* yp = y + m * y_stride + c;
  const float z = Elem<T>::load(g + m * g_stride + c);
  Elem<T>::store(yp, Elem<T>::load(yp) / (1.f + expf(-z)));
}
template <typename T>
static int sigmoid_gate_launch(void* y, const void* g, int m, int cols, int y_stride, int g_stride,
                               hipStream_t s) {
  const size_t total = static_cast<size_t>(m) * cols;
  if (total == 0) return 0;
  hipLaunchKernelGGL(sigmoid_gate_kernel<T>, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0,
                     s, static_cast<T*>(y), static_cast<const T*>(g), cols, y_stride, g_stride, total);
  return kvf_last_error();
}
KVF_EXPORT int kvf_sigmoid_gate_f32(void* y, const void* g, int m, int cols, int ys, int gs, hipStream_t s) {
  return sigmoid_gate_launch<float>(y, g, m, cols, ys, gs, s);
}
KVF_EXPORT int kvf_sigmoid_gate_bf16(void* y, const void* g, int m, int cols, int ys, int gs, hipStream_t s) {
  return sigmoid_gate_launch<bf16_t>(y, g, m, cols, ys, gs, s);
}

// ----------------------------------------------------------------------------- bias on the stream
// x[m, :] += bias (fp32) for every row.
__global__ void add_bias_kernel(float* __restrict__ x, const float* __restrict__ bias, int h, size_t total) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < total) x[i] += bias[i % h];
}
KVF_EXPORT int kvf_add_bias(float* x, const float* bias, int m, int h, hipStream_t s) {
  const size_t total = static_cast<size_t>(m) * h;
  if (total == 0) return 0;
  hipLaunchKernelGGL(add_bias_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, s, x,
                     bias, h, total);
  return kvf_last_error();
}

// ----------------------------------------------------------------------------- per-layer token input
// For every token row m of the fp32 stream x (first brought up to date: x[m] += bias, += owed[m],
// either may be null), with e = side[token[m], col0 .. col0 + dim):
//   a = gate x[m]                      gate  [dim, h]
//   g = gelu_tanh(a) * e
//   y = proj g                         proj  [h, dim]
//   x[m] += y * rsqrt(mean(y^2) + eps) * w
// all sums in fp32.  One workgroup per row: the row and g live in LDS; a wave takes every
// fourth row of `gate` with its lanes side by side along h, a thread takes elements of y with
// a row of `proj` to itself.  A token id outside the table adds nothing but bias and owed.
template <typename T, typename D>
__global__ __launch_bounds__(256) void token_side_kernel(
    float* __restrict__ x, const float* __restrict__ bias, const D* __restrict__ owed,
    const int* __restrict__ tokens, const T* __restrict__ side, const T* __restrict__ gate,
    const T* __restrict__ proj, const float* __restrict__ w, float eps, int h, int dim, int vocab,
    int side_stride, int col0) {
  extern __shared__ float side_lds[];  // [h] the row, [dim] g
  __shared__ float scratch[16];
  float* row = side_lds;
  float* g = side_lds + h;
  const int m = blockIdx.x;
  const int lane = threadIdx.x % KVF_WAVE, wave = threadIdx.x / KVF_WAVE, waves = blockDim.x / KVF_WAVE;
  float* xr = x + static_cast<size_t>(m) * h;
  const D* orow = owed ? owed + static_cast<size_t>(m) * h : nullptr;
  for (int i = threadIdx.x; i < h; i += blockDim.x) {
    float v = xr[i];
    if (bias) v += bias[i];
    if (orow) v += Elem<D>::load(orow + i);
    row[i] = v;
  }
  __syncthreads();
  const int tok = tokens[m];
  const bool known = tok >= 0 && tok < vocab;
  const T* e = side + static_cast<size_t>(known ? tok : 0) * side_stride + col0;
  for (int j = wave; j < dim; j += waves) {
    const T* gr = gate + static_cast<size_t>(j) * h;
    float a = 0.f;
    for (int i = lane; i < h; i += KVF_WAVE) a = fmaf(Elem<T>::load(gr + i), row[i], a);
    a = wave_sum(a);
    if (lane == 0) g[j] = known ? gelu_tanh_f(a) * Elem<T>::load(e + j) : 0.f;
  }
  __syncthreads();
  // y stays in registers where the row is short enough, otherwise it is computed twice
  constexpr int KEEP = 8;
  float y[KEEP];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < KEEP; ++k) {
    const int i = threadIdx.x + k * blockDim.x;
    y[k] = 0.f;
    if (i < h) {
      const T* pr = proj + static_cast<size_t>(i) * dim;
      float acc = 0.f;
      for (int j = 0; j < dim; ++j) acc = fmaf(Elem<T>::load(pr + j), g[j], acc);
      y[k] = acc;
      ss = fmaf(acc, acc, ss);
    }
  }
  for (int i = threadIdx.x + KEEP * blockDim.x; i < h; i += blockDim.x) {
    const T* pr = proj + static_cast<size_t>(i) * dim;
    float acc = 0.f;
    for (int j = 0; j < dim; ++j) acc = fmaf(Elem<T>::load(pr + j), g[j], acc);
    ss = fmaf(acc, acc, ss);
  }
  const float r = rsqrtf(block_sum(ss, scratch) / static_cast<float>(h) + eps);
#pragma unroll
  for (int k = 0; k < KEEP; ++k) {
    const int i = threadIdx.x + k * blockDim.x;
    if (i < h) xr[i] = fmaf(y[k] * r, w[i], row[i]);
  }
  for (int i = threadIdx.x + KEEP * blockDim.x; i < h; i += blockDim.x) {
    const T* pr = proj + static_cast<size_t>(i) * dim;
    float acc = 0.f;
    for (int j = 0; j < dim; ++j) acc = fmaf(Elem<T>::load(pr + j), g[j], acc);
    xr[i] = fmaf(acc * r, w[i], row[i]);
  }
}
// The same for rows of a multiple of 8 elements (h and dim), 1,024 threads and 16-byte loads: what
// a decode step runs.  `proj_t` is the projection transposed, [dim, h], so that the lanes of a
// wave read neighbouring elements of y's row.  The sixteen waves take the rows of `gate` in
// turn; for y a thread owns eight neighbouring elements and one of JG shares of the sum over
// dim, the shares are added in LDS in a fixed order.
template <typename T, typename D>
__global__ __launch_bounds__(1024) void token_side_wide_kernel(
    float* __restrict__ x, const float* __restrict__ bias, const D* __restrict__ owed,
    const int* __restrict__ tokens, const T* __restrict__ side, const T* __restrict__ gate,
    const T* __restrict__ proj_t, const float* __restrict__ w, float eps, int h, int dim, int vocab,
    int side_stride, int col0, int CC, int JG) {
  extern __shared__ __align__(16) float side_lds[];  // [h] the row, [JG][h] shares of y, [dim] g
  __shared__ float scratch[16];
  float* row = side_lds;
  float* part = side_lds + h;
  float* g = part + static_cast<size_t>(JG) * h;
  const int m = blockIdx.x, tid = threadIdx.x;
  const int lane = tid % KVF_WAVE, wave = tid / KVF_WAVE, waves = blockDim.x / KVF_WAVE;
  float* xr = x + static_cast<size_t>(m) * h;
  const D* orow = owed ? owed + static_cast<size_t>(m) * h : nullptr;
  for (int i = tid; i < h; i += blockDim.x) {
    float v = xr[i];
    if (bias) v += bias[i];
    if (orow) v += Elem<D>::load(orow + i);
    row[i] = v;
  }
  __syncthreads();
  const int tok = tokens[m];
  const bool known = tok >= 0 && tok < vocab;
  const T* e = side + static_cast<size_t>(known ? tok : 0) * side_stride + col0;
  const int chunks = h / 8;
  // a wave takes four rows of `gate` at a time, so that their loads are in flight together
  // (rows past dim are read again from row 0 and dropped)
  constexpr int RB = 4;
  for (int j0 = wave; j0 < dim; j0 += RB * waves) {
    float a[RB] = {0.f, 0.f, 0.f, 0.f};
    for (int c = lane; c < chunks; c += KVF_WAVE) {
      float v[RB][8];
#pragma unroll
      for (int u = 0; u < RB; ++u) {
        const int j = j0 + u * waves;
        load8(gate + static_cast<size_t>(j < dim ? j : 0) * h + 8 * c, v[u]);
      }
      const float4 r0 = *reinterpret_cast<const float4*>(row + 8 * c);
      const float4 r1 = *reinterpret_cast<const float4*>(row + 8 * c + 4);
#pragma unroll
      for (int u = 0; u < RB; ++u) {
        float t = a[u];
        t = fmaf(v[u][0], r0.x, t); t = fmaf(v[u][1], r0.y, t); t = fmaf(v[u][2], r0.z, t); t = fmaf(v[u][3], r0.w, t);
        t = fmaf(v[u][4], r1.x, t); t = fmaf(v[u][5], r1.y, t); t = fmaf(v[u][6], r1.z, t); t = fmaf(v[u][7], r1.w, t);
        a[u] = t;
      }
    }
#pragma unroll
    for (int u = 0; u < RB; ++u) {
      const int j = j0 + u * waves;
      const float t = wave_sum(a[u]);
      if (lane == 0 && j < dim) g[j] = known ? gelu_tanh_f(t) * Elem<T>::load(e + j) : 0.f;
    }
  }
  __syncthreads();
  // shares of y: thread (c, jg) sums g[j] * proj_t[j][8c .. 8c+7] over j = jg, jg + JG, ...
  const int jg = tid / CC, c0 = tid - jg * CC;
  if (jg < JG) {
    for (int c = c0; c < chunks; c += CC) {
      float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      // four rows of the transposed projection in flight (rows past dim count with g = 0)
      for (int j0 = jg; j0 < dim; j0 += RB * JG) {
        float v[RB][8], gj[RB];
#pragma unroll
        for (int u = 0; u < RB; ++u) {
          const int j = j0 + u * JG;
          load8(proj_t + static_cast<size_t>(j < dim ? j : 0) * h + 8 * c, v[u]);
          gj[u] = j < dim ? g[j] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < RB; ++u)
#pragma unroll
          for (int k = 0; k < 8; ++k) acc[k] = fmaf(v[u][k], gj[u], acc[k]);
      }
      float* p = part + static_cast<size_t>(jg) * h + 8 * c;
      *reinterpret_cast<float4*>(p) = make_float4(acc[0], acc[1], acc[2], acc[3]);
      *reinterpret_cast<float4*>(p + 4) = make_float4(acc[4], acc[5], acc[6], acc[7]);
    }
  }
  __syncthreads();
  float ss = 0.f;
  for (int i = tid; i < h; i += blockDim.x) {
    float y = part[i];
    for (int q = 1; q < JG; ++q) y += part[static_cast<size_t>(q) * h + i];
    part[i] = y;   // this thread's own element: read back below by the same thread
    ss = fmaf(y, y, ss);
  }
  const float r = rsqrtf(block_sum(ss, scratch) / static_cast<float>(h) + eps);
  for (int i = tid; i < h; i += blockDim.x) xr[i] = fmaf(part[i] * r, w[i], row[i]);
}

template <typename T, typename D>
static int token_side_launch(float* x, const float* bias, const void* owed, const int* tokens,
                             const void* side, const void* gate, const void* proj, const float* w,
                             float eps, int n, int h, int dim, int vocab, int side_stride, int col0,
                             const void* proj_t, hipStream_t s) {
  if (n <= 0) return 0;
  auto at16 = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  if (proj_t && h % 8 == 0 && dim % 8 == 0 && at16(gate) && at16(proj_t)) {
    const int chunks = h / 8;
    const int CC = chunks < 1024 ? chunks : 1024;
    int JG = 1024 / CC;
    if (JG > dim) JG = dim;
    const size_t wide = (static_cast<size_t>(1 + JG) * h + dim) * sizeof(float);
    if (wide <= 64 * 1024) {
      hipLaunchKernelGGL((token_side_wide_kernel<T, D>), dim3(n), dim3(1024), wide, s, x, bias,
                         static_cast<const D*>(owed), tokens, static_cast<const T*>(side),
                         static_cast<const T*>(gate), static_cast<const T*>(proj_t), w, eps, h, dim, vocab,
                         side_stride, col0, CC, JG);
      return kvf_last_error();
    }
  }
  const size_t lds = static_cast<size_t>(h + dim) * sizeof(float);
  if (lds > 64 * 1024) return static_cast<int>(hipErrorInvalidValue);
  hipLaunchKernelGGL((token_side_kernel<T, D>), dim3(n), dim3(256), lds, s, x, bias,
                     static_cast<const D*>(owed), tokens, static_cast<const T*>(side),
                     static_cast<const T*>(gate), static_cast<const T*>(proj), w, eps, h, dim, vocab,
                     side_stride, col0);
  return kvf_last_error();
}
#define TOKEN_SIDE_DECL                                                                          \
  float *x, const float *bias, const void *owed, int owed_f32, const int *tokens,               \
      const void *side, const void *gate, const void *proj, const float *w, float eps, int n,   \
      int h, int dim, int vocab, int side_stride, int col0, const void *proj_t, hipStream_t s
// proj_t (may be null): proj transposed, [dim, h]; with it, rows of a multiple of 8 elements take
// the kernel of 1,024 threads
KVF_EXPORT int kvf_token_side_f32(TOKEN_SIDE_DECL) {
  (void)owed_f32;
  return token_side_launch<float, float>(x, bias, owed, tokens, side, gate, proj, w, eps, n, h, dim,
                                         vocab, side_stride, col0, proj_t, s);
}
KVF_EXPORT int kvf_token_side_bf16(TOKEN_SIDE_DECL) {
  if (owed_f32)
    return token_side_launch<bf16_t, float>(x, bias, owed, tokens, side, gate, proj, w, eps, n, h, dim,
                                            vocab, side_stride, col0, proj_t, s);
  return token_side_launch<bf16_t, bf16_t>(x, bias, owed, tokens, side, gate, proj, w, eps, n, h, dim,
                                           vocab, side_stride, col0, proj_t, s);
}

// ----------------------------------------------------------------------------- the same, in pieces
// With many rows the two products of the per-layer token input go to the matrix kernels, and
// three row-wise kernels stand around them:
//   settle_cast: x[m] += bias + owed[m] (either may be null); copy[m] = x[m] in T (copy may be null)
//   side_gate:   g[m, j] = gelu_tanh(a[m, j]) * side[token[m], col0 + j]
//   rms_add:     x[m] += y[m] * rsqrt(mean(y[m]^2) + eps) * w
//   rms_add_norm: the same, and out[m] = x[m] * rsqrt(mean(x[m]^2) + eps2) * w2 of the new x
template <typename T, typename D>
__global__ void settle_cast_kernel(float* __restrict__ x, const float* __restrict__ bias,
                                   const D* __restrict__ owed, T* __restrict__ copy, int h, size_t total) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  float v = x[i];
  if (bias) v += bias[i % h];
  if (owed) v += Elem<D>::load(owed + i);
  if (bias || owed) x[i] = v;
  if (copy) Elem<T>::store(copy + i, v);
}
template <typename T, typename D>
static int settle_cast_launch(float* x, const float* bias, const void* owed, void* copy, int m, int h,
                              hipStream_t s) {
  const size_t total = static_cast<size_t>(m) * h;
  if (total == 0 || (!bias && !owed && !copy)) return 0;
  hipLaunchKernelGGL((settle_cast_kernel<T, D>), dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256),
                     0, s, x, bias, static_cast<const D*>(owed), static_cast<T*>(copy), h, total);
  return kvf_last_error();
}
KVF_EXPORT int kvf_settle_cast_f32(float* x, const float* bias, const void* owed, int owed_f32, void* copy,
                                   int m, int h, hipStream_t s) {
  (void)owed_f32;
  return settle_cast_launch<float, float>(x, bias, owed, copy, m, h, s);
}
KVF_EXPORT int kvf_settle_cast_bf16(float* x, const float* bias, const void* owed, int owed_f32, void* copy,
                                    int m, int h, hipStream_t s) {
  if (owed_f32) return settle_cast_launch<bf16_t, float>(x, bias, owed, copy, m, h, s);
  return settle_cast_launch<bf16_t, bf16_t>(x, bias, owed, copy, m, h, s);
}

template <typename T>
__global__ void side_gate_kernel(const T* __restrict__ a, const int* __restrict__ tokens,
                                 const T* __restrict__ side, T* __restrict__ g, int dim, int vocab,
                                 int side_stride, int col0, size_t total) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t m = idx / dim;
  const int j = static_cast<int>(idx - m * dim);
  const int tok = tokens[m];
  float v = 0.f;
  if (tok >= 0 && tok < vocab)
    v = gelu_tanh_f(Elem<T>::load(a + idx)) * Elem<T>::load(side + static_cast<size_t>(tok) * side_stride + col0 + j);
  Elem<T>::store(g + idx, v);
}
template <typename T>
static int side_gate_launch(const void* a, const int* tokens, const void* side, void* g, int m, int dim,
                            int vocab, int side_stride, int col0, hipStream_t s) {
  const size_t total = static_cast<size_t>(m) * dim;
  if (total == 0) return 0;
  hipLaunchKernelGGL(side_gate_kernel<T>, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, s,
                     static_cast<const T*>(a), tokens, static_cast<const T*>(side), static_cast<T*>(g), dim,
                     vocab, side_stride, col0, total);
  return kvf_last_error();
}
KVF_EXPORT int kvf_side_gate_f32(const void* a, const int* t, const void* side, void* g, int m, int dim,
                                 int vocab, int ss, int col0, hipStream_t s) {
  return side_gate_launch<float>(a, t, side, g, m, dim, vocab, ss, col0, s);
}
KVF_EXPORT int kvf_side_gate_bf16(const void* a, const int* t, const void* side, void* g, int m, int dim,
                                  int vocab, int ss, int col0, hipStream_t s) {
  return side_gate_launch<bf16_t>(a, t, side, g, m, dim, vocab, ss, col0, s);
}

__global__ __launch_bounds__(256) void rms_add_kernel(float* __restrict__ x, const float* __restrict__ y,
                                                      const float* __restrict__ w, float eps, int h) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  float* xr = x + static_cast<size_t>(m) * h;
  const float* yr = y + static_cast<size_t>(m) * h;
  float ss = 0.f;
  for (int i = threadIdx.x; i < h; i += blockDim.x) ss = fmaf(yr[i], yr[i], ss);
  const float r = rsqrtf(block_sum(ss, scratch) / static_cast<float>(h) + eps);
  for (int i = threadIdx.x; i < h; i += blockDim.x) xr[i] = fmaf(yr[i] * r, w[i], xr[i]);
}
KVF_EXPORT int kvf_rms_add(float* x, const float* y, const float* w, float eps, int m, int h, hipStream_t s) {
  if (m <= 0) return 0;
  hipLaunchKernelGGL(rms_add_kernel, dim3(m), dim3(256), 0, s, x, y, w, eps, h);
  return kvf_last_error();
}

// A sublayer's rows join the stream through their norm, and the next sublayer's input is the norm
// of the sum: one pass over the row for both (a thread reads back only what it wrote itself).
// EPT > 0: rows of at most 256 * EPT elements, which a thread then holds in registers: every load is
// asked for before the first sum, and the row is read once.  EPT = 0: any width, three passes.
template <typename T, int EPT>
__global__ __launch_bounds__(256) void rms_add_norm_kernel(float* __restrict__ x, const float* __restrict__ y,
                                                           const float* __restrict__ w, float eps,
                                                           const float* __restrict__ w2, float eps2,
                                                           T* __restrict__ out, int h) {
  __shared__ float scratch[16], scratch2[16];
  const int m = blockIdx.x;
  float* xr = x + static_cast<size_t>(m) * h;
  const float* yr = y + static_cast<size_t>(m) * h;
  T* o = out + static_cast<size_t>(m) * h;
  if (EPT > 0) {
    constexpr int N = EPT > 0 ? EPT : 1;
    float yv[N], xv[N], wv[N], w2v[N];
#pragma unroll
    for (int k = 0; k < N; ++k) {
      const int i = k * 256 + threadIdx.x;
      const bool ok = i < h;
      yv[k] = ok ? yr[i] : 0.f;
      xv[k] = ok ? xr[i] : 0.f;
      wv[k] = ok ? w[i] : 0.f;
      w2v[k] = ok ? w2[i] : 0.f;
    }
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < N; ++k) ss = fmaf(yv[k], yv[k], ss);
    const float r = rsqrtf(block_sum(ss, scratch) / static_cast<float>(h) + eps);
    float ss2 = 0.f;
#pragma unroll
    for (int k = 0; k < N; ++k) {
      xv[k] = fmaf(yv[k] * r, wv[k], xv[k]);
      ss2 = fmaf(xv[k], xv[k], ss2);
    }
    const float r2 = rsqrtf(block_sum(ss2, scratch2) / static_cast<float>(h) + eps2);
#pragma unroll
    for (int k = 0; k < N; ++k) {
      const int i = k * 256 + threadIdx.x;
      if (i < h) {
        xr[i] = xv[k];
        Elem<T>::store(o + i, xv[k] * r2 * w2v[k]);
      }
    }
    return;
  }
  float ss = 0.f;
  for (int i = threadIdx.x; i < h; i += blockDim.x) ss = fmaf(yr[i], yr[i], ss);
  const float r = rsqrtf(block_sum(ss, scratch) / static_cast<float>(h) + eps);
  float ss2 = 0.f;
  for (int i = threadIdx.x; i < h; i += blockDim.x) {
    const float v = fmaf(yr[i] * r, w[i], xr[i]);
    xr[i] = v;
    ss2 = fmaf(v, v, ss2);
  }
  const float r2 = rsqrtf(block_sum(ss2, scratch2) / static_cast<float>(h) + eps2);
  for (int i = threadIdx.x; i < h; i += blockDim.x) Elem<T>::store(o + i, xr[i] * r2 * w2[i]);
}
template <typename T>
static int rms_add_norm_launch(float* x, const float* y, const float* w, float eps, const float* w2, float eps2,
                               void* out, int m, int h, hipStream_t s) {
  if (h <= 256 * 4)
    hipLaunchKernelGGL((rms_add_norm_kernel<T, 4>), dim3(m), dim3(256), 0, s, x, y, w, eps, w2, eps2,
                       static_cast<T*>(out), h);
  else if (h <= 256 * 16)
    hipLaunchKernelGGL((rms_add_norm_kernel<T, 16>), dim3(m), dim3(256), 0, s, x, y, w, eps, w2, eps2,
                       static_cast<T*>(out), h);
  else
    hipLaunchKernelGGL((rms_add_norm_kernel<T, 0>), dim3(m), dim3(256), 0, s, x, y, w, eps, w2, eps2,
                       static_cast<T*>(out), h);
  return kvf_last_error();
}
// dtype of out: 0 = fp32, 1 = bf16
KVF_EXPORT int kvf_rms_add_norm(int dtype, float* x, const float* y, const float* w, float eps, const float* w2,
                                float eps2, void* out, int m, int h, hipStream_t s) {
  if (m <= 0) return 0;
  if (dtype == 0) return rms_add_norm_launch<float>(x, y, w, eps, w2, eps2, out, m, h, s);
  if (dtype == 1) return rms_add_norm_launch<bf16_t>(x, y, w, eps, w2, eps2, out, m, h, s);
  return static_cast<int>(hipErrorInvalidValue);
}

// ----------------------------------------------------------------------------- whole-row q/k norm
// Projected rows in fp32, `row_len` apart: H q heads of d elements, then KV k heads of d (then,
// unless values are keys, KV v heads of d); of a head's d elements the first dk are real, the
// rest padding.  Per token:
//   q <- q + q_bias, k <- k + k_bias (fp32 vectors over the real elements, or null);
//   the values are v's columns, or (v_from_k) the keys as they are here, before norm and rotation;
//   q and k are each divided by the root mean square over *all* their real elements (every head
//   at once, eps inside the root) and multiplied by weights qw [H dk], kw [KV dk];
//   the first `rot` elements of every head are rotated in neighbouring pairs by the position's
//   cos/sin row; q goes to q_out (rounded once), k and v to the token's place in the pages.
// A workgroup takes a token, or (blockIdx.y, few tokens) a share of a token's heads after it has
// summed the whole row's squares for itself.
template <typename T>
__global__ __launch_bounds__(256) void rownorm_rope_kvwrite_kernel(
    const float* __restrict__ proj, const float* __restrict__ q_bias, const float* __restrict__ k_bias,
    const float* __restrict__ qw, const float* __restrict__ kw, const int* __restrict__ positions,
    const int* __restrict__ seq_of_token, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ block_table, T* __restrict__ q_out, int q_stride, T* __restrict__ k_pages,
    T* __restrict__ v_pages, int dk, float eps, int v_from_k, RopeArgs a) {
  __shared__ float scratch[2][16];
  const int n = blockIdx.x;
  const int p = positions[n];
  const int half = a.rot / 2, d2 = a.d / 2;
  const float* row = proj + static_cast<size_t>(n) * a.row_len;
  const bool pos_ok = p >= 0 && p < a.table_len;
  const float* cs = cos_t ? cos_t + static_cast<size_t>(pos_ok ? p : 0) * half : nullptr;
  const float* sn = sin_t ? sin_t + static_cast<size_t>(pos_ok ? p : 0) * half : nullptr;
  int page = -1, off = 0;
  if (a.write_kv && pos_ok) {
    const int seq = seq_of_token[n];
    const int blk = p / a.block_size;
    if (seq >= 0 && seq < a.n_seqs && blk < a.table_stride) {
      page = block_table[static_cast<size_t>(seq) * a.table_stride + blk];
      if (page >= a.num_blocks) page = -1;
      off = p - blk * a.block_size;
    }
  }
  // the sums of squares over all of q and all of k: a wave a head in turn, its lanes along the
  // head (no index is divided), the waves' sums joined through LDS
  const int lane = threadIdx.x % KVF_WAVE, wave = threadIdx.x / KVF_WAVE, waves = blockDim.x / KVF_WAVE;
  float ssq = 0.f, ssk = 0.f;
  for (int hh = wave; hh < a.H + a.KV; hh += waves) {
    const bool is_k = hh >= a.H;
    const float* x = row + hh * a.d;
    const float* b = is_k ? (k_bias ? k_bias + (hh - a.H) * dk : nullptr) : (q_bias ? q_bias + hh * dk : nullptr);
    float ss = 0.f;
    for (int e = lane; e < dk; e += KVF_WAVE) {
      const float v = x[e] + (b ? b[e] : 0.f);
      ss = fmaf(v, v, ss);
    }
    if (is_k) ssk += ss; else ssq += ss;
  }
  ssq = wave_sum(ssq);
  ssk = wave_sum(ssk);
  if (lane == 0) {
    scratch[0][wave] = ssq;
    scratch[1][wave] = ssk;
  }
  __syncthreads();
  float tq = 0.f, tk = 0.f;
  for (int w = 0; w < waves; ++w) {
    tq += scratch[0][w];
    tk += scratch[1][w];
  }
  const float rq = 1.f / sqrtf(tq / static_cast<float>(a.H * dk) + eps);
  const float rk = 1.f / sqrtf(tk / static_cast<float>(a.KV * dk) + eps);
  // a wave a head in turn (blockIdx.y names a share of the heads); a lane holds the pairs lane and lane + 64
  for (int hh = blockIdx.y * waves + wave; hh < a.H + a.KV; hh += gridDim.y * waves) {
    const bool is_k = hh >= a.H;
    if (is_k && page < 0) continue;
    const int kh = hh - a.H;
    const float* x = row + hh * a.d;
    const float* b = is_k ? (k_bias ? k_bias + kh * dk : nullptr) : (q_bias ? q_bias + hh * dk : nullptr);
    const float* w = is_k ? kw + kh * dk : qw + hh * dk;
    const float r = is_k ? rk : rq;
    T* dst = is_k ? k_pages + ((static_cast<size_t>(page) * a.KV + kh) * a.block_size + off) * a.d
                  : q_out + static_cast<size_t>(n) * q_stride + hh * a.d;
    const float* vx = row + (a.H + a.KV + (is_k ? kh : 0)) * a.d;
    T* vdst = is_k ? v_pages + (static_cast<size_t>(page) * a.KV + kh) * a.d * a.block_size + off : nullptr;
    for (int i = lane; i < d2; i += KVF_WAVE) {
      const int e = 2 * i;
      const float x0 = e < dk ? x[e] + (b ? b[e] : 0.f) : 0.f;
      const float x1 = e + 1 < dk ? x[e + 1] + (b ? b[e + 1] : 0.f) : 0.f;
      float y0 = e < dk ? x0 * r * w[e] : 0.f;
      float y1 = e + 1 < dk ? x1 * r * w[e + 1] : 0.f;
      if (e < a.rot && pos_ok && cs) {
        const float c = cs[i], sv = sn[i];
        const float t0 = y0 * c - y1 * sv, t1 = y1 * c + y0 * sv;
        y0 = t0;
        y1 = t1;
      }
      Elem<T>::store(dst + e, y0);
      Elem<T>::store(dst + e + 1, y1);
      if (is_k) {
        Elem<T>::store(vdst + static_cast<size_t>(e) * a.block_size, v_from_k ? x0 : vx[e]);
        Elem<T>::store(vdst + static_cast<size_t>(e + 1) * a.block_size, v_from_k ? x1 : vx[e + 1]);
      }
    }
  }
}
#define ROWNORM_ARGS_DECL                                                                                    \
  int dtype, const float *proj, const float *q_bias, const float *k_bias, const float *qw, const float *kw, \
      const int *positions, const int *seq_of_token, const float *cos_t, const float *sin_t,                \
      const int *block_table, void *q_out, int q_stride, void *k_pages, void *v_pages, int dk, float eps,   \
      int v_from_k, int n, int H, int KV, int d, int rot, int table_len, int block_size, int table_stride,  \
      int num_blocks, int write_kv, int n_seqs, int row_len, hipStream_t s
// dtype of q_out and the pages: 0 = fp32, 1 = bf16
KVF_EXPORT int kvf_rownorm_rope_kvwrite(ROWNORM_ARGS_DECL) {
  if (n <= 0) return 0;
  if (d % 2 || dk > d || dk <= 0 || rot > dk || rot % 2 || !qw || !kw || !q_out)
    return static_cast<int>(hipErrorInvalidValue);
  const RopeArgs a{ROPE_ARGS_PACK};
  // few tokens: several workgroups share a token's pairs, so that the chip has work
  int shares = n >= 1024 ? 1 : (H + KV + 3) / 4;
  if (shares > 64) shares = 64;
  const dim3 grid(n, shares);
  if (dtype == 0)
    hipLaunchKernelGGL(rownorm_rope_kvwrite_kernel<float>, grid, dim3(256), 0, s, proj, q_bias, k_bias, qw, kw,
                       positions, seq_of_token, cos_t, sin_t, block_table, static_cast<float*>(q_out), q_stride,
                       static_cast<float*>(k_pages), static_cast<float*>(v_pages), dk, eps, v_from_k, a);
  else if (dtype == 1)
    hipLaunchKernelGGL(rownorm_rope_kvwrite_kernel<bf16_t>, grid, dim3(256), 0, s, proj, q_bias, k_bias, qw, kw,
                       positions, seq_of_token, cos_t, sin_t, block_table, static_cast<bf16_t*>(q_out), q_stride,
                       static_cast<bf16_t*>(k_pages), static_cast<bf16_t*>(v_pages), dk, eps, v_from_k, a);
  else
    return static_cast<int>(hipErrorInvalidValue);
  return kvf_last_error();
}

// ----------------------------------------------------------------------------- one gate per head
// y[m, h * d + e] *= sigmoid(g[m, h]) * scale for h < H, e < d; g fp32, rows g_stride apart
// (g null: y *= scale).
template <typename T>
__global__ void head_gate_kernel(T* __restrict__ y, const float* __restrict__ g, int H, int d, int y_stride,
                                 int g_stride, float scale, size_t total) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int cols = H * d;
  const size_t m = idx / cols;
  const int c = static_cast<int>(idx - m * cols);
  T* yp = y + m * y_stride + c;
  const float gate = g ? 1.f / (1.f + expf(-g[m * g_stride + c / d])) : 1.f;
  Elem<T>::store(yp, Elem<T>::load(yp) * (gate * scale));
}
// eight neighbouring elements of one head a thread (d a multiple of 8, rows that start on 16 / 32 bytes)
template <typename T>
__global__ void head_gate8_kernel(T* __restrict__ y, const float* __restrict__ g, int H, int d, int y_stride,
                                  int g_stride, float scale, int rows) {
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (c >= H * d) return;
  const int head = c / d;
  for (int m = blockIdx.y; m < rows; m += gridDim.y) {
    const float gate = g ? 1.f / (1.f + expf(-g[static_cast<size_t>(m) * g_stride + head])) : 1.f;
    T* yp = y + static_cast<size_t>(m) * y_stride + c;
    float v[8];
    load8(yp, v);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] *= gate * scale;
    store8(yp, v);
  }
}
KVF_EXPORT int kvf_head_gate(int dtype, void* y, const float* g, int m, int H, int d, int y_stride, int g_stride,
                             float scale, hipStream_t s) {
  const size_t total = static_cast<size_t>(m) * H * d;
  if (total == 0) return 0;
  if (d % 8 == 0 && y_stride % 8 == 0 && reinterpret_cast<uintptr_t>(y) % 32 == 0 && (dtype == 0 || dtype == 1)) {
    const int threads = H * d / 8 >= 256 ? 256 : 64;
    const dim3 grid8((H * d / 8 + threads - 1) / threads, m < 65535 ? m : 65535);
    if (dtype == 0)
      hipLaunchKernelGGL(head_gate8_kernel<float>, grid8, dim3(threads), 0, s, static_cast<float*>(y), g, H, d,
                         y_stride, g_stride, scale, m);
    else
      hipLaunchKernelGGL(head_gate8_kernel<bf16_t>, grid8, dim3(threads), 0, s, static_cast<bf16_t*>(y), g, H, d,
                         y_stride, g_stride, scale, m);
    return kvf_last_error();
  }
  const dim3 grid(static_cast<unsigned>((total + 255) / 256));
  if (dtype == 0)
    hipLaunchKernelGGL(head_gate_kernel<float>, grid, dim3(256), 0, s, static_cast<float*>(y), g, H, d, y_stride,
                       g_stride, scale, total);
  else if (dtype == 1)
    hipLaunchKernelGGL(head_gate_kernel<bf16_t>, grid, dim3(256), 0, s, static_cast<bf16_t*>(y), g, H, d, y_stride,
                       g_stride, scale, total);
  else
    return static_cast<int>(hipErrorInvalidValue);
  return kvf_last_error();
}

// ----------------------------------------------------------------------------- plain activations
// out = act(x) element by element in fp32, rounded once.  act: 0 silu, 1 the tanh form of gelu,
// 2 the square of relu.
__device__ __forceinline__ float plain_act_f(int act, float z) {
  if (act == 2) {
    const float r = fmaxf(z, 0.f);
    return r * r;
  }
  return act_f(act, z);
}
template <typename T>
__global__ void plain_act_kernel(const T* __restrict__ x, T* __restrict__ out, size_t total, int act) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < total) Elem<T>::store(out + i, plain_act_f(act, Elem<T>::load(x + i)));
}
// eight neighbouring elements a thread (16 bytes of bf16 in and out)
template <typename T>
__global__ void plain_act8_kernel(const T* __restrict__ x, T* __restrict__ out, size_t groups, int act) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= groups) return;
  float v[8];
  load8(x + 8 * i, v);
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = plain_act_f(act, v[e]);
  store8(out + 8 * i, v);
}
KVF_EXPORT int kvf_plain_act(int dtype, const void* x, void* out, long total, int act, hipStream_t s) {
  if (total <= 0) return 0;
  if (total % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 32 == 0 && reinterpret_cast<uintptr_t>(out) % 32 == 0 &&
      dtype >= 0 && dtype <= 1) {
    const size_t groups = static_cast<size_t>(total / 8);
    const dim3 grid8(static_cast<unsigned>((groups + 255) / 256));
    if (dtype == 0)
      hipLaunchKernelGGL(plain_act8_kernel<float>, grid8, dim3(256), 0, s, static_cast<const float*>(x),
                         static_cast<float*>(out), groups, act);
    else
      hipLaunchKernelGGL(plain_act8_kernel<bf16_t>, grid8, dim3(256), 0, s, static_cast<const bf16_t*>(x),
                         static_cast<bf16_t*>(out), groups, act);
    return kvf_last_error();
  }
  const dim3 grid(static_cast<unsigned>((total + 255) / 256));
  if (dtype == 0)
    hipLaunchKernelGGL(plain_act_kernel<float>, grid, dim3(256), 0, s, static_cast<const float*>(x),
                       static_cast<float*>(out), static_cast<size_t>(total), act);
  else if (dtype == 1)
    hipLaunchKernelGGL(plain_act_kernel<bf16_t>, grid, dim3(256), 0, s, static_cast<const bf16_t*>(x),
                       static_cast<bf16_t*>(out), static_cast<size_t>(total), act);
  else
    return static_cast<int>(hipErrorInvalidValue);
  return kvf_last_error();
}

// ----------------------------------------------------------------------------- gate per row
// out[m, i] = act(gate_i) * up_i * sigmoid(rg[m]) with (gate, up) at (2i, 2i + 1) of the input
// row; rg fp32, one number per row, rg_stride apart.  A feed-forward whose output is multiplied
// by a number per token takes the number here, ahead of its (linear) down projection.
template <typename T>
__global__ void gated_act_rowgate_kernel(const T* __restrict__ gu, const float* __restrict__ rg, int rg_stride,
                                         T* __restrict__ out, int inter, size_t total, int act) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t m = idx / inter;
  const int i = static_cast<int>(idx - m * inter);
  const T* row = gu + m * 2 * static_cast<size_t>(inter);
  const float g = Elem<T>::load(row + 2 * i), u = Elem<T>::load(row + 2 * i + 1);
  const float z = rg[m * rg_stride];
  Elem<T>::store(out + idx, act_f(act, g) * u * (1.f / (1.f + expf(-z))));
}
// bf16: a thread takes four neighbouring (gate, up) pairs (16 bytes in, 8 bytes out); the grid's x
// runs along a row, its y over the rows
__global__ void gated_act_rowgate4_kernel(const bf16_t* __restrict__ gu, const float* __restrict__ rg, int rg_stride,
                                          bf16_t* __restrict__ out, int inter, int rows, int act) {
  const int i0 = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i0 >= inter) return;
  for (int m = blockIdx.y; m < rows; m += gridDim.y) {
    const float gate = 1.f / (1.f + expf(-rg[static_cast<size_t>(m) * rg_stride]));
    float v[8];
    load8(gu + (static_cast<size_t>(m) * inter + i0) * 2, v);
    uint32_t hh[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) hh[i] = f32_to_bf16(act_f(act, v[2 * i]) * v[2 * i + 1] * gate);
    uint2 packed;
    packed.x = hh[0] | (hh[1] << 16);
    packed.y = hh[2] | (hh[3] << 16);
    *reinterpret_cast<uint2*>(out + static_cast<size_t>(m) * inter + i0) = packed;
  }
}
KVF_EXPORT int kvf_gated_act_rowgate(int dtype, const void* gu, const float* rg, int rg_stride, void* out, int m,
                                     int inter, int act, hipStream_t s) {
  const size_t total = static_cast<size_t>(m) * inter;
  if (total == 0) return 0;
  if (dtype == 1 && inter % 4 == 0 && reinterpret_cast<uintptr_t>(gu) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(out) % 8 == 0) {
    const int threads = inter / 4 >= 256 ? 256 : 64;
    const dim3 grid4((inter / 4 + threads - 1) / threads, m < 65535 ? m : 65535);
    hipLaunchKernelGGL(gated_act_rowgate4_kernel, grid4, dim3(threads), 0, s, static_cast<const bf16_t*>(gu), rg,
                       rg_stride, static_cast<bf16_t*>(out), inter, m, act);
    return kvf_last_error();
  }
  const dim3 grid(static_cast<unsigned>((total + 255) / 256));
  if (dtype == 0)
    hipLaunchKernelGGL(gated_act_rowgate_kernel<float>, grid, dim3(256), 0, s, static_cast<const float*>(gu), rg,
                       rg_stride, static_cast<float*>(out), inter, total, act);
  else if (dtype == 1)
    hipLaunchKernelGGL(gated_act_rowgate_kernel<bf16_t>, grid, dim3(256), 0, s, static_cast<const bf16_t*>(gu), rg,
                       rg_stride, static_cast<bf16_t*>(out), inter, total, act);
  else
    return static_cast<int>(hipErrorInvalidValue);
  return kvf_last_error();
}
