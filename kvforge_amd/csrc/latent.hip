// Latent attention: what lies between the projections and the paged attention kernels.
//
// A token's keys and values of all heads are read out of one latent vector c [rank] (RMS-normed)
// and one rotated key part k_r [rot] that the heads share.  With W_uk the read-out of the
// unrotated keys, q_h . (W_uk_h c) = (W_uk_h^T q_h) . c, so attention runs over ONE key per
// token, [k_r | c], with per-head queries [q_r_h | W_uk_h^T q_h]; the weighted sum of the c is
// taken by the same kernels (the value is the key's c part) and read out per head by W_uv_h
// afterwards.  The cache holds k_r and c and nothing per head.
//
//   latent_split : a projected row [q heads (dim | rot) ... | c_raw (rank) | k_r (rot)] becomes
//                  the attention kernels' row [H q heads | k | v] of heads of d elements:
//                  q head h = [q_r_h | (left for head_product) | 0], k = [k_r | norm(c) | 0],
//                  v = [0 | norm(c) | 0]; the norm in fp32 with one rounding.
//   head_product : out[n, h, :] = W[h] in[n, h, :] for per-head matrices W [H, O, I].  bf16 rows and
//                  weights whose heads start on 16 bytes go to the matrix cores (a workgroup
//                  per 64 rows x 64 outputs of a head, a wave per 16 outputs, operands straight
//                  from memory, fp32 sums); everything else is fp32 multiply and add on the
//                  vector ALUs, tiles of 32 rows x 64 outputs through LDS.
#include "common.h"

namespace {

template <typename T>
__global__ __launch_bounds__(256) void latent_split_kernel(const T* __restrict__ proj, int ld_in,
                                                           T* __restrict__ qkv, int ld_out,
                                                           const float* __restrict__ w, float eps, int H,
                                                           int dim, int rot, int rank, int d) {
  __shared__ float scratch[16];
  const int n = blockIdx.x, tid = threadIdx.x;
  const T* in = proj + static_cast<size_t>(n) * ld_in;
  T* out = qkv + static_cast<size_t>(n) * ld_out;
  const T* down = in + H * (dim + rot);
  float ss = 0.f;
  for (int i = tid; i < rank; i += blockDim.x) {
    const float v = Elem<T>::load(down + i);
    ss = fmaf(v, v, ss);
  }
  const float r = 1.f / sqrtf(block_sum(ss, scratch) / static_cast<float>(rank) + eps);
  // q heads: the rotated part to the front, zeros behind what head_product fills
  for (int i = tid; i < H * d; i += blockDim.x) {
    const int h = i / d, e = i - h * d;
    if (e < rot)
      out[i] = in[h * (dim + rot) + dim + e];
    else if (e >= rot + rank || dim == 0)   // (heads without a plain part: nothing fills the middle)
      Elem<T>::store(out + i, 0.f);
  }
  T* k = out + H * d;
  T* v = k + d;
  for (int e = tid; e < d; e += blockDim.x) {
    if (e < rot) {
      k[e] = down[rank + e];
      Elem<T>::store(v + e, 0.f);
    } else if (e < rot + rank) {
      const float c = Elem<T>::load(down + e - rot) * r * w[e - rot];
      Elem<T>::store(k + e, c);
      Elem<T>::store(v + e, c);
    } else {
      Elem<T>::store(k + e, 0.f);
      Elem<T>::store(v + e, 0.f);
    }
  }
}

constexpr int HP_M = 32, HP_N = 64, HP_K = 32;

// grid (row tiles, output tiles, heads); 256 threads, thread (ty, tx) owns rows ty, ty + 16 and
// outputs tx + 16 j (j = 0..3) of the tile.
template <typename T, typename TW>
__global__ __launch_bounds__(256) void head_product_kernel(const T* __restrict__ in, int ld_in, int in_head,
                                                           const TW* __restrict__ W, T* __restrict__ out,
                                                           int ld_out, int out_head, int N, int O, int I) {
  __shared__ float As[HP_M][HP_K + 1];
  __shared__ float Bs[HP_N][HP_K + 1];
  const int n0 = blockIdx.x * HP_M, o0 = blockIdx.y * HP_N, h = blockIdx.z;
  const int tid = threadIdx.x, ty = tid / 16, tx = tid % 16;
  const T* a = in + static_cast<size_t>(h) * in_head;
  const TW* w = W + static_cast<size_t>(h) * O * I;
  float acc[2][4] = {};
  for (int k0 = 0; k0 < I; k0 += HP_K) {
    for (int i = tid; i < HP_M * HP_K; i += 256) {
      const int r = i / HP_K, c = i % HP_K;
      As[r][c] = (n0 + r < N && k0 + c < I) ? Elem<T>::load(a + static_cast<size_t>(n0 + r) * ld_in + k0 + c) : 0.f;
    }
    for (int i = tid; i < HP_N * HP_K; i += 256) {
      const int r = i / HP_K, c = i % HP_K;
      Bs[r][c] = (o0 + r < O && k0 + c < I) ? Elem<TW>::load(w + static_cast<size_t>(o0 + r) * I + k0 + c) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < HP_K; ++c) {
      const float a0 = As[ty][c], a1 = As[ty + 16][c];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float b = Bs[tx + 16 * j][c];
        acc[0][j] = fmaf(a0, b, acc[0][j]);
        acc[1][j] = fmaf(a1, b, acc[1][j]);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int n = n0 + ty + 16 * i;
    if (n >= N) continue;
    T* o = out + static_cast<size_t>(n) * ld_out + static_cast<size_t>(h) * out_head;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (o0 + tx + 16 * j < O) Elem<T>::store(o + o0 + tx + 16 * j, acc[i][j]);
  }
}

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

// a lane's four neighbouring outputs: one 8-byte store where the output rows allow it (`wide`:
// every head's outputs start on 8 bytes) and all four lie inside the head, else one by one
__device__ __forceinline__ void store4(bf16_t* o, const f32x4& a, int left, bool wide) {
  if (wide && left >= 4) {
    uint2 p;
    p.x = static_cast<unsigned>(f32_to_bf16(a[0])) | (static_cast<unsigned>(f32_to_bf16(a[1])) << 16);
    p.y = static_cast<unsigned>(f32_to_bf16(a[2])) | (static_cast<unsigned>(f32_to_bf16(a[3])) << 16);
    *reinterpret_cast<uint2*>(o) = p;
    return;
  }
#pragma unroll
  for (int v = 0; v < 4; ++v)
    if (v < left) Elem<bf16_t>::store(o + v, a[v]);
}

// v_mfma_f32_16x16x32_bf16 computes D[i][j] += sum_k A[i][k] B[j][k]; lane 16 c + r gives row r,
// elements 8c..8c+7 of the step's 32 of either operand, and holds D[4 (l / 16) + v][l % 16].
// A: 16 rows of the head's matrix (outputs), B: 16 rows of the input.  Grid (tiles of 64 rows,
// tiles of 64 outputs, heads); wave w takes outputs 16w..16w+15 of the tile for all its rows, so a
// weight fragment is loaded once for up to four row fragments.  I, in_head and ld_in are
// multiples of 8 and both bases lie on 16 bytes (the host checks), so a fragment is one 16-byte
// load that lies inside its row or is left zero.
__global__ __launch_bounds__(256) void head_product_mfma_kernel(const bf16_t* __restrict__ in, int ld_in,
                                                                int in_head, const bf16_t* __restrict__ W,
                                                                bf16_t* __restrict__ out, int ld_out, int out_head,
                                                                int N, int O, int I, bool wide) {
  const int n0 = blockIdx.x * 64, h = blockIdx.z;
  const int lane = threadIdx.x % KVF_WAVE, wave = threadIdx.x / KVF_WAVE;
  const int j = lane % 16, c = lane / 16;
  const int o0 = blockIdx.y * 64 + wave * 16;
  if (o0 >= O) return;
  const int subs = min(4, (N - n0 + 15) / 16);
  const bf16_t* wrow = o0 + j < O ? W + (static_cast<size_t>(h) * O + o0 + j) * I + 8 * c : nullptr;
  const bf16_t* xr[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int n = n0 + 16 * r + j;
    xr[r] = (r < subs && n < N) ? in + static_cast<size_t>(n) * ld_in + static_cast<size_t>(h) * in_head + 8 * c
                                : nullptr;
  }
  f32x4 acc[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) acc[r] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < I; k0 += 32) {
    const bool inside = k0 + 8 * c + 8 <= I;
    uint4 wf = make_uint4(0u, 0u, 0u, 0u);
    if (wrow && inside) wf = *reinterpret_cast<const uint4*>(wrow + k0);
    uint4 xf[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      xf[r] = make_uint4(0u, 0u, 0u, 0u);
      if (xr[r] && inside) xf[r] = *reinterpret_cast<const uint4*>(xr[r] + k0);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (r < subs)
        acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wf),
                                                         __builtin_bit_cast(bf16x8, xf[r]), acc[r], 0, 0, 0);
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int n = n0 + 16 * r + j;
    if (r >= subs || n >= N) continue;
    bf16_t* o = out + static_cast<size_t>(n) * ld_out + static_cast<size_t>(h) * out_head + o0 + 4 * c;
    store4(o, acc[r], O - (o0 + 4 * c), wide);
  }
}

// The same for many rows: a workgroup takes 64 rows of a head and ALL its outputs.  The rows'
// fragments (KS steps of 32 elements cover I) are loaded once and stay in registers while the
// wave goes through its groups of 16 outputs (w, w + 4, ...), so a row is read once per wave
// and not once per wave and output tile.  Sums run over the steps in the same order as above.
template <int KS>
__global__ __launch_bounds__(256) void head_product_mfma_rows_kernel(const bf16_t* __restrict__ in, int ld_in,
                                                                     int in_head, const bf16_t* __restrict__ W,
                                                                     bf16_t* __restrict__ out, int ld_out,
                                                                     int out_head, int N, int O, int I, bool wide) {
  const int n0 = blockIdx.x * 64, h = blockIdx.y;
  const int lane = threadIdx.x % KVF_WAVE, wave = threadIdx.x / KVF_WAVE;
  const int j = lane % 16, c = lane / 16;
  const int subs = min(4, (N - n0 + 15) / 16);
  uint4 xf[KS][4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int n = n0 + 16 * r + j;
    const bf16_t* x = (r < subs && n < N)
                          ? in + static_cast<size_t>(n) * ld_in + static_cast<size_t>(h) * in_head + 8 * c
                          : nullptr;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      xf[s][r] = make_uint4(0u, 0u, 0u, 0u);
      if (x && 32 * s + 8 * c + 8 <= I) xf[s][r] = *reinterpret_cast<const uint4*>(x + 32 * s);
    }
  }
  const int groups = (O + 15) / 16;
  for (int g = wave; g < groups; g += 4) {
    const int o0 = 16 * g;
    const bf16_t* wrow = o0 + j < O ? W + (static_cast<size_t>(h) * O + o0 + j) * I + 8 * c : nullptr;
    uint4 wf[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      wf[s] = make_uint4(0u, 0u, 0u, 0u);
      if (wrow && 32 * s + 8 * c + 8 <= I) wf[s] = *reinterpret_cast<const uint4*>(wrow + 32 * s);
    }
    f32x4 acc[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[r] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (r < subs)
          acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wf[s]),
                                                           __builtin_bit_cast(bf16x8, xf[s][r]), acc[r], 0, 0, 0);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int n = n0 + 16 * r + j;
      if (r >= subs || n >= N) continue;
      bf16_t* o = out + static_cast<size_t>(n) * ld_out + static_cast<size_t>(h) * out_head + o0 + 4 * c;
      store4(o, acc[r], O - (o0 + 4 * c), wide);
    }
  }
}

template <typename T, typename TW>
int head_product_launch(const void* in, int ld_in, int in_head, const void* W, void* out, int ld_out,
                        int out_head, int N, int H, int O, int I, hipStream_t s) {
  const dim3 grid((N + HP_M - 1) / HP_M, (O + HP_N - 1) / HP_N, H);
  hipLaunchKernelGGL((head_product_kernel<T, TW>), grid, dim3(256), 0, s, static_cast<const T*>(in), ld_in, in_head,
                     static_cast<const TW*>(W), static_cast<T*>(out), ld_out, out_head, N, O, I);
  return kvf_last_error();
}
}  // namespace

// dtype: 0 = fp32, 1 = bf16 (rows in and out).  d >= rot + rank.
KVF_EXPORT int kvf_latent_split(int dtype, const void* proj, int ld_in, void* qkv, int ld_out, const float* w,
                                float eps, int n, int H, int dim, int rot, int rank, int d, hipStream_t s) {
  if (n <= 0) return 0;
  if (H <= 0 || dim < 0 || rot < 0 || rank <= 0 || d < rot + rank || ld_in < H * (dim + rot) + rank + rot ||
      ld_out < (H + 2) * d || !w)
    return static_cast<int>(hipErrorInvalidValue);
  if (dtype == 0)
    hipLaunchKernelGGL(latent_split_kernel<float>, dim3(n), dim3(256), 0, s, static_cast<const float*>(proj), ld_in,
                       static_cast<float*>(qkv), ld_out, w, eps, H, dim, rot, rank, d);
  else if (dtype == 1)
    hipLaunchKernelGGL(latent_split_kernel<bf16_t>, dim3(n), dim3(256), 0, s, static_cast<const bf16_t*>(proj), ld_in,
                       static_cast<bf16_t*>(qkv), ld_out, w, eps, H, dim, rot, rank, d);
  else
    return static_cast<int>(hipErrorInvalidValue);
  return kvf_last_error();
}

// out[n, h * out_head + o] = sum_i W[h, o, i] * in[n * ld_in + h * in_head + i]; dtype of rows
// and wtype of W: 0 = fp32, 1 = bf16.
KVF_EXPORT int kvf_head_product(int dtype, int wtype, const void* in, int ld_in, int in_head, const void* W,
                                void* out, int ld_out, int out_head, int N, int H, int O, int I,
                                hipStream_t s) {
  if (N <= 0) return 0;
  if (H <= 0 || O <= 0 || I <= 0 || H > 65535 || (O + HP_N - 1) / HP_N > 65535)
    return static_cast<int>(hipErrorInvalidValue);
  if (dtype == 1 && wtype == 1 && I % 8 == 0 && in_head % 8 == 0 && ld_in % 8 == 0 &&
      reinterpret_cast<uintptr_t>(in) % 16 == 0 && reinterpret_cast<uintptr_t>(W) % 16 == 0) {
    const bf16_t* x = static_cast<const bf16_t*>(in);
    const bf16_t* w = static_cast<const bf16_t*>(W);
    bf16_t* y = static_cast<bf16_t*>(out);
    const dim3 rows((N + 63) / 64, H);
    const bool wide = ld_out % 4 == 0 && out_head % 4 == 0 && reinterpret_cast<uintptr_t>(out) % 8 == 0;
    if (N < 256 || I > 256) {   // few rows: more workgroups, each with one tile of outputs
      const dim3 grid((N + 63) / 64, (O + 63) / 64, H);
      hipLaunchKernelGGL(head_product_mfma_kernel, grid, dim3(256), 0, s, x, ld_in, in_head, w, y, ld_out, out_head, N,
                         O, I, wide);
    } else if (I <= 64) {
      hipLaunchKernelGGL(head_product_mfma_rows_kernel<2>, rows, dim3(256), 0, s, x, ld_in, in_head, w, y, ld_out,
                         out_head, N, O, I, wide);
    } else if (I <= 128) {
      hipLaunchKernelGGL(head_product_mfma_rows_kernel<4>, rows, dim3(256), 0, s, x, ld_in, in_head, w, y, ld_out,
                         out_head, N, O, I, wide);
    } else if (I <= 192) {
      hipLaunchKernelGGL(head_product_mfma_rows_kernel<6>, rows, dim3(256), 0, s, x, ld_in, in_head, w, y, ld_out,
                         out_head, N, O, I, wide);
    } else {
      hipLaunchKernelGGL(head_product_mfma_rows_kernel<8>, rows, dim3(256), 0, s, x, ld_in, in_head, w, y, ld_out,
                         out_head, N, O, I, wide);
    }
    return kvf_last_error();
  }
  if (dtype == 0 && wtype == 0)
    return head_product_launch<float, float>(in, ld_in, in_head, W, out, ld_out, out_head, N, H, O, I, s);
  if (dtype == 1 && wtype == 1)
    return head_product_launch<bf16_t, bf16_t>(in, ld_in, in_head, W, out, ld_out, out_head, N, H, O, I, s);
  if (dtype == 1 && wtype == 0)
    return head_product_launch<bf16_t, float>(in, ld_in, in_head, W, out, ld_out, out_head, N, H, O, I, s);
  if (dtype == 0 && wtype == 1)
    return head_product_launch<float, bf16_t>(in, ld_in, in_head, W, out, ld_out, out_head, N, H, O, I, s);
  return static_cast<int>(hipErrorInvalidValue);
}
