// A matrix memory with a data-dependent decay per key channel (RWKV-style time mixing).
//
// Per head a state S [dk, dk] (key channel by value channel), zero before a sequence's first
// token.  For a token with rows r, k, v [dk], decay w = exp(-exp(z + w0)) [dk] and bonus u [dk]:
//     o_j = sum_i r_i (S_ij + u_i k_i v_j)        S_ij <- w_i S_ij + k_i v_j
// A request's slot holds [S of all heads | the last token's input row h].
//
//   wkv_mix  : the five inputs of a token, h + (h_prev - h) * mu_s, where h_prev is the row before
//              in the same query run, the slot's row for a run that continues a sequence, zeros at
//              position 0; the workgroup of a run's first token leaves the run's last row in
//              the slot after it has read the slot (no other workgroup touches it).
//   wkv_scan : token by token.  A workgroup per (64 value columns, head, sequence); a thread
//              owns one value column of up to 64 key rows of S in registers (a wave per 64 key
//              rows); r, k, w of a stage of tokens go through LDS.  Everything is fp32; the
//              order of every sum is fixed by the shapes, so a token's output does not depend
//              on how its sequence was cut into runs.
//   wkv_out  : o / rms(o) * weight * silu(g) per head.
#include "common.h"

namespace {

template <typename T>
__global__ __launch_bounds__(256) void wkv_mix_kernel(const T* __restrict__ h, const float* __restrict__ mu,
                                                      float* __restrict__ state, int slot_floats, int prev_off,
                                                      const int* __restrict__ slot_ids,
                                                      const int* __restrict__ seq_of_token,
                                                      const int* __restrict__ cu_q,
                                                      const int* __restrict__ positions, T* __restrict__ out,
                                                      int width, int n_mix, int n_seqs, int n_slots,
                                                      int n_tokens) {
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
  // where the predecessor comes from: 0 nothing, 1 the row before, 2 the state slot
  const int from = pos <= 0 ? 0 : (!first ? 1 : (slot >= 0 ? 2 : 0));
  const T* row = h + static_cast<size_t>(t) * width;
  const T* before = row - width;
  float* st = slot >= 0 ? state + static_cast<size_t>(slot) * slot_floats + prev_off : nullptr;
  const T* last = h + static_cast<size_t>(q_last) * width;
  const bool save = first && slot >= 0;
  const size_t plane = static_cast<size_t>(n_tokens) * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float y = Elem<T>::load(row + i);
    const float p = from == 1 ? Elem<T>::load(before + i) : (from == 2 ? st[i] : 0.f);
    for (int m = 0; m < n_mix; ++m)
      Elem<T>::store(out + m * plane + static_cast<size_t>(t) * width + i, fmaf(p - y, mu[m * width + i], y));
    if (save) st[i] = Elem<T>::load(last + i);   // this thread has read the element it writes
  }
}

struct ScanArgs {
  int H, dk, n_seqs, n_slots, slot_floats;
  int row_len, r_off, k_off, v_off;   // where r, k, v of a token lie in a row of `rows`
  int z_stride;                        // row stride of the decay's pre-activations [tokens, >= H * dk]
  int stage;                           // tokens staged in LDS at a time
};


// ROWS: key rows a thread keeps (32 or 64); blockDim.x = 64 * ceil(dk / ROWS).
template <typename T, int ROWS>
__global__ __launch_bounds__(256) void wkv_scan_kernel(const T* __restrict__ rows, const float* __restrict__ z,
                                                       const float* __restrict__ w0, const float* __restrict__ u,
                                                       const int* __restrict__ cu_q,
                                                       const int* __restrict__ positions,
                                                       const int* __restrict__ slot_ids, float* __restrict__ state,
                                                       float* __restrict__ out, ScanArgs a) {
  extern __shared__ float lds[];
  const int dk = a.dk, head = blockIdx.y, seq = blockIdx.z, SCAN_STAGE = a.stage;
  const int lane = threadIdx.x % KVF_WAVE, part = threadIdx.x / KVF_WAVE, parts = blockDim.x / KVF_WAVE;
  const int col = blockIdx.x * KVF_WAVE + lane;
  const bool col_ok = col < dk;
  float* rs = lds;                         // [STAGE][dk]
  float* ks = rs + SCAN_STAGE * dk;        // [STAGE][dk]
  float* ws = ks + SCAN_STAGE * dk;        // [STAGE][dk]
  float* vs = ws + SCAN_STAGE * dk;        // [STAGE][64]
  float* bonus = vs + SCAN_STAGE * KVF_WAVE;   // [STAGE]
  float* psum = bonus + SCAN_STAGE;        // [STAGE][parts][64]
  const int t0 = cu_q[seq], t1 = cu_q[seq + 1];
  if (t1 <= t0) return;
  int slot = slot_ids[seq];
  if (slot < 0 || slot >= a.n_slots) slot = -1;
  const int row0 = part * ROWS;
  float* S_slot = slot >= 0 ? state + static_cast<size_t>(slot) * a.slot_floats +
                                  static_cast<size_t>(head) * dk * dk
                            : nullptr;
  float S[ROWS];
  const bool resume = positions[t0] > 0 && slot >= 0;
#pragma unroll
  for (int i = 0; i < ROWS; ++i)
    S[i] = (resume && col_ok && row0 + i < dk) ? S_slot[static_cast<size_t>(row0 + i) * dk + col] : 0.f;
  const float* w0h = w0 + head * dk;
  const float* uh = u + head * dk;
  for (int tb = t0; tb < t1; tb += SCAN_STAGE) {
    const int cnt = min(SCAN_STAGE, t1 - tb);
    __syncthreads();
    for (int i = threadIdx.x; i < cnt * dk; i += blockDim.x) {
      const int t = i / dk, e = i - t * dk;
      const T* row = rows + static_cast<size_t>(tb + t) * a.row_len + head * dk + e;
      rs[i] = Elem<T>::load(row + a.r_off);
      ks[i] = Elem<T>::load(row + a.k_off);
      ws[i] = expf(-expf(z[static_cast<size_t>(tb + t) * a.z_stride + head * dk + e] + w0h[e]));
    }
    for (int i = threadIdx.x; i < cnt * KVF_WAVE; i += blockDim.x) {
      const int t = i / KVF_WAVE, c = blockIdx.x * KVF_WAVE + i % KVF_WAVE;
      vs[i] = c < dk ? Elem<T>::load(rows + static_cast<size_t>(tb + t) * a.row_len + a.v_off + head * dk + c) : 0.f;
    }
    __syncthreads();
    // the bonus of a token, sum_i r_i u_i k_i: a wave a token, lanes side by side along i
    for (int t = part; t < cnt; t += parts) {
      float b = 0.f;
      for (int e = lane; e < dk; e += KVF_WAVE) b = fmaf(rs[t * dk + e] * uh[e], ks[t * dk + e], b);
      b = wave_sum(b);
      if (lane == 0) bonus[t] = b;
    }
    for (int t = 0; t < cnt; ++t) {
      const float v = vs[t * KVF_WAVE + lane];
      const float* r = rs + t * dk + row0;
      const float* k = ks + t * dk + row0;
      const float* w = ws + t * dk + row0;
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < ROWS; ++i) {
        if (row0 + i < dk) {
          acc = fmaf(r[i], S[i], acc);
          S[i] = fmaf(w[i], S[i], k[i] * v);
        }
      }
      psum[(t * parts + part) * KVF_WAVE + lane] = acc;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < cnt * KVF_WAVE; i += blockDim.x) {
      const int t = i / KVF_WAVE, l = i % KVF_WAVE, c = blockIdx.x * KVF_WAVE + l;
      if (c >= dk) continue;
      float o = 0.f;
      for (int p = 0; p < parts; ++p) o += psum[(t * parts + p) * KVF_WAVE + l];
      out[(static_cast<size_t>(tb + t) * a.H + head) * dk + c] = fmaf(vs[i], bonus[t], o);
    }
  }
  if (slot >= 0 && col_ok) {
#pragma unroll
    for (int i = 0; i < ROWS; ++i)
      if (row0 + i < dk) S_slot[static_cast<size_t>(row0 + i) * dk + col] = S[i];
  }
}

template <typename T>
__global__ __launch_bounds__(KVF_WAVE) void wkv_out_kernel(const float* __restrict__ o, const T* __restrict__ g,
                                                           int g_stride, const float* __restrict__ w, float eps,
                                                           T* __restrict__ out, int H, int dk) {
  const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const float* orow = o + (static_cast<size_t>(t) * H + head) * dk;
  float ss = 0.f;
  for (int e = lane; e < dk; e += KVF_WAVE) ss = fmaf(orow[e], orow[e], ss);
  const float r = 1.f / sqrtf(wave_sum(ss) / static_cast<float>(dk) + eps);
  const T* grow = g + static_cast<size_t>(t) * g_stride + head * dk;
  T* dst = out + (static_cast<size_t>(t) * H + head) * dk;
  for (int e = lane; e < dk; e += KVF_WAVE) {
    const float gv = Elem<T>::load(grow + e);
    Elem<T>::store(dst + e, orow[e] * r * w[head * dk + e] * (gv / (1.f + expf(-gv))));
  }
}

// out = tanh(in), fp32 in, rounded once to the rows' type
template <typename T>
__global__ void wkv_tanh_kernel(const float* __restrict__ in, T* __restrict__ out, long total) {
  const long i = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < total) Elem<T>::store(out + i, tanhf(in[i]));
}

template <typename T>
int scan_launch(const void* rows, const float* z, const float* w0, const float* u, const int* cu_q,
                const int* positions, const int* slot_ids, float* state, float* out, int num_seqs, ScanArgs a,
                hipStream_t s) {
  const int rows_per = a.dk <= 32 ? 32 : 64;
  const int parts = (a.dk + rows_per - 1) / rows_per;
  const dim3 grid((a.dk + KVF_WAVE - 1) / KVF_WAVE, a.H, num_seqs), block(parts * KVF_WAVE);
  const size_t lds = sizeof(float) * (static_cast<size_t>(a.stage) * (3 * a.dk + KVF_WAVE + 1 + parts * KVF_WAVE));
  if (rows_per == 32)
    hipLaunchKernelGGL((wkv_scan_kernel<T, 32>), grid, block, lds, s, static_cast<const T*>(rows), z, w0, u, cu_q,
                       positions, slot_ids, state, out, a);
  else
    hipLaunchKernelGGL((wkv_scan_kernel<T, 64>), grid, block, lds, s, static_cast<const T*>(rows), z, w0, u, cu_q,
                       positions, slot_ids, state, out, a);
  return kvf_last_error();
}
}  // namespace

// dtype: 0 = fp32, 1 = bf16 (rows h and out).  out holds n_mix planes of [n_tokens, width].
KVF_EXPORT int kvf_wkv_mix(int dtype, const void* h, const float* mu, float* state, int slot_floats, int prev_off,
                           const int* slot_ids, const int* seq_of_token, const int* cu_q, const int* positions,
                           void* out, int width, int n_mix, int n_seqs, int n_slots, int n_tokens,
                           hipStream_t s) {
  if (n_tokens <= 0) return 0;
  if (width <= 0 || n_mix <= 0 || prev_off < 0 || prev_off + width > slot_floats)
    return static_cast<int>(hipErrorInvalidValue);
  if (dtype == 0)
    hipLaunchKernelGGL(wkv_mix_kernel<float>, dim3(n_tokens), dim3(256), 0, s, static_cast<const float*>(h), mu, state,
                       slot_floats, prev_off, slot_ids, seq_of_token, cu_q, positions, static_cast<float*>(out),
                       width, n_mix, n_seqs, n_slots, n_tokens);
  else if (dtype == 1)
    hipLaunchKernelGGL(wkv_mix_kernel<bf16_t>, dim3(n_tokens), dim3(256), 0, s, static_cast<const bf16_t*>(h), mu, state,
                       slot_floats, prev_off, slot_ids, seq_of_token, cu_q, positions, static_cast<bf16_t*>(out),
                       width, n_mix, n_seqs, n_slots, n_tokens);
  else
    return static_cast<int>(hipErrorInvalidValue);
  return kvf_last_error();
}

KVF_EXPORT int kvf_wkv_scan(int dtype, const void* rows, const float* z, const float* w0, const float* u,
                            const int* cu_q, const int* positions, const int* slot_ids, float* state, float* out,
                            int num_seqs, int H, int dk, int n_slots, int slot_floats, int row_len, int r_off,
                            int k_off, int v_off, int z_stride, hipStream_t s) {
  if (num_seqs <= 0) return 0;
  if (H <= 0 || dk <= 0 || dk > 256 || num_seqs > 65535 || H > 65535 || slot_floats < H * dk * dk ||
      z_stride < H * dk)
    return static_cast<int>(hipErrorInvalidValue);
  ScanArgs a{H, dk, num_seqs, n_slots, slot_floats, row_len, r_off, k_off, v_off, z_stride, dk > 128 ? 8 : 16};
  if (dtype == 0)
    return scan_launch<float>(rows, z, w0, u, cu_q, positions, slot_ids, state, out, num_seqs, a, s);
  if (dtype == 1)
    return scan_launch<bf16_t>(rows, z, w0, u, cu_q, positions, slot_ids, state, out, num_seqs, a, s);
  return static_cast<int>(hipErrorInvalidValue);
}

KVF_EXPORT int kvf_wkv_out(int dtype, const float* o, const void* g, int g_stride, const float* w, float eps,
                           void* out, int n, int H, int dk, hipStream_t s) {
  if (n <= 0) return 0;
  if (H <= 0 || H > 65535 || dk <= 0) return static_cast<int>(hipErrorInvalidValue);
  if (dtype == 0)
    hipLaunchKernelGGL(wkv_out_kernel<float>, dim3(n, H), dim3(KVF_WAVE), 0, s, o, static_cast<const float*>(g),
                       g_stride, w, eps, static_cast<float*>(out), H, dk);
  else if (dtype == 1)
    hipLaunchKernelGGL(wkv_out_kernel<bf16_t>, dim3(n, H), dim3(KVF_WAVE), 0, s, o, static_cast<const bf16_t*>(g),
                       g_stride, w, eps, static_cast<bf16_t*>(out), H, dk);
  else
    return static_cast<int>(hipErrorInvalidValue);
  return kvf_last_error();
}

KVF_EXPORT int kvf_wkv_tanh(int dtype, const float* in, void* out, long total, hipStream_t s) {
  if (total <= 0) return 0;
  const dim3 grid(static_cast<unsigned>((total + 255) / 256));
  if (dtype == 0)
    hipLaunchKernelGGL(wkv_tanh_kernel<float>, grid, dim3(256), 0, s, in, static_cast<float*>(out), total);
  else if (dtype == 1)
    hipLaunchKernelGGL(wkv_tanh_kernel<bf16_t>, grid, dim3(256), 0, s, in, static_cast<bf16_t*>(out), total);
  else
    return static_cast<int>(hipErrorInvalidValue);
  return kvf_last_error();
}
