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
//              rows); r, k, w of a stage of tokens go through LDS, from where lane l takes row
//              l's and the wave passes them round lane by lane.  Everything is fp32; the
//              order of every sum is fixed by the shapes, so a token's output does not depend
//              on how its sequence was cut into runs.
//   wkv_chunks : long runs, cut into chunks of 16 tokens that go side by side.  Over a chunk that
//              starts from S the recurrence ends in D S + G with D = prod_t diag(w_t) and G what
//              the chunk alone leaves behind from zeros.  Pass 1 (a workgroup per chunk, the
//              scan kernel without outputs) leaves every chunk's G and D; pass 2 (a thread per
//              element of S) walks a run's chunks in order and leaves in G's place the state
//              *before* each chunk, and the run's last state in the slot; pass 3 (the scan
//              kernel again) computes every chunk's outputs from that.  A prompt of 2,048
//              tokens is 128 x heads workgroups of 16 steps instead of heads workgroups of 2,048.
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
  const int i = blockIdx.y * blockDim.x + threadIdx.x;     // one element a thread: no loop to wait in
  if (i >= width) return;
  const float y = Elem<T>::load(row + i);
  const float p = from == 1 ? Elem<T>::load(before + i) : (from == 2 ? st[i] : 0.f);
  const float keep = save ? Elem<T>::load(last + i) : 0.f;
  for (int m = 0; m < n_mix; ++m)
    Elem<T>::store(out + m * plane + static_cast<size_t>(t) * width + i, fmaf(p - y, mu[m * width + i], y));
  if (save) st[i] = keep;   // this thread has read the element it writes
}

struct ScanArgs {
  int H, dk, n_seqs, n_slots, slot_floats;
  int row_len, r_off, k_off, v_off;   // where r, k, v of a token lie in a row of `rows`
  int z_stride;                        // row stride of the decay's pre-activations [tokens, >= H * dk]
  int stage;                           // tokens staged in LDS at a time
  int skip_from;                       // whole runs: those of at least this many tokens are another kernel's (0: none)
};

// What a workgroup of the scan kernel walks: a sequence's whole run from and to its slot
// (WHOLE), one chunk from zeros leaving G and D and no outputs (CHUNK_STATE), or one chunk from
// the state left in G's place, leaving outputs and no state (CHUNK_OUT).
enum ScanMode { WHOLE = 0, CHUNK_STATE = 1, CHUNK_OUT = 2 };


// ROWS: key rows a thread keeps (32 or 64); blockDim.x = 64 * ceil(dk / ROWS) >= dk.
// chunks: rows (sequence, first token, tokens, 0); G [chunks, H, dk, dk]; D [chunks, H, dk].
template <typename T, int ROWS, int MODE>
__global__ __launch_bounds__(256) void wkv_scan_kernel(const T* __restrict__ rows, const float* __restrict__ z,
                                                       const float* __restrict__ w0, const float* __restrict__ u,
                                                       const int* __restrict__ cu_q,
                                                       const int* __restrict__ positions,
                                                       const int* __restrict__ slot_ids, float* __restrict__ state,
                                                       float* __restrict__ out, ScanArgs a,
                                                       const int* __restrict__ chunks, float* __restrict__ G,
                                                       float* __restrict__ D) {
  extern __shared__ float lds[];
  const int dk = a.dk, head = blockIdx.y, SCAN_STAGE = a.stage;
  const int lane = threadIdx.x % KVF_WAVE, part = threadIdx.x / KVF_WAVE, parts = blockDim.x / KVF_WAVE;
  const int col = blockIdx.x * KVF_WAVE + lane;
  const bool col_ok = col < dk;
  float* rs = lds;                         // [STAGE][dk]
  float* ks = rs + SCAN_STAGE * dk;        // [STAGE][dk]
  float* ws = ks + SCAN_STAGE * dk;        // [STAGE][dk]
  float* vs = ws + SCAN_STAGE * dk;        // [STAGE][64]
  float* bonus = vs + SCAN_STAGE * KVF_WAVE;   // [STAGE]
  float* psum = bonus + SCAN_STAGE;        // [STAGE][parts][64]
  int t0, t1, slot = -1;
  if (MODE == WHOLE) {
    const int seq = blockIdx.z;
    t0 = cu_q[seq], t1 = cu_q[seq + 1];
    if (t1 <= t0 || (a.skip_from > 0 && t1 - t0 >= a.skip_from)) return;
    slot = slot_ids[seq];
    if (slot < 0 || slot >= a.n_slots) slot = -1;
  } else {
    t0 = chunks[4 * blockIdx.z + 1], t1 = t0 + chunks[4 * blockIdx.z + 2];
    if (t1 <= t0) return;
  }
  const int row0 = part * ROWS;
  // WHOLE: the head's memory in the slot; otherwise the chunk's place in G
  float* S_slot = MODE != WHOLE ? G + (static_cast<size_t>(blockIdx.z) * a.H + head) * dk * dk
                  : slot >= 0   ? state + static_cast<size_t>(slot) * a.slot_floats +
                                    static_cast<size_t>(head) * dk * dk
                                : nullptr;
  float S[ROWS];
  const bool resume = MODE == CHUNK_OUT || (MODE == WHOLE && slot >= 0 && positions[t0] > 0);
#pragma unroll
  for (int i = 0; i < ROWS; ++i)
    S[i] = (resume && col_ok && row0 + i < dk) ? S_slot[static_cast<size_t>(row0 + i) * dk + col] : 0.f;
  float decayed = 1.f;    // CHUNK_STATE: thread e < dk multiplies up the chunk's decays of row e
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
    if (MODE == CHUNK_STATE && static_cast<int>(threadIdx.x) < dk)
      for (int t = 0; t < cnt; ++t) decayed *= ws[t * dk + threadIdx.x];
    // the bonus of a token, sum_i r_i u_i k_i: a wave a token, lanes side by side along i
    for (int t = part; MODE != CHUNK_STATE && parts > 1 && t < cnt; t += parts) {
      float b = 0.f;
      for (int e = lane; e < dk; e += KVF_WAVE) b = fmaf(rs[t * dk + e] * uh[e], ks[t * dk + e], b);
      b = wave_sum(b);
      if (lane == 0) bonus[t] = b;
    }
    // lane l of a wave takes r, k, w of the wave's row l out of LDS once per token; every row's
    // three numbers then reach all lanes as scalars (v_readlane), not as 64 broadcast reads
    const int my_row = row0 + lane;
    const bool row_ok = lane < ROWS && my_row < dk;
    const float ul = row_ok ? uh[my_row] : 0.f;
    for (int t = 0; t < cnt; ++t) {
      const float v = vs[t * KVF_WAVE + lane];
      const int rl = row_ok ? __float_as_int(rs[t * dk + my_row]) : 0;
      const int kl = row_ok ? __float_as_int(ks[t * dk + my_row]) : 0;
      const int wl = row_ok ? __float_as_int(ws[t * dk + my_row]) : 0;   // rows past dk: S stays 0
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < ROWS; ++i) {
        const float ri = __int_as_float(__builtin_amdgcn_readlane(rl, i));
        const float ki = __int_as_float(__builtin_amdgcn_readlane(kl, i));
        const float wi = __int_as_float(__builtin_amdgcn_readlane(wl, i));
        acc = fmaf(ri, S[i], acc);
        S[i] = fmaf(wi, S[i], ki * v);
      }
      if (MODE == CHUNK_STATE) continue;
      if (parts == 1) {
        // one wave has all rows: the token's output is complete here (the bonus summed over the
        // lanes' own rows, in the order the wider case sums it)
        const float b = wave_sum(__int_as_float(rl) * ul * __int_as_float(kl));
        if (col_ok) out[(static_cast<size_t>(tb + t) * a.H + head) * dk + col] = fmaf(v, b, acc);
      } else {
        psum[(t * parts + part) * KVF_WAVE + lane] = acc;
      }
    }
    if (MODE == CHUNK_STATE || parts == 1) continue;     // (the next stage starts with a barrier)
    __syncthreads();
    for (int i = threadIdx.x; i < cnt * KVF_WAVE; i += blockDim.x) {
      const int t = i / KVF_WAVE, l = i % KVF_WAVE, c = blockIdx.x * KVF_WAVE + l;
      if (c >= dk) continue;
      float o = 0.f;
      for (int p = 0; p < parts; ++p) o += psum[(t * parts + p) * KVF_WAVE + l];
      out[(static_cast<size_t>(tb + t) * a.H + head) * dk + c] = fmaf(vs[i], bonus[t], o);
    }
  }
  if (MODE == CHUNK_OUT) return;
  if (S_slot != nullptr && col_ok) {
#pragma unroll
    for (int i = 0; i < ROWS; ++i)
      if (row0 + i < dk) S_slot[static_cast<size_t>(row0 + i) * dk + col] = S[i];
  }
  if (MODE == CHUNK_STATE && blockIdx.x == 0 && static_cast<int>(threadIdx.x) < dk)
    D[(static_cast<size_t>(blockIdx.z) * a.H + head) * dk + threadIdx.x] = decayed;
}

// runs: rows (sequence, first chunk, chunks).  A thread per element (i, j) of a head's memory walks
// the run's chunks in order: G[c] becomes the state before chunk c, the state after the last one
// goes to the slot.  Four chunks' loads are asked for before the chain of four steps uses them.
__global__ __launch_bounds__(256) void wkv_carry_kernel(const int* __restrict__ runs, const int* __restrict__ cu_q,
                                                        const int* __restrict__ positions,
                                                        const int* __restrict__ slot_ids, float* __restrict__ state,
                                                        float* __restrict__ G, const float* __restrict__ D, int H,
                                                        int dk, int n_slots, int slot_floats) {
  const int run = blockIdx.z, head = blockIdx.y, e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= dk * dk) return;
  const int seq = runs[3 * run], c0 = runs[3 * run + 1], nc = runs[3 * run + 2];
  int slot = slot_ids[seq];
  if (slot < 0 || slot >= n_slots) slot = -1;
  float* S_slot = slot >= 0 ? state + static_cast<size_t>(slot) * slot_floats + static_cast<size_t>(head) * dk * dk + e
                            : nullptr;
  float S = (slot >= 0 && positions[cu_q[seq]] > 0) ? *S_slot : 0.f;
  const size_t gs = static_cast<size_t>(H) * dk * dk, ds = static_cast<size_t>(H) * dk;
  float* g = G + (static_cast<size_t>(c0) * H + head) * dk * dk + e;
  const float* d = D + (static_cast<size_t>(c0) * H + head) * dk + e / dk;
  int c = 0;
  for (; c + 4 <= nc; c += 4, g += 4 * gs, d += 4 * ds) {
    const float g0 = g[0], g1 = g[gs], g2 = g[2 * gs], g3 = g[3 * gs];
    const float d0 = d[0], d1 = d[ds], d2 = d[2 * ds], d3 = d[3 * ds];
    g[0] = S;
    S = fmaf(d0, S, g0);
    g[gs] = S;
    S = fmaf(d1, S, g1);
    g[2 * gs] = S;
    S = fmaf(d2, S, g2);
    g[3 * gs] = S;
    S = fmaf(d3, S, g3);
  }
  for (; c < nc; ++c, g += gs, d += ds) {
    const float g0 = g[0], d0 = d[0];
    g[0] = S;
    S = fmaf(d0, S, g0);
  }
  if (S_slot != nullptr) *S_slot = S;
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

template <typename T, int MODE>
int scan_launch(const void* rows, const float* z, const float* w0, const float* u, const int* cu_q,
                const int* positions, const int* slot_ids, float* state, float* out, int grid_z, ScanArgs a,
                const int* chunks, float* G, float* D, hipStream_t s) {
  const int rows_per = a.dk <= 32 ? 32 : 64;
  const int parts = (a.dk + rows_per - 1) / rows_per;
  const dim3 grid((a.dk + KVF_WAVE - 1) / KVF_WAVE, a.H, grid_z), block(parts * KVF_WAVE);
  const size_t lds = sizeof(float) * (static_cast<size_t>(a.stage) * (3 * a.dk + KVF_WAVE + 1 + parts * KVF_WAVE));
  if (rows_per == 32)
    hipLaunchKernelGGL((wkv_scan_kernel<T, 32, MODE>), grid, block, lds, s, static_cast<const T*>(rows), z, w0, u,
                       cu_q, positions, slot_ids, state, out, a, chunks, G, D);
  else
    hipLaunchKernelGGL((wkv_scan_kernel<T, 64, MODE>), grid, block, lds, s, static_cast<const T*>(rows), z, w0, u,
                       cu_q, positions, slot_ids, state, out, a, chunks, G, D);
  return kvf_last_error();
}

template <typename T>
int chunks_launch(const void* rows, const float* z, const float* w0, const float* u, const int* cu_q,
                  const int* positions, const int* slot_ids, float* state, float* out, const int* chunks,
                  int n_chunks, const int* runs, int n_runs, float* G, float* D, ScanArgs a, hipStream_t s) {
  int rc = scan_launch<T, CHUNK_STATE>(rows, z, w0, u, cu_q, positions, slot_ids, state, out, n_chunks, a, chunks, G,
                                       D, s);
  if (rc) return rc;
  hipLaunchKernelGGL(wkv_carry_kernel, dim3((a.dk * a.dk + 255) / 256, a.H, n_runs), dim3(256), 0, s, runs, cu_q,
                     positions, slot_ids, state, G, D, a.H, a.dk, a.n_slots, a.slot_floats);
  rc = kvf_last_error();
  if (rc) return rc;
  return scan_launch<T, CHUNK_OUT>(rows, z, w0, u, cu_q, positions, slot_ids, state, out, n_chunks, a, chunks, G, D,
                                   s);
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
    hipLaunchKernelGGL(wkv_mix_kernel<float>, dim3(n_tokens, (width + 255) / 256), dim3(256), 0, s, static_cast<const float*>(h), mu, state,
                       slot_floats, prev_off, slot_ids, seq_of_token, cu_q, positions, static_cast<float*>(out),
                       width, n_mix, n_seqs, n_slots, n_tokens);
  else if (dtype == 1)
    hipLaunchKernelGGL(wkv_mix_kernel<bf16_t>, dim3(n_tokens, (width + 255) / 256), dim3(256), 0, s, static_cast<const bf16_t*>(h), mu, state,
                       slot_floats, prev_off, slot_ids, seq_of_token, cu_q, positions, static_cast<bf16_t*>(out),
                       width, n_mix, n_seqs, n_slots, n_tokens);
  else
    return static_cast<int>(hipErrorInvalidValue);
  return kvf_last_error();
}

// skip_from: runs of at least this many tokens are left alone (kvf_wkv_chunks takes them); 0: none.
KVF_EXPORT int kvf_wkv_scan(int dtype, const void* rows, const float* z, const float* w0, const float* u,
                            const int* cu_q, const int* positions, const int* slot_ids, float* state, float* out,
                            int num_seqs, int H, int dk, int n_slots, int slot_floats, int row_len, int r_off,
                            int k_off, int v_off, int z_stride, int skip_from, hipStream_t s) {
  if (num_seqs <= 0) return 0;
  if (H <= 0 || dk <= 0 || dk > 256 || num_seqs > 65535 || H > 65535 || slot_floats < H * dk * dk ||
      z_stride < H * dk || skip_from < 0)
    return static_cast<int>(hipErrorInvalidValue);
  ScanArgs a{H, dk, num_seqs, n_slots, slot_floats, row_len, r_off, k_off, v_off, z_stride, dk > 128 ? 8 : 16,
             skip_from};
  if (dtype == 0)
    return scan_launch<float, WHOLE>(rows, z, w0, u, cu_q, positions, slot_ids, state, out, num_seqs, a, nullptr,
                                     nullptr, nullptr, s);
  if (dtype == 1)
    return scan_launch<bf16_t, WHOLE>(rows, z, w0, u, cu_q, positions, slot_ids, state, out, num_seqs, a, nullptr,
                                      nullptr, nullptr, s);
  return static_cast<int>(hipErrorInvalidValue);
}

// The runs named in `runs` (sequence, first chunk, chunks), cut into `chunks` (sequence, first token,
// tokens, 0; a run's chunks in order and one after another), all chunks side by side.  G
// [n_chunks, H, dk, dk] and D [n_chunks, H, dk] are scratch.
KVF_EXPORT int kvf_wkv_chunks(int dtype, const void* rows, const float* z, const float* w0, const float* u,
                              const int* cu_q, const int* positions, const int* slot_ids, float* state, float* out,
                              const int* chunks, int n_chunks, const int* runs, int n_runs, float* G, float* D,
                              int num_seqs, int H, int dk, int n_slots, int slot_floats, int row_len, int r_off,
                              int k_off, int v_off, int z_stride, hipStream_t s) {
  if (n_chunks <= 0 || n_runs <= 0) return 0;
  if (H <= 0 || dk <= 0 || dk > 256 || n_chunks > 65535 || n_runs > 65535 || H > 65535 ||
      slot_floats < H * dk * dk || z_stride < H * dk || !chunks || !runs || !G || !D)
    return static_cast<int>(hipErrorInvalidValue);
  ScanArgs a{H, dk, num_seqs, n_slots, slot_floats, row_len, r_off, k_off, v_off, z_stride, dk > 128 ? 8 : 16, 0};
  if (dtype == 0)
    return chunks_launch<float>(rows, z, w0, u, cu_q, positions, slot_ids, state, out, chunks, n_chunks, runs, n_runs,
                                G, D, a, s);
  if (dtype == 1)
    return chunks_launch<bf16_t>(rows, z, w0, u, cu_q, positions, slot_ids, state, out, chunks, n_chunks, runs,
                                 n_runs, G, D, a, s);
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
