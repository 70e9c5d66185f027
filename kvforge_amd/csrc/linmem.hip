// A linear-attention memory: per head a matrix S [dk, dv] (key channel by value channel) whose
// key rows decay, zero before a sequence's first token.  For a token with rows q, k [dk], v [dv]
// and decays a [dk]:
//     S_ij <- a_i S_ij + k_i v_j            o_j = sum_i q_i S_ij      (the output sees the token itself)
// The decays are either constants (one number per head and key channel, handed in) or gates,
//     a = sigmoid(z + b)^(1/tau) = exp(logsigmoid(z + b) / tau),
// formed here in fp32 from pre-activations z [tokens, H * dk] (fp32) and a bias b [H * dk].
// q and k may be rotated first: the first `rot` elements of every head in neighbouring pairs
// (2i, 2i + 1) by the cos/sin row of the token's position, in fp32 as they are staged; then they
// are multiplied by constants (q_scale, k_scale).  A request's slot holds S of all heads, fp32.
//
//   linmem_scan   : token by token.  A workgroup per (64 value columns, head, sequence); a thread
//                   owns one value column of up to 64 key rows of S in registers (a wave per 64
//                   key rows); q, k, a of a stage of tokens go through LDS, from where lane l
//                   takes row l's and the wave passes them round lane by lane.
//   linmem_chunks : long runs, cut into chunks that go side by side.  Over a chunk that starts
//                   from S the recurrence ends in D S + G with D the product of the chunk's decays
//                   and G what the chunk alone leaves from zeros.  Pass 1 (the scan kernel without
//                   outputs) leaves every chunk's G and D; pass 2 (a thread per element of S)
//                   walks a run's chunks in order and leaves in G's place the state *before* each
//                   chunk, and the run's last state in the slot; pass 3 (the scan kernel again)
//                   computes every chunk's outputs from that.
//   linmem_out    : o / rms(o) * weight * silu(g) * scale per head (weight [dv] shared by the
//                   heads, or none).
// Everything is fp32; the order of every sum is fixed by the shapes.
#include "common.h"

namespace {

struct LmArgs {
  int H, dk, dv, n_seqs, n_slots, slot_floats;
  int q_stride, k_stride, v_stride;   // elements from one token's q (k, v) to the next token's
  int gated;                          // 0: `decay` holds constants [H * dk]; 1: z [tokens, z_stride] and a bias
  int z_stride;
  float inv_tau, q_scale, k_scale;
  int rot, table_len;                 // rotary width (0: none) and the positions the tables cover
  int stage;                          // tokens staged in LDS at a time
  int skip_from;                      // whole runs: those of at least this many tokens are another kernel's (0: none)
};

enum LmMode { LM_WHOLE = 0, LM_CHUNK_STATE = 1, LM_CHUNK_OUT = 2 };

__device__ __forceinline__ float log_sigmoid(float x) {
  return fminf(x, 0.f) - log1pf(expf(-fabsf(x)));
}

// ROWS: key rows a thread keeps (32 or 64); blockDim.x = 64 * ceil(dk / ROWS) >= dk.
// chunks: rows (sequence, first token, tokens, 0); G [chunks, H, dk, dv]; D [chunks, H, dk].
template <typename T, int ROWS, int MODE>
__global__ __launch_bounds__(256) void linmem_scan_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                          const T* __restrict__ v, const float* __restrict__ decay,
                                                          const float* __restrict__ bias,
                                                          const float* __restrict__ cos_t,
                                                          const float* __restrict__ sin_t,
                                                          const int* __restrict__ cu_q,
                                                          const int* __restrict__ positions,
                                                          const int* __restrict__ slot_ids,
                                                          float* __restrict__ state, float* __restrict__ out,
                                                          LmArgs a, const int* __restrict__ chunks,
                                                          float* __restrict__ G, float* __restrict__ D) {
  extern __shared__ float lds[];
  const int dk = a.dk, dv = a.dv, head = blockIdx.y, STAGE = a.stage;
  const int lane = threadIdx.x % KVF_WAVE, part = threadIdx.x / KVF_WAVE, parts = blockDim.x / KVF_WAVE;
  const int col = blockIdx.x * KVF_WAVE + lane;
  const bool col_ok = col < dv;
  float* qs = lds;                         // [STAGE][dk]
  float* ks = qs + STAGE * dk;             // [STAGE][dk]
  float* as = ks + STAGE * dk;             // [STAGE][dk]
  float* vs = as + STAGE * dk;             // [STAGE][64]
  float* psum = vs + STAGE * KVF_WAVE;     // [STAGE][parts][64]
  int t0, t1, slot = -1;
  if (MODE == LM_WHOLE) {
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
  const size_t head_floats = static_cast<size_t>(dk) * dv;
  // WHOLE: the head's memory in the slot; otherwise the chunk's place in G
  float* S_slot = MODE != LM_WHOLE ? G + (static_cast<size_t>(blockIdx.z) * a.H + head) * head_floats
                  : slot >= 0      ? state + static_cast<size_t>(slot) * a.slot_floats + head * head_floats
                                   : nullptr;
  float S[ROWS];
  const bool resume = MODE == LM_CHUNK_OUT || (MODE == LM_WHOLE && slot >= 0 && positions[t0] > 0);
#pragma unroll
  for (int i = 0; i < ROWS; ++i)
    S[i] = (resume && col_ok && row0 + i < dk) ? S_slot[static_cast<size_t>(row0 + i) * dv + col] : 0.f;
  float decayed = 1.f;    // CHUNK_STATE: thread e < dk multiplies up the chunk's decays of row e
  const float* dh = decay + (a.gated ? 0 : head * dk);
  const float* bh = bias ? bias + head * dk : nullptr;
  for (int tb = t0; tb < t1; tb += STAGE) {
    const int cnt = min(STAGE, t1 - tb);
    __syncthreads();
    for (int i = threadIdx.x; i < cnt * dk; i += blockDim.x) {
      const int t = i / dk, e = i - t * dk;
      const T* qp = q + static_cast<size_t>(tb + t) * a.q_stride + head * dk + e;
      const T* kp = k + static_cast<size_t>(tb + t) * a.k_stride + head * dk + e;
      float qv = Elem<T>::load(qp), kv = Elem<T>::load(kp);
      if (e < a.rot) {
        const int p = positions[tb + t];
        if (p >= 0 && p < a.table_len) {
          // the pair's other element, and the sign its product with the sine takes
          const int o = (e & 1) ? -1 : 1;
          const float c = cos_t[static_cast<size_t>(p) * (a.rot / 2) + e / 2];
          const float sn = sin_t[static_cast<size_t>(p) * (a.rot / 2) + e / 2] * static_cast<float>(-o);
          qv = fmaf(Elem<T>::load(qp + o), sn, qv * c);
          kv = fmaf(Elem<T>::load(kp + o), sn, kv * c);
        }
      }
      qs[i] = qv * a.q_scale;
      ks[i] = kv * a.k_scale;
      if (a.gated) {
        const float z = dh[static_cast<size_t>(tb + t) * a.z_stride + head * dk + e] + (bh ? bh[e] : 0.f);
        as[i] = expf(log_sigmoid(z) * a.inv_tau);
      } else {
        as[i] = dh[e];
      }
    }
    for (int i = threadIdx.x; i < cnt * KVF_WAVE; i += blockDim.x) {
      const int t = i / KVF_WAVE, c = blockIdx.x * KVF_WAVE + i % KVF_WAVE;
      vs[i] = c < dv ? Elem<T>::load(v + static_cast<size_t>(tb + t) * a.v_stride + head * dv + c) : 0.f;
    }
    __syncthreads();
    if (MODE == LM_CHUNK_STATE && static_cast<int>(threadIdx.x) < dk)
      for (int t = 0; t < cnt; ++t) decayed *= as[t * dk + threadIdx.x];
    // lane l of a wave takes q, k, a of the wave's row l out of LDS once per token; every row's
    // three numbers then reach all lanes as scalars (v_readlane), not as 64 broadcast reads
    const int my_row = row0 + lane;
    const bool row_ok = lane < ROWS && my_row < dk;
    for (int t = 0; t < cnt; ++t) {
      const float vv = vs[t * KVF_WAVE + lane];
      const int ql = row_ok ? __float_as_int(qs[t * dk + my_row]) : 0;
      const int kl = row_ok ? __float_as_int(ks[t * dk + my_row]) : 0;
      const int al = row_ok ? __float_as_int(as[t * dk + my_row]) : 0;   // rows past dk: S stays 0
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < ROWS; ++i) {
        const float qi = __int_as_float(__builtin_amdgcn_readlane(ql, i));
        const float ki = __int_as_float(__builtin_amdgcn_readlane(kl, i));
        const float ai = __int_as_float(__builtin_amdgcn_readlane(al, i));
        S[i] = fmaf(ai, S[i], ki * vv);
        acc = fmaf(qi, S[i], acc);
      }
      if (MODE == LM_CHUNK_STATE) continue;
      if (parts == 1) {
        if (col_ok) out[(static_cast<size_t>(tb + t) * a.H + head) * dv + col] = acc;
      } else {
        psum[(t * parts + part) * KVF_WAVE + lane] = acc;
      }
    }
    if (MODE == LM_CHUNK_STATE || parts == 1) continue;     // (the next stage starts with a barrier)
    __syncthreads();
    for (int i = threadIdx.x; i < cnt * KVF_WAVE; i += blockDim.x) {
      const int t = i / KVF_WAVE, l = i % KVF_WAVE, c = blockIdx.x * KVF_WAVE + l;
      if (c >= dv) continue;
      float o = 0.f;
      for (int p = 0; p < parts; ++p) o += psum[(t * parts + p) * KVF_WAVE + l];
      out[(static_cast<size_t>(tb + t) * a.H + head) * dv + c] = o;
    }
  }
  if (MODE == LM_CHUNK_OUT) return;
  if (S_slot != nullptr && col_ok) {
#pragma unroll
    for (int i = 0; i < ROWS; ++i)
      if (row0 + i < dk) S_slot[static_cast<size_t>(row0 + i) * dv + col] = S[i];
  }
  if (MODE == LM_CHUNK_STATE && blockIdx.x == 0 && static_cast<int>(threadIdx.x) < dk)
    D[(static_cast<size_t>(blockIdx.z) * a.H + head) * dk + threadIdx.x] = decayed;
}

// runs: rows (sequence, first chunk, chunks).  A thread per element (i, j) of a head's memory walks
// the run's chunks in order: G[c] becomes the state before chunk c, the state after the last one
// goes to the slot.  Four chunks' loads are asked for before the chain of four steps uses them.
__global__ __launch_bounds__(256) void linmem_carry_kernel(const int* __restrict__ runs, const int* __restrict__ cu_q,
                                                           const int* __restrict__ positions,
                                                           const int* __restrict__ slot_ids,
                                                           float* __restrict__ state, float* __restrict__ G,
                                                           const float* __restrict__ D, int H, int dk, int dv,
                                                           int n_slots, int slot_floats) {
  const int run = blockIdx.z, head = blockIdx.y, e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= dk * dv) return;
  const int seq = runs[3 * run], c0 = runs[3 * run + 1], nc = runs[3 * run + 2];
  int slot = slot_ids[seq];
  if (slot < 0 || slot >= n_slots) slot = -1;
  const size_t head_floats = static_cast<size_t>(dk) * dv;
  float* S_slot = slot >= 0 ? state + static_cast<size_t>(slot) * slot_floats + head * head_floats + e : nullptr;
  float S = (slot >= 0 && positions[cu_q[seq]] > 0) ? *S_slot : 0.f;
  const size_t gs = static_cast<size_t>(H) * head_floats, ds = static_cast<size_t>(H) * dk;
  float* g = G + (static_cast<size_t>(c0) * H + head) * head_floats + e;
  const float* d = D + (static_cast<size_t>(c0) * H + head) * dk + e / dv;
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

// A wave per (token, head): the head's root mean square, then weight, gate and scale.
template <typename T>
__global__ __launch_bounds__(KVF_WAVE) void linmem_out_kernel(const float* __restrict__ o, const T* __restrict__ g,
                                                              int g_stride, const float* __restrict__ w, float eps,
                                                              float scale, T* __restrict__ out, int H, int dv) {
  const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const float* orow = o + (static_cast<size_t>(t) * H + head) * dv;
  float ss = 0.f;
  for (int e = lane; e < dv; e += KVF_WAVE) ss = fmaf(orow[e], orow[e], ss);
  const float r = 1.f / sqrtf(wave_sum(ss) / static_cast<float>(dv) + eps);
  const T* grow = g + static_cast<size_t>(t) * g_stride + head * dv;
  T* dst = out + (static_cast<size_t>(t) * H + head) * dv;
  for (int e = lane; e < dv; e += KVF_WAVE) {
    const float gv = Elem<T>::load(grow + e);
    const float y = orow[e] * r * (w ? w[e] : 1.f);
    Elem<T>::store(dst + e, y * (gv / (1.f + expf(-gv))) * scale);
  }
}

template <typename T, int MODE>
int scan_launch(const void* q, const void* k, const void* v, const float* decay, const float* bias,
                const float* cos_t, const float* sin_t, const int* cu_q,
                const int* positions, const int* slot_ids, float* state, float* out, int grid_z, LmArgs a,
                const int* chunks, float* G, float* D, hipStream_t s) {
  const int rows_per = a.dk <= 32 ? 32 : 64;
  const int parts = (a.dk + rows_per - 1) / rows_per;
  const dim3 grid((a.dv + KVF_WAVE - 1) / KVF_WAVE, a.H, grid_z), block(parts * KVF_WAVE);
  const size_t lds = sizeof(float) * (static_cast<size_t>(a.stage) * (3 * a.dk + KVF_WAVE + parts * KVF_WAVE));
  if (rows_per == 32)
    hipLaunchKernelGGL((linmem_scan_kernel<T, 32, MODE>), grid, block, lds, s, static_cast<const T*>(q),
                       static_cast<const T*>(k), static_cast<const T*>(v), decay, bias, cos_t, sin_t, cu_q, positions, slot_ids,
                       state, out, a, chunks, G, D);
  else
    hipLaunchKernelGGL((linmem_scan_kernel<T, 64, MODE>), grid, block, lds, s, static_cast<const T*>(q),
                       static_cast<const T*>(k), static_cast<const T*>(v), decay, bias, cos_t, sin_t, cu_q, positions, slot_ids,
                       state, out, a, chunks, G, D);
  return kvf_last_error();
}

template <typename T>
int chunks_launch(const void* q, const void* k, const void* v, const float* decay, const float* bias,
                  const float* cos_t, const float* sin_t, const int* cu_q,
                  const int* positions, const int* slot_ids, float* state, float* out, const int* chunks,
                  int n_chunks, const int* runs, int n_runs, float* G, float* D, LmArgs a, hipStream_t s) {
  int rc = scan_launch<T, LM_CHUNK_STATE>(q, k, v, decay, bias, cos_t, sin_t, cu_q, positions, slot_ids, state, out, n_chunks, a,
                                          chunks, G, D, s);
  if (rc) return rc;
  hipLaunchKernelGGL(linmem_carry_kernel, dim3((a.dk * a.dv + 255) / 256, a.H, n_runs), dim3(256), 0, s, runs, cu_q,
                     positions, slot_ids, state, G, D, a.H, a.dk, a.dv, a.n_slots, a.slot_floats);
  rc = kvf_last_error();
  if (rc) return rc;
  return scan_launch<T, LM_CHUNK_OUT>(q, k, v, decay, bias, cos_t, sin_t, cu_q, positions, slot_ids, state, out, n_chunks, a,
                                      chunks, G, D, s);
}

bool args_ok(int H, int dk, int dv, int slot_floats, int gated, int z_stride, const float* decay, int rot,
             const float* cos_t, const float* sin_t) {
  if (rot < 0 || rot % 2 || rot > dk || (rot > 0 && (!cos_t || !sin_t))) return false;
  return H > 0 && dk > 0 && dk <= 256 && dv > 0 && H <= 65535 && decay != nullptr &&
         static_cast<long>(slot_floats) >= static_cast<long>(H) * dk * dv && (!gated || z_stride >= H * dk);
}
}  // namespace

#define LINMEM_ARGS_DECL                                                                                          \
  int dtype, const void *q, const void *k, const void *v, const float *decay, const float *bias,                 \
      const float *cos_t, const float *sin_t, int rot, int table_len, const int *cu_q, const int *positions, const int *slot_ids, float *state, float *out, int num_seqs, int H, int dk, int dv,   \
      int n_slots, int slot_floats, int q_stride, int k_stride, int v_stride, int gated, int z_stride,            \
      float inv_tau, float q_scale, float k_scale

// dtype: 0 = fp32, 1 = bf16 (q, k, v).  skip_from: runs of at least this many tokens are left alone
// (kvf_linmem_chunks takes them); 0: none.
KVF_EXPORT int kvf_linmem_scan(LINMEM_ARGS_DECL, int skip_from, hipStream_t s) {
  if (num_seqs <= 0) return 0;
  if (!args_ok(H, dk, dv, slot_floats, gated, z_stride, decay, rot, cos_t, sin_t) || num_seqs > 65535 || skip_from < 0)
    return static_cast<int>(hipErrorInvalidValue);
  LmArgs a{H, dk, dv, num_seqs, n_slots, slot_floats, q_stride, k_stride, v_stride, gated, z_stride, inv_tau,
           q_scale, k_scale, rot, table_len, dk > 128 ? 8 : 16, skip_from};
  if (dtype == 0)
    return scan_launch<float, LM_WHOLE>(q, k, v, decay, bias, cos_t, sin_t, cu_q, positions, slot_ids, state, out, num_seqs, a,
                                        nullptr, nullptr, nullptr, s);
  if (dtype == 1)
    return scan_launch<bf16_t, LM_WHOLE>(q, k, v, decay, bias, cos_t, sin_t, cu_q, positions, slot_ids, state, out, num_seqs, a,
                                         nullptr, nullptr, nullptr, s);
  return static_cast<int>(hipErrorInvalidValue);
}

// The runs named in `runs` (sequence, first chunk, chunks), cut into `chunks` (sequence, first token,
// tokens, 0; a run's chunks in order and one after another), all chunks side by side.  G
// [n_chunks, H, dk, dv] and D [n_chunks, H, dk] are scratch.
KVF_EXPORT int kvf_linmem_chunks(LINMEM_ARGS_DECL, const int* chunks, int n_chunks, const int* runs, int n_runs,
                                 float* G, float* D, hipStream_t s) {
  if (n_chunks <= 0 || n_runs <= 0) return 0;
  if (!args_ok(H, dk, dv, slot_floats, gated, z_stride, decay, rot, cos_t, sin_t) || n_chunks > 65535 || n_runs > 65535 || !chunks ||
      !runs || !G || !D)
    return static_cast<int>(hipErrorInvalidValue);
  LmArgs a{H, dk, dv, num_seqs, n_slots, slot_floats, q_stride, k_stride, v_stride, gated, z_stride, inv_tau,
           q_scale, k_scale, rot, table_len, dk > 128 ? 8 : 16, 0};
  if (dtype == 0)
    return chunks_launch<float>(q, k, v, decay, bias, cos_t, sin_t, cu_q, positions, slot_ids, state, out, chunks, n_chunks, runs,
                                n_runs, G, D, a, s);
  if (dtype == 1)
    return chunks_launch<bf16_t>(q, k, v, decay, bias, cos_t, sin_t, cu_q, positions, slot_ids, state, out, chunks, n_chunks, runs,
                                 n_runs, G, D, a, s);
  return static_cast<int>(hipErrorInvalidValue);
}

// w: null (no weight) or [dv] shared by the heads.
KVF_EXPORT int kvf_linmem_out(int dtype, const float* o, const void* g, int g_stride, const float* w, float eps,
                              float scale, void* out, int n, int H, int dv, hipStream_t s) {
  if (n <= 0) return 0;
  if (H <= 0 || H > 65535 || dv <= 0) return static_cast<int>(hipErrorInvalidValue);
  if (dtype == 0)
    hipLaunchKernelGGL(linmem_out_kernel<float>, dim3(n, H), dim3(KVF_WAVE), 0, s, o, static_cast<const float*>(g),
                       g_stride, w, eps, scale, static_cast<float*>(out), H, dv);
  else if (dtype == 1)
    hipLaunchKernelGGL(linmem_out_kernel<bf16_t>, dim3(n, H), dim3(KVF_WAVE), 0, s, o, static_cast<const bf16_t*>(g),
                       g_stride, w, eps, scale, static_cast<bf16_t*>(out), H, dv);
  else
    return static_cast<int>(hipErrorInvalidValue);
  return kvf_last_error();
}
