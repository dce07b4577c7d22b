// Matrix-memory recurrence (mLSTM) over the tokens of every sequence of a step, with the state
// carried in per-request slots; everything but the projected q, k, v rows is fp32.
//
// Per head: a matrix S [dk, dv], a vector n [dk] and a running maximum m, all zero at position
// 0.  For a token with log input gate li and log forget gate lf (both from capped
// pre-activations):  a = lf + m;  m' = max(a, li);  S' = e^(a - m') S + e^(li - m') k v^T;
// n' likewise with k alone;  o = S'^T q / (max(|n' . q|, e^(-m')) + 1e-6).
//
// A slot holds, per head, S row-major, then n, then m: dk * dv + dk + 1 floats.
#include "common.h"

namespace {
constexpr int TB = 8;          // tokens staged in LDS at a time
constexpr int COLS = KVF_WAVE; // columns of S (elements of v) per workgroup: one per lane

struct ScanArgs {
  int H, dk, dv, row_len;   // row_len: elements from one token's projected row to the next
  int q_off, k_off, v_off;  // where q, k and v begin in a row (heads side by side)
  int n_seqs, n_slots;
  float cap, q_scale;
};

__device__ __forceinline__ float capped(float z, float cap) { return cap * tanhf(z / cap); }
__device__ __forceinline__ float log_sigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

// Workgroup (column block, head, sequence) of RG waves; wave w holds rows w*ROWS .. w*ROWS+ROWS-1
// of the block's 64 columns of S, a lane one column (ROWS registers), and lanes 0..ROWS-1 the
// wave's rows of n (row lane + 64 j).  A stage of TB tokens (k, q scaled, the block's elements of
// v, the two log gates) goes through LDS; within a stage nothing waits for memory.  With one
// wave there is no barrier per token; with several, the waves' shares of o and of n . q are
// added through LDS in wave order.
template <typename T, int ROWS>
__global__ __launch_bounds__(ROWS > KVF_WAVE ? 2 * KVF_WAVE : KVF_WAVE) void mlstm_scan_kernel(const T* __restrict__ qkv, const float* __restrict__ zif,
                                  const float* __restrict__ bias_if, const int* __restrict__ cu_q,
                                  const int* __restrict__ positions, const int* __restrict__ slot_ids,
                                  float* __restrict__ state, float* __restrict__ out, ScanArgs a) {
  extern __shared__ float lds[];
  const int seq = blockIdx.z, head = blockIdx.y, col0 = blockIdx.x * COLS;
  const int lane = threadIdx.x % KVF_WAVE, wave = threadIdx.x / KVF_WAVE, RG = blockDim.x / KVF_WAVE;
  const int slot = slot_ids[seq];
  const int t0 = cu_q[seq], t1 = cu_q[seq + 1];
  if (t1 <= t0) return;
  if (slot < 0 || slot >= a.n_slots) {   // the same for the whole workgroup
    // a sequence without a slot (the padding of a captured batch): zeros, so that its rows
    // never hold what an earlier step left there
    if (wave == 0 && col0 + lane < a.dv)
      for (int t = t0; t < t1; ++t) out[static_cast<size_t>(t) * a.H * a.dv + head * a.dv + col0 + lane] = 0.f;
    return;
  }
  const int dk = a.dk, dv = a.dv;
  float* ks = lds;                    // [TB][dk]
  float* qs = ks + TB * dk;           // [TB][dk]
  float* vs = qs + TB * dk;           // [TB][COLS]
  float* gs = vs + TB * COLS;         // [TB][2]: li, lf
  float* red = gs + TB * 2;           // [RG][COLS + 1]: shares of o, then of n . q
  const bool fresh = positions[t0] == 0;   // a sequence's first token: whatever the slot holds is not its own
  const int c = col0 + lane;
  const bool col_ok = c < dv;
  const int r0 = wave * ROWS;
  float* st = state + (static_cast<size_t>(slot) * a.H + head) * (static_cast<size_t>(dk) * dv + dk + 1);
  float S[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r)
    S[r] = (!fresh && col_ok && r0 + r < dk) ? st[static_cast<size_t>(r0 + r) * dv + c] : 0.f;
  constexpr int NJ = ROWS > KVF_WAVE ? ROWS / KVF_WAVE : 1;
  float nv[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int r = lane + KVF_WAVE * j;
    nv[j] = (!fresh && r < ROWS && r0 + r < dk) ? st[static_cast<size_t>(dk) * dv + r0 + r] : 0.f;
  }
  float m = fresh ? 0.f : st[static_cast<size_t>(dk) * dv + dk];

  for (int tb = t0; tb < t1; tb += TB) {
    const int cnt = min(TB, t1 - tb);
    __syncthreads();   // the stage before is consumed
    for (int i = threadIdx.x; i < cnt * dk; i += blockDim.x) {
      const int t = i / dk, e = i - t * dk;
      const T* row = qkv + static_cast<size_t>(tb + t) * a.row_len;
      ks[t * dk + e] = Elem<T>::load(row + a.k_off + head * dk + e);
      qs[t * dk + e] = Elem<T>::load(row + a.q_off + head * dk + e) * a.q_scale;
    }
    for (int i = threadIdx.x; i < cnt * COLS; i += blockDim.x) {
      const int t = i / COLS, e = i - t * COLS;
      vs[i] = col0 + e < dv
                  ? Elem<T>::load(qkv + static_cast<size_t>(tb + t) * a.row_len + a.v_off + head * dv + col0 + e)
                  : 0.f;
    }
    if (threadIdx.x < cnt) {
      const float* z = zif + static_cast<size_t>(tb + threadIdx.x) * 2 * a.H;
      gs[2 * threadIdx.x] = capped(z[head] + bias_if[head], a.cap);
      gs[2 * threadIdx.x + 1] = log_sigmoid(capped(z[a.H + head] + bias_if[a.H + head], a.cap));
    }
    __syncthreads();
    for (int t = 0; t < cnt; ++t) {
      const float li = gs[2 * t], lf = gs[2 * t + 1];
      const float al = lf + m;
      const float m_new = fmaxf(al, li);
      const float keep = expf(al - m_new), take = expf(li - m_new);
      const float tv = take * vs[t * COLS + lane];
      const float* kt = ks + t * dk + r0;
      const float* qt = qs + t * dk + r0;
      float o = 0.f;
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        if (r0 + r < dk) {
          S[r] = fmaf(keep, S[r], kt[r] * tv);
          o = fmaf(S[r], qt[r], o);
        }
      }
      float nq = 0.f;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int r = lane + KVF_WAVE * j;
        if (r < ROWS && r0 + r < dk) {
          nv[j] = fmaf(keep, nv[j], take * kt[r]);
          nq = fmaf(nv[j], qt[r], nq);
        }
      }
      nq = wave_sum(nq);
      if (RG > 1) {
        __syncthreads();
        red[wave * (COLS + 1) + lane] = o;
        if (lane == 0) red[wave * (COLS + 1) + COLS] = nq;
        __syncthreads();
        o = 0.f;
        nq = 0.f;
        for (int w = 0; w < RG; ++w) {
          o += red[w * (COLS + 1) + lane];
          nq += red[w * (COLS + 1) + COLS];
        }
      }
      m = m_new;
      const float den = fmaxf(fabsf(nq), expf(-m)) + 1e-6f;
      if (wave == 0 && col_ok)
        out[static_cast<size_t>(tb + t) * a.H * dv + head * dv + c] = o / den;
    }
  }
#pragma unroll
  for (int r = 0; r < ROWS; ++r)
    if (col_ok && r0 + r < dk) st[static_cast<size_t>(r0 + r) * dv + c] = S[r];
  if (blockIdx.x == 0) {
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int r = lane + KVF_WAVE * j;
      if (r < ROWS && r0 + r < dk) st[static_cast<size_t>(dk) * dv + r0 + r] = nv[j];
    }
    if (threadIdx.x == 0) st[static_cast<size_t>(dk) * dv + dk] = m;
  }
}

template <typename T>
int scan_launch(const void* qkv, const float* zif, const float* bias_if, const int* cu_q, const int* positions,
                const int* slot_ids, float* state, float* out, int num_seqs, ScanArgs a, hipStream_t s) {
  if (num_seqs <= 0) return 0;
  const int rows = a.dk <= 32 ? 32 : (a.dk <= 64 ? 64 : 128);
  const int rg = (a.dk + rows - 1) / rows;
  const dim3 grid((a.dv + COLS - 1) / COLS, a.H, num_seqs), block(rg * KVF_WAVE);
  const size_t lds = sizeof(float) * (static_cast<size_t>(TB) * (2 * a.dk + COLS + 2) + rg * (COLS + 1));
#define GO(ROWS)                                                                                  \
  hipLaunchKernelGGL((mlstm_scan_kernel<T, ROWS>), grid, block, lds, s, static_cast<const T*>(qkv), zif, \
                     bias_if, cu_q, positions, slot_ids, state, out, a)
  if (rows == 32) GO(32);
  else if (rows == 64) GO(64);
  else GO(128);
#undef GO
  return kvf_last_error();
}

// out[t, head, :] = o / rms(o) * w[head, :] * sigmoid(g[t, head, :]) for the raw heads o of the
// scan: a wave per (token, head); the root mean square is over the head's dv elements.
template <typename T>
__global__ __launch_bounds__(KVF_WAVE) void mlstm_out_kernel(const float* __restrict__ o, const T* __restrict__ g,
                                                             int g_stride, const float* __restrict__ w,
                                                             float eps, T* __restrict__ out, int H, int dv) {
  const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const float* orow = o + (static_cast<size_t>(t) * H + head) * dv;
  float ss = 0.f;
  for (int e = lane; e < dv; e += KVF_WAVE) ss = fmaf(orow[e], orow[e], ss);
  const float r = 1.f / sqrtf(wave_sum(ss) / static_cast<float>(dv) + eps);
  const T* grow = g + static_cast<size_t>(t) * g_stride + head * dv;
  T* dst = out + (static_cast<size_t>(t) * H + head) * dv;
  for (int e = lane; e < dv; e += KVF_WAVE) {
    const float gate = 1.f / (1.f + expf(-Elem<T>::load(grow + e)));
    Elem<T>::store(dst + e, orow[e] * r * w[head * dv + e] * gate);
  }
}

template <typename T>
int out_launch(const float* o, const void* g, int g_stride, const float* w, float eps, void* out, int n,
               int H, int dv, hipStream_t s) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL(mlstm_out_kernel<T>, dim3(n, H), dim3(KVF_WAVE), 0, s, o, static_cast<const T*>(g),
                     g_stride, w, eps, static_cast<T*>(out), H, dv);
  return kvf_last_error();
}
}  // namespace

// dtype: 0 = fp32, 1 = bf16 rows.  qkv [tokens, row_len]; zif [tokens, 2 H] fp32 (input gates,
// then forget gates, before bias and cap); bias_if [2 H]; state [n_slots, H, dk dv + dk + 1];
// out [tokens, H dv] fp32.  Sequence s owns tokens cu_q[s] .. cu_q[s+1]-1 and slot slot_ids[s]
// (negative: skipped); it starts from zeros when its first token's position is 0.
KVF_EXPORT int kvf_mlstm_scan(int dtype, const void* qkv, const float* zif, const float* bias_if,
                              const int* cu_q, const int* positions, const int* slot_ids, float* state,
                              float* out, int num_seqs, int H, int dk, int dv, int row_len, int q_off,
                              int k_off, int v_off, int n_slots, float cap, float q_scale, hipStream_t s) {
  if (H <= 0 || dk <= 0 || dk > 256 || dv <= 0 || !(cap > 0.f) || num_seqs > 65535 || H > 65535)
    return static_cast<int>(hipErrorInvalidValue);
  const ScanArgs a{H, dk, dv, row_len, q_off, k_off, v_off, num_seqs, n_slots, cap, q_scale};
  if (dtype == 0) return scan_launch<float>(qkv, zif, bias_if, cu_q, positions, slot_ids, state, out, num_seqs, a, s);
  if (dtype == 1) return scan_launch<bf16_t>(qkv, zif, bias_if, cu_q, positions, slot_ids, state, out, num_seqs, a, s);
  return static_cast<int>(hipErrorInvalidValue);
}

KVF_EXPORT int kvf_mlstm_out(int dtype, const float* o, const void* g, int g_stride, const float* w, float eps,
                             void* out, int n, int H, int dv, hipStream_t s) {
  if (H <= 0 || H > 65535 || dv <= 0) return static_cast<int>(hipErrorInvalidValue);
  if (dtype == 0) return out_launch<float>(o, g, g_stride, w, eps, out, n, H, dv, s);
  if (dtype == 1) return out_launch<bf16_t>(o, g, g_stride, w, eps, out, n, H, dv, s);
  return static_cast<int>(hipErrorInvalidValue);
}
