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
  int gate_stride;          // numbers from one token's gate row to the next (at least 2 H)
  int chunk_from;           // runs of at least so many tokens are the chunk kernel's, shorter ones the scan kernel's
  int multi_from;           // and runs of at least so many are taken by the kernels that work on all chunks at once
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
  extern __shared__ __align__(16) float lds[];
  const int seq = blockIdx.z, head = blockIdx.y, col0 = blockIdx.x * COLS;
  const int lane = threadIdx.x % KVF_WAVE, wave = threadIdx.x / KVF_WAVE, RG = blockDim.x / KVF_WAVE;
  const int slot = slot_ids[seq];
  const int t0 = cu_q[seq], t1 = cu_q[seq + 1];
  if (t1 <= t0 || t1 - t0 >= a.chunk_from) return;   // long runs belong to the chunk kernel
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
      const float* z = zif + static_cast<size_t>(tb + threadIdx.x) * a.gate_stride;
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

// ---------------------------------------------------------------------------------------------
// The same recurrence for long runs, a chunk of CL tokens at a time on the matrix cores, all in
// fp32 (v_mfma_f32_16x16x4_f32: D[i][j] += sum_k A[i][k] B[k][j], k = 0..3; lane l gives
// A[l % 16][l / 16] and B[l / 16][l % 16] and holds D[4 (l / 16) + v][l % 16], v = 0..3).
//
// With the state (S, n, m_c) at the chunk's start, b_t the sum of the log forget gates of the
// chunk's tokens up to t, and m_t from the recurrence itself (one thread walks it, so that it is
// the number the token-by-token kernel gets):
//   D[t][s] = exp(b_t - b_s + li_s - m_t) for s <= t (0 otherwise),  g_t = exp(b_t + m_c - m_t)
//   A = (Q K^T) * D;   O = A V + diag(g) Q S;   n_t . q_t = rowsum(A)_t + g_t q_t . n
//   S' = g_L S + K^T diag(D[L]) V;   n' = g_L n + K^T D[L];   m_c' = m_L        (L: the last token)
// which is the recurrence written out over the chunk.  A workgroup of four waves takes 32 columns
// of S for one (sequence, head); Q, K, A (fp32, token-major) and V, S (column-major: Vt[c][token],
// St[c][k]) live in LDS with row strides of 4 mod 32 floats.  The four lane groups of the
// instruction stand for four *neighbouring* k each (group g takes k = k0 + 4 g + e in
// instruction e of four), so that a lane's operands for four instructions are 16 consecutive
// bytes of a row: one LDS read for four matrix instructions, spread evenly over the banks.
typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr int CCOLS = 32;

template <typename T, int DKP, int CL>
__global__ __launch_bounds__(256) void mlstm_chunk_kernel(const T* __restrict__ qkv, const float* __restrict__ zif,
                                                          const float* __restrict__ bias_if,
                                                          const int* __restrict__ cu_q,
                                                          const int* __restrict__ positions,
                                                          const int* __restrict__ slot_ids,
                                                          float* __restrict__ state, float* __restrict__ out,
                                                          ScanArgs a) {
  extern __shared__ __align__(16) float lds[];
  constexpr int QLD = DKP + 4, ALD = CL + 4, VLD = CL + 4, SLD = DKP + 4;
  // the running sum of the log forget gates is kept in 64 bits: its differences b_t - b_s are
  // what the weights are made of, and a sum that has passed a nearly closed gate is hundreds
  // of times larger than the differences that matter behind it
  double* bc = reinterpret_cast<double*>(lds);   // [CL] log forget gates, then their running sum
  float* Qs = lds + 2 * CL;              // [CL][QLD], q times its scale
  float* Ks = Qs + CL * QLD;             // [CL][QLD]
  float* Vt = Ks + CL * QLD;             // [CCOLS][VLD]: the block's columns of v, a column's tokens side by side
  float* As = Vt + CCOLS * VLD;          // [CL][ALD]
  float* St = As + CL * ALD;             // [CCOLS][SLD]: the block's columns of S, a column's rows side by side
  float* ns = St + CCOLS * SLD;          // [DKP]
  float* li = ns + DKP;                  // [CL] log input gates
  float* mt = li + CL;                   // [CL] running maximum after each token
  float* gt = mt + CL;                   // [CL] weight of the chunk's first state for token t
  float* wl = gt + CL;                   // [CL] weight of token s in the chunk's last state
  float* den = wl + CL;                  // [CL]
  float* part = den + CL;                // [256 / CL][CL] shares of n . q
  __shared__ float m_c;
  const int seq = blockIdx.z, head = blockIdx.y, col0 = blockIdx.x * CCOLS;
  const int tid = threadIdx.x, lane = tid % KVF_WAVE, wave = tid / KVF_WAVE;
  const int l16 = lane % 16, lq = lane / 16;
  const int slot = slot_ids[seq];
  const int t0 = cu_q[seq], t1 = cu_q[seq + 1];
  if (t1 - t0 < a.chunk_from || t1 - t0 >= a.multi_from) return;    // short runs belong to the scan kernel, the longest to the passes
  const int dk = a.dk, dv = a.dv;
  if (slot < 0 || slot >= a.n_slots) {
    for (int i = tid; i < (t1 - t0) * CCOLS; i += blockDim.x) {
      const int t = i / CCOLS, c = col0 + i % CCOLS;
      if (c < dv) out[static_cast<size_t>(t0 + t) * a.H * dv + head * dv + c] = 0.f;
    }
    return;
  }
  const bool fresh = positions[t0] == 0;
  const bool vec8 = dk % 8 == 0 && a.row_len % 8 == 0 && a.q_off % 8 == 0 && a.k_off % 8 == 0 &&
                    reinterpret_cast<uintptr_t>(qkv) % (8 * sizeof(T)) == 0;
  float* st = state + (static_cast<size_t>(slot) * a.H + head) * (static_cast<size_t>(dk) * dv + dk + 1);
  for (int i = tid; i < DKP * CCOLS; i += blockDim.x) {
    const int r = i / CCOLS, cl = i % CCOLS, c = col0 + cl;
    St[cl * SLD + r] = (!fresh && r < dk && c < dv) ? st[static_cast<size_t>(r) * dv + c] : 0.f;
  }
  for (int r = tid; r < DKP; r += blockDim.x) ns[r] = (!fresh && r < dk) ? st[static_cast<size_t>(dk) * dv + r] : 0.f;
  if (tid == 0) m_c = fresh ? 0.f : st[static_cast<size_t>(dk) * dv + dk];

  for (int tb = t0; tb < t1; tb += CL) {
    const int cnt = min(CL, t1 - tb);
    __syncthreads();   // the chunk before is done with everything
    if (vec8) {
      // eight elements a load: the heads' rows start on 16 bytes (32 for fp32) and dk is a multiple of 8
      for (int i = tid; i < CL * (DKP / 8); i += blockDim.x) {
        const int t = i / (DKP / 8), e = 8 * (i - t * (DKP / 8));
        float qv[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, kv[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (t < cnt && e < dk) {
          const T* row = qkv + static_cast<size_t>(tb + t) * a.row_len;
          load8(row + a.q_off + head * dk + e, qv);
          load8(row + a.k_off + head * dk + e, kv);
        }
#pragma unroll
        for (int x = 0; x < 8; ++x) {
          Qs[t * QLD + e + x] = qv[x] * a.q_scale;
          Ks[t * QLD + e + x] = kv[x];
        }
      }
    } else {
      for (int i = tid; i < CL * DKP; i += blockDim.x) {
        const int t = i / DKP, e = i - t * DKP;
        float qv = 0.f, kv = 0.f;
        if (t < cnt && e < dk) {
          const T* row = qkv + static_cast<size_t>(tb + t) * a.row_len;
          qv = Elem<T>::load(row + a.q_off + head * dk + e) * a.q_scale;
          kv = Elem<T>::load(row + a.k_off + head * dk + e);
        }
        Qs[t * QLD + e] = qv;
        Ks[t * QLD + e] = kv;
      }
    }
    for (int i = tid; i < CL * CCOLS; i += blockDim.x) {
      const int t = i / CCOLS, cl = i % CCOLS, c = col0 + cl;
      Vt[cl * VLD + t] = (t < cnt && c < dv)
                             ? Elem<T>::load(qkv + static_cast<size_t>(tb + t) * a.row_len + a.v_off + head * dv + c)
                             : 0.f;
    }
    if (wave == 0) {
      // a lane per token: the gates, the running sum of the log forget gates (64-bit) and the
      // running maximum, which the recurrence m_t = max(lf_t + m_(t-1), li_t) gives as
      // m_t = b_t + max(m_c, max over s <= t of (li_s - b_s)): two scans over the wave
      const int t = lane;
      float i_gate = 0.f, f_gate = 0.f;
      if (t < cnt) {
        const float* z = zif + static_cast<size_t>(tb + t) * a.gate_stride;
        i_gate = capped(z[head] + bias_if[head], a.cap);
        f_gate = log_sigmoid(capped(z[a.H + head] + bias_if[a.H + head], a.cap));
      }
      double b = static_cast<double>(f_gate);
#pragma unroll
      for (int o = 1; o < KVF_WAVE; o <<= 1) {
        const double up = __shfl_up(b, o, KVF_WAVE);
        if (lane >= o) b += up;
      }
      double u = t < cnt ? static_cast<double>(i_gate) - b : -1e300;
#pragma unroll
      for (int o = 1; o < KVF_WAVE; o <<= 1) {
        const double up = __shfl_up(u, o, KVF_WAVE);
        if (lane >= o) u = fmax(u, up);
      }
      const float mc = m_c;
      const float m = static_cast<float>(b + fmax(static_cast<double>(mc), u));
      const int last_t = cnt - 1;
      const double b_last = __shfl(b, last_t, KVF_WAVE);
      const float m_last = __shfl(m, last_t, KVF_WAVE);
      if (t < CL) {
        li[t] = i_gate;
        bc[t] = b;
        mt[t] = t < cnt ? m : m_last;
        gt[t] = t < cnt ? expf(static_cast<float>(b + static_cast<double>(mc) - static_cast<double>(m))) : 0.f;
        wl[t] = t < cnt ? expf(static_cast<float>(b_last - b) + i_gate - m_last) : 0.f;
      }
    }
    __syncthreads();
    const int last = cnt - 1;
    // ---- A = (Q K^T) * D, tile by tile; tiles above the diagonal are zero
    constexpr int RT = CL / 16;
    for (int tile = wave; tile < RT * RT; tile += 4) {
      const int rt = tile / RT, ct = tile - rt * RT;
      f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
      if (ct <= rt) {
        const float* qa = Qs + (16 * rt + l16) * QLD + 4 * lq;
        const float* kb = Ks + (16 * ct + l16) * QLD + 4 * lq;
#pragma unroll 4
        for (int k0 = 0; k0 < DKP; k0 += 16) {
          const f32x4 a4 = *reinterpret_cast<const f32x4*>(qa + k0), b4 = *reinterpret_cast<const f32x4*>(kb + k0);
#pragma unroll
          for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[e], b4[e], acc, 0, 0, 0);
        }
      }
      const int s = 16 * ct + l16;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int t = 16 * rt + 4 * lq + v;
        const bool vis = s <= t && t < cnt;
        As[t * ALD + s] = vis ? acc[v] * expf(static_cast<float>(bc[t] - bc[s]) + li[s] - mt[t]) : 0.f;
      }
    }
    __syncthreads();
    // ---- n . q per token: rowsum(A) + g_t q_t . n, in four shares
    {
      const int t = tid % CL, share = tid / CL;
      constexpr int SH = 256 / CL;
      float sum = 0.f;
      for (int s2 = share; s2 < CL; s2 += SH) sum += As[t * ALD + s2];
      float dot = 0.f;
      for (int k = share; k < DKP; k += SH) dot = fmaf(Qs[t * QLD + k], ns[k], dot);
      part[share * CL + t] = fmaf(gt[t], dot, sum);
    }
    __syncthreads();
    if (tid < CL) {
      constexpr int SH = 256 / CL;
      float nq = 0.f;
      for (int sh = 0; sh < SH; ++sh) nq += part[sh * CL + tid];
      den[tid] = fmaxf(fabsf(nq), expf(-mt[min(tid, last)])) + 1e-6f;
    }
    __syncthreads();
    // ---- O = A V + diag(g) Q S, divided by the denominator, to memory
    for (int tile = wave; tile < RT * (CCOLS / 16); tile += 4) {
      const int rt = tile / (CCOLS / 16), ct = tile - rt * (CCOLS / 16);
      f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
      const float* aa = As + (16 * rt + l16) * ALD + 4 * lq;
      const float* vb = Vt + (16 * ct + l16) * VLD + 4 * lq;
      for (int k0 = 0; k0 < 16 * (rt + 1); k0 += 16) {
        const f32x4 a4 = *reinterpret_cast<const f32x4*>(aa + k0), b4 = *reinterpret_cast<const f32x4*>(vb + k0);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[e], b4[e], acc, 0, 0, 0);
      }
      const float g = gt[16 * rt + l16];
      const float* qa = Qs + (16 * rt + l16) * QLD + 4 * lq;
      const float* sb = St + (16 * ct + l16) * SLD + 4 * lq;
#pragma unroll 4
      for (int k0 = 0; k0 < DKP; k0 += 16) {
        const f32x4 a4 = *reinterpret_cast<const f32x4*>(qa + k0) * g, b4 = *reinterpret_cast<const f32x4*>(sb + k0);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[e], b4[e], acc, 0, 0, 0);
      }
      const int c = col0 + 16 * ct + l16;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int t = 16 * rt + 4 * lq + v;
        if (t < cnt && c < dv) out[static_cast<size_t>(tb + t) * a.H * dv + head * dv + c] = acc[v] / den[t];
      }
    }
    __syncthreads();   // every read of S and n for this chunk is done
    // ---- S' = g_L S + K^T diag(w) V;  n' = g_L n + K^T w
    const float g_last = gt[last];
    for (int tile = wave; tile < (DKP / 16) * (CCOLS / 16); tile += 4) {
      const int kt = tile / (CCOLS / 16), ct = tile - kt * (CCOLS / 16);
      // the lane's four rows of S are neighbours in St: one read, one write
      f32x4* mine = reinterpret_cast<f32x4*>(St + (16 * ct + l16) * SLD + 16 * kt + 4 * lq);
      f32x4 acc = *mine * g_last;
      const float* ka = Ks + (4 * lq) * QLD + 16 * kt + l16;
      const float* vb = Vt + (16 * ct + l16) * VLD + 4 * lq;
#pragma unroll 2
      for (int k0 = 0; k0 < CL; k0 += 16) {
        const f32x4 b4 = *reinterpret_cast<const f32x4*>(vb + k0) * *reinterpret_cast<const f32x4*>(wl + k0 + 4 * lq);
#pragma unroll
        for (int e = 0; e < 4; ++e)
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(ka[(k0 + e) * QLD], b4[e], acc, 0, 0, 0);
      }
      *mine = acc;
    }
    for (int k = tid; k < DKP; k += blockDim.x) {
      float nk = g_last * ns[k];
      for (int s2 = 0; s2 < cnt; ++s2) nk = fmaf(wl[s2], Ks[s2 * QLD + k], nk);
      ns[k] = nk;
    }
    if (tid == 0) m_c = mt[last];
  }
  __syncthreads();
  for (int i = tid; i < DKP * CCOLS; i += blockDim.x) {
    const int r = i / CCOLS, cl = i % CCOLS, c = col0 + cl;
    if (r < dk && c < dv) st[static_cast<size_t>(r) * dv + c] = St[cl * SLD + r];
  }
  if (blockIdx.x == 0) {
    for (int r = tid; r < dk; r += blockDim.x) st[static_cast<size_t>(dk) * dv + r] = ns[r];
    if (tid == 0) st[static_cast<size_t>(dk) * dv + dk] = m_c;
  }
}

template <int DKP, int CL> constexpr size_t chunk_lds() {
  return sizeof(float) * (2 * CL + 2 * CL * (DKP + 4) + CCOLS * (CL + 4) + CL * (CL + 4) + CCOLS * (DKP + 4) + DKP +
                          5 * CL + 256);
}

template <typename T, int DKP, int CL>
int chunk_go(const void* qkv, const float* zif, const float* bias_if, const int* cu_q, const int* positions,
             const int* slot_ids, float* state, float* out, int num_seqs, ScanArgs a, hipStream_t s) {
  constexpr size_t lds = chunk_lds<DKP, CL>();
  static bool allowed = false;   // more LDS than a kernel gets unasked: asked for once per kernel
  if (!allowed) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&mlstm_chunk_kernel<T, DKP, CL>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    if (e != hipSuccess) return static_cast<int>(e);
    allowed = true;
  }
  const dim3 grid((a.dv + CCOLS - 1) / CCOLS, a.H, num_seqs);
  hipLaunchKernelGGL((mlstm_chunk_kernel<T, DKP, CL>), grid, dim3(256), lds, s, static_cast<const T*>(qkv), zif,
                     bias_if, cu_q, positions, slot_ids, state, out, a);
  return kvf_last_error();
}

template <typename T>
int chunk_launch(const void* qkv, const float* zif, const float* bias_if, const int* cu_q, const int* positions,
                 const int* slot_ids, float* state, float* out, int num_seqs, ScanArgs a, hipStream_t s) {
  if (num_seqs <= 0) return 0;
#define GO(DKP, CL) return chunk_go<T, DKP, CL>(qkv, zif, bias_if, cu_q, positions, slot_ids, state, out, num_seqs, a, s)
  if (a.dk <= 32) GO(32, 64);
  if (a.dk <= 64) GO(64, 64);
  if (a.dk <= 128) GO(128, 64);
  GO(256, 32);
#undef GO
}

// ---------------------------------------------------------------------------------------------
// The longest runs: all chunks of all sequences at once, in four passes (same formulas as above).
//   gates:  per (sequence, head) one wave walks the chunks: li, b (64-bit), m per token; per chunk
//           the maximum it starts from (m_c) and the weight of its first state in its last (g_L)
//   local:  per chunk, U = K^T diag(D[L]) V and u = K^T D[L]: what the chunk adds to the state
//   carry:  per element of S (and n), over the sequence's chunks in order: the chunk's slot in the
//           workspace gets the state *before* the chunk, the state becomes g_L S + U
//   output: per chunk, A = (Q K^T) * D, O = A V + diag(g) Q S_c, the denominator, to memory
// `chunks` rows: (sequence, first token, tokens, -); `runs` rows: (sequence, first chunk, chunks).
struct MultiArgs {
  const int* chunks;
  const int* runs;
  float* li;      // [tokens, H]
  float* mt;      // [tokens, H]
  double* bc;     // [tokens, H]
  float* mc;      // [chunks, H] the maximum before the chunk
  float* gl;      // [chunks, H] exp(b_L + m_c - m_L)
  float* W;       // [chunks, H, dk, dv]: U after `local`, the state before the chunk after `carry`
  float* un;      // [chunks, H, dk] likewise for n
};

template <int CL>
__global__ __launch_bounds__(KVF_WAVE) void mlstm_gates_kernel(const float* __restrict__ zif,
                                                               const float* __restrict__ bias_if,
                                                               const int* __restrict__ cu_q,
                                                               const int* __restrict__ positions,
                                                               const int* __restrict__ slot_ids,
                                                               float* __restrict__ state, ScanArgs a, MultiArgs w) {
  const int head = blockIdx.x, lane = threadIdx.x;
  const int seq = w.runs[3 * blockIdx.y], c0 = w.runs[3 * blockIdx.y + 1], nc = w.runs[3 * blockIdx.y + 2];
  const int slot = slot_ids[seq];
  if (slot < 0 || slot >= a.n_slots) return;
  const int t0 = cu_q[seq], t1 = cu_q[seq + 1];
  float* st = state + (static_cast<size_t>(slot) * a.H + head) * (static_cast<size_t>(a.dk) * a.dv + a.dk + 1);
  float m_c = positions[t0] == 0 ? 0.f : st[static_cast<size_t>(a.dk) * a.dv + a.dk];
  for (int j = 0; j < nc; ++j) {
    const int tb = t0 + j * CL, cnt = min(CL, t1 - tb), t = lane;
    float i_gate = 0.f, f_gate = 0.f;
    if (t < cnt) {
      const float* z = zif + static_cast<size_t>(tb + t) * a.gate_stride;
      i_gate = capped(z[head] + bias_if[head], a.cap);
      f_gate = log_sigmoid(capped(z[a.H + head] + bias_if[a.H + head], a.cap));
    }
    double b = static_cast<double>(f_gate);
#pragma unroll
    for (int o = 1; o < KVF_WAVE; o <<= 1) {
      const double up = __shfl_up(b, o, KVF_WAVE);
      if (lane >= o) b += up;
    }
    double u = t < cnt ? static_cast<double>(i_gate) - b : -1e300;
#pragma unroll
    for (int o = 1; o < KVF_WAVE; o <<= 1) {
      const double up = __shfl_up(u, o, KVF_WAVE);
      if (lane >= o) u = fmax(u, up);
    }
    const float m = static_cast<float>(b + fmax(static_cast<double>(m_c), u));
    const double b_last = __shfl(b, cnt - 1, KVF_WAVE);
    const float m_last = __shfl(m, cnt - 1, KVF_WAVE);
    if (t < cnt) {
      const size_t at = static_cast<size_t>(tb + t) * a.H + head;
      w.li[at] = i_gate;
      w.bc[at] = b;
      w.mt[at] = m;
    }
    if (lane == 0) {
      w.mc[static_cast<size_t>(c0 + j) * a.H + head] = m_c;
      w.gl[static_cast<size_t>(c0 + j) * a.H + head] =
          expf(static_cast<float>(b_last + static_cast<double>(m_c) - static_cast<double>(m_last)));
    }
    m_c = m_last;
  }
  if (lane == 0) st[static_cast<size_t>(a.dk) * a.dv + a.dk] = m_c;
}

// K (token-major) and the block's columns of V (column-major) of one chunk into LDS, as the
// chunk kernel keeps them; rows past the chunk's tokens and elements past dk, dv are zero.
template <typename T, int DKP, int CL>
__device__ __forceinline__ void stage_kv(const T* __restrict__ qkv, const ScanArgs& a, int head, int tb, int cnt,
                                         int col0, float* Qs, float* Ks, float* Vt, bool vec8) {
  constexpr int QLD = DKP + 4, VLD = CL + 4;
  const int tid = threadIdx.x, dk = a.dk, dv = a.dv;
  if (vec8) {
    for (int i = tid; i < CL * (DKP / 8); i += blockDim.x) {
      const int t = i / (DKP / 8), e = 8 * (i - t * (DKP / 8));
      float qv[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, kv[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (t < cnt && e < dk) {
        const T* row = qkv + static_cast<size_t>(tb + t) * a.row_len;
        if (Qs) load8(row + a.q_off + head * dk + e, qv);
        load8(row + a.k_off + head * dk + e, kv);
      }
#pragma unroll
      for (int x = 0; x < 8; ++x) {
        if (Qs) Qs[t * QLD + e + x] = qv[x] * a.q_scale;
        Ks[t * QLD + e + x] = kv[x];
      }
    }
  } else {
    for (int i = tid; i < CL * DKP; i += blockDim.x) {
      const int t = i / DKP, e = i - t * DKP;
      float qv = 0.f, kv = 0.f;
      if (t < cnt && e < dk) {
        const T* row = qkv + static_cast<size_t>(tb + t) * a.row_len;
        if (Qs) qv = Elem<T>::load(row + a.q_off + head * dk + e) * a.q_scale;
        kv = Elem<T>::load(row + a.k_off + head * dk + e);
      }
      if (Qs) Qs[t * QLD + e] = qv;
      Ks[t * QLD + e] = kv;
    }
  }
  for (int i = tid; i < CL * CCOLS; i += blockDim.x) {
    const int t = i / CCOLS, cl = i % CCOLS, c = col0 + cl;
    Vt[cl * VLD + t] = (t < cnt && c < dv)
                           ? Elem<T>::load(qkv + static_cast<size_t>(tb + t) * a.row_len + a.v_off + head * dv + c)
                           : 0.f;
  }
}

template <typename T, int DKP, int CL>
__global__ __launch_bounds__(256) void mlstm_local_kernel(const T* __restrict__ qkv, const int* __restrict__ slot_ids,
                                                          ScanArgs a, MultiArgs w) {
  extern __shared__ __align__(16) float lds[];
  constexpr int QLD = DKP + 4, VLD = CL + 4;
  float* Ks = lds;                 // [CL][QLD]
  float* Vt = Ks + CL * QLD;       // [CCOLS][VLD]
  float* wl = Vt + CCOLS * VLD;    // [CL]
  const int chunk = blockIdx.z, head = blockIdx.y, col0 = blockIdx.x * CCOLS;
  const int seq = w.chunks[4 * chunk], tb = w.chunks[4 * chunk + 1], cnt = w.chunks[4 * chunk + 2];
  const int slot = slot_ids[seq];
  if (slot < 0 || slot >= a.n_slots) return;
  const int tid = threadIdx.x, lane = tid % KVF_WAVE, wave = tid / KVF_WAVE, l16 = lane % 16, lq = lane / 16;
  const int dk = a.dk, dv = a.dv;
  const bool vec8 = dk % 8 == 0 && a.row_len % 8 == 0 && a.k_off % 8 == 0 &&
                    reinterpret_cast<uintptr_t>(qkv) % (8 * sizeof(T)) == 0;
  stage_kv<T, DKP, CL>(qkv, a, head, tb, cnt, col0, nullptr, Ks, Vt, vec8);
  if (tid < CL) {
    float v = 0.f;
    if (tid < cnt) {
      const size_t at = static_cast<size_t>(tb + tid) * a.H + head, last = static_cast<size_t>(tb + cnt - 1) * a.H + head;
      v = expf(static_cast<float>(w.bc[last] - w.bc[at]) + w.li[at] - w.mt[last]);
    }
    wl[tid] = v;
  }
  __syncthreads();
  float* U = w.W + (static_cast<size_t>(chunk) * a.H + head) * dk * dv;
  for (int tile = wave; tile < (DKP / 16) * (CCOLS / 16); tile += 4) {
    const int kt = tile / (CCOLS / 16), ct = tile - kt * (CCOLS / 16);
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
    const float* ka = Ks + (4 * lq) * QLD + 16 * kt + l16;
    const float* vb = Vt + (16 * ct + l16) * VLD + 4 * lq;
#pragma unroll 2
    for (int k0 = 0; k0 < CL; k0 += 16) {
      const f32x4 b4 = *reinterpret_cast<const f32x4*>(vb + k0) * *reinterpret_cast<const f32x4*>(wl + k0 + 4 * lq);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(ka[(k0 + e) * QLD], b4[e], acc, 0, 0, 0);
    }
    const int c = col0 + 16 * ct + l16;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int k = 16 * kt + 4 * lq + v;
      if (k < dk && c < dv) U[static_cast<size_t>(k) * dv + c] = acc[v];
    }
  }
  if (blockIdx.x == 0) {
    float* u = w.un + (static_cast<size_t>(chunk) * a.H + head) * dk;
    for (int k = tid; k < dk; k += blockDim.x) {
      float nk = 0.f;
      for (int s2 = 0; s2 < cnt; ++s2) nk = fmaf(wl[s2], Ks[s2 * QLD + k], nk);
      u[k] = nk;
    }
  }
}

// One thread per element of a head's S and n, over the run's chunks in order.
__global__ __launch_bounds__(256) void mlstm_carry_kernel(const int* __restrict__ cu_q, const int* __restrict__ positions,
                                                          const int* __restrict__ slot_ids, float* __restrict__ state,
                                                          ScanArgs a, MultiArgs w) {
  const int head = blockIdx.y;
  const int seq = w.runs[3 * blockIdx.z], c0 = w.runs[3 * blockIdx.z + 1], nc = w.runs[3 * blockIdx.z + 2];
  const int slot = slot_ids[seq];
  if (slot < 0 || slot >= a.n_slots) return;
  const size_t mat = static_cast<size_t>(a.dk) * a.dv;
  const size_t e = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (e >= mat + a.dk) return;
  float* st = state + (static_cast<size_t>(slot) * a.H + head) * (mat + a.dk + 1);
  float S = positions[cu_q[seq]] == 0 ? 0.f : st[e];
  for (int j = 0; j < nc; ++j) {
    const size_t ch = static_cast<size_t>(c0 + j) * a.H + head;
    float* slot_of = e < mat ? w.W + ch * mat + e : w.un + ch * a.dk + (e - mat);
    const float add = *slot_of;
    *slot_of = S;
    S = fmaf(w.gl[ch], S, add);
  }
  st[e] = S;
}

template <typename T, int DKP, int CL>
__global__ __launch_bounds__(256) void mlstm_output_kernel(const T* __restrict__ qkv, const int* __restrict__ slot_ids,
                                                           float* __restrict__ out, ScanArgs a, MultiArgs w) {
  extern __shared__ __align__(16) float lds[];
  constexpr int QLD = DKP + 4, ALD = CL + 4, VLD = CL + 4, SLD = DKP + 4;
  double* bc = reinterpret_cast<double*>(lds);   // [CL]
  float* Qs = lds + 2 * CL;
  float* Ks = Qs + CL * QLD;
  float* Vt = Ks + CL * QLD;
  float* As = Vt + CCOLS * VLD;
  float* St = As + CL * ALD;
  float* ns = St + CCOLS * SLD;
  float* li = ns + DKP;
  float* mt = li + CL;
  float* gt = mt + CL;
  float* den = gt + CL;
  float* part = den + CL;   // [256 / CL][CL]
  const int chunk = blockIdx.z, head = blockIdx.y, col0 = blockIdx.x * CCOLS;
  const int seq = w.chunks[4 * chunk], tb = w.chunks[4 * chunk + 1], cnt = w.chunks[4 * chunk + 2];
  const int tid = threadIdx.x, lane = tid % KVF_WAVE, wave = tid / KVF_WAVE, l16 = lane % 16, lq = lane / 16;
  const int dk = a.dk, dv = a.dv;
  const int slot = slot_ids[seq];
  if (slot < 0 || slot >= a.n_slots) {
    for (int i = tid; i < cnt * CCOLS; i += blockDim.x) {
      const int t = i / CCOLS, c = col0 + i % CCOLS;
      if (c < dv) out[static_cast<size_t>(tb + t) * a.H * dv + head * dv + c] = 0.f;
    }
    return;
  }
  const bool vec8 = dk % 8 == 0 && a.row_len % 8 == 0 && a.q_off % 8 == 0 && a.k_off % 8 == 0 &&
                    reinterpret_cast<uintptr_t>(qkv) % (8 * sizeof(T)) == 0;
  stage_kv<T, DKP, CL>(qkv, a, head, tb, cnt, col0, Qs, Ks, Vt, vec8);
  const size_t ch = static_cast<size_t>(chunk) * a.H + head;
  const float* Sc = w.W + ch * dk * dv;
  for (int i = tid; i < DKP * CCOLS; i += blockDim.x) {
    const int r = i / CCOLS, cl = i % CCOLS, c = col0 + cl;
    St[cl * SLD + r] = (r < dk && c < dv) ? Sc[static_cast<size_t>(r) * dv + c] : 0.f;
  }
  for (int r = tid; r < DKP; r += blockDim.x) ns[r] = r < dk ? w.un[ch * dk + r] : 0.f;
  const int last = cnt - 1;
  if (tid < CL) {
    const int t = min(tid, last);
    const size_t at = static_cast<size_t>(tb + t) * a.H + head;
    const float m_c = w.mc[ch];
    li[tid] = w.li[at];
    bc[tid] = w.bc[at];
    mt[tid] = w.mt[at];
    gt[tid] = tid < cnt ? expf(static_cast<float>(w.bc[at] + static_cast<double>(m_c) - static_cast<double>(w.mt[at]))) : 0.f;
  }
  __syncthreads();
  constexpr int RT = CL / 16;
  for (int tile = wave; tile < RT * RT; tile += 4) {
    const int rt = tile / RT, ct = tile - rt * RT;
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
    if (ct <= rt) {
      const float* qa = Qs + (16 * rt + l16) * QLD + 4 * lq;
      const float* kb = Ks + (16 * ct + l16) * QLD + 4 * lq;
#pragma unroll 4
      for (int k0 = 0; k0 < DKP; k0 += 16) {
        const f32x4 a4 = *reinterpret_cast<const f32x4*>(qa + k0), b4 = *reinterpret_cast<const f32x4*>(kb + k0);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[e], b4[e], acc, 0, 0, 0);
      }
    }
    const int s = 16 * ct + l16;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int t = 16 * rt + 4 * lq + v;
      const bool vis = s <= t && t < cnt;
      As[t * ALD + s] = vis ? acc[v] * expf(static_cast<float>(bc[t] - bc[s]) + li[s] - mt[t]) : 0.f;
    }
  }
  __syncthreads();
  {
    const int t = tid % CL, share = tid / CL;
    constexpr int SH = 256 / CL;
    float sum = 0.f;
    for (int s2 = share; s2 < CL; s2 += SH) sum += As[t * ALD + s2];
    float dot = 0.f;
    for (int k = share; k < DKP; k += SH) dot = fmaf(Qs[t * QLD + k], ns[k], dot);
    part[share * CL + t] = fmaf(gt[t], dot, sum);
  }
  __syncthreads();
  if (tid < CL) {
    constexpr int SH = 256 / CL;
    float nq = 0.f;
    for (int sh = 0; sh < SH; ++sh) nq += part[sh * CL + tid];
    den[tid] = fmaxf(fabsf(nq), expf(-mt[tid])) + 1e-6f;
  }
  __syncthreads();
  for (int tile = wave; tile < RT * (CCOLS / 16); tile += 4) {
    const int rt = tile / (CCOLS / 16), ct = tile - rt * (CCOLS / 16);
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
    const float* aa = As + (16 * rt + l16) * ALD + 4 * lq;
    const float* vb = Vt + (16 * ct + l16) * VLD + 4 * lq;
    for (int k0 = 0; k0 < 16 * (rt + 1); k0 += 16) {
      const f32x4 a4 = *reinterpret_cast<const f32x4*>(aa + k0), b4 = *reinterpret_cast<const f32x4*>(vb + k0);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[e], b4[e], acc, 0, 0, 0);
    }
    const float g = gt[16 * rt + l16];
    const float* qa = Qs + (16 * rt + l16) * QLD + 4 * lq;
    const float* sb = St + (16 * ct + l16) * SLD + 4 * lq;
#pragma unroll 4
    for (int k0 = 0; k0 < DKP; k0 += 16) {
      const f32x4 a4 = *reinterpret_cast<const f32x4*>(qa + k0) * g, b4 = *reinterpret_cast<const f32x4*>(sb + k0);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[e], b4[e], acc, 0, 0, 0);
    }
    const int c = col0 + 16 * ct + l16;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int t = 16 * rt + 4 * lq + v;
      if (t < cnt && c < dv) out[static_cast<size_t>(tb + t) * a.H * dv + head * dv + c] = acc[v] / den[t];
    }
  }
}

template <int DKP, int CL> constexpr size_t output_lds() {
  return sizeof(float) * (2 * CL + 2 * CL * (DKP + 4) + CCOLS * (CL + 4) + CL * (CL + 4) + CCOLS * (DKP + 4) + DKP +
                          4 * CL + 256);
}
template <int DKP, int CL> constexpr size_t local_lds() {
  return sizeof(float) * (CL * (DKP + 4) + CCOLS * (CL + 4) + CL);
}

template <typename T, int DKP, int CL>
int multi_go(const void* qkv, const float* zif, const float* bias_if, const int* cu_q, const int* positions,
             const int* slot_ids, float* state, float* out, int n_chunks, int n_runs, ScanArgs a, MultiArgs w,
             hipStream_t s) {
  static bool allowed = false;
  if (!allowed) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&mlstm_output_kernel<T, DKP, CL>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(output_lds<DKP, CL>()));
    if (e == hipSuccess)
      e = hipFuncSetAttribute(reinterpret_cast<const void*>(&mlstm_local_kernel<T, DKP, CL>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(local_lds<DKP, CL>()));
    if (e != hipSuccess) return static_cast<int>(e);
    allowed = true;
  }
  const T* rows = static_cast<const T*>(qkv);
  constexpr size_t lds_local = local_lds<DKP, CL>(), lds_output = output_lds<DKP, CL>();
  const int slices = (a.dv + CCOLS - 1) / CCOLS;
  hipLaunchKernelGGL(mlstm_gates_kernel<CL>, dim3(a.H, n_runs), dim3(KVF_WAVE), 0, s, zif, bias_if, cu_q, positions,
                     slot_ids, state, a, w);
  hipLaunchKernelGGL((mlstm_local_kernel<T, DKP, CL>), dim3(slices, a.H, n_chunks), dim3(256), lds_local, s,
                     rows, slot_ids, a, w);
  const unsigned per_head = static_cast<unsigned>((static_cast<size_t>(a.dk) * a.dv + a.dk + 255) / 256);
  hipLaunchKernelGGL(mlstm_carry_kernel, dim3(per_head, a.H, n_runs), dim3(256), 0, s, cu_q, positions, slot_ids, state,
                     a, w);
  hipLaunchKernelGGL((mlstm_output_kernel<T, DKP, CL>), dim3(slices, a.H, n_chunks), dim3(256), lds_output, s,
                     rows, slot_ids, out, a, w);
  return kvf_last_error();
}

template <typename T>
int multi_launch(const void* qkv, const float* zif, const float* bias_if, const int* cu_q, const int* positions,
                 const int* slot_ids, float* state, float* out, int n_chunks, int n_runs, ScanArgs a, MultiArgs w,
                 hipStream_t s) {
  if (n_chunks <= 0 || n_runs <= 0) return 0;
  if (n_chunks > 65535 || n_runs > 65535) return static_cast<int>(hipErrorInvalidValue);
#define GO(DKP, CL) \
  return multi_go<T, DKP, CL>(qkv, zif, bias_if, cu_q, positions, slot_ids, state, out, n_chunks, n_runs, a, w, s)
  if (a.dk <= 32) GO(32, 64);
  if (a.dk <= 64) GO(64, 64);
  if (a.dk <= 128) GO(128, 64);
  GO(256, 32);
#undef GO
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

// dtype: 0 = fp32, 1 = bf16 rows.  qkv [tokens, row_len]; zif [tokens, gate_stride >= 2 H] fp32 (input gates,
// then forget gates, before bias and cap); bias_if [2 H]; state [n_slots, H, dk dv + dk + 1];
// out [tokens, H dv] fp32.  Sequence s owns tokens cu_q[s] .. cu_q[s+1]-1 and slot slot_ids[s]
// (negative: skipped); it starts from zeros when its first token's position is 0.
// Runs of fewer than chunk_from tokens are walked token by token (`short_runs`: launch that
// kernel), runs of chunk_from to multi_from - 1 tokens chunk by chunk in one kernel (`long_runs`),
// runs of at least multi_from tokens by the four passes over all chunks at once (n_chunks > 0:
// `chunks` [n_chunks, 4] and `runs` [n_runs, 3] name them, the other pointers are their scratch);
// each kernel leaves the others' sequences alone.
KVF_EXPORT int kvf_mlstm_scan(int dtype, const void* qkv, const float* zif, const float* bias_if,
                              const int* cu_q, const int* positions, const int* slot_ids, float* state,
                              float* out, int num_seqs, int H, int dk, int dv, int row_len, int q_off,
                              int k_off, int v_off, int n_slots, int gate_stride, float cap, float q_scale, int chunk_from,
                              int short_runs, int long_runs, int multi_from, int n_chunks, int n_runs,
                              const int* chunks, const int* runs, float* w_li, float* w_mt, double* w_bc,
                              float* w_mc, float* w_gl, float* w_W, float* w_un, hipStream_t s) {
  if (H <= 0 || dk <= 0 || dk > 256 || dv <= 0 || !(cap > 0.f) || num_seqs > 65535 || H > 65535 || chunk_from < 1 ||
      gate_stride < 2 * H || multi_from < chunk_from)
    return static_cast<int>(hipErrorInvalidValue);
  if (dtype != 0 && dtype != 1) return static_cast<int>(hipErrorInvalidValue);
  const ScanArgs a{H, dk, dv, row_len, q_off, k_off, v_off, num_seqs, n_slots, cap, q_scale, gate_stride, chunk_from,
                   multi_from};
  int code = 0;
  if (short_runs)
    code = dtype == 0 ? scan_launch<float>(qkv, zif, bias_if, cu_q, positions, slot_ids, state, out, num_seqs, a, s)
                      : scan_launch<bf16_t>(qkv, zif, bias_if, cu_q, positions, slot_ids, state, out, num_seqs, a, s);
  if (code == 0 && long_runs)
    code = dtype == 0 ? chunk_launch<float>(qkv, zif, bias_if, cu_q, positions, slot_ids, state, out, num_seqs, a, s)
                      : chunk_launch<bf16_t>(qkv, zif, bias_if, cu_q, positions, slot_ids, state, out, num_seqs, a, s);
  if (code == 0 && n_chunks > 0) {
    if (!chunks || !runs || !w_li || !w_mt || !w_bc || !w_mc || !w_gl || !w_W || !w_un)
      return static_cast<int>(hipErrorInvalidValue);
    const MultiArgs w{chunks, runs, w_li, w_mt, w_bc, w_mc, w_gl, w_W, w_un};
    code = dtype == 0 ? multi_launch<float>(qkv, zif, bias_if, cu_q, positions, slot_ids, state, out, n_chunks, n_runs, a, w, s)
                      : multi_launch<bf16_t>(qkv, zif, bias_if, cu_q, positions, slot_ids, state, out, n_chunks, n_runs, a, w, s);
  }
  return code;
}

KVF_EXPORT int kvf_mlstm_chunk_len(int dk) { return dk <= 128 ? 64 : 32; }

KVF_EXPORT int kvf_mlstm_out(int dtype, const float* o, const void* g, int g_stride, const float* w, float eps,
                             void* out, int n, int H, int dv, hipStream_t s) {
  if (H <= 0 || H > 65535 || dv <= 0) return static_cast<int>(hipErrorInvalidValue);
  if (dtype == 0) return out_launch<float>(o, g, g_stride, w, eps, out, n, H, dv, s);
  if (dtype == 1) return out_launch<bf16_t>(o, g, g_stride, w, eps, out, n, H, dv, s);
  return static_cast<int>(hipErrorInvalidValue);
}
