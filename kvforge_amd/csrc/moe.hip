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
}  // namespace

KVF_EXPORT int kvf_moe_topk(const float* z, int z_stride, const float* correction, int* sel, float* wgt,
                            int n, int R, int top, hipStream_t s) {
  if (n <= 0) return 0;
  if (R <= 0 || R > MAX_PER_LANE * KVF_WAVE || top <= 0 || top > MAX_TOP || top > R)
    return static_cast<int>(hipErrorInvalidValue);
  hipLaunchKernelGGL(moe_topk_kernel, dim3(n), dim3(KVF_WAVE), 0, s, z, z_stride, correction, sel, wgt, R, top);
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
