// A feed-forward layer made of many small experts, of which every token uses a few.
//
//   router:  z = R h + r            32-bit; the `top` largest z are chosen (the lower index
//            wins a tie), and their weights are the soft-max over the chosen z alone
//   expert:  g = min(Wg h, limit), u = clamp(Wu h, -limit, limit)      (limit <= 0: no clamp)
//            y = g * sigmoid(alpha * g) * (u + shift)
//            out = Wd y
//   layer:   out[t] = sum over the chosen experts of weight * expert(h[t])
//
// Expert matrices are stacked: gate_up [E, 2 * ff, W] (an expert's gate rows, then its up
// rows) and down [E, W, ff].  Three kernels that stream the weights of the chosen experts
// token by token; every token's result depends on that token alone and its sums run in a
// fixed order, so a token gives the same bits whatever else is in the batch:
//
//  * moe_route         one wave per token
//  * moe_gate_up       grid (token * slot, groups of outputs): y[t, slot, :] of the expert in
//                      that slot, the token's row staged in LDS as 32-bit numbers
//  * moe_down          grid (token, groups of outputs): out[t, n] (=, or += into) the weighted
//                      sum over the slots in slot order, 32-bit
//
// With `ids` null every token uses expert 0 with weight 1 (an expert that all tokens share).
#include "zf_common.h"

#define MOE_MAX_EXPERTS 1024

template <typename T>
__global__ __launch_bounds__(ZF_WAVE) void moe_route_kernel(
    const T* __restrict__ h, const float* __restrict__ router, const float* __restrict__ bias,
    int* __restrict__ ids, float* __restrict__ weights, int W, int E, int top) {
  __shared__ float z[MOE_MAX_EXPERTS], share[MOE_MAX_EXPERTS];
  __shared__ int chosen[MOE_MAX_EXPERTS];
  const int t = blockIdx.x, lane = threadIdx.x;
  const T* row = h + (size_t)t * W;
  for (int e = 0; e < E; ++e) {
    const float* r = router + (size_t)e * W;
    float dot = 0.f;
    for (int i = lane; i < W; i += ZF_WAVE) dot = fmaf(load_as_float<T>(row + i), r[i], dot);
    dot = wave_sum(dot);
    if (lane == 0) z[e] = dot + (bias != nullptr ? bias[e] : 0.f);
  }
  __syncthreads();
  // `top` rounds of: the largest remaining logit, the lowest index among equals
  float first = 0.f, sum = 0.f;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int arg = 0x7fffffff;
    for (int e = lane; e < E; e += ZF_WAVE) {
      const float v = z[e];
      if (v > best) { best = v; arg = e; }
    }
#pragma unroll
    for (int off = ZF_WAVE / 2; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, ZF_WAVE);
      const int oa = __shfl_xor(arg, off, ZF_WAVE);
      if (ob > best || (ob == best && oa < arg)) { best = ob; arg = oa; }
    }
    if (arg == 0x7fffffff) arg = 0;            // nothing but NaN or -inf left
    if (k == 0) first = best;
    const float e_k = expf(best - first);       // the first chosen logit is the largest
    sum += e_k;
    __syncthreads();
    if (lane == 0) {
      chosen[k] = arg;
      share[k] = e_k;
      z[arg] = -INFINITY;
    }
    __syncthreads();
  }
  for (int k = lane; k < top; k += ZF_WAVE) {
    ids[(size_t)t * top + k] = chosen[k];
    weights[(size_t)t * top + k] = share[k] / sum;
  }
}

extern "C" int zf_moe_route(const void* h, int dtype, const float* router, const float* bias,
                            int* ids, float* weights, int T, int W, int E, int top,
                            hipStream_t stream) {
  if (T <= 0) return 0;
  if (E <= 0 || E > MOE_MAX_EXPERTS || top <= 0 || top > E) return -2;
  if (dtype == ZF_F32)
    hipLaunchKernelGGL(moe_route_kernel<float>, dim3(T), dim3(ZF_WAVE), 0, stream,
                       (const float*)h, router, bias, ids, weights, W, E, top);
  else
    hipLaunchKernelGGL(moe_route_kernel<bf16_t>, dim3(T), dim3(ZF_WAVE), 0, stream,
                       (const bf16_t*)h, router, bias, ids, weights, W, E, top);
  ZF_CHECK_LAUNCH();
}

// the activation of an expert's two products
__device__ __forceinline__ float gated_unit(float g, float u, float limit, float alpha,
                                            float shift) {
  if (limit > 0.f) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
  }
  return g * (1.0f / (1.0f + expf(-alpha * g))) * (u + shift);
}

// dot product of a weight row with a vector held in LDS as floats, lanes side by side
template <typename T>
__device__ __forceinline__ float row_dot_lds(const T* __restrict__ w, const float* __restrict__ x,
                                             int n, int lane) {
  float dot = 0.f;
  for (int i = lane; i < n; i += ZF_WAVE) dot = fmaf(load_as_float<T>(w + i), x[i], dot);
  return dot;
}

#define MOE_WAVES 4
#define MOE_GU_PER_WAVE 4      // outputs of y a wave computes, one after the other

template <typename T>
__global__ __launch_bounds__(MOE_WAVES * ZF_WAVE) void moe_gate_up_kernel(
    const T* __restrict__ h, const T* __restrict__ gate_up, const int* __restrict__ ids,
    T* __restrict__ y, int W, int ff, int slots, float limit, float alpha, float shift) {
  extern __shared__ float xs[];                    // the token's row, [W]
  const int ts = blockIdx.x, t = ts / slots;
  const int e = ids != nullptr ? ids[ts] : 0;
  const int wave = threadIdx.x / ZF_WAVE, lane = threadIdx.x % ZF_WAVE;
  const T* row = h + (size_t)t * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) xs[i] = load_as_float<T>(row + i);
  __syncthreads();
  const T* we = gate_up + (size_t)e * 2 * ff * W;
  const int j0 = (blockIdx.y * MOE_WAVES + wave) * MOE_GU_PER_WAVE;
  for (int j = j0; j < j0 + MOE_GU_PER_WAVE && j < ff; ++j) {
    const float g = wave_sum(row_dot_lds<T>(we + (size_t)j * W, xs, W, lane));
    const float u = wave_sum(row_dot_lds<T>(we + (size_t)(ff + j) * W, xs, W, lane));
    if (lane == 0)
      store_from_float<T>(y + (size_t)ts * ff + j, gated_unit(g, u, limit, alpha, shift));
  }
}

extern "C" int zf_moe_gate_up(const void* h, const void* gate_up, int dtype, const int* ids,
                              void* y, int T, int W, int ff, int slots, float limit, float alpha,
                              float shift, hipStream_t stream) {
  if (T <= 0) return 0;
  if (W <= 0 || ff <= 0 || slots <= 0 || (size_t)W * sizeof(float) > 64 * 1024) return -2;
  const int per_wg = MOE_WAVES * MOE_GU_PER_WAVE;
  dim3 grid(T * slots, (ff + per_wg - 1) / per_wg);
  const size_t smem = (size_t)W * sizeof(float);
  if (dtype == ZF_F32)
    hipLaunchKernelGGL(moe_gate_up_kernel<float>, grid, dim3(MOE_WAVES * ZF_WAVE), smem, stream,
                       (const float*)h, (const float*)gate_up, ids, (float*)y, W, ff, slots,
                       limit, alpha, shift);
  else
    hipLaunchKernelGGL(moe_gate_up_kernel<bf16_t>, grid, dim3(MOE_WAVES * ZF_WAVE), smem, stream,
                       (const bf16_t*)h, (const bf16_t*)gate_up, ids, (bf16_t*)y, W, ff, slots,
                       limit, alpha, shift);
  ZF_CHECK_LAUNCH();
}

#define MOE_DOWN_PER_WAVE 4

template <typename T>
__global__ __launch_bounds__(MOE_WAVES * ZF_WAVE) void moe_down_kernel(
    const T* __restrict__ y, const T* __restrict__ down, const int* __restrict__ ids,
    const float* __restrict__ weights, float* __restrict__ out, int W, int ff, int slots,
    int add) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x / ZF_WAVE, lane = threadIdx.x % ZF_WAVE;
  const int n0 = (blockIdx.y * MOE_WAVES + wave) * MOE_DOWN_PER_WAVE;
  for (int n = n0; n < n0 + MOE_DOWN_PER_WAVE && n < W; ++n) {
    float total = 0.f;
    for (int s = 0; s < slots; ++s) {
      const int ts = t * slots + s;
      const int e = ids != nullptr ? ids[ts] : 0;
      const T* wr = down + ((size_t)e * W + n) * ff;
      const T* yr = y + (size_t)ts * ff;
      float dot = 0.f;
      for (int i = lane; i < ff; i += ZF_WAVE)
        dot = fmaf(load_as_float<T>(wr + i), load_as_float<T>(yr + i), dot);
      dot = wave_sum(dot);
      total += (weights != nullptr ? weights[ts] : 1.0f) * dot;
    }
    if (lane == 0) {
      float* o = out + (size_t)t * W + n;
      *o = add ? *o + total : total;
    }
  }
}

extern "C" int zf_moe_down(const void* y, const void* down, int dtype, const int* ids,
                           const float* weights, float* out, int T, int W, int ff, int slots,
                           int add, hipStream_t stream) {
  if (T <= 0) return 0;
  if (W <= 0 || ff <= 0 || slots <= 0) return -2;
  const int per_wg = MOE_WAVES * MOE_DOWN_PER_WAVE;
  dim3 grid(T, (W + per_wg - 1) / per_wg);
  if (dtype == ZF_F32)
    hipLaunchKernelGGL(moe_down_kernel<float>, grid, dim3(MOE_WAVES * ZF_WAVE), 0, stream,
                       (const float*)y, (const float*)down, ids, weights, out, W, ff, slots, add);
  else
    hipLaunchKernelGGL(moe_down_kernel<bf16_t>, grid, dim3(MOE_WAVES * ZF_WAVE), 0, stream,
                       (const bf16_t*)y, (const bf16_t*)down, ids, weights, out, W, ff, slots,
                       add);
  ZF_CHECK_LAUNCH();
}
