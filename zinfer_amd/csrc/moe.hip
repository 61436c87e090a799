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

// dot product of a weight row with a vector held in LDS as floats, lanes side by side; a
// bfloat16 row whose length is a multiple of 8 comes as 16-byte loads
template <typename T>
__device__ __forceinline__ float row_dot_lds(const T* __restrict__ w, const float* __restrict__ x,
                                             int n, int lane) {
  float dot = 0.f;
  if constexpr (sizeof(T) == 2) {
    if (n % 8 == 0) {
      for (int i = lane * 8; i < n; i += ZF_WAVE * 8) {
        const uint4 v = *(const uint4*)(w + i);
        const uint32_t p[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          dot = fmaf(__uint_as_float(p[c] << 16), x[i + 2 * c], dot);
          dot = fmaf(__uint_as_float(p[c] & 0xffff0000u), x[i + 2 * c + 1], dot);
        }
      }
      return dot;
    }
  }
  for (int i = lane; i < n; i += ZF_WAVE) dot = fmaf(load_as_float<T>(w + i), x[i], dot);
  return dot;
}

// the same between two rows in global memory
template <typename T>
__device__ __forceinline__ float row_dot(const T* __restrict__ w, const T* __restrict__ y, int n,
                                         int lane) {
  float dot = 0.f;
  if constexpr (sizeof(T) == 2) {
    if (n % 8 == 0) {
      for (int i = lane * 8; i < n; i += ZF_WAVE * 8) {
        const uint4 a = *(const uint4*)(w + i);
        const uint4 b = *(const uint4*)(y + i);
        const uint32_t p[4] = {a.x, a.y, a.z, a.w}, q[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          dot = fmaf(__uint_as_float(p[c] << 16), __uint_as_float(q[c] << 16), dot);
          dot = fmaf(__uint_as_float(p[c] & 0xffff0000u), __uint_as_float(q[c] & 0xffff0000u), dot);
        }
      }
      return dot;
    }
  }
  for (int i = lane; i < n; i += ZF_WAVE)
    dot = fmaf(load_as_float<T>(w + i), load_as_float<T>(y + i), dot);
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
      const float dot = wave_sum(row_dot<T>(wr, yr, ff, lane));
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

// ---------------------------------------------------------------- the activation alone
// out[t, j] = act(gu[t, j], gu[t, ff + j]) for a gate/up product that a plain matrix kernel
// made (an expert that every token uses)
template <typename T>
__global__ void gated_act_kernel(const T* __restrict__ gu, T* __restrict__ out, int ff, size_t n,
                                 float limit, float alpha, float shift) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const size_t t = i / ff, j = i % ff;
  const float g = load_as_float<T>(gu + t * 2 * ff + j);
  const float u = load_as_float<T>(gu + t * 2 * ff + ff + j);
  store_from_float<T>(out + i, gated_unit(g, u, limit, alpha, shift));
}

extern "C" int zf_gated_act(const void* gu, void* out, int dtype, int T, int ff, float limit,
                            float alpha, float shift, hipStream_t stream) {
  const size_t n = (size_t)T * ff;
  if (n == 0) return 0;
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (dtype == ZF_F32)
    hipLaunchKernelGGL(gated_act_kernel<float>, dim3(blocks), dim3(256), 0, stream,
                       (const float*)gu, (float*)out, ff, n, limit, alpha, shift);
  else
    hipLaunchKernelGGL(gated_act_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream,
                       (const bf16_t*)gu, (bf16_t*)out, ff, n, limit, alpha, shift);
  ZF_CHECK_LAUNCH();
}

// =====================================================================================
//  Many tokens (bfloat16): the (token, slot) pairs are sorted by expert, and every expert's
//  pairs run through MFMA tiles of 128 pairs against that expert's matrices.
//
//  * moe_sort      one workgroup: counts per expert, the pairs in expert order (`sorted`: the
//                  pair at a place, `place`: the place of a pair), and the list of tiles
//                  (expert, first place, places), their number in n_tiles[0].
//  * moe_grouped   grid (tile, columns): GATED: y[place, j] = act(gate, up) of the pair's token
//                  (rows of h gathered through `sorted`); else o[place, n] = down y[place] in
//                  32-bit.  A row's result depends on that row and the expert's matrix alone
//                  (sums along K in a fixed order), not on the rows beside it in the tile.
//  * moe_combine   out[t] (=, +=) sum over the slots, in slot order, of weight * o[place].
// =====================================================================================
#define MOE_TILE_ROWS 128

__global__ __launch_bounds__(1024) void moe_sort_kernel(
    const int* __restrict__ ids, int P, int E, int* __restrict__ sorted, int* __restrict__ place,
    int* __restrict__ tile_expert, int* __restrict__ tile_row0, int* __restrict__ tile_rows,
    int* __restrict__ n_tiles) {
  __shared__ int count[MOE_MAX_EXPERTS], start[MOE_MAX_EXPERTS], cursor[MOE_MAX_EXPERTS];
  for (int e = threadIdx.x; e < E; e += blockDim.x) { count[e] = 0; cursor[e] = 0; }
  __syncthreads();
  for (int i = threadIdx.x; i < P; i += blockDim.x) atomicAdd(&count[ids[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, tiles = 0;
    for (int e = 0; e < E; ++e) {
      start[e] = at;
      for (int r = 0; r < count[e]; r += MOE_TILE_ROWS) {
        tile_expert[tiles] = e;
        tile_row0[tiles] = at + r;
        tile_rows[tiles] = min(MOE_TILE_ROWS, count[e] - r);
        ++tiles;
      }
      at += count[e];
    }
    n_tiles[0] = tiles;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < P; i += blockDim.x) {
    const int e = ids[i];
    const int at = start[e] + atomicAdd(&cursor[e], 1);
    sorted[at] = i;
    place[i] = at;
  }
}

extern "C" int zf_moe_sort(const int* ids, int P, int E, int* sorted, int* place, int* tile_expert,
                           int* tile_row0, int* tile_rows, int* n_tiles, hipStream_t stream) {
  if (P <= 0) return 0;
  if (E <= 0 || E > MOE_MAX_EXPERTS) return -2;
  hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, stream, ids, P, E, sorted, place,
                     tile_expert, tile_row0, tile_rows, n_tiles);
  ZF_CHECK_LAUNCH();
}

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 moe_bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float moe_f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t moe_u32x4_t;

#define MOE_BK 64
#define MOE_LD (MOE_BK + 8)      // row stride in LDS (bfloat16): 16-byte reads of 8 lanes cover all banks

// 4 waves as 2 x 2: a wave takes 64 of the tile's 128 rows and 32 of the 64 columns of each of
// the two weight tiles (GATED: gate rows and up rows of the same 64 outputs; else two
// neighbouring groups of 64 outputs).  v_mfma_f32_32x32x16_bf16: a lane holds row (or column)
// lane % 32 and k 8 (lane / 32) .. + 8 of an operand, and of the result column lane % 32, rows
// 8 (r / 4) + 4 (lane / 32) + r % 4.
template <bool GATED>
__global__ __launch_bounds__(256) void moe_grouped_kernel(
    const bf16_t* __restrict__ a, long long lda, const int* __restrict__ sorted, int top,
    const bf16_t* __restrict__ w, const int* __restrict__ tile_expert,
    const int* __restrict__ tile_row0, const int* __restrict__ tile_rows,
    const int* __restrict__ n_tiles, void* __restrict__ out, int N, int K, float limit,
    float alpha, float shift) {
  __shared__ __attribute__((aligned(16))) bf16_t as[MOE_TILE_ROWS * MOE_LD];
  __shared__ __attribute__((aligned(16))) bf16_t bs[2 * 64 * MOE_LD];
  const int tile = blockIdx.x;
  if (tile >= n_tiles[0]) return;
  const int e = tile_expert[tile], row0 = tile_row0[tile], nrows = tile_rows[tile];
  const int c0 = blockIdx.y * (GATED ? 64 : 128);
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int wm = wave / 2, wn = wave % 2;

  // what this thread stages: rows tid / 8 + 32 i (i < 4) of the pairs' tile and of the two
  // weight tiles, 8 values at k0 + 8 (tid % 8)
  const int sr = tid / 8, sk = (tid % 8) * 8;
  const bf16_t* ap[4];
  const bf16_t* bp[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = sr + 32 * i;
    ap[i] = nullptr;
    if (r < nrows) {
      const int src = GATED ? sorted[row0 + r] / top : row0 + r;
      ap[i] = a + (size_t)src * lda;
    }
    const int br = r % 64, bt = r / 64;              // row of weight tile bt
    size_t wrow;
    bool ok;
    if (GATED) {
      ok = c0 + br < N;
      wrow = (size_t)e * 2 * N + (size_t)bt * N + c0 + br;
    } else {
      ok = c0 + bt * 64 + br < N;
      wrow = (size_t)e * N + c0 + bt * 64 + br;
    }
    bp[i] = ok ? w + wrow * K : nullptr;
  }
  moe_f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const moe_u32x4_t zero = {0u, 0u, 0u, 0u};
  moe_u32x4_t ra[4], rb[4];
  auto fetch = [&](int k0) {
    const bool in_k = k0 + sk < K;                   // K is a multiple of 8
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ra[i] = (ap[i] != nullptr && in_k) ? *(const moe_u32x4_t*)(ap[i] + k0 + sk) : zero;
      rb[i] = (bp[i] != nullptr && in_k) ? *(const moe_u32x4_t*)(bp[i] + k0 + sk) : zero;
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += MOE_BK) {
    __syncthreads();                                 // the tiles of the step before are done with
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      *(moe_u32x4_t*)(as + (sr + 32 * i) * MOE_LD + sk) = ra[i];
      *(moe_u32x4_t*)(bs + (sr + 32 * i) * MOE_LD + sk) = rb[i];
    }
    __syncthreads();
    if (k0 + MOE_BK < K) fetch(k0 + MOE_BK);         // in flight while the MFMAs run
#pragma unroll
    for (int ks = 0; ks < MOE_BK; ks += 16) {
      moe_bf16x8_t af[2], bf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
        af[i] = *(const moe_bf16x8_t*)(as + (wm * 64 + i * 32 + lane % 32) * MOE_LD + ks + 8 * (lane / 32));
#pragma unroll
      for (int j = 0; j < 2; ++j)
        bf[j] = *(const moe_bf16x8_t*)(bs + (j * 64 + wn * 32 + lane % 32) * MOE_LD + ks + 8 * (lane / 32));
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
  }
  const int col = wn * 32 + lane % 32;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = wm * 64 + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + r % 4;
      if (row >= nrows) continue;
      if (GATED) {
        if (c0 + col < N)
          ((bf16_t*)out)[(size_t)(row0 + row) * N + c0 + col] =
              float_to_bf16(gated_unit(acc[i][0][r], acc[i][1][r], limit, alpha, shift));
      } else {
#pragma unroll
        for (int j = 0; j < 2; ++j)
          if (c0 + j * 64 + col < N)
            ((float*)out)[(size_t)(row0 + row) * N + c0 + j * 64 + col] = acc[i][j][r];
      }
    }
}

// GATED: a = h [T, K] (rows gathered), w = gate_up [E, 2 N, K], out = y bfloat16 [P, N];
// else a = y [P, K], w = down [E, N, K], out = o float32 [P, N].  K a multiple of 8.
extern "C" int zf_moe_grouped(const void* a, long long lda, const int* sorted, int top,
                              const void* w, const int* tile_expert, const int* tile_row0,
                              const int* tile_rows, const int* n_tiles, void* out, int max_tiles,
                              int N, int K, int gated, float limit, float alpha, float shift,
                              hipStream_t stream) {
  if (max_tiles <= 0) return 0;
  if (N <= 0 || K <= 0 || K % 8 != 0 || top <= 0) return -2;
  if (gated)
    hipLaunchKernelGGL(moe_grouped_kernel<true>, dim3(max_tiles, (N + 63) / 64), dim3(256), 0,
                       stream, (const bf16_t*)a, lda, sorted, top, (const bf16_t*)w, tile_expert,
                       tile_row0, tile_rows, n_tiles, out, N, K, limit, alpha, shift);
  else
    hipLaunchKernelGGL(moe_grouped_kernel<false>, dim3(max_tiles, (N + 127) / 128), dim3(256), 0,
                       stream, (const bf16_t*)a, lda, sorted, top, (const bf16_t*)w, tile_expert,
                       tile_row0, tile_rows, n_tiles, out, N, K, limit, alpha, shift);
  ZF_CHECK_LAUNCH();
}

__global__ __launch_bounds__(256) void moe_combine_kernel(
    const float* __restrict__ o, const int* __restrict__ place, const float* __restrict__ weights,
    float* __restrict__ out, int W, int slots, int add) {
  const int t = blockIdx.x;
  for (int n = blockIdx.y * blockDim.x + threadIdx.x; n < W; n += gridDim.y * blockDim.x) {
    float total = 0.f;
    for (int s = 0; s < slots; ++s) {
      const int ts = t * slots + s;
      total += weights[ts] * o[(size_t)place[ts] * W + n];
    }
    float* dst = out + (size_t)t * W + n;
    *dst = add ? *dst + total : total;
  }
}

extern "C" int zf_moe_combine(const float* o, const int* place, const float* weights, float* out,
                              int T, int W, int slots, int add, hipStream_t stream) {
  if (T <= 0) return 0;
  if (W <= 0 || slots <= 0) return -2;
  int gy = (W + 255) / 256;
  if (gy > 64) gy = 64;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(T, gy), dim3(256), 0, stream, o, place, weights,
                     out, W, slots, add);
  ZF_CHECK_LAUNCH();
}
