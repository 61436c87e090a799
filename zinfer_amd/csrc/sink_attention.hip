// Causal grouped-query attention whose values are its keys, over a paged cache that holds the
// keys only, with an optional silent term in the soft-max and an optional output gate:
//
//   s_ij = scale * q_i . k_j          for max(0, i - window + 1) <= j <= i   (window 0: all)
//   a_ij = exp(s_ij) / (sink + sum_j exp(s_ij))        sink = 1: one more key of score 0 that
//                                                      brings no value; sink = 0: plain soft-max
//   o_i  = sum_j a_ij k_j,   then o_i * sigmoid(gate_i) element by element if a gate is given
//
// The key pool is laid out [page, kv head, row, hd]; token p of a sequence lies in page
// block_table[seq][p / page_size], row p % page_size.  Query head h reads kv head h / G.
//
//  * kv_rows_write: a step's key rows go from the rows of a product (any row stride, any
//    column offset) into the pool at slot_mapping.
//  * shared_kv_attention: one workgroup per (token, kv head, 16 query heads of its group), one
//    wave per query head.  The keys of a chunk are staged once in LDS as 32-bit numbers and
//    serve both products of all the group's heads.  Scores, weights and sums are 32-bit with
//    a running maximum; a token's result depends only on its own keys (the chunks start at
//    the first key it sees), never on how the batch was cut, so a prompt's portion and a
//    decoded token run the same arithmetic.  Any head size up to 512, any page size.
#include "zf_common.h"

template <typename T>
__global__ __launch_bounds__(256) void kv_rows_write_kernel(
    const T* __restrict__ src, long long row_stride, int col_offset,
    const int* __restrict__ slot_mapping, T* __restrict__ k_pool, int nKV, int hd,
    int page_size) {
  const int t = blockIdx.x;
  const int slot = slot_mapping[t];
  if (slot < 0) return;
  const int page = slot / page_size, r = slot % page_size;
  const T* s = src + (size_t)t * row_stride + col_offset;
  for (int i = threadIdx.x; i < nKV * hd; i += blockDim.x) {
    const int kvh = i / hd, d = i % hd;
    k_pool[(((size_t)page * nKV + kvh) * page_size + r) * hd + d] = s[i];
  }
}

extern "C" int zf_kv_rows_write(const void* src, int dtype, long long row_stride, int col_offset,
                                const int* slot_mapping, void* k_pool, int T, int nKV, int hd,
                                int page_size, hipStream_t stream) {
  if (T <= 0) return 0;
  if (nKV <= 0 || hd <= 0 || page_size <= 0) return -2;
  if (dtype == ZF_F32)
    hipLaunchKernelGGL(kv_rows_write_kernel<float>, dim3(T), dim3(256), 0, stream,
                       (const float*)src, row_stride, col_offset, slot_mapping, (float*)k_pool,
                       nKV, hd, page_size);
  else
    hipLaunchKernelGGL(kv_rows_write_kernel<bf16_t>, dim3(T), dim3(256), 0, stream,
                       (const bf16_t*)src, row_stride, col_offset, slot_mapping, (bf16_t*)k_pool,
                       nKV, hd, page_size);
  ZF_CHECK_LAUNCH();
}

#define SKA_MAX_WAVES 16

// keys staged per chunk: the tile [chunk][hd + 1] of floats stays within 33 KB
__host__ __device__ static inline int ska_chunk(int hd) { return hd <= 128 ? 64 : hd <= 256 ? 32 : 16; }

template <typename T>
__global__ __launch_bounds__(SKA_MAX_WAVES * ZF_WAVE) void shared_kv_attention_kernel(
    const T* __restrict__ q, long long q_stride, const T* __restrict__ gate,
    long long gate_stride, const T* __restrict__ k_pool, const int* __restrict__ block_table,
    const int* __restrict__ q_start, const int* __restrict__ ctx_len,
    const int* __restrict__ seq_index, T* __restrict__ out, float scale, int window, int sink,
    int nH, int nKV, int hd, int page_size, int max_pages) {
  extern __shared__ float smem[];
  const int KC = ska_chunk(hd);
  const int ld = hd + 1;                          // odd row stride: a lane per key, no conflicts
  const int n_waves = blockDim.x / ZF_WAVE;
  float* ks = smem;                               // [KC][ld]
  float* qs = ks + KC * ld;                       // [n_waves][hd]
  float* ps = qs + n_waves * hd;                  // [n_waves][ZF_WAVE]
  int* rows = (int*)(ps + n_waves * ZF_WAVE);     // [KC]: row of each key in the pool, or -1

  const int t = blockIdx.x, kvh = blockIdx.y;
  const int G = nH / nKV;
  const int wave = threadIdx.x / ZF_WAVE, lane = threadIdx.x % ZF_WAVE;
  const int g = blockIdx.z * SKA_MAX_WAVES + wave;      // this wave's head within the group
  const bool live = g < G;
  const int h = kvh * G + (live ? g : 0);
  const int s = seq_index[t];
  const int q_len = q_start[s + 1] - q_start[s];
  const int pos = ctx_len[s] - q_len + (t - q_start[s]);
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int* table = block_table + (size_t)s * max_pages;

  const T* qrow = q + (size_t)t * q_stride + (size_t)h * hd;
  float* qw = qs + wave * hd;
  for (int i = lane; i < hd; i += ZF_WAVE) qw[i] = load_as_float<T>(qrow + i);

  // a lane owns the output elements d = lane, lane + 64, ... (up to 8: hd <= 512)
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  // the silent term is a key of score 0 that is there before the first real one
  float m = sink ? 0.f : -INFINITY, l = sink ? 1.f : 0.f;

  for (int base = lo; base <= pos; base += KC) {
    const int nk = min(KC, pos - base + 1);
    __syncthreads();                               // the tile of the chunk before is done with
    if ((int)threadIdx.x < KC) {
      const int key = base + threadIdx.x;
      rows[threadIdx.x] = key <= pos
          ? (table[key / page_size] * nKV + kvh) * page_size + key % page_size : -1;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nk * hd; i += blockDim.x) {
      const int j = i / hd, d = i % hd;
      ks[j * ld + d] = load_as_float<T>(k_pool + (size_t)rows[j] * hd + d);
    }
    __syncthreads();
    float sc = -INFINITY;
    if (lane < nk) {
      const float* kr = ks + lane * ld;
      float dot = 0.f;
      for (int d = 0; d < hd; ++d) dot = fmaf(qw[d], kr[d], dot);
      sc = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(sc));
    const float corr = expf(m - m_new);            // exp(-inf) = 0 on a first chunk without sink
    const float p = lane < nk ? expf(sc - m_new) : 0.f;
    l = l * corr + wave_sum(p);
    m = m_new;
    ps[wave * ZF_WAVE + lane] = p;                 // read back by this wave only
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] *= corr;
    const float* pw = ps + wave * ZF_WAVE;
    for (int j = 0; j < nk; ++j) {
      const float pj = pw[j];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int d = lane + i * ZF_WAVE;
        if (d < hd) acc[i] = fmaf(pj, ks[j * ld + d], acc[i]);
      }
    }
  }
  if (!live) return;
  const float inv = 1.0f / l;
  T* orow = out + ((size_t)t * nH + h) * hd;
  const T* grow = gate != nullptr ? gate + (size_t)t * gate_stride + (size_t)h * hd : nullptr;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int d = lane + i * ZF_WAVE;
    if (d < hd) {
      float v = acc[i] * inv;
      if (grow != nullptr) v *= 1.0f / (1.0f + expf(-load_as_float<T>(grow + d)));
      store_from_float<T>(orow + d, v);
    }
  }
}

extern "C" int zf_shared_kv_attention(const void* q, long long q_stride, const void* gate,
                                      long long gate_stride, const void* k_pool, int dtype,
                                      const int* block_table, const int* q_start,
                                      const int* ctx_len, const int* seq_index, void* out,
                                      float scale, int window, int sink, int T, int nH, int nKV,
                                      int hd, int page_size, int max_pages, hipStream_t stream) {
  if (T <= 0) return 0;
  if (hd <= 0 || hd > 512 || nKV <= 0 || nH % nKV != 0 || page_size <= 0) return -2;
  const int G = nH / nKV;
  const int n_waves = G < SKA_MAX_WAVES ? G : SKA_MAX_WAVES;
  const int KC = ska_chunk(hd);
  dim3 grid(T, nKV, (G + SKA_MAX_WAVES - 1) / SKA_MAX_WAVES);
  const size_t smem = ((size_t)KC * (hd + 1) + (size_t)n_waves * hd + (size_t)n_waves * ZF_WAVE
                       + KC) * sizeof(float);
  if (smem > 64 * 1024) return -3;
  if (dtype == ZF_F32)
    hipLaunchKernelGGL(shared_kv_attention_kernel<float>, grid, dim3(n_waves * ZF_WAVE), smem,
                       stream, (const float*)q, q_stride, (const float*)gate, gate_stride,
                       (const float*)k_pool, block_table, q_start, ctx_len, seq_index,
                       (float*)out, scale, window, sink, nH, nKV, hd, page_size, max_pages);
  else
    hipLaunchKernelGGL(shared_kv_attention_kernel<bf16_t>, grid, dim3(n_waves * ZF_WAVE), smem,
                       stream, (const bf16_t*)q, q_stride, (const bf16_t*)gate, gate_stride,
                       (const bf16_t*)k_pool, block_table, q_start, ctx_len, seq_index,
                       (bf16_t*)out, scale, window, sink, nH, nKV, hd, page_size, max_pages);
  ZF_CHECK_LAUNCH();
}
