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

// =====================================================================================
//  bfloat16 MFMA kernel (head sizes 32, 64, 96, 128, 192, 256; up to 128 query heads per kv
//  head).  A workgroup takes one kv head and a tile of query positions of one sequence: its
//  128 rows are (position, head of the group) pairs, 32 to a wave.  Keys come in chunks of 32,
//  staged once in LDS in two forms, [key][d] and [d][key], and serve both products of all
//  rows.  As in the other attention kernels the score tile is computed transposed,
//  S^T = K Q^T (v_mfma_f32_32x32x16_bf16), so that a lane's 16 scores belong to one row and
//  the soft-max runs in registers in 32-bit; the second product O^T = K^T P^T takes the
//  weights from those registers as they lie.  Each weight enters it as the sum of two
//  bfloat16 numbers (its rounding and the rounding of what that leaves), so what the weights
//  lose against 32 bits is below 2^-16 of each; the running maximum, the sums and the
//  accumulators are 32-bit.  With n_splits > 1 (few rows, long contexts: decoding) a
//  workgroup takes one range of the keys and leaves an un-normalised partial result that
//  tied_attention_merge_kernel combines in split order; the silent term belongs to split 0.
// =====================================================================================
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 ta_bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float ta_f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t ta_u32x4_t;

#define TA_ROWS 128
#define TA_KEYS 32

// where key j of row d lies in the [d][key] tile: the row's eight groups of four keys are
// permuted by the row's group of eight, so that the lanes that write one key of 16 groups of
// rows (and those that read four keys of 32 rows) spread over the banks
// 2^x for x <= 0 as the bare instruction (-inf gives 0)
__device__ __forceinline__ float ta_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ int ta_swz(int j, int d) { return (((j >> 2) ^ ((d >> 3) & 7)) << 2) | (j & 3); }

template <int HD>
__global__ __launch_bounds__(256) void tied_attention_mfma_kernel(
    const bf16_t* __restrict__ q, long long q_stride, const bf16_t* __restrict__ gate,
    long long gate_stride, const bf16_t* __restrict__ k_pool, const int* __restrict__ block_table,
    const int* __restrict__ q_start, const int* __restrict__ ctx_len, bf16_t* __restrict__ out,
    float* __restrict__ ws_o, float* __restrict__ ws_ml, float scale, int window, int sink,
    int n_seqs, int nH, int nKV, int page_size, int max_pages, int QT, int n_splits,
    int split_keys) {
  constexpr int LDK = HD + 8;              // [key][d]: 16-byte reads of 8 lanes cover all banks
  constexpr int LDT = TA_KEYS + 4;         // [d][key]
  constexpr int CH = TA_KEYS * HD / 8;     // 16-byte pieces of a chunk of keys
  constexpr int PER = (CH + 255) / 256;
  __shared__ __attribute__((aligned(16))) bf16_t ks[TA_KEYS * LDK];
  __shared__ __attribute__((aligned(16))) bf16_t kt[HD * LDT];

  // which sequence and which of its tiles of QT positions this workgroup has
  int s = 0, tile = blockIdx.x;
  for (; s < n_seqs; ++s) {
    const int n = (q_start[s + 1] - q_start[s] + QT - 1) / QT;
    if (tile < n) break;
    tile -= n;
  }
  if (s >= n_seqs) return;
  const int kvh = blockIdx.y, split = blockIdx.z;
  const int G = nH / nKV;
  const int q_len = q_start[s + 1] - q_start[s];
  const int first = tile * QT;
  const int npos = min(QT, q_len - first);
  const int pos0 = ctx_len[s] - q_len + first;
  const int nrows = npos * G;
  const int* table = block_table + (size_t)s * max_pages;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int c = lane % 32, hl = lane / 32;

  // this lane's row: a (position, head) pair; both halves of the wave hold the same rows
  const int row = wave * 32 + c;
  const bool row_ok = row < nrows;
  const int qi = row_ok ? row / G : 0, g = row_ok ? row % G : 0;
  const int h = kvh * G + g;
  const int tok = q_start[s] + first + qi;
  const int pos_r = pos0 + qi;
  const int lo_r = (window > 0 && pos_r - window + 1 > 0) ? pos_r - window + 1 : 0;
  const bool wave_on = wave * 32 < nrows;

  ta_bf16x8_t qf[HD / 16];
  {
    const bf16_t* qrow = q + (size_t)tok * q_stride + (size_t)h * HD;
#pragma unroll
    for (int i = 0; i < HD / 16; ++i) {
      ta_u32x4_t v = {0u, 0u, 0u, 0u};
      if (row_ok) v = *(const ta_u32x4_t*)(qrow + 16 * i + 8 * hl);
      qf[i] = *(const ta_bf16x8_t*)&v;
    }
  }
  ta_f32x16_t acc[HD / 32];
#pragma unroll
  for (int i = 0; i < HD / 32; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  // scores are kept times log2(e), so that every weight is one v_exp_f32; the silent term's
  // score 0 stays 0
  const float scale_log2 = scale * 1.4426950408889634f;
  const bool has_sink = sink && split == 0;
  float m = has_sink ? 0.f : -INFINITY, l = has_sink ? 1.f : 0.f;

  // the keys any row of the tile sees, from a multiple of 32 on; this split's part of them
  const int k_first = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
  const int k_last = pos0 + npos - 1;
  int k_begin = k_first / TA_KEYS * TA_KEYS, k_end = k_last + 1;
  if (n_splits > 1) {
    k_begin += split * split_keys;
    k_end = min(k_end, k_begin + split_keys);
  }

  // three chunks of keys are on their way from memory at any time: a workgroup is alone on its
  // CU when a prompt has few tiles, so nothing else hides that latency
  ta_u32x4_t st0[PER], st1[PER], st2[PER];
  auto fetch = [&](ta_u32x4_t (&stage)[PER], int base) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int ci = tid + i * 256;
      ta_u32x4_t v = {0u, 0u, 0u, 0u};
      if (ci < CH) {
        const int key = base + ci / (HD / 8);
        // (a chunk starts at a multiple of 32: the keys of its first chunk that lie before
        // the window may be on a page that has gone back, whose table entry is no page)
        if (key >= k_first && key <= k_last) {
          const size_t prow = ((size_t)table[key / page_size] * nKV + kvh) * page_size + key % page_size;
          v = *(const ta_u32x4_t*)(k_pool + prow * HD + (ci % (HD / 8)) * 8);
        }
      }
      stage[i] = v;
    }
  };
  auto chunk = [&](ta_u32x4_t (&stage)[PER], int base) {
    __syncthreads();                               // the chunk before is done with
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int ci = tid + i * 256;
      if (ci < CH) {
        const int j = ci / (HD / 8), d0 = (ci % (HD / 8)) * 8;
        *(ta_u32x4_t*)(ks + j * LDK + d0) = stage[i];
        const bf16_t* e = (const bf16_t*)&stage[i];
#pragma unroll
        for (int x = 0; x < 8; ++x) kt[(d0 + x) * LDT + ta_swz(j, d0)] = e[x];
      }
    }
    __syncthreads();
    if (base + 3 * TA_KEYS < k_end) fetch(stage, base + 3 * TA_KEYS);
    if (!wave_on) return;
    // S^T = K Q^T: this lane gets, for its row, the keys base + 8 (r / 4) + 4 hl + r % 4
    ta_f32x16_t sc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sc[r] = 0.f;
#pragma unroll
    for (int i = 0; i < HD / 16; ++i) {
      const ta_bf16x8_t kf = *(const ta_bf16x8_t*)(ks + c * LDK + 16 * i + 8 * hl);
      sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[i], sc, 0, 0, 0);
    }
    float cmax = -INFINITY;
    // a chunk that every row of the wave sees whole needs no mask
    const bool whole = row_ok && base >= lo_r && base + TA_KEYS - 1 <= pos_r;
    if (__all(whole)) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        sc[r] *= scale_log2;
        cmax = fmaxf(cmax, sc[r]);
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = base + 8 * (r / 4) + 4 * hl + r % 4;
        const bool seen = row_ok && key <= pos_r && key >= lo_r;
        sc[r] = seen ? sc[r] * scale_log2 : -INFINITY;
        cmax = fmaxf(cmax, sc[r]);
      }
    }
    cmax = fmaxf(cmax, __shfl_xor(cmax, 32, 64));
    const float m_new = fmaxf(m, cmax);
    // nothing seen yet (and no silent term): every weight below is exp(-inf) = 0
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float corr = ta_exp2(m - m_use);
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      sc[r] = ta_exp2(sc[r] - m_use);
      psum += sc[r];
    }
    psum += __shfl_xor(psum, 32, 64);
    l = l * corr + psum;
    m = m_new;
    if (__any(corr != 1.0f)) {                     // (the maximum of some row moved)
#pragma unroll
      for (int i = 0; i < HD / 32; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] *= corr;
    }
    // O^T += K^T P^T over the chunk's two groups of 16 keys; the registers 8 t .. 8 t + 7 hold
    // the weights of the keys 16 t + {0..3, 8..11} + 4 hl, and K^T is read in that same order
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      ta_bf16x8_t p_hi, p_lo;
#pragma unroll
      for (int x = 0; x < 8; ++x) {
        const float p = sc[8 * t + x];
        const __bf16 hi = (__bf16)p;
        p_hi[x] = hi;
        p_lo[x] = (__bf16)(p - (float)hi);
      }
#pragma unroll
      for (int i = 0; i < HD / 32; ++i) {
        const bf16_t* src = kt + (i * 32 + c) * LDT;
        const uint2 a0 = *(const uint2*)(src + ta_swz(16 * t + 4 * hl, i * 32 + c));
        const uint2 a1 = *(const uint2*)(src + ta_swz(16 * t + 8 + 4 * hl, i * 32 + c));
        ta_u32x4_t av = {a0.x, a0.y, a1.x, a1.y};
        const ta_bf16x8_t vf = *(const ta_bf16x8_t*)&av;
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, p_hi, acc[i], 0, 0, 0);
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, p_lo, acc[i], 0, 0, 0);
      }
    }
  };
  if (k_begin < k_end) fetch(st0, k_begin);
  if (k_begin + TA_KEYS < k_end) fetch(st1, k_begin + TA_KEYS);
  if (k_begin + 2 * TA_KEYS < k_end) fetch(st2, k_begin + 2 * TA_KEYS);
  for (int base = k_begin; base < k_end; base += 3 * TA_KEYS) {
    chunk(st0, base);
    if (base + TA_KEYS < k_end) chunk(st1, base + TA_KEYS);
    if (base + 2 * TA_KEYS < k_end) chunk(st2, base + 2 * TA_KEYS);
  }
  if (!row_ok) return;
  // acc[i][r] is element d = 32 i + 8 (r / 4) + 4 hl + r % 4 of this lane's row
  if (n_splits > 1) {
    const size_t slot = ((size_t)tok * nH + h) * n_splits + split;
    float* po = ws_o + slot * HD;
#pragma unroll
    for (int i = 0; i < HD / 32; ++i)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4)
        *(float4*)(po + 32 * i + 8 * r4 + 4 * hl) = make_float4(acc[i][4 * r4], acc[i][4 * r4 + 1],
                                                                acc[i][4 * r4 + 2], acc[i][4 * r4 + 3]);
    if (hl == 0) {
      ws_ml[2 * slot] = m;
      ws_ml[2 * slot + 1] = l;
    }
    return;
  }
  const float inv = 1.0f / l;
  bf16_t* orow = out + ((size_t)tok * nH + h) * HD;
  const bf16_t* grow = gate != nullptr ? gate + (size_t)tok * gate_stride + (size_t)h * HD : nullptr;
#pragma unroll
  for (int i = 0; i < HD / 32; ++i)
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      const int d = 32 * i + 8 * r4 + 4 * hl;
      float v[4];
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        v[x] = acc[i][4 * r4 + x] * inv;
        if (grow != nullptr) v[x] *= 1.0f / (1.0f + expf(-bf16_to_float(grow[d + x])));
      }
      *(uint2*)(orow + d) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
    }
}

// ---------------------------------------------------------------- decode: one token a sequence
// Grid (sequence, kv head, split); every wave of a workgroup is a split of its own: wave w of
// workgroup z takes the keys [first + (4 z + w) * wave_keys, + wave_keys) of the context (first:
// the window's first key, down to a multiple of 32), in chunks of 32.  The token's G rows (its
// query heads of this kv head) are the first G of the 32 columns.  A lane loads the 8 values of
// its key that its operand of S^T = K Q^T needs straight from the pool (every value of the
// chunk exactly once in the wave), and writes them transposed into the wave's own LDS tile
// for O^T = K^T P^T: no barrier between waves anywhere.  Each wave leaves an un-normalised
// partial (maximum, sum, O) for tied_attention_merge_kernel; the silent term belongs to the
// first wave of the first workgroup.
template <int HD, bool DECODE>
__global__ __launch_bounds__(256, 2) void tied_attention_wave_kernel(
    const bf16_t* __restrict__ q, long long q_stride, const bf16_t* __restrict__ gate,
    long long gate_stride, const bf16_t* __restrict__ k_pool, const int* __restrict__ block_table,
    const int* __restrict__ q_start, const int* __restrict__ ctx_len, bf16_t* __restrict__ out,
    float* __restrict__ ws_o, float* __restrict__ ws_ml, float scale, int window, int sink,
    int n_seqs, int nH, int nKV, int page_size, int max_pages, int QT, int wave_keys) {
  constexpr int LDT = TA_KEYS + 4;
  __shared__ __attribute__((aligned(16))) bf16_t kt_all[4 * HD * LDT];
  const int kvh = blockIdx.y;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int c = lane % 32, hl = lane / 32;
  bf16_t* kt = kt_all + wave * HD * LDT;
  const int G = nH / nKV;

  // the wave's 32 rows: (position, head of the group) pairs of one sequence
  int s, tok, pos_r, lo_r, h, split = 0, n_splits = 1;
  int k_first, k_end;          // the keys the wave walks: [k_first down to a multiple of 32, k_end)
  bool row_ok;
  if constexpr (DECODE) {
    // one token a sequence; the workgroup's four waves are four splits of its context
    s = blockIdx.x;
    split = blockIdx.z * 4 + wave;
    n_splits = gridDim.z * 4;
    row_ok = c < G;
    h = kvh * G + (row_ok ? c : 0);
    tok = s;
    pos_r = ctx_len[s] - 1;
    lo_r = (window > 0 && pos_r - window + 1 > 0) ? pos_r - window + 1 : 0;
    k_first = lo_r;
    k_end = pos_r + 1;
  } else {
    // a tile of QT positions of a sequence; the four waves take 32 rows each, and with
    // gridDim.z > 1 the z-th part of their keys (a prompt's last rows see the most keys and
    // its first the fewest: parts even out what the waves have to do, and let a SIMD hold two)
    split = blockIdx.z;
    n_splits = gridDim.z;
    s = 0;
    int tile = blockIdx.x;
    for (; s < n_seqs; ++s) {
      const int n = (q_start[s + 1] - q_start[s] + QT - 1) / QT;
      if (tile < n) break;
      tile -= n;
    }
    if (s >= n_seqs) return;
    const int q_len = q_start[s + 1] - q_start[s];
    const int first = tile * QT;
    const int npos = min(QT, q_len - first);
    const int nrows = npos * G;
    if (wave * 32 >= nrows) return;                // (no barrier follows: waves are on their own)
    const int pos0 = ctx_len[s] - q_len + first;
    const int row = wave * 32 + c;
    row_ok = row < nrows;
    const int qi = row_ok ? row / G : 0;
    h = kvh * G + (row_ok ? row % G : 0);
    tok = q_start[s] + first + qi;
    pos_r = pos0 + qi;
    lo_r = (window > 0 && pos_r - window + 1 > 0) ? pos_r - window + 1 : 0;
    const int p_lo = pos0 + (wave * 32) / G;                       // the wave's first position
    const int p_hi = pos0 + (min(nrows, wave * 32 + 32) - 1) / G;  // and its last
    k_first = (window > 0 && p_lo - window + 1 > 0) ? p_lo - window + 1 : 0;
    k_end = p_hi + 1;
  }
  const int* table = block_table + (size_t)s * max_pages;

  ta_bf16x8_t qf[HD / 16];
  {
    const bf16_t* qrow = q + (size_t)tok * q_stride + (size_t)h * HD;
#pragma unroll
    for (int i = 0; i < HD / 16; ++i) {
      ta_u32x4_t v = {0u, 0u, 0u, 0u};
      if (row_ok) v = *(const ta_u32x4_t*)(qrow + 16 * i + 8 * hl);
      qf[i] = *(const ta_bf16x8_t*)&v;
    }
  }
  ta_f32x16_t acc[HD / 32];
#pragma unroll
  for (int i = 0; i < HD / 32; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  const float scale_log2 = scale * 1.4426950408889634f;
  const bool has_sink = sink && split == 0;
  float m = has_sink ? 0.f : -INFINITY, l = has_sink ? 1.f : 0.f;

  int k_begin = k_first / TA_KEYS * TA_KEYS;
  if constexpr (DECODE) {
    k_begin += split * wave_keys;
    k_end = min(k_end, k_begin + wave_keys);
  } else if (n_splits > 1) {
    const int share = (k_end - k_begin + n_splits * TA_KEYS - 1) / (n_splits * TA_KEYS) * TA_KEYS;
    k_begin += split * share;
    k_end = min(k_end, k_begin + share);
  }

  // this lane's key of a chunk: key base + c, values 16 i + 8 hl .. + 8 of it for every i
  ta_u32x4_t kf[HD / 16], kn[HD / 16];
  auto fetch = [&](ta_u32x4_t (&dst)[HD / 16], int base) {
    const int key = base + c;
    const bool ok = key >= k_first && key < k_end;
    size_t prow = 0;
    if (ok) prow = ((size_t)table[key / page_size] * nKV + kvh) * page_size + key % page_size;
#pragma unroll
    for (int i = 0; i < HD / 16; ++i) {
      ta_u32x4_t v = {0u, 0u, 0u, 0u};
      if (ok) v = *(const ta_u32x4_t*)(k_pool + prow * HD + 16 * i + 8 * hl);
      dst[i] = v;
    }
  };
  if (k_begin < k_end) fetch(kf, k_begin);
  for (int base = k_begin; base < k_end; base += TA_KEYS) {
    if (base + TA_KEYS < k_end) fetch(kn, base + TA_KEYS);      // in flight while this chunk runs
    ta_f32x16_t sc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sc[r] = 0.f;
#pragma unroll
    for (int i = 0; i < HD / 16; ++i)
      sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const ta_bf16x8_t*)&kf[i], qf[i], sc, 0, 0, 0);
    // the chunk transposed into the wave's tile
#pragma unroll
    for (int i = 0; i < HD / 16; ++i) {
      const bf16_t* e = (const bf16_t*)&kf[i];
#pragma unroll
      for (int x = 0; x < 8; ++x)
        kt[(16 * i + 8 * hl + x) * LDT + ta_swz(c, 16 * i + 8 * hl)] = e[x];
    }
    float cmax = -INFINITY;
    // a chunk that every row of the wave sees whole needs no mask
    const bool whole = row_ok && base >= lo_r && base + TA_KEYS - 1 <= pos_r &&
                       base >= k_first && base + TA_KEYS <= k_end;
    if (__all(whole)) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        sc[r] *= scale_log2;
        cmax = fmaxf(cmax, sc[r]);
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = base + 8 * (r / 4) + 4 * hl + r % 4;
        const bool seen = row_ok && key >= lo_r && key <= pos_r && key >= k_first && key < k_end;
        sc[r] = seen ? sc[r] * scale_log2 : -INFINITY;
        cmax = fmaxf(cmax, sc[r]);
      }
    }
    cmax = fmaxf(cmax, __shfl_xor(cmax, 32, 64));
    const float m_new = fmaxf(m, cmax);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float corr = ta_exp2(m - m_use);
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      sc[r] = ta_exp2(sc[r] - m_use);
      psum += sc[r];
    }
    psum += __shfl_xor(psum, 32, 64);
    l = l * corr + psum;
    m = m_new;
    if (__any(corr != 1.0f)) {
#pragma unroll
      for (int i = 0; i < HD / 32; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] *= corr;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();               // the wave's transposed tile is written
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      ta_bf16x8_t p_hi, p_lo;
#pragma unroll
      for (int x = 0; x < 8; ++x) {
        const float p = sc[8 * t + x];
        const __bf16 hi = (__bf16)p;
        p_hi[x] = hi;
        p_lo[x] = (__bf16)(p - (float)hi);
      }
#pragma unroll
      for (int i = 0; i < HD / 32; ++i) {
        const bf16_t* src = kt + (i * 32 + c) * LDT;
        const uint2 a0 = *(const uint2*)(src + ta_swz(16 * t + 4 * hl, i * 32 + c));
        const uint2 a1 = *(const uint2*)(src + ta_swz(16 * t + 8 + 4 * hl, i * 32 + c));
        ta_u32x4_t av = {a0.x, a0.y, a1.x, a1.y};
        const ta_bf16x8_t vf = *(const ta_bf16x8_t*)&av;
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, p_hi, acc[i], 0, 0, 0);
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, p_lo, acc[i], 0, 0, 0);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    __builtin_amdgcn_wave_barrier();               // the tile is read before it is written again
#pragma unroll
    for (int i = 0; i < HD / 16; ++i) kf[i] = kn[i];
  }
  if (!row_ok) return;
  // acc[i][r] is element d = 32 i + 8 (r / 4) + 4 hl + r % 4 of this lane's row
  if (DECODE || n_splits > 1) {
    const size_t slot = ((size_t)tok * nH + h) * n_splits + split;
    float* po = ws_o + slot * HD;
#pragma unroll
    for (int i = 0; i < HD / 32; ++i)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4)
        *(float4*)(po + 32 * i + 8 * r4 + 4 * hl) = make_float4(acc[i][4 * r4], acc[i][4 * r4 + 1],
                                                                acc[i][4 * r4 + 2], acc[i][4 * r4 + 3]);
    if (hl == 0) {
      ws_ml[2 * slot] = m;
      ws_ml[2 * slot + 1] = l;
    }
  } else {
    const float inv = 1.0f / l;
    bf16_t* orow = out + ((size_t)tok * nH + h) * HD;
    const bf16_t* grow = gate != nullptr ? gate + (size_t)tok * gate_stride + (size_t)h * HD : nullptr;
#pragma unroll
    for (int i = 0; i < HD / 32; ++i)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        const int d = 32 * i + 8 * r4 + 4 * hl;
        float v[4];
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          v[x] = acc[i][4 * r4 + x] * inv;
          if (grow != nullptr) v[x] *= 1.0f / (1.0f + expf(-bf16_to_float(grow[d + x])));
        }
        *(uint2*)(orow + d) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
      }
  }
}

#define TA_WAVE_LAUNCH(HD, DEC)                                                                   \
  case HD:                                                                                       \
    hipLaunchKernelGGL((tied_attention_wave_kernel<HD, DEC>), grid, dim3(256), 0, stream,        \
                       (const bf16_t*)q, q_stride, (const bf16_t*)gate, gate_stride,             \
                       (const bf16_t*)k_pool, block_table, q_start, ctx_len, (bf16_t*)out, ws_o, \
                       ws_ml, scale, window, sink, n_seqs, nH, nKV, page_size, max_pages, QT,    \
                       wave_keys);                                                               \
    break;

// one wave per (token, head): the splits' partials in split order (their maxima are scores
// times log2(e)), then the gate
__global__ __launch_bounds__(ZF_WAVE) void tied_attention_merge_kernel(
    const float* __restrict__ ws_o, const float* __restrict__ ws_ml,
    const bf16_t* __restrict__ gate, long long gate_stride, bf16_t* __restrict__ out, int nH,
    int hd, int n_splits) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const size_t slot0 = ((size_t)t * nH + h) * n_splits;
  // lane z holds split z's maximum and sum (at most 64 splits); a split without keys has the
  // maximum -inf and counts for nothing
  float mz = -INFINITY, lz = 0.f;
  if (lane < n_splits) {
    mz = ws_ml[2 * (slot0 + lane)];
    lz = ws_ml[2 * (slot0 + lane) + 1];
  }
  const float M = wave_max(mz);
  __shared__ float w[ZF_WAVE], lw[ZF_WAVE];
  w[lane] = mz == -INFINITY ? 0.f : exp2f(mz - M);
  lw[lane] = lz * w[lane];
  __syncthreads();
  // the sums in split order
  float L = 0.f;
  for (int z = 0; z < n_splits; ++z) L += lw[z];
  const float inv = 1.0f / L;
  for (int d = lane; d < hd; d += ZF_WAVE) {
    float o = 0.f;
    for (int z = 0; z < n_splits; ++z) o += ws_o[(slot0 + z) * hd + d] * w[z];
    o *= inv;
    if (gate != nullptr)
      o *= 1.0f / (1.0f + expf(-bf16_to_float(gate[(size_t)t * gate_stride + (size_t)h * hd + d])));
    out[((size_t)t * nH + h) * hd + d] = float_to_bf16(o);
  }
}

#define TA_LAUNCH(HD)                                                                            \
  case HD:                                                                                       \
    hipLaunchKernelGGL(tied_attention_mfma_kernel<HD>, grid, dim3(256), 0, stream,               \
                       (const bf16_t*)q, q_stride, (const bf16_t*)gate, gate_stride,             \
                       (const bf16_t*)k_pool, block_table, q_start, ctx_len, (bf16_t*)out, ws_o, \
                       ws_ml, scale, window, sink, n_seqs, nH, nKV, page_size, max_pages, QT,    \
                       n_splits, split_keys);                                                    \
    break;

// n_tiles: an upper bound of the tiles of QT = max(1, 128 / G) positions over all sequences
// (workgroups beyond the real number leave at once).  n_splits > 1: ws_o [T * nH * n_splits *
// hd] and ws_ml [T * nH * n_splits * 2] floats; split_keys a multiple of 32.
extern "C" int zf_tied_attention_mfma(const void* q, long long q_stride, const void* gate,
                                      long long gate_stride, const void* k_pool,
                                      const int* block_table, const int* q_start,
                                      const int* ctx_len, void* out, float* ws_o, float* ws_ml,
                                      float scale, int window, int sink, int T, int n_seqs,
                                      int n_tiles, int nH, int nKV, int hd, int page_size,
                                      int max_pages, int n_splits, int split_keys,
                                      hipStream_t stream) {
  if (T <= 0 || n_tiles <= 0) return 0;
  if (nKV <= 0 || nH % nKV != 0 || nH / nKV > TA_ROWS || page_size <= 0 || n_splits < 1 ||
      n_splits > ZF_WAVE ||
      (n_splits > 1 && (split_keys <= 0 || split_keys % TA_KEYS != 0 || !ws_o || !ws_ml)))
    return -2;
  const int G = nH / nKV;
  const int QT = TA_ROWS / G;
  dim3 grid(n_tiles, nKV, n_splits);
  switch (hd) {
    TA_LAUNCH(32) TA_LAUNCH(64) TA_LAUNCH(96) TA_LAUNCH(128) TA_LAUNCH(192) TA_LAUNCH(256)
    default: return -3;
  }
  if (n_splits > 1)
    hipLaunchKernelGGL(tied_attention_merge_kernel, dim3(T, nH), dim3(ZF_WAVE), 0, stream, ws_o,
                       ws_ml, (const bf16_t*)gate, gate_stride, (bf16_t*)out, nH, hd, n_splits);
  ZF_CHECK_LAUNCH();
}

// A step in which every sequence brings one token (token s is sequence s's): n_blocks
// workgroups a (sequence, kv head), every wave a split of wave_keys keys (a multiple of 32);
// ws_o [n_seqs * nH * 4 n_blocks * hd], ws_ml [n_seqs * nH * 4 n_blocks * 2] floats;
// 4 n_blocks <= 64; at most 32 query heads a kv head; head sizes up to 128 (the wave's tile and
// operands in registers).
extern "C" int zf_tied_attention_decode(const void* q, long long q_stride, const void* gate,
                                        long long gate_stride, const void* k_pool,
                                        const int* block_table, const int* ctx_len, void* out,
                                        float* ws_o, float* ws_ml, float scale, int window,
                                        int sink, int n_seqs, int nH, int nKV, int hd,
                                        int page_size, int max_pages, int n_blocks, int wave_keys,
                                        hipStream_t stream) {
  if (n_seqs <= 0) return 0;
  if (nKV <= 0 || nH % nKV != 0 || nH / nKV > 32 || page_size <= 0 || n_blocks < 1 ||
      4 * n_blocks > ZF_WAVE || wave_keys <= 0 || wave_keys % TA_KEYS != 0 || !ws_o || !ws_ml)
    return -2;
  dim3 grid(n_seqs, nKV, n_blocks);
  const int* q_start = nullptr;
  const int QT = 1;
  switch (hd) {
    TA_WAVE_LAUNCH(32, true) TA_WAVE_LAUNCH(64, true) TA_WAVE_LAUNCH(96, true)
    TA_WAVE_LAUNCH(128, true)
    default: return -3;
  }
  hipLaunchKernelGGL(tied_attention_merge_kernel, dim3(n_seqs, nH), dim3(ZF_WAVE), 0, stream,
                     ws_o, ws_ml, (const bf16_t*)gate, gate_stride, (bf16_t*)out, nH, hd,
                     4 * n_blocks);
  ZF_CHECK_LAUNCH();
}

// Prompt portions by the same waves-on-their-own scheme: a workgroup's four waves take 32 rows
// each of a tile of 128 / G positions and walk their own keys (no barrier; the keys a
// workgroup's waves share come to each through the caches).  Head sizes up to 128, at most 32
// query heads a kv head.  n_tiles as for zf_tied_attention_mfma.  n_splits > 1: every wave's
// keys in that many parts, the partial results in ws_o / ws_ml (as above) and merged.
extern "C" int zf_tied_attention_rows(const void* q, long long q_stride, const void* gate,
                                      long long gate_stride, const void* k_pool,
                                      const int* block_table, const int* q_start,
                                      const int* ctx_len, void* out, float* ws_o, float* ws_ml,
                                      float scale, int window, int sink, int T, int n_seqs,
                                      int n_tiles, int nH, int nKV, int hd, int page_size,
                                      int max_pages, int n_splits, hipStream_t stream) {
  if (T <= 0 || n_tiles <= 0) return 0;
  if (nKV <= 0 || nH % nKV != 0 || nH / nKV > 32 || page_size <= 0 || n_splits < 1 ||
      n_splits > ZF_WAVE || (n_splits > 1 && (!ws_o || !ws_ml)))
    return -2;
  const int QT = TA_ROWS / (nH / nKV);
  dim3 grid(n_tiles, nKV, n_splits);
  const int wave_keys = 0;
  switch (hd) {
    TA_WAVE_LAUNCH(32, false) TA_WAVE_LAUNCH(64, false) TA_WAVE_LAUNCH(96, false)
    TA_WAVE_LAUNCH(128, false)
    default: return -3;
  }
  if (n_splits > 1)
    hipLaunchKernelGGL(tied_attention_merge_kernel, dim3(T, nH), dim3(ZF_WAVE), 0, stream, ws_o,
                       ws_ml, (const bf16_t*)gate, gate_stride, (bf16_t*)out, nH, hd, n_splits);
  ZF_CHECK_LAUNCH();
}
