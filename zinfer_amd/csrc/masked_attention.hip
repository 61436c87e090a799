// Causal attention over a paged cache with the pieces that newer decoders add to it, each a
// parameter of its own:
//
//   s_ij = scale * q_i . k_j,  then  s_ij = cap * tanh(s_ij / cap)          (cap 0: not capped)
//   key j is seen by query i when j <= i and
//       i - j < window                         (window 0: no window)
//       floor(i / chunk) == floor(j / chunk)   (chunk 0: no chunks; counted from position 0)
//   a_ij = exp(s_ij) / (exp(sink_h) + sum_j exp(s_ij))   sink: one learned number a head that
//                                                        has no key and no value (null: none)
//   o_i  = sum_j a_ij v_j;  then o_i * sigmoid(gate) with one gate an element or one a head
//
// Keys lie in a pool [page, kv head, row, KW]; values in a pool of their own [page, kv head,
// row, VW], or (no value pool) they are the first VW columns of the key rows: that is what
// attention over a shared latent row looks like once the per-head key and value matrices have
// been moved to the query's and the output's side (one kv head, a key row = the latent and the
// rotated part, the value = the latent).
//
//  * project_rows: the rows of a projection, segment by segment: an RMS norm over the whole
//    segment, a rotation of some leading elements of every head by the token's position
//    (angle = position * frequency in 32-bit, pairs (i, i + dims / 2)), then to plain rows or
//    into the pools at slot_mapping.
//  * masked_attention: any sizes, both dtypes, all arithmetic 32-bit; one workgroup a (token,
//    kv head), one wave a query head.  A token's chunks of keys start at the first key it sees,
//    so its result never depends on how the batch was cut.
//  * head_products: out[t, h, :] = W_h a[t, h, :], a matrix a head (the products that move a
//    latent attention's per-head matrices out of the attention), 32-bit sums in ascending k,
//    with an optional gate sigmoid(g) on the output.
#include "zf_common.h"

#define PR_MAX_SEGMENTS 4

struct RowSegment {
  int src_off, width;        // columns [src_off, src_off + width) of a source row
  const float* gain;         // [width]: RMS norm over the whole segment; null: none
  float eps;
  int hd;                    // head size inside the segment (width % hd == 0)
  int rot_off, rot_dims;     // elements [rot_off, rot_off + rot_dims) of a head are rotated
  const float* freq;         // [rot_dims / 2]
  float mag;                 // cosine and sine are multiplied by this
  int skip;                  // elements of a head below this are not written
  int to_pool;               // 0: plain rows, 1: pages
  void* dst;
  long long dst_stride;      // plain rows: elements from one row to the next
  int dst_off;               // first column in the destination row (pool: in the key row)
  int dst_hd;                // width a head takes in the destination (pool: of a pool row)
  int pool_heads;            // pool: kv heads
};
struct RowSegments {
  RowSegment s[PR_MAX_SEGMENTS];
  int n;
};

template <typename T>
__global__ __launch_bounds__(256) void project_rows_kernel(
    const T* __restrict__ src, long long src_stride, const int* __restrict__ positions,
    const int* __restrict__ slot_mapping, int page_size, RowSegments segs) {
#pragma clang fp contract(off)
  __shared__ float red[16];
  const int t = blockIdx.x;
  const T* row = src + (size_t)t * src_stride;
  const float pos = (float)positions[t];
  for (int si = 0; si < segs.n; ++si) {
    const RowSegment& g = segs.s[si];
    const T* x = row + g.src_off;
    float inv = 1.f;
    if (g.gain != nullptr) {
      float ss = 0.f;
      for (int i = threadIdx.x; i < g.width; i += blockDim.x) {
        const float v = load_as_float<T>(x + i);
        ss += v * v;
      }
      ss = block_sum(ss, red);
      inv = 1.0f / sqrtf(ss / (float)g.width + g.eps);
    }
    size_t pool_base = 0;
    int pool_row = 0;
    if (g.to_pool) {
      const int slot = slot_mapping[t];
      if (slot < 0) continue;                       // the same for the whole workgroup
      pool_base = (size_t)(slot / page_size) * g.pool_heads;
      pool_row = slot % page_size;
    }
    const int half = g.rot_dims / 2;
    for (int i = threadIdx.x; i < g.width; i += blockDim.x) {
      const int head = i / g.hd, d = i % g.hd;
      if (d < g.skip) continue;
      float a = load_as_float<T>(x + i);
      if (g.gain != nullptr) a = a * inv * g.gain[i];
      const int r = d - g.rot_off;
      if (r >= 0 && r < g.rot_dims) {
        const bool first = r < half;
        const int pi = first ? i + half : i - half;
        float b = load_as_float<T>(x + pi);
        if (g.gain != nullptr) b = b * inv * g.gain[pi];
        const float ang = pos * g.freq[first ? r : r - half];
        float sn, cs;
        sincosf(ang, &sn, &cs);
        cs = cs * g.mag;
        sn = sn * g.mag;
        a = first ? a * cs - b * sn : a * cs + b * sn;
      }
      if (g.to_pool) {
        T* o = (T*)g.dst + ((pool_base + head) * page_size + pool_row) * (size_t)g.dst_hd
               + g.dst_off + (d - g.skip);
        store_from_float<T>(o, a);
      } else {
        T* o = (T*)g.dst + (size_t)t * g.dst_stride + g.dst_off + (size_t)head * g.dst_hd
               + (d - g.skip);
        store_from_float<T>(o, a);
      }
    }
  }
}

// ints: 11 a segment (src_off, width, hd, rot_off, rot_dims, skip, to_pool, dst_off, dst_hd,
// pool_heads, 0); floats: 2 a segment (eps, mag); ptrs: 3 a segment (gain, freq, dst);
// strides: 1 a segment
extern "C" int zf_project_rows(const void* src, int dtype, long long src_stride,
                               const int* positions, const int* slot_mapping, int T,
                               int page_size, int n_segs, const int* ints, const float* floats,
                               void* const* ptrs, const long long* strides, hipStream_t stream) {
  if (T <= 0 || n_segs <= 0) return 0;
  if (n_segs > PR_MAX_SEGMENTS) return -2;
  RowSegments segs;
  segs.n = n_segs;
  for (int i = 0; i < n_segs; ++i) {
    RowSegment& g = segs.s[i];
    const int* v = ints + 11 * i;
    g.src_off = v[0]; g.width = v[1]; g.hd = v[2]; g.rot_off = v[3]; g.rot_dims = v[4];
    g.skip = v[5]; g.to_pool = v[6]; g.dst_off = v[7]; g.dst_hd = v[8]; g.pool_heads = v[9];
    g.eps = floats[2 * i]; g.mag = floats[2 * i + 1];
    g.gain = (const float*)ptrs[3 * i]; g.freq = (const float*)ptrs[3 * i + 1];
    g.dst = ptrs[3 * i + 2];
    g.dst_stride = strides[i];
    if (g.width <= 0 || g.hd <= 0 || g.width % g.hd != 0 || g.rot_dims < 0 || g.rot_dims % 2 != 0
        || g.rot_off < 0 || g.rot_off + g.rot_dims > g.hd || g.skip < 0 || g.skip >= g.hd
        || (g.rot_dims > 0 && g.freq == nullptr) || g.dst == nullptr
        || (g.to_pool && (slot_mapping == nullptr || page_size <= 0 || g.pool_heads <= 0)))
      return -2;
  }
  if (dtype == ZF_F32)
    hipLaunchKernelGGL(project_rows_kernel<float>, dim3(T), dim3(256), 0, stream,
                       (const float*)src, src_stride, positions, slot_mapping, page_size, segs);
  else
    hipLaunchKernelGGL(project_rows_kernel<bf16_t>, dim3(T), dim3(256), 0, stream,
                       (const bf16_t*)src, src_stride, positions, slot_mapping, page_size, segs);
  ZF_CHECK_LAUNCH();
}

// =====================================================================================
//  masked_attention: the 32-bit kernel for every size
// =====================================================================================
#define MA_MAX_WAVES 16
#define MA_GATE_NONE 0
#define MA_GATE_ELEMENT 1
#define MA_GATE_HEAD 2

struct MaskedAttentionArgs {
  long long q_stride, gate_stride;
  float scale, cap;
  int window, chunk, gate_mode;
  int nH, nKV, KW, VW, page_size, max_pages, KC;
};

template <typename T>
__global__ __launch_bounds__(MA_MAX_WAVES * ZF_WAVE) void masked_attention_kernel(
    const T* __restrict__ q, const T* __restrict__ gate, const T* __restrict__ k_pool,
    const T* __restrict__ v_pool, const float* __restrict__ sink,
    const int* __restrict__ block_table, const int* __restrict__ q_start,
    const int* __restrict__ ctx_len, const int* __restrict__ seq_index, T* __restrict__ out,
    MaskedAttentionArgs a) {
  extern __shared__ float smem[];
  const int KC = a.KC, KW = a.KW, VW = a.VW;
  const int ldk = KW + 1;                          // odd row stride: a lane a key, no conflicts
  const int ldv = VW + 1;
  const int n_waves = blockDim.x / ZF_WAVE;
  float* ks = smem;                                // [KC][ldk]
  float* vs = ks + KC * ldk;                       // [KC][ldv] when the values have a pool
  float* qs = vs + (v_pool != nullptr ? KC * ldv : 0);   // [n_waves][KW]
  float* ps = qs + n_waves * KW;                   // [n_waves][ZF_WAVE]
  int* rows = (int*)(ps + n_waves * ZF_WAVE);      // [KC]: row of each key in the pools

  const int t = blockIdx.x, kvh = blockIdx.y;
  const int G = a.nH / a.nKV;
  const int wave = threadIdx.x / ZF_WAVE, lane = threadIdx.x % ZF_WAVE;
  const int g = blockIdx.z * MA_MAX_WAVES + wave;  // this wave's head within the group
  const bool live = g < G;
  const int h = kvh * G + (live ? g : 0);
  const int s = seq_index[t];
  const int q_len = q_start[s + 1] - q_start[s];
  const int pos = ctx_len[s] - q_len + (t - q_start[s]);
  int lo = 0;
  if (a.window > 0 && pos - a.window + 1 > lo) lo = pos - a.window + 1;
  if (a.chunk > 0 && pos / a.chunk * a.chunk > lo) lo = pos / a.chunk * a.chunk;
  const int* table = block_table + (size_t)s * a.max_pages;

  const T* qrow = q + (size_t)t * a.q_stride + (size_t)h * KW;
  float* qw = qs + wave * KW;
  for (int i = lane; i < KW; i += ZF_WAVE) qw[i] = load_as_float<T>(qrow + i);

  // a lane owns the output elements d = lane, lane + 64, ... (up to 8: VW <= 512)
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  // the sink is a key of score sink_h that is there before the first real one
  float m = -INFINITY, l = 0.f;
  if (sink != nullptr) {
    m = sink[h];
    l = 1.f;
  }
  const float* vsrc = v_pool != nullptr ? vs : ks;
  const int ldvs = v_pool != nullptr ? ldv : ldk;

  for (int base = lo; base <= pos; base += KC) {
    const int nk = min(KC, pos - base + 1);
    __syncthreads();                               // the tiles of the chunk before are done with
    if ((int)threadIdx.x < KC) {
      const int key = base + threadIdx.x;
      rows[threadIdx.x] = key <= pos
          ? (table[key / a.page_size] * a.nKV + kvh) * a.page_size + key % a.page_size : -1;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nk * KW; i += blockDim.x) {
      const int j = i / KW, d = i % KW;
      ks[j * ldk + d] = load_as_float<T>(k_pool + (size_t)rows[j] * KW + d);
    }
    if (v_pool != nullptr)
      for (int i = threadIdx.x; i < nk * VW; i += blockDim.x) {
        const int j = i / VW, d = i % VW;
        vs[j * ldv + d] = load_as_float<T>(v_pool + (size_t)rows[j] * VW + d);
      }
    __syncthreads();
    float sc = -INFINITY;
    if (lane < nk) {
      const float* kr = ks + lane * ldk;
      float dot = 0.f;
      for (int d = 0; d < KW; ++d) dot = fmaf(qw[d], kr[d], dot);
      sc = dot * a.scale;
      if (a.cap > 0.f) sc = a.cap * tanhf(sc / a.cap);
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
        if (d < VW) acc[i] = fmaf(pj, vsrc[j * ldvs + d], acc[i]);
      }
    }
  }
  if (!live) return;
  const float inv = 1.0f / l;
  T* orow = out + ((size_t)t * a.nH + h) * VW;
  float head_gate = 1.f;
  if (a.gate_mode == MA_GATE_HEAD)
    head_gate = 1.0f / (1.0f + expf(-load_as_float<T>(gate + (size_t)t * a.gate_stride + h)));
  const T* grow = a.gate_mode == MA_GATE_ELEMENT
      ? gate + (size_t)t * a.gate_stride + (size_t)h * VW : nullptr;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int d = lane + i * ZF_WAVE;
    if (d < VW) {
      float v = acc[i] * inv * head_gate;
      if (grow != nullptr) v *= 1.0f / (1.0f + expf(-load_as_float<T>(grow + d)));
      store_from_float<T>(orow + d, v);
    }
  }
}

// floats a key of a chunk takes in LDS, and the chunk that fits 40 KB beside the queries
static int ma_chunk_keys(int KW, int VW, bool v_pool, int n_waves) {
  const long per_key = (KW + 1) + (v_pool ? VW + 1 : 0) + 1;
  const long fixed = (long)n_waves * (KW + ZF_WAVE);
  long kc = (40 * 1024 / 4 - fixed) / per_key;
  if (kc > ZF_WAVE) kc = ZF_WAVE;
  return (int)kc;
}

extern "C" int zf_masked_attention(const void* q, long long q_stride, const void* gate,
                                   long long gate_stride, int gate_mode, const void* k_pool,
                                   const void* v_pool, int dtype, const float* sink,
                                   const int* block_table, const int* q_start,
                                   const int* ctx_len, const int* seq_index, void* out,
                                   float scale, float cap, int window, int chunk, int T, int nH,
                                   int nKV, int KW, int VW, int page_size, int max_pages,
                                   hipStream_t stream) {
  if (T <= 0) return 0;
  if (KW <= 0 || VW <= 0 || VW > 512 || nKV <= 0 || nH % nKV != 0 || page_size <= 0
      || (v_pool == nullptr && VW > KW) || (gate_mode != MA_GATE_NONE && gate == nullptr)
      || gate_mode < 0 || gate_mode > 2 || window < 0 || chunk < 0 || cap < 0.f)
    return -2;
  const int G = nH / nKV;
  const int n_waves = G < MA_MAX_WAVES ? G : MA_MAX_WAVES;
  const int KC = ma_chunk_keys(KW, VW, v_pool != nullptr, n_waves);
  if (KC < 4) return -3;
  MaskedAttentionArgs a;
  a.q_stride = q_stride; a.gate_stride = gate_stride; a.scale = scale; a.cap = cap;
  a.window = window; a.chunk = chunk; a.gate_mode = gate_mode; a.nH = nH; a.nKV = nKV;
  a.KW = KW; a.VW = VW; a.page_size = page_size; a.max_pages = max_pages; a.KC = KC;
  dim3 grid(T, nKV, (G + MA_MAX_WAVES - 1) / MA_MAX_WAVES);
  const size_t smem = ((size_t)KC * (KW + 1) + (v_pool != nullptr ? (size_t)KC * (VW + 1) : 0)
                       + (size_t)n_waves * (KW + ZF_WAVE) + KC) * sizeof(float);
  if (dtype == ZF_F32)
    hipLaunchKernelGGL(masked_attention_kernel<float>, grid, dim3(n_waves * ZF_WAVE), smem,
                       stream, (const float*)q, (const float*)gate, (const float*)k_pool,
                       (const float*)v_pool, sink, block_table, q_start, ctx_len, seq_index,
                       (float*)out, a);
  else
    hipLaunchKernelGGL(masked_attention_kernel<bf16_t>, grid, dim3(n_waves * ZF_WAVE), smem,
                       stream, (const bf16_t*)q, (const bf16_t*)gate, (const bf16_t*)k_pool,
                       (const bf16_t*)v_pool, sink, block_table, q_start, ctx_len, seq_index,
                       (bf16_t*)out, a);
  ZF_CHECK_LAUNCH();
}

// =====================================================================================
//  head_products: a matrix a head
// =====================================================================================
// out[t, h, n] = sum_k a[t, h, k] * w[h, n, k]  (n < N, k < K), then times sigmoid(gate[t, h, n])
// if a gate is given.  a: row t at a + t * a_stride, head h at + a_off + h * a_hd; out: row t at
// out + t * out_stride, head h at + out_off + h * out_hd; w [H, N, K]; gate [T, H * N] rows of
// stride gate_stride.  A workgroup takes 16 tokens x 64 outputs of one head; k runs upwards in
// one accumulator an output, so a token's result does not depend on the tokens beside it.
#define HP_TOK 16
#define HP_OUT 64
#define HP_K 64

template <typename T, typename TW>
__global__ __launch_bounds__(256) void head_products_kernel(
    const T* __restrict__ a, long long a_stride, int a_off, int a_hd, const TW* __restrict__ w,
    const T* __restrict__ gate, long long gate_stride, T* __restrict__ out, long long out_stride,
    int out_off, int out_hd, int n_tok, int N, int K) {
  __shared__ float as[HP_TOK][HP_K + 1];
  __shared__ float ws[HP_OUT][HP_K + 1];
  const int t0 = blockIdx.x * HP_TOK, h = blockIdx.y, n0 = blockIdx.z * HP_OUT;
  const int nl = threadIdx.x % HP_OUT, tg = threadIdx.x / HP_OUT;    // 4 groups of 4 tokens
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  const TW* wh = w + (size_t)h * N * K;
  for (int k0 = 0; k0 < K; k0 += HP_K) {
    const int kn = min(HP_K, K - k0);
    __syncthreads();
    for (int i = threadIdx.x; i < HP_TOK * HP_K; i += 256) {
      const int r = i / HP_K, c = i % HP_K;
      float v = 0.f;
      if (t0 + r < n_tok && c < kn)
        v = load_as_float<T>(a + (size_t)(t0 + r) * a_stride + a_off + (size_t)h * a_hd + k0 + c);
      as[r][c] = v;
    }
    for (int i = threadIdx.x; i < HP_OUT * HP_K; i += 256) {
      const int r = i / HP_K, c = i % HP_K;
      float v = 0.f;
      if (n0 + r < N && c < kn) v = load_as_float<TW>(wh + (size_t)(n0 + r) * K + k0 + c);
      ws[r][c] = v;
    }
    __syncthreads();
    for (int c = 0; c < kn; ++c) {
      const float wv = ws[nl][c];
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = fmaf(as[tg * 4 + i][c], wv, acc[i]);
    }
  }
  const int n = n0 + nl;
  if (n >= N) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = t0 + tg * 4 + i;
    if (t >= n_tok) continue;
    float v = acc[i];
    if (gate != nullptr)
      v *= 1.0f / (1.0f + expf(-load_as_float<T>(gate + (size_t)t * gate_stride
                                                  + (size_t)h * N + n)));
    store_from_float<T>(out + (size_t)t * out_stride + out_off + (size_t)h * out_hd + n, v);
  }
}

extern "C" int zf_head_products(const void* a, int dtype, long long a_stride, int a_off, int a_hd,
                                const void* w, int w_dtype, const void* gate,
                                long long gate_stride, void* out, long long out_stride,
                                int out_off, int out_hd, int T, int H, int N, int K,
                                hipStream_t stream) {
  if (T <= 0) return 0;
  if (H <= 0 || N <= 0 || K <= 0 || a_hd < K || out_hd < N) return -2;
  dim3 grid((T + HP_TOK - 1) / HP_TOK, H, (N + HP_OUT - 1) / HP_OUT);
#define HP_LAUNCH(TA, TWT)                                                                      \
  hipLaunchKernelGGL((head_products_kernel<TA, TWT>), grid, dim3(256), 0, stream, (const TA*)a, \
                     a_stride, a_off, a_hd, (const TWT*)w, (const TA*)gate, gate_stride,        \
                     (TA*)out, out_stride, out_off, out_hd, T, N, K)
  if (dtype == ZF_F32 && w_dtype == ZF_F32) HP_LAUNCH(float, float);
  else if (dtype == ZF_F32) HP_LAUNCH(float, bf16_t);
  else if (w_dtype == ZF_F32) HP_LAUNCH(bf16_t, float);
  else HP_LAUNCH(bf16_t, bf16_t);
#undef HP_LAUNCH
  ZF_CHECK_LAUNCH();
}
