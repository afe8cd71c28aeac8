// Talking-heads attention over the paged KV cache, gfx950.
//
// Causal attention whose H per-head score planes are mixed across heads
// before the softmax:
//
//   s_g(i, j)  = scale * q_g(i) . k_kv(g)(j)          all heads g
//   s'_h(i, j) = sum_g talk[h, g] * s_g(i, j)
//   w_h(i, .)  = exp(s'_h) / (sum_{j <= i} exp(s'_h) + exp(sink_h))
//   o_h(i)     = sum_j w_h(i, j) * v_kv(h)(j)
//
// The mix couples the heads, so one workgroup owns ALL heads of its
// queries. Scores, the mix, softmax statistics and the sink are fp32
// whatever the I/O type T (bf16 or fp32) is.
//
//   talking_attention_kernel   any D, Dv, H, G, page size, dtype: one
//       workgroup per (query token, key split); 64-key tiles: raw scores
//       -> LDS, mix + online softmax (one wave per head), P.V with the
//       accumulators in registers. Decode-only batches split the keys
//       over several workgroups (partials + talking_merge_kernel).
//   talking_mfma_kernel        bf16, D == Dv in {32, 64, 96, 128}, up to
//       16 heads, batches with prompt portions: 16 queries of one
//       sequence per workgroup, K/V tiles of 32 keys staged through LDS,
//       Q K^T and P V on 16x16x32 MFMA; the raw score planes of all
//       heads pass through LDS for the fp32 mix.

#include <torch/extension.h>
#include <ATen/cuda/CUDAContext.h>
#include "common.h"

namespace {

constexpr int TK_BLOCK = 256;
constexpr int TK_KEYS = 64;   // keys per tile = one wave of scores

// which sequence owns flat token t: largest b with qsl[b] <= t
DEV_INLINE int owner_of(const int *__restrict__ qsl, int B, int t) {
  int lo = 0, hi = B - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (qsl[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

template <typename T>
DEV_INLINE float dot_row(const float *__restrict__ qs,
                         const T *__restrict__ kr, int D) {
  float dot = 0.f;
  if (sizeof(T) == 2 && D % 8 == 0) {
    for (int d = 0; d < D; d += 8) {
      float kf[8];
      unpack8<T>(*reinterpret_cast<const shortx8 *>(kr + d), kf);
#pragma unroll
      for (int e = 0; e < 8; ++e) dot += qs[d + e] * kf[e];
    }
  } else if (sizeof(T) == 4 && D % 4 == 0) {
    for (int d = 0; d < D; d += 4) {
      const floatx4 kf = *reinterpret_cast<const floatx4 *>(kr + d);
#pragma unroll
      for (int e = 0; e < 4; ++e) dot += qs[d + e] * kf[e];
    }
  } else {
    for (int d = 0; d < D; ++d) dot += qs[d] * ScalarOps<T>::to_f32(kr[d]);
  }
  return dot;
}

// grid (tokens, splits). NACC = ceil(H * Dv / 256) rounded up to a power
// of two: output element o = tid + c * 256 (head o / Dv, column o % Dv).
template <typename T, int NACC>
__global__ __launch_bounds__(TK_BLOCK) void talking_attention_kernel(
    T *__restrict__ out, float *__restrict__ part_acc,
    float *__restrict__ part_ml, const T *__restrict__ q, long q_stride,
    const T *__restrict__ k_cache, const T *__restrict__ v_cache,
    const int *__restrict__ block_table, int bt_stride,
    const int *__restrict__ seq_lens, const int *__restrict__ qsl, int B,
    int H, int G, int D, int Dv, int page, float scale,
    const float *__restrict__ talk, const float *__restrict__ sink,
    int splits) {
  extern __shared__ float smem[];
  const int HD = (H * D + 3) & ~3;
  float *qs = smem;                    // [H * D]
  float *tk = qs + HD;                 // [H * H]
  float *sraw = tk + ((H * H + 3) & ~3);  // [H][64] raw scores
  float *pp = sraw + H * TK_KEYS;      // [H][64] softmax numerators
  float *mrun = pp + H * TK_KEYS;      // [H] running max
  float *lrun = mrun + H;              // [H] running sum
  float *corr = lrun + H;              // [H] rescale of this tile
  long *rows = reinterpret_cast<long *>(
      smem + ((HD + ((H * H + 3) & ~3) + 2 * H * TK_KEYS + 3 * H + 1) & ~1));

  const int t = blockIdx.x, sp = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int b = owner_of(qsl, B, t);
  const int i = seq_lens[b] - (qsl[b + 1] - t);   // position of row t
  const int total = i + 1;                         // keys 0..i
  const int *bt = block_table + (long)b * bt_stride;
  const int rep = H / G;

  const int tiles = (total + TK_KEYS - 1) / TK_KEYS;
  const int tiles_per = (tiles + splits - 1) / splits;
  const int j0 = sp * tiles_per * TK_KEYS;
  const int j1 = min(total, j0 + tiles_per * TK_KEYS);

  for (int d = tid; d < H * D; d += TK_BLOCK)
    qs[d] = ScalarOps<T>::to_f32(q[(long)t * q_stride + d]);
  for (int d = tid; d < H * H; d += TK_BLOCK) tk[d] = talk[d];
  for (int h = tid; h < H; h += TK_BLOCK) {
    mrun[h] = -INFINITY;
    lrun[h] = 0.f;
  }
  float acc[NACC];
#pragma unroll
  for (int c = 0; c < NACC; ++c) acc[c] = 0.f;

  for (int base = j0; base < j1; base += TK_KEYS) {
    const int n_tile = min(TK_KEYS, j1 - base);
    __syncthreads();   // q/talk staged; last tile's pp/rows are done with
    if (tid < TK_KEYS) {
      const int j = base + tid;
      rows[tid] = tid < n_tile ? (long)bt[j / page] * page + j % page : 0;
    }
    __syncthreads();
    // raw scores: lane = key, wave strides over the heads
    for (int h = wave; h < H; h += TK_BLOCK / 64) {
      float s = 0.f;
      if (lane < n_tile)
        s = dot_row<T>(qs + h * D, k_cache + (rows[lane] * G + h / rep) * D,
                       D) * scale;
      sraw[h * TK_KEYS + lane] = s;
    }
    __syncthreads();
    // mix + online softmax: a wave owns head h for this tile
    for (int h = wave; h < H; h += TK_BLOCK / 64) {
      float s = 0.f;
      for (int g = 0; g < H; ++g) s += tk[h * H + g] * sraw[g * TK_KEYS + lane];
      if (lane >= n_tile) s = -INFINITY;
      const float m_old = mrun[h];
      const float m_new = fmaxf(m_old, wave_reduce_max(s));
      const float p = lane < n_tile ? expf(s - m_new) : 0.f;
      const float psum = wave_reduce_sum(p);
      const float c = m_old == -INFINITY ? 0.f : expf(m_old - m_new);
      pp[h * TK_KEYS + lane] = p;
      if (lane == 0) {
        mrun[h] = m_new;
        lrun[h] = lrun[h] * c + psum;
        corr[h] = c;
      }
    }
    __syncthreads();
    // P.V
#pragma unroll
    for (int c = 0; c < NACC; ++c) {
      const int o = tid + c * TK_BLOCK;
      if (o < H * Dv) {
        const int h = o / Dv, d = o - h * Dv;
        const float *ph = pp + h * TK_KEYS;
        const T *vb = v_cache + (long)(h / rep) * Dv + d;
        float a = acc[c] * corr[h];
        for (int jj = 0; jj < n_tile; ++jj)
          a += ph[jj] * ScalarOps<T>::to_f32(vb[rows[jj] * G * Dv]);
        acc[c] = a;
      }
    }
  }
  __syncthreads();
  if (splits == 1) {
#pragma unroll
    for (int c = 0; c < NACC; ++c) {
      const int o = tid + c * TK_BLOCK;
      if (o < H * Dv) {
        const int h = o / Dv;
        float m = mrun[h], l = lrun[h], a = acc[c];
        if (sink != nullptr) {
          const float sk = sink[h];
          const float M = fmaxf(m, sk);
          const float w = expf(m - M);
          l = l * w + expf(sk - M);
          a *= w;
        }
        out[(long)t * H * Dv + o] = ScalarOps<T>::from_f32(a / l);
      }
    }
  } else {
    const long pbase = (long)t * splits + sp;
#pragma unroll
    for (int c = 0; c < NACC; ++c) {
      const int o = tid + c * TK_BLOCK;
      if (o < H * Dv) part_acc[pbase * H * Dv + o] = acc[c];
    }
    for (int h = tid; h < H; h += TK_BLOCK) {
      part_ml[(pbase * H + h) * 2] = mrun[h];
      part_ml[(pbase * H + h) * 2 + 1] = lrun[h];
    }
  }
}

// grid (tokens, heads): combine the key splits of one (query, head),
// sink included; the first ``splits`` threads form the split weights
constexpr int MERGE_MAX_SPLITS = 64;

template <typename T>
__global__ __launch_bounds__(128) void talking_merge_kernel(
    T *__restrict__ out, const float *__restrict__ part_acc,
    const float *__restrict__ part_ml, const float *__restrict__ sink, int H,
    int Dv, int splits) {
  __shared__ float wgt[MERGE_MAX_SPLITS];
  __shared__ float inv_l;
  const int t = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x;
  if (tid < 64) {
    float m = -INFINITY, l = 0.f;
    if (tid < splits) {
      const long pb = ((long)t * splits + tid) * H + h;
      m = part_ml[pb * 2];
      l = part_ml[pb * 2 + 1];
    }
    float M = wave_reduce_max(m);
    if (sink != nullptr) M = fmaxf(M, sink[h]);
    const float w = m == -INFINITY ? 0.f : expf(m - M);
    if (tid < splits) wgt[tid] = w;
    float lsum = wave_reduce_sum(l * w);
    if (sink != nullptr) lsum += expf(sink[h] - M);
    if (tid == 0) inv_l = lsum > 0.f ? 1.0f / lsum : 0.f;
  }
  __syncthreads();
  for (int d = tid; d < Dv; d += 128) {
    float a = 0.f;
    for (int s = 0; s < splits; ++s)
      a += part_acc[(((long)t * splits + s) * H + h) * Dv + d] * wgt[s];
    out[((long)t * H + h) * Dv + d] = ScalarOps<T>::from_f32(a * inv_l);
  }
}

bool rows_ok2(const torch::Tensor &t) {
  return t.dim() == 2 && t.stride(1) == 1;
}

}  // namespace

bool talking_attention_mfma(torch::Tensor &out, torch::Tensor &q,
                            torch::Tensor &k_cache, torch::Tensor &v_cache,
                            torch::Tensor &block_table,
                            torch::Tensor &seq_lens,
                            torch::Tensor &query_start_loc, double scale,
                            torch::Tensor &talk, const float *sink,
                            long max_query_len);

bool talking_attention_decode_mfma(torch::Tensor &out, torch::Tensor &q,
                                   torch::Tensor &k_cache,
                                   torch::Tensor &v_cache,
                                   torch::Tensor &block_table,
                                   torch::Tensor &seq_lens, double scale,
                                   torch::Tensor &talk, const float *sink,
                                   int splits, float *part_acc,
                                   float *part_ml);

void talking_attention(torch::Tensor out, torch::Tensor q,
                       torch::Tensor k_cache, torch::Tensor v_cache,
                       torch::Tensor block_table, torch::Tensor seq_lens,
                       torch::Tensor query_start_loc, double scale,
                       torch::Tensor talk, c10::optional<torch::Tensor> sink,
                       long max_query_len) {
  const long T = q.size(0);
  if (T == 0) return;
  const auto st = q.scalar_type();
  TORCH_CHECK(q.is_cuda() && k_cache.dim() == 4 && v_cache.dim() == 4);
  const int page = k_cache.size(1), G = k_cache.size(2), D = k_cache.size(3);
  const int Dv = v_cache.size(3);
  TORCH_CHECK(rows_ok2(q) && q.size(1) % D == 0);
  const int H = q.size(1) / D;
  TORCH_CHECK(G > 0 && H % G == 0,
              "query heads must be a multiple of kv heads");
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() &&
              k_cache.scalar_type() == st && v_cache.scalar_type() == st);
  TORCH_CHECK(v_cache.size(0) == k_cache.size(0) && v_cache.size(1) == page &&
              v_cache.size(2) == G);
  TORCH_CHECK(out.is_contiguous() && out.scalar_type() == st &&
              out.numel() == T * H * Dv);
  TORCH_CHECK(block_table.scalar_type() == at::kInt && block_table.dim() == 2 &&
              block_table.stride(1) == 1);
  TORCH_CHECK(seq_lens.scalar_type() == at::kInt && seq_lens.is_contiguous());
  TORCH_CHECK(query_start_loc.scalar_type() == at::kInt &&
              query_start_loc.is_contiguous());
  const int B = seq_lens.numel();
  TORCH_CHECK(query_start_loc.numel() >= B + 1 && block_table.size(0) >= B);
  TORCH_CHECK(talk.is_cuda() && talk.scalar_type() == at::kFloat &&
              talk.is_contiguous() && talk.numel() == (long)H * H,
              "talk must be fp32 [H, H]");
  const float *sp = nullptr;
  if (sink.has_value()) {
    TORCH_CHECK(sink->is_cuda() && sink->scalar_type() == at::kFloat &&
                sink->is_contiguous() && sink->numel() == H,
                "sink must be fp32 [H]");
    sp = sink->data_ptr<float>();
  }
  TORCH_CHECK((long)H * Dv <= 32 * TK_BLOCK,
              "talking_attention: heads * value size <= 8192");

  if (st == at::kBFloat16 && max_query_len > 1 &&
      talking_attention_mfma(out, q, k_cache, v_cache, block_table, seq_lens,
                             query_start_loc, scale, talk, sp,
                             max_query_len))
    return;

  // decode-only batches: spread the keys of each query over workgroups
  // (fixed by the batch size alone, so a captured graph keeps its shape)
  int splits = 1;
  if (max_query_len == 1 && T < 512)
    splits = (int)std::min<long>(16, (1024 + T - 1) / T);
  torch::Tensor pacc, pml;
  float *paccp = nullptr, *pmlp = nullptr;
  if (splits > 1) {
    auto opts = torch::TensorOptions().dtype(at::kFloat).device(q.device());
    pacc = torch::empty({T, splits, (long)H * Dv}, opts);
    pml = torch::empty({T, splits, (long)H, 2}, opts);
    paccp = pacc.data_ptr<float>();
    pmlp = pml.data_ptr<float>();
  }
  auto stream = at::cuda::getCurrentCUDAStream();
  auto merge = [&]() {
    if (splits == 1) return;
    if (st == at::kBFloat16)
      hipLaunchKernelGGL((talking_merge_kernel<__hip_bfloat16>), dim3(T, H),
                         dim3(128), 0, stream,
                         (__hip_bfloat16 *)out.data_ptr(), paccp, pmlp, sp, H,
                         Dv, splits);
    else
      hipLaunchKernelGGL((talking_merge_kernel<float>), dim3(T, H),
                         dim3(128), 0, stream, (float *)out.data_ptr(),
                         paccp, pmlp, sp, H, Dv, splits);
    HIP_CHECK_KERNEL();
  };
  // bf16 decode-only batch: one token per sequence, the heads of a GQA
  // group ride the MFMA rows
  if (st == at::kBFloat16 && max_query_len == 1 && T == B &&
      talking_attention_decode_mfma(out, q, k_cache, v_cache, block_table,
                                    seq_lens, scale, talk, sp, splits, paccp,
                                    pmlp)) {
    merge();
    return;
  }
  const int HD = (H * D + 3) & ~3, HH = (H * H + 3) & ~3;
  const int nf = (HD + HH + 2 * H * TK_KEYS + 3 * H + 1) & ~1;
  const size_t lds = (size_t)nf * sizeof(float) + TK_KEYS * sizeof(long);
  TORCH_CHECK(lds <= 64 * 1024, "talking_attention: heads * dim too large");
  int nacc = 1;
  while (nacc * TK_BLOCK < H * Dv) nacc *= 2;
#define RUN(TT, N)                                                           \
  hipLaunchKernelGGL((talking_attention_kernel<TT, N>), dim3(T, splits),     \
                     dim3(TK_BLOCK), lds, stream, (TT *)out.data_ptr(),      \
                     paccp, pmlp, (const TT *)q.data_ptr(),                  \
                     (long)q.stride(0), (const TT *)k_cache.data_ptr(),      \
                     (const TT *)v_cache.data_ptr(),                         \
                     block_table.data_ptr<int>(), (int)block_table.stride(0), \
                     seq_lens.data_ptr<int>(),                               \
                     query_start_loc.data_ptr<int>(), B, H, G, D, Dv, page,  \
                     (float)scale, talk.data_ptr<float>(), sp, splits)
#define RUN_N(TT)                                                            \
  switch (nacc) {                                                            \
    case 1: RUN(TT, 1); break;                                               \
    case 2: RUN(TT, 2); break;                                               \
    case 4: RUN(TT, 4); break;                                               \
    case 8: RUN(TT, 8); break;                                               \
    case 16: RUN(TT, 16); break;                                             \
    default: RUN(TT, 32); break;                                             \
  }
  if (st == at::kBFloat16) { RUN_N(__hip_bfloat16) }
  else if (st == at::kFloat) { RUN_N(float) }
  else TORCH_CHECK(false, "talking_attention: bf16 or fp32");
#undef RUN_N
#undef RUN
  HIP_CHECK_KERNEL();
  merge();
}

// ------------------------------------------------------------------
// MFMA tile form (bf16). One workgroup = 16 queries of one sequence x
// all H heads; 4 waves, wave w owns heads w, w+4, ... (HPW per wave).
// Per 32-key tile:
//   stage K (all kv heads) -> LDS
//   S_h = Q_h K^T on 16x16x32 MFMA, scaled, -> sraw[h] (fp32, LDS)
//   stage V over K; meanwhile mix: s'_h = sum_g talk[h,g] sraw[g]
//   (lane = query row x 8 keys, 16 B LDS reads), causal mask, online
//   softmax in fp32, P_h -> pbuf[h] (bf16), rescale factors -> LDS
//   O_h += P_h V on MFMA (B fragments gathered from the linear V tile)
// Softmax weights are fp32 until they become the matrix core's left
// operand (bf16, fp32 accumulation); scores, mix, max/sum and the sink
// never leave fp32.
typedef __attribute__((ext_vector_type(8))) __bf16 tk_bf8;
typedef __attribute__((ext_vector_type(4))) float tk_f4;

namespace {

constexpr int MQ = 16;   // queries per workgroup
constexpr int MK = 32;   // keys per tile
constexpr int MWAVES = 4;
constexpr int SR = 36;   // sraw row stride (floats), 16 B aligned rows
constexpr int PR = 40;   // pbuf row stride (bf16), 16 B aligned rows

constexpr int VS = 40;   // V^T row stride (bf16): 32 keys + pad

DEV_INLINE long cache_row(const int *__restrict__ bt, int page, int tok) {
  return (long)bt[tok / page] * page + tok % page;
}

// K tile of MK keys, all kv heads, into LDS as [g][key][D + 8]: 16 B
// chunks, a thread keeps the same (key, column chunk) for every kv head
// (one page lookup per chunk), loads of two heads fly before their stores.
template <int D>
DEV_INLINE void stage_k_tile(__hip_bfloat16 *__restrict__ kvbuf,
                             const __hip_bfloat16 *__restrict__ src,
                             const int *__restrict__ bt, int page, int G,
                             int kv0, int last_tok, int tid) {
  constexpr int CPR = D / 8, KS = D + 8, NCH = MK * CPR;
  constexpr int NTH = MWAVES * 64, UU = (NCH + NTH - 1) / NTH;
  long off[UU];
  int dst[UU];
#pragma unroll
  for (int u = 0; u < UU; ++u) {
    const int c = tid + u * NTH;
    const int key = c / CPR, dc = c - key * CPR;
    dst[u] = c < NCH ? key * KS + dc * 8 : -1;
    off[u] = cache_row(bt, page, min(kv0 + min(key, MK - 1), last_tok)) * G *
                 D + dc * 8;
  }
  for (int g0 = 0; g0 < G; g0 += 2) {
    shortx8 v[2][UU];
#pragma unroll
    for (int gg = 0; gg < 2; ++gg)
#pragma unroll
      for (int u = 0; u < UU; ++u)
        if (g0 + gg < G && dst[u] >= 0)
          v[gg][u] = *reinterpret_cast<const shortx8 *>(src + off[u] +
                                                        (g0 + gg) * D);
#pragma unroll
    for (int gg = 0; gg < 2; ++gg)
#pragma unroll
      for (int u = 0; u < UU; ++u)
        if (g0 + gg < G && dst[u] >= 0)
          *reinterpret_cast<shortx8 *>(
              &kvbuf[(g0 + gg) * MK * KS + dst[u]]) = v[gg][u];
  }
}

// V tile transposed into LDS as [g][column][VS]: the P.V right operand
// (8 consecutive keys of one column) is then one 16 B read, shared by
// every head of the kv group. A thread owns one key (tid % 32) and
// walks that key's 16 B chunks; the 2-byte stores of neighbouring lanes
// fall into neighbouring keys of one column.
template <int D>
DEV_INLINE void stage_vt_tile(__hip_bfloat16 *__restrict__ kvbuf,
                              const __hip_bfloat16 *__restrict__ src,
                              const int *__restrict__ bt, int page, int G,
                              int kv0, int last_tok, int tid) {
  constexpr int CPR = D / 8, NTH = MWAVES * 64, SUBS = NTH / MK, U = 4;
  const int key = tid & (MK - 1), sub = tid / MK;
  const __hip_bfloat16 *rowp =
      src + cache_row(bt, page, min(kv0 + key, last_tok)) * G * D;
  const int nch = G * CPR;
  for (int c0 = sub; c0 < nch; c0 += SUBS * U) {
    shortx8 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = c0 + u * SUBS;
      if (c < nch) v[u] = *reinterpret_cast<const shortx8 *>(rowp + c * 8);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = c0 + u * SUBS;
      if (c < nch) {
        // chunk c covers columns c*8 .. c*8+7 of the [G*D] row
        const short *e = reinterpret_cast<const short *>(&v[u]);
        short *dstp = reinterpret_cast<short *>(kvbuf) + (c * 8) * VS + key;
#pragma unroll
        for (int j = 0; j < 8; ++j) dstp[j * VS] = e[j];
      }
    }
  }
}

// Split forms of the two stagings for tiles small enough to ride in
// registers (at most PF 16 B chunks per thread): the loads are issued
// early and their stores come after independent work, so the global
// latency hides behind the matrix and mix phases.
constexpr int PF = 4;

template <int D>
DEV_INLINE bool tile_fits_regs(int G) {
  constexpr int CPR = D / 8, NTH = MWAVES * 64;
  constexpr int UU = (MK * CPR + NTH - 1) / NTH;
  return G * UU <= PF && G * CPR <= PF * (NTH / MK);
}

template <int D>
DEV_INLINE void k_tile_load(shortx8 (&v)[PF],
                            const __hip_bfloat16 *__restrict__ src,
                            const int *__restrict__ bt, int page, int G,
                            int kv0, int last_tok, int tid) {
  constexpr int CPR = D / 8, NCH = MK * CPR, NTH = MWAVES * 64;
  constexpr int UU = (NCH + NTH - 1) / NTH;
#pragma unroll
  for (int u = 0; u < UU; ++u) {
    const int c = tid + u * NTH;
    const int key = c / CPR, dc = c - key * CPR;
    if (c < NCH) {
      const __hip_bfloat16 *rowp =
          src + cache_row(bt, page, min(kv0 + key, last_tok)) * G * D + dc * 8;
#pragma unroll
      for (int g = 0; g < PF / UU; ++g)
        if (g < G)
          v[g * UU + u] = *reinterpret_cast<const shortx8 *>(rowp + g * D);
    }
  }
}

template <int D>
DEV_INLINE void k_tile_store(__hip_bfloat16 *__restrict__ kvbuf,
                             const shortx8 (&v)[PF], int G, int tid) {
  constexpr int CPR = D / 8, KS = D + 8, NCH = MK * CPR, NTH = MWAVES * 64;
  constexpr int UU = (NCH + NTH - 1) / NTH;
#pragma unroll
  for (int u = 0; u < UU; ++u) {
    const int c = tid + u * NTH;
    const int key = c / CPR, dc = c - key * CPR;
    if (c < NCH) {
#pragma unroll
      for (int g = 0; g < PF / UU; ++g)
        if (g < G)
          *reinterpret_cast<shortx8 *>(
              &kvbuf[(g * MK + key) * KS + dc * 8]) = v[g * UU + u];
    }
  }
}

template <int D>
DEV_INLINE void vt_tile_load(shortx8 (&v)[PF],
                             const __hip_bfloat16 *__restrict__ src,
                             const int *__restrict__ bt, int page, int G,
                             int kv0, int last_tok, int tid) {
  constexpr int CPR = D / 8, SUBS = MWAVES * 64 / MK;
  const int key = tid & (MK - 1), sub = tid / MK;
  const __hip_bfloat16 *rowp =
      src + cache_row(bt, page, min(kv0 + key, last_tok)) * G * D;
  const int nch = G * CPR;
#pragma unroll
  for (int u = 0; u < PF; ++u) {
    const int c = sub + u * SUBS;
    if (c < nch) v[u] = *reinterpret_cast<const shortx8 *>(rowp + c * 8);
  }
}

template <int D>
DEV_INLINE void vt_tile_store(__hip_bfloat16 *__restrict__ kvbuf,
                              const shortx8 (&v)[PF], int G, int tid) {
  constexpr int CPR = D / 8, SUBS = MWAVES * 64 / MK;
  const int key = tid & (MK - 1), sub = tid / MK;
  const int nch = G * CPR;
#pragma unroll
  for (int u = 0; u < PF; ++u) {
    const int c = sub + u * SUBS;
    if (c < nch) {
      const short *e = reinterpret_cast<const short *>(&v[u]);
      short *dstp = reinterpret_cast<short *>(kvbuf) + (c * 8) * VS + key;
#pragma unroll
      for (int j = 0; j < 8; ++j) dstp[j * VS] = e[j];
    }
  }
}

template <int D, int HPW>
__global__ __launch_bounds__(MWAVES * 64) void talking_mfma_kernel(
    __hip_bfloat16 *__restrict__ out, const __hip_bfloat16 *__restrict__ q,
    long q_stride, const __hip_bfloat16 *__restrict__ k_cache,
    const __hip_bfloat16 *__restrict__ v_cache,
    const int *__restrict__ block_table, int bt_stride,
    const int *__restrict__ seq_lens, const int *__restrict__ qsl, int H,
    int G, int page, float scale, const float *__restrict__ talk,
    const float *__restrict__ sink) {
  constexpr int KT = D / 32, NT = D / 16, KS = D + 8;
  extern __shared__ __attribute__((aligned(16))) char tk_lds[];
  __hip_bfloat16 *kvbuf = reinterpret_cast<__hip_bfloat16 *>(tk_lds);
  constexpr int KV_ELEMS = MK * KS > D * VS ? MK * KS : D * VS;
  float *sraw = reinterpret_cast<float *>(tk_lds + (size_t)G * KV_ELEMS * 2);
  __hip_bfloat16 *pbuf =
      reinterpret_cast<__hip_bfloat16 *>(sraw + H * MQ * SR);
  float *alpha_s = reinterpret_cast<float *>(pbuf + H * MQ * PR);
  float *tks = alpha_s + H * MQ;

  const int tile = blockIdx.x, b = blockIdx.y;
  const int q_start = qsl[b];
  const int q_len = qsl[b + 1] - q_start;
  if (tile * MQ >= q_len) return;
  const int seq_len = seq_lens[b];
  const int past = seq_len - q_len;
  const int rep = H / G;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int l16 = lane & 15, lhi = lane >> 4;
  const int mi = lane >> 2, mc = lane & 3;   // mix layout: row, key octet
  const int *bt = block_table + (long)b * bt_stride;

  for (int d = tid; d < H * H; d += MWAVES * 64) tks[d] = talk[d];

  float m_run[HPW], l_run[HPW];
  tk_f4 o_acc[HPW][NT];
#pragma unroll
  for (int hs = 0; hs < HPW; ++hs) {
    m_run[hs] = -INFINITY;
    l_run[hs] = 0.f;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) o_acc[hs][nt] = tk_f4{0, 0, 0, 0};
  }
  const int qrow_a = tile * MQ + l16;          // A-fragment row
  const bool qrow_a_ok = qrow_a < q_len;
  const __hip_bfloat16 *qa =
      q + (long)(q_start + (qrow_a_ok ? qrow_a : 0)) * q_stride + lhi * 8;
  const int qrow_m = tile * MQ + mi;
  const int qpos_m = past + qrow_m;
  const bool qrow_m_ok = qrow_m < q_len;
  const int kv_max = min(seq_len, past + min(q_len, (tile + 1) * MQ));


  // the query fragments of this wave's heads stay in registers
  tk_bf8 qf[HPW][KT];
#pragma unroll
  for (int hs = 0; hs < HPW; ++hs) {
    const int h = min(wave + hs * MWAVES, H - 1);
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
      qf[hs][kt] = tk_bf8{0, 0, 0, 0, 0, 0, 0, 0};
      if (qrow_a_ok)
        qf[hs][kt] = *reinterpret_cast<const tk_bf8 *>(qa + h * D + kt * 32);
    }
  }
  // small tiles travel through registers: K of the next tile is fetched
  // under P V, V^T of this tile under Q K^T and the mix
  const bool piped = tile_fits_regs<D>(G);
  shortx8 kreg[PF], vreg[PF];
  if (piped && kv_max > 0)
    k_tile_load<D>(kreg, k_cache, bt, page, G, 0, seq_len - 1, tid);
  for (int kv0 = 0; kv0 < kv_max; kv0 += MK) {
    if (piped) {
      k_tile_store<D>(kvbuf, kreg, G, tid);
      vt_tile_load<D>(vreg, v_cache, bt, page, G, kv0, seq_len - 1, tid);
    } else {
      stage_k_tile<D>(kvbuf, k_cache, bt, page, G, kv0, seq_len - 1, tid);
    }
    __syncthreads();
    // ---- raw scores of this wave's heads ----
#pragma unroll
    for (int hs = 0; hs < HPW; ++hs) {
      const int h = wave + hs * MWAVES;
      if (h < H) {
        const int g = h / rep;
        tk_f4 s0 = tk_f4{0, 0, 0, 0}, s1 = tk_f4{0, 0, 0, 0};
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
          const tk_bf8 a = qf[hs][kt];
          const tk_bf8 b0 = *reinterpret_cast<const tk_bf8 *>(
              &kvbuf[(g * MK + l16) * KS + kt * 32 + lhi * 8]);
          const tk_bf8 b1 = *reinterpret_cast<const tk_bf8 *>(
              &kvbuf[(g * MK + 16 + l16) * KS + kt * 32 + lhi * 8]);
          s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b0, s0, 0, 0, 0);
          s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b1, s1, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float *row = sraw + (h * MQ + lhi * 4 + r) * SR;
          row[l16] = s0[r] * scale;
          row[16 + l16] = s1[r] * scale;
        }
      }
    }
    __syncthreads();
    // K is done with; V^T lands while the heads talk
    if (!piped)
      stage_vt_tile<D>(kvbuf, v_cache, bt, page, G, kv0, seq_len - 1, tid);
    // ---- mix + online softmax ----
    const bool full_tile = kv0 + MK - 1 <= past + tile * MQ &&
                           tile * MQ + MQ <= q_len;
    // every raw plane is read once and feeds all heads of this wave
    float svs[HPW][8];
#pragma unroll
    for (int hs = 0; hs < HPW; ++hs)
#pragma unroll
      for (int e = 0; e < 8; ++e) svs[hs][e] = 0.f;
#pragma unroll 2
    for (int g2 = 0; g2 < H; ++g2) {
      const float *row = sraw + (g2 * MQ + mi) * SR + mc * 8;
      const floatx4 a0 = *reinterpret_cast<const floatx4 *>(row);
      const floatx4 a1 = *reinterpret_cast<const floatx4 *>(row + 4);
#pragma unroll
      for (int hs = 0; hs < HPW; ++hs) {
        const int h = min(wave + hs * MWAVES, H - 1);
        const float t = tks[h * H + g2];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          svs[hs][e] += t * a0[e];
          svs[hs][4 + e] += t * a1[e];
        }
      }
    }
#pragma unroll
    for (int hs = 0; hs < HPW; ++hs) {
      const int h = wave + hs * MWAVES;
      if (h < H) {
        float sv[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) sv[e] = svs[hs][e];
        float mx = -INFINITY;
        if (full_tile) {   // every key visible to every row: no mask lanes
#pragma unroll
          for (int e = 0; e < 8; ++e) mx = fmaxf(mx, sv[e]);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int kvp = kv0 + mc * 8 + e;
            if (!qrow_m_ok || kvp > qpos_m || kvp >= seq_len)
              sv[e] = -INFINITY;
            mx = fmaxf(mx, sv[e]);
          }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 1, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 2, 64));
        const float m_old = m_run[hs];
        const float m_new = fmaxf(m_old, mx);
        float pv[8], psum = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          pv[e] = sv[e] == -INFINITY ? 0.f : __expf(sv[e] - m_new);
          psum += pv[e];
        }
        psum += __shfl_xor(psum, 1, 64);
        psum += __shfl_xor(psum, 2, 64);
        const float alpha = m_old == -INFINITY ? 0.f : __expf(m_old - m_new);
        l_run[hs] = l_run[hs] * alpha + psum;
        m_run[hs] = m_new;
        if (mc == 0) alpha_s[h * MQ + mi] = alpha;
        *reinterpret_cast<shortx8 *>(&pbuf[(h * MQ + mi) * PR + mc * 8]) =
            pack8<__hip_bfloat16>(pv);
      }
    }
    if (piped) {
      vt_tile_store<D>(kvbuf, vreg, G, tid);
      if (kv0 + MK < kv_max)
        k_tile_load<D>(kreg, k_cache, bt, page, G, kv0 + MK, seq_len - 1,
                       tid);
    }
    __syncthreads();
    // ---- O += P V ----
#pragma unroll
    for (int hs = 0; hs < HPW; ++hs) {
      const int h = wave + hs * MWAVES;
      if (h < H) {
        const int g = h / rep;
        float a4[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) a4[r] = alpha_s[h * MQ + lhi * 4 + r];
        const tk_bf8 pf = *reinterpret_cast<const tk_bf8 *>(
            &pbuf[(h * MQ + l16) * PR + lhi * 8]);
        const __hip_bfloat16 *vt = kvbuf + (g * D + l16) * VS + lhi * 8;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          const tk_bf8 vf =
              *reinterpret_cast<const tk_bf8 *>(vt + nt * 16 * VS);
          tk_f4 acc = o_acc[hs][nt];
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[r] *= a4[r];
          o_acc[hs][nt] =
              __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, vf, acc, 0, 0, 0);
        }
      }
    }
    __syncthreads();
  }

  // ---- epilogue: sink joins the denominator, rows leave as bf16 ----
#pragma unroll
  for (int hs = 0; hs < HPW; ++hs) {
    const int h = wave + hs * MWAVES;
    if (h < H && mc == 0) {
      float m = m_run[hs], l = l_run[hs], w = 1.f;
      if (sink != nullptr) {
        const float sk = sink[h];
        const float M = fmaxf(m, sk);
        w = m == -INFINITY ? 0.f : expf(m - M);
        l = l * w + expf(sk - M);
      }
      alpha_s[h * MQ + mi] = l > 0.f ? w / l : 0.f;
    }
  }
  __syncthreads();
#pragma unroll
  for (int hs = 0; hs < HPW; ++hs) {
    const int h = wave + hs * MWAVES;
    if (h < H) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int qrow = tile * MQ + lhi * 4 + r;
        if (qrow >= q_len) continue;
        const float f = alpha_s[h * MQ + lhi * 4 + r];
        __hip_bfloat16 *op = out + ((long)(q_start + qrow) * H + h) * D + l16;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          op[nt * 16] = __float2bfloat16(o_acc[hs][nt][r] * f);
      }
    }
  }
}

template <int D, int HPW>
bool launch_talking_mfma(torch::Tensor &out, torch::Tensor &q,
                         torch::Tensor &k_cache, torch::Tensor &v_cache,
                         torch::Tensor &block_table, torch::Tensor &seq_lens,
                         torch::Tensor &query_start_loc, double scale,
                         torch::Tensor &talk, const float *sink,
                         long max_query_len, int H, int G, int page) {
  constexpr size_t kv_elems = MK * (D + 8) > D * VS ? MK * (D + 8) : D * VS;
  const size_t lds = (size_t)G * kv_elems * 2 + (size_t)H * MQ * SR * 4 +
                     (size_t)H * MQ * PR * 2 + (size_t)H * MQ * 4 +
                     (size_t)H * H * 4;
  if (lds > 160 * 1024) return false;
  auto kern = talking_mfma_kernel<D, HPW>;
  if (lds > 48 * 1024) {
    static size_t granted = 0;   // per instantiation
    if (lds > granted) {
      if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                              hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)lds) != hipSuccess) {
        (void)hipGetLastError();
        return false;
      }
      granted = lds;
    }
  }
  const int B = seq_lens.numel();
  const int q_tiles = (int)((max_query_len + MQ - 1) / MQ);
  auto stream = at::cuda::getCurrentCUDAStream();
  hipLaunchKernelGGL(kern, dim3(q_tiles, B), dim3(MWAVES * 64), lds, stream,
                     (__hip_bfloat16 *)out.data_ptr(),
                     (const __hip_bfloat16 *)q.data_ptr(), (long)q.stride(0),
                     (const __hip_bfloat16 *)k_cache.data_ptr(),
                     (const __hip_bfloat16 *)v_cache.data_ptr(),
                     block_table.data_ptr<int>(), (int)block_table.stride(0),
                     seq_lens.data_ptr<int>(),
                     query_start_loc.data_ptr<int>(), H, G, page,
                     (float)scale, talk.data_ptr<float>(), sink);
  HIP_CHECK_KERNEL();
  return true;
}

}  // namespace

// false = this geometry has no MFMA instantiation (the caller runs the
// generic kernel)
bool talking_attention_mfma(torch::Tensor &out, torch::Tensor &q,
                            torch::Tensor &k_cache, torch::Tensor &v_cache,
                            torch::Tensor &block_table,
                            torch::Tensor &seq_lens,
                            torch::Tensor &query_start_loc, double scale,
                            torch::Tensor &talk, const float *sink,
                            long max_query_len) {
  const int page = k_cache.size(1), G = k_cache.size(2), D = k_cache.size(3);
  const int H = q.size(1) / D;
  if (v_cache.size(3) != D || H > 4 * MWAVES) return false;
  // 16 B fragment loads straight from q rows
  if (reinterpret_cast<uintptr_t>(q.data_ptr()) % 16 != 0 ||
      (q.stride(0) * 2) % 16 != 0)
    return false;
  const int hpw = H <= MWAVES ? 1 : H <= 2 * MWAVES ? 2 : 4;
#define GO(DV, HP)                                                          \
  return launch_talking_mfma<DV, HP>(out, q, k_cache, v_cache, block_table, \
                                     seq_lens, query_start_loc, scale,      \
                                     talk, sink, max_query_len, H, G, page)
#define GO_D(DV)                                                            \
  if (D == DV) {                                                            \
    if (hpw == 1) GO(DV, 1);                                                \
    if (hpw == 2) GO(DV, 2);                                                \
    GO(DV, 4);                                                              \
  }
  GO_D(32)
  GO_D(64)
  GO_D(96)
  GO_D(128)
#undef GO_D
#undef GO
  return false;
}

// ------------------------------------------------------------------
// bf16 decode-only batches (one new token per sequence). One workgroup =
// (token, key split); the rep = H / G heads that share a kv head are the
// MFMA rows, so a K/V tile is staged once and serves the whole group:
//   stage K tile [G][32][D] -> LDS; S_grp = Q_grp K_g^T (16x16x32 MFMA)
//   -> sraw[H][32]; stage V; mix + online softmax over the [H][32] plane
//   (thread = head x key, stats in LDS); P -> pbuf (bf16);
//   O_grp += P_grp V_g per (kv head, 16-column block) item, IT items per
//   wave. Partials go through talking_merge_kernel when keys are split.
namespace {

constexpr int DSR = 33;   // sraw row stride (floats)

template <int D, int IT>
__global__ __launch_bounds__(MWAVES * 64) void talking_decode_mfma_kernel(
    __hip_bfloat16 *__restrict__ out, float *__restrict__ part_acc,
    float *__restrict__ part_ml, const __hip_bfloat16 *__restrict__ q,
    long q_stride, const __hip_bfloat16 *__restrict__ k_cache,
    const __hip_bfloat16 *__restrict__ v_cache,
    const int *__restrict__ block_table, int bt_stride,
    const int *__restrict__ seq_lens, int H, int G, int page, float scale,
    const float *__restrict__ talk, const float *__restrict__ sink,
    int splits) {
  constexpr int KT = D / 32, NT = D / 16, KS = D + 8;
  extern __shared__ __attribute__((aligned(16))) char tk_lds[];
  __hip_bfloat16 *kvbuf = reinterpret_cast<__hip_bfloat16 *>(tk_lds);
  constexpr int KV_ELEMS = MK * KS > D * VS ? MK * KS : D * VS;
  float *sraw = reinterpret_cast<float *>(tk_lds + (size_t)G * KV_ELEMS * 2);
  __hip_bfloat16 *pbuf = reinterpret_cast<__hip_bfloat16 *>(
      sraw + (H * DSR + 3) / 4 * 4);
  float *alpha_s = reinterpret_cast<float *>(pbuf + H * PR);
  float *mrun = alpha_s + H;
  float *lrun = mrun + H;
  float *tks = lrun + H;

  const int t = blockIdx.x, sp = blockIdx.y;
  const int total = seq_lens[t];            // keys 0 .. position
  const int rep = H / G;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int l16 = lane & 15, lhi = lane >> 4;
  const int *bt = block_table + (long)t * bt_stride;
  const int tiles = (total + MK - 1) / MK;
  const int tiles_per = (tiles + splits - 1) / splits;
  const int j0 = sp * tiles_per * MK;
  const int j1 = min(total, j0 + tiles_per * MK);

  for (int d = tid; d < H * H; d += MWAVES * 64) tks[d] = talk[d];
  for (int h = tid; h < H; h += MWAVES * 64) {
    mrun[h] = -INFINITY;
    lrun[h] = 0.f;
  }
  tk_f4 o_acc[IT];
#pragma unroll
  for (int ii = 0; ii < IT; ++ii) o_acc[ii] = tk_f4{0, 0, 0, 0};
  const __hip_bfloat16 *qt = q + (long)t * q_stride;


  for (int kv0 = j0; kv0 < j1; kv0 += MK) {
    stage_k_tile<D>(kvbuf, k_cache, bt, page, G, kv0, total - 1, tid);
    __syncthreads();
    // ---- raw scores: item = (kv head, 16-key half) ----
    for (int it = wave; it < 2 * G; it += MWAVES) {
      const int g = it >> 1, f = it & 1;
      tk_f4 s = tk_f4{0, 0, 0, 0};
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) {
        tk_bf8 a = tk_bf8{0, 0, 0, 0, 0, 0, 0, 0};
        if (l16 < rep)
          a = *reinterpret_cast<const tk_bf8 *>(
              qt + (g * rep + l16) * D + kt * 32 + lhi * 8);
        const tk_bf8 bk = *reinterpret_cast<const tk_bf8 *>(
            &kvbuf[(g * MK + f * 16 + l16) * KS + kt * 32 + lhi * 8]);
        s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bk, s, 0, 0, 0);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (lhi * 4 + r < rep)
          sraw[(g * rep + lhi * 4 + r) * DSR + f * 16 + l16] = s[r] * scale;
    }
    __syncthreads();
    stage_vt_tile<D>(kvbuf, v_cache, bt, page, G, kv0, total - 1, tid);
    // ---- mix + online softmax: thread = (head, key) ----
    {
      const int key = tid & 31;
      const bool live = kv0 + key < j1;
      for (int h = tid >> 5; h < H; h += MWAVES * 2) {
        float sv = 0.f;
#pragma unroll 4
        for (int g2 = 0; g2 < H; ++g2)
          sv += tks[h * H + g2] * sraw[g2 * DSR + key];
        if (!live) sv = -INFINITY;
        float mx = sv;
#pragma unroll
        for (int off = 16; off > 0; off >>= 1)
          mx = fmaxf(mx, __shfl_xor(mx, off, 64));
        const float m_old = mrun[h];
        const float m_new = fmaxf(m_old, mx);
        const float p = live ? __expf(sv - m_new) : 0.f;
        float psum = p;
#pragma unroll
        for (int off = 16; off > 0; off >>= 1)
          psum += __shfl_xor(psum, off, 64);
        const float alpha = m_old == -INFINITY ? 0.f : __expf(m_old - m_new);
        pbuf[h * PR + key] = __float2bfloat16(p);
        if (key == 0) {
          mrun[h] = m_new;
          lrun[h] = lrun[h] * alpha + psum;
          alpha_s[h] = alpha;
        }
      }
    }
    __syncthreads();
    // ---- O += P V: item = (kv head, 16-column block) ----
#pragma unroll
    for (int ii = 0; ii < IT; ++ii) {
      const int it = wave + ii * MWAVES;
      if (it < G * NT) {
        const int g = it / NT, nt = it - g * NT;
        tk_bf8 pf = tk_bf8{0, 0, 0, 0, 0, 0, 0, 0};
        if (l16 < rep)
          pf = *reinterpret_cast<const tk_bf8 *>(
              &pbuf[(g * rep + l16) * PR + lhi * 8]);
        const tk_bf8 vf = *reinterpret_cast<const tk_bf8 *>(
            kvbuf + (g * D + nt * 16 + l16) * VS + lhi * 8);
        tk_f4 acc = o_acc[ii];
#pragma unroll
        for (int r = 0; r < 4; ++r)
          acc[r] *= lhi * 4 + r < rep ? alpha_s[g * rep + lhi * 4 + r] : 0.f;
        o_acc[ii] =
            __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, vf, acc, 0, 0, 0);
      }
    }
    __syncthreads();
  }

  // ---- epilogue ----
  if (splits == 1) {
    __syncthreads();
    for (int h = tid; h < H; h += MWAVES * 64) {
      float m = mrun[h], l = lrun[h], w = 1.f;
      if (sink != nullptr) {
        const float sk = sink[h];
        const float M = fmaxf(m, sk);
        w = m == -INFINITY ? 0.f : expf(m - M);
        l = l * w + expf(sk - M);
      }
      alpha_s[h] = l > 0.f ? w / l : 0.f;
    }
    __syncthreads();
  } else {
    __syncthreads();
    const long pbase = (long)t * splits + sp;
    for (int h = tid; h < H; h += MWAVES * 64) {
      part_ml[(pbase * H + h) * 2] = mrun[h];
      part_ml[(pbase * H + h) * 2 + 1] = lrun[h];
    }
  }
#pragma unroll
  for (int ii = 0; ii < IT; ++ii) {
    const int it = wave + ii * MWAVES;
    if (it < G * NT) {
      const int g = it / NT, nt = it - g * NT;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (lhi * 4 + r >= rep) continue;
        const int h = g * rep + lhi * 4 + r;
        const int col = h * D + nt * 16 + l16;
        if (splits == 1)
          out[(long)t * H * D + col] =
              __float2bfloat16(o_acc[ii][r] * alpha_s[h]);
        else
          part_acc[((long)t * splits + sp) * H * D + col] = o_acc[ii][r];
      }
    }
  }
}

template <int D, int IT>
bool launch_talking_decode(torch::Tensor &out, torch::Tensor &q,
                           torch::Tensor &k_cache, torch::Tensor &v_cache,
                           torch::Tensor &block_table,
                           torch::Tensor &seq_lens, double scale,
                           torch::Tensor &talk, const float *sink, int splits,
                           float *part_acc, float *part_ml, int H, int G,
                           int page) {
  const size_t sraw_f = ((size_t)H * DSR + 3) / 4 * 4;
  constexpr size_t kv_elems = MK * (D + 8) > D * VS ? MK * (D + 8) : D * VS;
  const size_t lds = (size_t)G * kv_elems * 2 + sraw_f * 4 +
                     (size_t)H * PR * 2 + (size_t)H * 3 * 4 +
                     (size_t)H * H * 4;
  if (lds > 160 * 1024) return false;
  auto kern = talking_decode_mfma_kernel<D, IT>;
  if (lds > 48 * 1024) {
    static size_t granted = 0;
    if (lds > granted) {
      if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                              hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)lds) != hipSuccess) {
        (void)hipGetLastError();
        return false;
      }
      granted = lds;
    }
  }
  const int B = seq_lens.numel();
  auto stream = at::cuda::getCurrentCUDAStream();
  hipLaunchKernelGGL(kern, dim3(B, splits), dim3(MWAVES * 64), lds, stream,
                     (__hip_bfloat16 *)out.data_ptr(), part_acc, part_ml,
                     (const __hip_bfloat16 *)q.data_ptr(), (long)q.stride(0),
                     (const __hip_bfloat16 *)k_cache.data_ptr(),
                     (const __hip_bfloat16 *)v_cache.data_ptr(),
                     block_table.data_ptr<int>(), (int)block_table.stride(0),
                     seq_lens.data_ptr<int>(), H, G, page, (float)scale,
                     talk.data_ptr<float>(), sink, splits);
  HIP_CHECK_KERNEL();
  return true;
}

}  // namespace

bool talking_attention_decode_mfma(torch::Tensor &out, torch::Tensor &q,
                                   torch::Tensor &k_cache,
                                   torch::Tensor &v_cache,
                                   torch::Tensor &block_table,
                                   torch::Tensor &seq_lens, double scale,
                                   torch::Tensor &talk, const float *sink,
                                   int splits, float *part_acc,
                                   float *part_ml) {
  const int page = k_cache.size(1), G = k_cache.size(2), D = k_cache.size(3);
  const int H = q.size(1) / D;
  if (v_cache.size(3) != D || H / G > 16) return false;
  if (reinterpret_cast<uintptr_t>(q.data_ptr()) % 16 != 0 ||
      (q.stride(0) * 2) % 16 != 0)
    return false;
  const int items = (G * (D / 16) + MWAVES - 1) / MWAVES;
  if (items > 16) return false;
  const int itc = items <= 2 ? 2 : items <= 4 ? 4 : items <= 8 ? 8 : 16;
#define GO(DV, I)                                                          \
  return launch_talking_decode<DV, I>(out, q, k_cache, v_cache,            \
                                      block_table, seq_lens, scale, talk,  \
                                      sink, splits, part_acc, part_ml, H,  \
                                      G, page)
#define GO_D(DV)                                                           \
  if (D == DV) {                                                           \
    if (itc == 2) GO(DV, 2);                                               \
    if (itc == 4) GO(DV, 4);                                               \
    if (itc == 8) GO(DV, 8);                                               \
    GO(DV, 16);                                                            \
  }
  GO_D(32)
  GO_D(64)
  GO_D(96)
  GO_D(128)
#undef GO_D
#undef GO
  return false;
}
