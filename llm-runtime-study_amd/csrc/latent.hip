// Latent attention: every position keeps one row [rank latent values | rot rotated key values] that all
// query heads share.  A head's key is a matrix times the latent values, and so is its value; both matrices are
// moved to the query's side, so that the kernels here work on the rows as they are kept:
//
//   query row of head h   [ W_uk[h]^T q_plain[h]  (rank) | rotated q part (rot) ]
//   score                 (query row . kept row) * scale
//   weights               softmax over the causal keys, with one more term exp(sink[h]) in the denominator
//                         that has no key and no value
//   latent output         sum of weight * kept row[:rank], times sigmoid(gate[h])
//   head output           W_uv[h] latent output
//
//   latent_prep       per token: RMS norm of the projected latent values and rotation of the shared key part,
//                     both written into the token's row of the pages; rotation of every head's rotated query part
//                     into the query rows.  Pairs (2i, 2i + 1) are rotated (the interleaved layout).
//   head_gemm         a small product per (token, head), with a matrix of the head's own: the two steps above that
//                     move between a head's own dims and the latent ones.
//   latent_attention  scores, softmax with the sink, weighted sum of latent rows and the gate.
//
// Scores, weights, sums, norms and rotations are float32.  Key tiles start at multiples of the tile size counted
// from position 0 and every sum runs in the order of its index, so a query's result depends on its position alone.
#include "common.h"

namespace {

// ------------------------------------------------------------------ preparation
template <typename T, typename TW>
__global__ __launch_bounds__(256) void latent_prep_kernel(
    const T* __restrict__ proj, int proj_stride, int q_col, int kv_col, int heads, int dim, int rot, int rank,
    const TW* __restrict__ norm_weight, float eps, const float* __restrict__ cosv, const float* __restrict__ sinv,
    T* __restrict__ pages, const int* __restrict__ slots, T* __restrict__ queries, int query_stride) {
  __shared__ float scratch[16];
  const int token = blockIdx.x, tid = threadIdx.x, half = rot / 2, width = rank + rot;
  const T* row = proj + (int64_t)token * proj_stride;
  const T* latent = row + kv_col;
  const int slot = slots[token];
  float ss = 0.f;
  for (int i = tid; i < rank; i += blockDim.x) {
    const float v = to_float(latent[i]);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)rank + eps);
  if (slot >= 0) {
    T* kept = pages + (int64_t)slot * width;
    for (int i = tid; i < rank; i += blockDim.x) kept[i] = from_float<T>(to_float(latent[i]) * inv * to_float(norm_weight[i]));
    for (int i = tid; i < half; i += blockDim.x) {
      const float u = to_float(latent[rank + 2 * i]), v = to_float(latent[rank + 2 * i + 1]);
      const float c = cosv ? cosv[(int64_t)token * half + i] : 1.f, s = sinv ? sinv[(int64_t)token * half + i] : 0.f;
      kept[rank + 2 * i] = from_float<T>(u * c - v * s);
      kept[rank + 2 * i + 1] = from_float<T>(v * c + u * s);
    }
    if (rot % 2 && tid == 0) kept[width - 1] = latent[width - 1];
  }
  for (int i = tid; i < heads * half; i += blockDim.x) {
    const int h = i / half, p = i % half;
    const T* q = row + q_col + (int64_t)h * (dim + rot) + dim;
    const float u = to_float(q[2 * p]), v = to_float(q[2 * p + 1]);
    const float c = cosv ? cosv[(int64_t)token * half + p] : 1.f, s = sinv ? sinv[(int64_t)token * half + p] : 0.f;
    T* dst = queries + (int64_t)token * query_stride + (int64_t)h * width + rank;
    dst[2 * p] = from_float<T>(u * c - v * s);
    dst[2 * p + 1] = from_float<T>(v * c + u * s);
  }
  if (rot % 2)
    for (int h = tid; h < heads; h += blockDim.x)
      queries[(int64_t)token * query_stride + (int64_t)h * width + width - 1] = row[q_col + (int64_t)h * (dim + rot) + dim + rot - 1];
}

// ------------------------------------------------------------------ per-head products
// out[t, h, j] = sum over k of a[t, h, k] * w[h](j, k); the head's matrix is stored [n, k] (TRANS false) or [k, n]
// (TRANS true).  A workgroup takes TT tokens of one head; the sum runs in the order of k.
constexpr int HG_TOKENS = 8;

template <typename T, bool TRANS>
__global__ __launch_bounds__(256) void head_gemm_kernel(T* __restrict__ out, int out_token, int out_head, const T* __restrict__ a,
                                                        int a_token, int a_head, const T* __restrict__ w, int64_t w_head, int tokens,
                                                        int n, int k) {
  extern __shared__ __attribute__((aligned(16))) float rows[];     // [HG_TOKENS][k]
  const int t0 = blockIdx.x * HG_TOKENS, h = blockIdx.y, tid = threadIdx.x;
  const int count = min(HG_TOKENS, tokens - t0);
  for (int i = tid; i < HG_TOKENS * k; i += blockDim.x) {
    const int t = i / k, c = i % k;
    rows[i] = t < count ? to_float(a[(int64_t)(t0 + t) * a_token + (int64_t)h * a_head + c]) : 0.f;
  }
  __syncthreads();
  const T* wh = w + (int64_t)h * w_head;
  for (int j = tid; j < n; j += blockDim.x) {
    float acc[HG_TOKENS];
#pragma unroll
    for (int t = 0; t < HG_TOKENS; ++t) acc[t] = 0.f;
    for (int c = 0; c < k; ++c) {
      const float wv = to_float(TRANS ? wh[(int64_t)c * n + j] : wh[(int64_t)j * k + c]);
#pragma unroll
      for (int t = 0; t < HG_TOKENS; ++t) acc[t] = fmaf(rows[t * k + c], wv, acc[t]);
    }
#pragma unroll
    for (int t = 0; t < HG_TOKENS; ++t)
      if (t < count) out[(int64_t)(t0 + t) * out_token + (int64_t)h * out_head + j] = from_float<T>(acc[t]);
  }
}

// ------------------------------------------------------------------ attention, any shape
// One workgroup per (query token, head).  rank <= MAX_OUT * THREADS.
constexpr int LA_THREADS = 128, LA_MAX_OUT = 8;

template <typename T>
__global__ __launch_bounds__(LA_THREADS) void latent_attention_kernel(
    T* __restrict__ out, int out_stride, const T* __restrict__ queries, int query_stride, const T* __restrict__ pages,
    const int* __restrict__ block_table, int table_stride, const int* __restrict__ token_request, const int* __restrict__ positions,
    const float* __restrict__ sink, const T* __restrict__ gate, int gate_stride, int heads, int rank, int width, int page_size,
    float scale, int window) {
  constexpr int THREADS = LA_THREADS;
  extern __shared__ __attribute__((aligned(16))) float smem[];
  float* qs = smem;                              // [width]
  float* probs = qs + width + width % 2;         // [THREADS]
  int64_t* bases = (int64_t*)(probs + THREADS);  // [THREADS] element offset of each key's row
  __shared__ float scratch[16];

  const int token = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
  const int request = token_request[token];
  const int pos = positions[token];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int* table = block_table + (int64_t)request * table_stride;
  for (int i = tid; i < width; i += THREADS) qs[i] = to_float(queries[(int64_t)token * query_stride + (int64_t)head * width + i]);
  __syncthreads();

  float acc[LA_MAX_OUT];
#pragma unroll
  for (int c = 0; c < LA_MAX_OUT; ++c) acc[c] = 0.f;
  float running_max = -INFINITY, running_sum = 0.f;
  const bool wide = (width * sizeof(T)) % 16 == 0 && ((uintptr_t)pages % 16) == 0;
  for (int tile = (lo / THREADS) * THREADS; tile <= pos; tile += THREADS) {
    const int key = tile + tid;
    const bool valid = key >= lo && key <= pos;
    float score = -INFINITY;
    int64_t base = 0;
    if (valid) {
      const int64_t page = table[key / page_size];
      base = (page * page_size + key % page_size) * (int64_t)width;
      const T* kr = pages + base;
      float dot = 0.f;
      if (wide) {
        constexpr int PER = 16 / sizeof(T);
        typedef T vec_t __attribute__((ext_vector_type(PER)));
        for (int i = 0; i < width; i += PER) {
          const vec_t kv = *(const vec_t*)(kr + i);
#pragma unroll
          for (int e = 0; e < PER; ++e) dot = fmaf(qs[i + e], to_float(kv[e]), dot);
        }
      } else {
        for (int i = 0; i < width; ++i) dot = fmaf(qs[i], to_float(kr[i]), dot);
      }
      score = dot * scale;
    }
    const float tile_max = block_max(score, scratch);
    const float new_max = fmaxf(running_max, tile_max);
    const float p = valid ? expf(score - new_max) : 0.f;
    const float tile_sum = block_sum(p, scratch);
    const float alpha = expf(running_max - new_max);  // exp(-inf) = 0 on the first tile
    running_sum = running_sum * alpha + tile_sum;
    running_max = new_max;
    probs[tid] = p;
    bases[tid] = base;
    __syncthreads();
    const int count = (pos - tile + 1 < THREADS) ? pos - tile + 1 : THREADS;
#pragma unroll
    for (int c = 0; c < LA_MAX_OUT; ++c) {
      const int dim = tid + c * THREADS;
      if (dim < rank) {
        float a = acc[c] * alpha;
        for (int j = 0; j < count; ++j) {
          const float pj = probs[j];
          if (pj != 0.f) a = fmaf(pj, to_float(pages[bases[j] + dim]), a);
        }
        acc[c] = a;
      }
    }
    __syncthreads();
  }
  // the sink: one more term of the denominator, with no key and no value
  float denominator = running_sum;
  if (sink) {
    const float s = sink[head];
    const float m = fmaxf(running_max, s);
    const float shrink = expf(running_max - m);
    denominator = running_sum * shrink + expf(s - m);
#pragma unroll
    for (int c = 0; c < LA_MAX_OUT; ++c) acc[c] *= shrink;
  }
  float factor = 1.0f / denominator;
  if (gate) factor *= 1.0f / (1.0f + expf(-to_float(gate[(int64_t)token * gate_stride + head])));
#pragma unroll
  for (int c = 0; c < LA_MAX_OUT; ++c) {
    const int dim = tid + c * THREADS;
    if (dim < rank) out[(int64_t)token * out_stride + (int64_t)head * rank + dim] = from_float<T>(acc[c] * factor);
  }
}

}  // namespace

// proj [tokens, >= columns] holds, per token, the heads' queries from column q_col on ([dim plain | rot rotated] a head)
// and [rank latent | rot shared key] from column kv_col on.  pages [P, page, rank + rot]; slots[t] the token's row
// (negative: not kept).  queries [tokens, heads, rank + rot]: the rotated parts are written, the others left.
LRS_API int lrs_latent_prep(const void* proj, int proj_stride, int dtype, int tokens, int q_col, int kv_col, int heads, int dim, int rot,
                            int rank, const void* norm_weight, int weight_dtype, float eps, const float* cosv, const float* sinv,
                            void* pages, const int* slots, void* queries, int query_stride, void* stream) {
  LRS_REQUIRE(tokens > 0 && heads > 0 && dim >= 0 && rot >= 0 && rank > 0, "latent_prep: bad sizes tokens=%d heads=%d dim=%d rot=%d rank=%d", tokens, heads,
              dim, rot, rank);
  LRS_REQUIRE(eps > 0.f, "latent_prep: eps must be positive");
  LRS_REQUIRE((cosv == nullptr) == (sinv == nullptr), "latent_prep: cos and sin come together");
  hipStream_t s = (hipStream_t)stream;
#define LRS_PREP(T, TW)                                                                                                              \
  latent_prep_kernel<T, TW><<<tokens, 256, 0, s>>>((const T*)proj, proj_stride, q_col, kv_col, heads, dim, rot, rank, (const TW*)norm_weight, \
                                                   eps, cosv, sinv, (T*)pages, slots, (T*)queries, query_stride)
  if (dtype == LRS_F32 && weight_dtype == LRS_F32) LRS_PREP(float, float);
  else if (dtype == LRS_F32 && weight_dtype == LRS_BF16) LRS_PREP(float, bf16);
  else if (dtype == LRS_BF16 && weight_dtype == LRS_F32) LRS_PREP(bf16, float);
  else if (dtype == LRS_BF16 && weight_dtype == LRS_BF16) LRS_PREP(bf16, bf16);
  else return lrs_fail("latent_prep: unknown dtypes %d %d", dtype, weight_dtype);
#undef LRS_PREP
  return lrs_check_launch("latent_prep");
}

// out[t, h, :n] = w[h] a[t, h, :k] with w[h] stored [n, k] (trans 0) or [k, n] (trans 1), w_head elements from one head's
// matrix to the next; strides in elements.
LRS_API int lrs_head_gemm(void* out, int out_token, int out_head, const void* a, int a_token, int a_head, const void* w, int64_t w_head,
                          int trans, int dtype, int tokens, int heads, int n, int k, void* stream) {
  LRS_REQUIRE(tokens > 0 && heads > 0 && n > 0 && k > 0, "head_gemm: bad sizes tokens=%d heads=%d n=%d k=%d", tokens, heads, n, k);
  LRS_REQUIRE(heads <= 65535, "head_gemm: at most 65535 heads");
  LRS_REQUIRE(k <= 4096, "head_gemm: k %d above the supported 4096", k);
  const dim3 grid((tokens + HG_TOKENS - 1) / HG_TOKENS, heads);
  const size_t lds = sizeof(float) * HG_TOKENS * k;
  hipStream_t s = (hipStream_t)stream;
#define LRS_HG(T, TR) \
  head_gemm_kernel<T, TR><<<grid, 256, lds, s>>>((T*)out, out_token, out_head, (const T*)a, a_token, a_head, (const T*)w, w_head, tokens, n, k)
  if (dtype == LRS_F32) { if (trans) LRS_HG(float, true); else LRS_HG(float, false); }
  else if (dtype == LRS_BF16) { if (trans) LRS_HG(bf16, true); else LRS_HG(bf16, false); }
  else return lrs_fail("head_gemm: unknown dtype %d", dtype);
#undef LRS_HG
  return lrs_check_launch("head_gemm");
}

// out [tokens, heads * rank]; queries [tokens, heads, width]; pages [P, page, width]; gate (may be null) holds a head's
// gate at gate[t * gate_stride + h]; sink (may be null) [heads] float32.
LRS_API int lrs_latent_attention(void* out, int out_stride, const void* queries, int query_stride, const void* pages, const int* block_table,
                                 int table_stride, const int* token_request, const int* positions, const float* sink, const void* gate,
                                 int gate_stride, int dtype, int tokens, int heads, int rank, int width, int page_size, float scale, int window,
                                 void* stream) {
  LRS_REQUIRE(tokens > 0 && heads > 0 && rank > 0 && width >= rank && page_size > 0, "latent_attention: bad sizes tokens=%d heads=%d rank=%d width=%d page=%d",
              tokens, heads, rank, width, page_size);
  LRS_REQUIRE(rank <= LA_THREADS * LA_MAX_OUT, "latent_attention: rank %d above the supported %d", rank, LA_THREADS * LA_MAX_OUT);
  LRS_REQUIRE(heads <= 65535 && window >= 0, "latent_attention: at most 65535 heads, window >= 0 (0 = none)");
  const dim3 grid(tokens, heads);
  const size_t lds = sizeof(float) * (width + width % 2 + LA_THREADS) + sizeof(int64_t) * LA_THREADS;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == LRS_F32)
    latent_attention_kernel<float><<<grid, LA_THREADS, lds, s>>>((float*)out, out_stride, (const float*)queries, query_stride, (const float*)pages,
                                                                 block_table, table_stride, token_request, positions, sink, (const float*)gate,
                                                                 gate_stride, heads, rank, width, page_size, scale, window);
  else if (dtype == LRS_BF16)
    latent_attention_kernel<bf16><<<grid, LA_THREADS, lds, s>>>((bf16*)out, out_stride, (const bf16*)queries, query_stride, (const bf16*)pages,
                                                                block_table, table_stride, token_request, positions, sink, (const bf16*)gate,
                                                                gate_stride, heads, rank, width, page_size, scale, window);
  else
    return lrs_fail("latent_attention: unknown dtype %d", dtype);
  return lrs_check_launch("latent_attention");
}
