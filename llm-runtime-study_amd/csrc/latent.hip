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
    T* __restrict__ pages, T* __restrict__ value_pages, int page_size, const int* __restrict__ slots, T* __restrict__ queries,
    int query_stride) {
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
    // value_pages: the latent values once more, transposed inside a page ([page, rank, slot]), for the kernel that wants the
    // keys of one latent column side by side
    T* across = value_pages ? value_pages + (int64_t)(slot / page_size) * rank * page_size + slot % page_size : nullptr;
    for (int i = tid; i < rank; i += blockDim.x) {
      const T v = from_float<T>(to_float(latent[i]) * inv * to_float(norm_weight[i]));
      kept[i] = v;
      if (across) across[(int64_t)i * page_size] = v;
    }
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


// ------------------------------------------------------------------ per-head products on the matrix cores
// bfloat16, w[h] stored [n, k]: a wave makes 16 tokens x 64 outputs with both operands straight from memory (16 bytes a lane).
__global__ __launch_bounds__(256) void head_gemm_bf16_kernel(bf16* __restrict__ out, int out_token, int out_head, const bf16* __restrict__ a,
                                                             int a_token, int a_head, const bf16* __restrict__ w, int64_t w_head, int tokens,
                                                             int n, int k) {
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, col = lane & 15, g = lane >> 4;
  const int h = blockIdx.z, n0 = blockIdx.y * 64, t0 = blockIdx.x * 64 + wave * 16;
  if (t0 >= tokens) return;
  const int t = t0 + col;
  const bf16* a_row = a + (int64_t)(t < tokens ? t : tokens - 1) * a_token + (int64_t)h * a_head + g * 8;
  const bf16* w_row = w + (int64_t)h * w_head + (int64_t)(n0 + col) * k + g * 8;
  floatx4 acc[4] = {};
  const bf16x8 zero = {};
  constexpr int KC = 4;       // products of 32 inputs whose operands are asked for together
  for (int ks = 0; ks < k; ks += 32 * KC) {
    bf16x8 af[KC], wf[KC][4];
#pragma unroll
    for (int u = 0; u < KC; ++u) {
      const bool inside = ks + 32 * u + g * 8 < k;
      af[u] = inside ? *(const bf16x8*)(a_row + ks + 32 * u) : zero;
#pragma unroll
      for (int c = 0; c < 4; ++c) wf[u][c] = inside && n0 + col + 16 * c < n ? *(const bf16x8*)(w_row + (int64_t)16 * c * k + ks + 32 * u) : zero;
    }
#pragma unroll
    for (int u = 0; u < KC; ++u)
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[u], wf[u][c], acc[c], 0, 0, 0);
  }
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = t0 + 4 * g + i, nn = n0 + 16 * c + col;
      if (row < tokens && nn < n) out[(int64_t)row * out_token + (int64_t)h * out_head + nn] = (bf16)acc[c][i];
    }
}

// ------------------------------------------------------------------ attention on the matrix cores
// bfloat16.  The rows of a query group (consecutive tokens of one request) are its (token, head) pairs, token by token;
// a wave takes 16 of them and walks the request's kept rows in tiles of 32 keys, every operand straight from memory:
//   scores   [16 rows x 32 keys]   = query rows . kept rows      (pages [P, page, width]: a key's values side by side)
//   output   [16 rows x rank]     += weights . latent values     (value pages [P, rank, page]: a column's keys side by side)
// The weights pass through a small piece of LDS of the wave's own on their way from the layout products leave to the one
// they take.  The four waves of a workgroup read the same keys.  Key tiles start at multiples of 32 from position 0.  With
// splits > 1 a workgroup walks one part of the tiles and leaves its maximum, sum and unscaled output for the merge.
constexpr float LOG2E = 1.4426950408889634f;
constexpr int LATENT_KC = 9, LATENT_VC = 16;

template <int CT>   // tiles of 16 latent columns: rank <= 16 * CT
__global__ __launch_bounds__(256) void latent_attention_bf16_kernel(
    bf16* __restrict__ out, int out_stride, float* __restrict__ part_o, float* __restrict__ part_ml, const bf16* __restrict__ queries,
    int query_stride, const bf16* __restrict__ pages, const bf16* __restrict__ value_pages, const int* __restrict__ block_table,
    int table_stride, const int* __restrict__ token_request, const int* __restrict__ positions, const int* __restrict__ group_token0,
    const int* __restrict__ group_count, const float* __restrict__ sink, const bf16* __restrict__ gate, int gate_stride, int heads, int rank,
    int width, int page_size, float scale, int window, int splits) {
  __shared__ __attribute__((aligned(16))) bf16 weights_lds[4][16][40];
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, col = lane & 15, g = lane >> 4;
  const int group = blockIdx.x, split = blockIdx.z;
  const int token0 = group_token0 ? group_token0[group] : group;
  const int rows = (group_count ? group_count[group] : 1) * heads;
  const int row0 = (blockIdx.y * 4 + wave) * 16;
  if (row0 >= rows) return;                     // the kernel has no barrier: a wave without rows leaves
  const int last_row = row0 + 15 < rows ? row0 + 15 : rows - 1;
  const int* table = block_table + (int64_t)token_request[token0] * table_stride;
  const int pos_first = positions[token0 + row0 / heads], pos_last = positions[token0 + last_row / heads];
  const int lo = (window > 0 && pos_first - window + 1 > 0) ? pos_first - window + 1 : 0;
  const int first_tile = lo / 32, last_tile = pos_last / 32;
  const int per_split = (last_tile - first_tile + splits) / splits;
  const int tile_begin = first_tile + split * per_split;
  const int tile_end = tile_begin + per_split <= last_tile + 1 ? tile_begin + per_split : last_tile + 1;

  // the row this lane feeds into the score products, and the four rows whose results it holds
  const int a_row = row0 + col;
  const bool a_valid = a_row < rows;
  const bf16* q_row = queries + (int64_t)(token0 + (a_valid ? a_row / heads : 0)) * query_stride + (int64_t)(a_valid ? a_row % heads : 0) * width + g * 8;
  int c_pos[4], c_lo[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = row0 + 4 * g + i;
    c_pos[i] = r < rows ? positions[token0 + r / heads] : -1;
    c_lo[i] = (window > 0 && c_pos[i] - window + 1 > 0) ? c_pos[i] - window + 1 : 0;
  }
  const float scale2 = scale * LOG2E;
  float top[4], total[4];
  floatx4 acc[CT];
#pragma unroll
  for (int i = 0; i < 4; ++i) top[i] = -INFINITY, total[i] = 0.f;
#pragma unroll
  for (int c = 0; c < CT; ++c) acc[c] = floatx4{0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = {};

  // the pages of a tile's keys are looked up a tile ahead: page_a / page_b of the keys whose kept rows this lane brings to the
  // scores (key0 + col, key0 + 16 + col), page_v of the eight keys whose latent values it brings to the weighted sum
  auto page_of = [&](int first_key, int last_key) -> int {
    return last_key >= lo && first_key <= pos_last ? table[first_key / page_size] : -1;
  };
  int next_a = -1, next_b = -1, next_v = -1;
  if (tile_begin < tile_end) {
    next_a = page_of(tile_begin * 32 + col, tile_begin * 32 + col);
    next_b = page_of(tile_begin * 32 + 16 + col, tile_begin * 32 + 16 + col);
    next_v = page_of(tile_begin * 32 + 8 * g, tile_begin * 32 + 8 * g + 7);
  }
  constexpr int KC = LATENT_KC;      // products of 32 dims whose operands are asked for together: a wave waits for memory once a chunk
  for (int tile = tile_begin; tile < tile_end; ++tile) {
    const int key0 = tile * 32;
    const int key_a = key0 + col, key_b = key_a + 16;
    const int page_a = next_a, page_b = next_b, page_v = next_v;
    if (tile + 1 < tile_end) {
      next_a = page_of(key_a + 32, key_a + 32);
      next_b = page_of(key_b + 32, key_b + 32);
      next_v = page_of(key0 + 32 + 8 * g, key0 + 32 + 8 * g + 7);
    }
    const bf16* row_a = pages + ((int64_t)(page_a < 0 ? 0 : page_a) * page_size + key_a % page_size) * width + g * 8;
    const bf16* row_b = pages + ((int64_t)(page_b < 0 ? 0 : page_b) * page_size + key_b % page_size) * width + g * 8;
    floatx4 s_a = {0.f, 0.f, 0.f, 0.f}, s_b = {0.f, 0.f, 0.f, 0.f};
    for (int ks = 0; ks < width; ks += 32 * KC) {
      bf16x8 qf[KC], ka[KC], kb[KC];
#pragma unroll
      for (int u = 0; u < KC; ++u) {
        const bool inside = ks + 32 * u + g * 8 < width;
        qf[u] = inside && a_valid ? *(const bf16x8*)(q_row + ks + 32 * u) : zero;
        ka[u] = inside && page_a >= 0 ? *(const bf16x8*)(row_a + ks + 32 * u) : zero;
        kb[u] = inside && page_b >= 0 ? *(const bf16x8*)(row_b + ks + 32 * u) : zero;
      }
#pragma unroll
      for (int u = 0; u < KC; ++u) {
        s_a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[u], ka[u], s_a, 0, 0, 0);
        s_b = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[u], kb[u], s_b, 0, 0, 0);
      }
    }
    // the running softmax of the lane's four rows (a row's 32 scores lie in the 16 lanes that share g)
    float shrink[4];
    bf16 w_a[4], w_b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool see_a = page_a >= 0 && key_a <= c_pos[i] && key_a >= c_lo[i], see_b = page_b >= 0 && key_b <= c_pos[i] && key_b >= c_lo[i];
      const float v_a = see_a ? s_a[i] * scale2 : -INFINITY, v_b = see_b ? s_b[i] * scale2 : -INFINITY;
      float most = fmaxf(v_a, v_b);
#pragma unroll
      for (int off = 8; off > 0; off >>= 1) most = fmaxf(most, __shfl_xor(most, off, WAVE));
      const float now = fmaxf(top[i], most);
      const float ref = now == -INFINITY ? 0.f : now;        // a row that has seen no key yet
      const float e_a = __builtin_amdgcn_exp2f(v_a - ref), e_b = __builtin_amdgcn_exp2f(v_b - ref);
      float sum = e_a + e_b;
#pragma unroll
      for (int off = 8; off > 0; off >>= 1) sum += __shfl_xor(sum, off, WAVE);
      shrink[i] = __builtin_amdgcn_exp2f(top[i] - ref);      // 0 while the old maximum is -inf
      total[i] = total[i] * shrink[i] + sum;
      top[i] = now;
      w_a[i] = (bf16)e_a;
      w_b[i] = (bf16)e_b;
    }
    // the weights from the layout the products left them in (rows 4g + i, key col) to the one they are taken in (row col, keys 8g ..)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      weights_lds[wave][4 * g + i][col] = w_a[i];
      weights_lds[wave][4 * g + i][16 + col] = w_b[i];
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    const bf16x8 pf = *(const bf16x8*)&weights_lds[wave][col][8 * g];
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    // the weighted sum: this lane brings, per tile of 16 columns, the latent values of column col at keys key0 + 8g .. + 7
    const int key_v = key0 + 8 * g;
    const bf16* column = value_pages + ((int64_t)(page_v < 0 ? 0 : page_v) * rank + col) * page_size + key_v % page_size;
    const bool rescale = shrink[0] != 1.f || shrink[1] != 1.f || shrink[2] != 1.f || shrink[3] != 1.f;
    constexpr int VC = CT % LATENT_VC == 0 ? LATENT_VC : CT % 6 == 0 ? 6 : CT % 4 == 0 ? 4 : 2;      // column tiles whose values are asked for together
#pragma unroll
    for (int c0 = 0; c0 < CT; c0 += VC) {
      bf16x8 vf[VC];
#pragma unroll
      for (int u = 0; u < VC; ++u)
        vf[u] = page_v >= 0 && 16 * (c0 + u) + col < rank ? *(const bf16x8*)(column + (int64_t)16 * (c0 + u) * page_size) : zero;
#pragma unroll
      for (int u = 0; u < VC; ++u) {
        if (rescale) {
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[c0 + u][i] *= shrink[i];
        }
        acc[c0 + u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, vf[u], acc[c0 + u], 0, 0, 0);
      }
    }
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = row0 + 4 * g + i;
    if (r >= rows) continue;
    const int token = token0 + r / heads, head = r % heads;
    if (splits > 1) {
      const int64_t at = ((int64_t)token * heads + head) * splits + split;
      if (col == 0) {
        part_ml[at * 2] = top[i];
        part_ml[at * 2 + 1] = total[i];
      }
#pragma unroll
      for (int c = 0; c < CT; ++c)
        if (16 * c + col < rank) part_o[at * rank + 16 * c + col] = acc[c][i];
      continue;
    }
    // the sink, one more term of the denominator, and the gate
    float most = top[i], denominator = total[i], shrunk = 1.f;
    if (sink) {
      const float s2 = sink[head] * LOG2E;
      most = fmaxf(top[i], s2);
      shrunk = __builtin_amdgcn_exp2f(top[i] - most);
      denominator = total[i] * shrunk + __builtin_amdgcn_exp2f(s2 - most);
    }
    float factor = shrunk / denominator;
    if (gate) factor *= 1.0f / (1.0f + expf(-(float)gate[(int64_t)token * gate_stride + head]));
#pragma unroll
    for (int c = 0; c < CT; ++c)
      if (16 * c + col < rank) out[(int64_t)token * out_stride + (int64_t)head * rank + 16 * c + col] = (bf16)(acc[c][i] * factor);
  }
}

// What the parts of one (token, head) left, put together: maxima and sums in powers of two.
__global__ __launch_bounds__(256) void latent_merge_kernel(bf16* __restrict__ out, int out_stride, const float* __restrict__ part_o,
                                                           const float* __restrict__ part_ml, const float* __restrict__ sink,
                                                           const bf16* __restrict__ gate, int gate_stride, int heads, int rank, int splits) {
  __shared__ float weight[64];          // of each part: 2^(its maximum - the maximum of all), over the denominator, times the gate
  const int token = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int64_t base = ((int64_t)token * heads + head) * splits;
  if (lane < WAVE) {                    // the first wave: a part a lane (splits <= 64)
    const float mine = lane < splits ? part_ml[(base + lane) * 2] : -INFINITY;
    const float sum = lane < splits ? part_ml[(base + lane) * 2 + 1] : 0.f;
    const float s2 = sink ? sink[head] * LOG2E : -INFINITY;
    const float most = fmaxf(wave_max(mine), s2);
    const float w = __builtin_amdgcn_exp2f(mine - most);
    const float denominator = wave_sum(sum * w) + (sink ? __builtin_amdgcn_exp2f(s2 - most) : 0.f);
    float factor = 1.0f / denominator;
    if (gate) factor *= 1.0f / (1.0f + expf(-(float)gate[(int64_t)token * gate_stride + head]));
    weight[lane] = w * factor;
  }
  __syncthreads();
  constexpr int AT_ONCE = 8;            // parts whose sums are asked for together
  for (int dim = lane; dim < rank; dim += blockDim.x) {
    float sum = 0.f;
    for (int s0 = 0; s0 < splits; s0 += AT_ONCE) {
      float o[AT_ONCE];
#pragma unroll
      for (int i = 0; i < AT_ONCE; ++i) o[i] = part_o[(base + (s0 + i < splits ? s0 + i : splits - 1)) * rank + dim];
#pragma unroll
      for (int i = 0; i < AT_ONCE; ++i)
        if (s0 + i < splits) sum = fmaf(o[i], weight[s0 + i], sum);
    }
    out[(int64_t)token * out_stride + (int64_t)head * rank + dim] = (bf16)sum;
  }
}

}  // namespace

// proj [tokens, >= columns] holds, per token, the heads' queries from column q_col on ([dim plain | rot rotated] a head)
// and [rank latent | rot shared key] from column kv_col on.  pages [P, page, rank + rot]; value_pages (may be null)
// [P, rank, page]; slots[t] the token's row (negative: not kept).  queries [tokens, heads, rank + rot]: the rotated parts are written, the others left.
LRS_API int lrs_latent_prep(const void* proj, int proj_stride, int dtype, int tokens, int q_col, int kv_col, int heads, int dim, int rot,
                            int rank, const void* norm_weight, int weight_dtype, float eps, const float* cosv, const float* sinv,
                            void* pages, void* value_pages, int page_size, const int* slots, void* queries, int query_stride, void* stream) {
  LRS_REQUIRE(tokens > 0 && heads > 0 && dim >= 0 && rot >= 0 && rank > 0, "latent_prep: bad sizes tokens=%d heads=%d dim=%d rot=%d rank=%d", tokens, heads,
              dim, rot, rank);
  LRS_REQUIRE(eps > 0.f, "latent_prep: eps must be positive");
  LRS_REQUIRE((cosv == nullptr) == (sinv == nullptr), "latent_prep: cos and sin come together");
  hipStream_t s = (hipStream_t)stream;
#define LRS_PREP(T, TW)                                                                                                              \
  latent_prep_kernel<T, TW><<<tokens, 256, 0, s>>>((const T*)proj, proj_stride, q_col, kv_col, heads, dim, rot, rank, (const TW*)norm_weight, \
                                                   eps, cosv, sinv, (T*)pages, (T*)value_pages, page_size, slots, (T*)queries, query_stride)
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
  hipStream_t s = (hipStream_t)stream;
  if (dtype == LRS_BF16 && !trans && k % 8 == 0 && a_token % 8 == 0 && a_head % 8 == 0 && (uintptr_t)a % 16 == 0 && (uintptr_t)w % 16 == 0 &&
      (n + 63) / 64 <= 65535) {
    head_gemm_bf16_kernel<<<dim3((tokens + 63) / 64, (n + 63) / 64, heads), 256, 0, s>>>((bf16*)out, out_token, out_head, (const bf16*)a, a_token, a_head,
                                                                                       (const bf16*)w, w_head, tokens, n, k);
    return lrs_check_launch("head_gemm");
  }
  const dim3 grid((tokens + HG_TOKENS - 1) / HG_TOKENS, heads);
  const size_t lds = sizeof(float) * HG_TOKENS * k;
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

// Whether lrs_latent_attention_groups takes the shape.
LRS_API int lrs_latent_attention_groups_takes(int rank, int width, int page_size) {
  return rank > 0 && rank <= 512 && width >= rank && width % 8 == 0 && page_size % 8 == 0;
}

// The same attention on the matrix cores, bfloat16: the step's tokens come as query groups (group_token0 / group_count
// [groups]: consecutive tokens of one request, at most max_count; both null: every token a group of its own), the keys of a
// group may be divided between `splits` workgroups (part_o [tokens, heads, splits, rank], part_ml [tokens, heads, splits, 2]
// float32).  value_pages [P, rank, page] holds the latent values once more, a column's keys side by side.
LRS_API int lrs_latent_attention_groups(void* out, int out_stride, const void* queries, int query_stride, const void* pages, const void* value_pages,
                                        const int* block_table, int table_stride, const int* token_request, const int* positions,
                                        const int* group_token0, const int* group_count, int groups, int max_count, const float* sink,
                                        const void* gate, int gate_stride, int tokens, int heads, int rank, int width, int page_size, float scale,
                                        int window, int splits, float* part_o, float* part_ml, void* stream) {
  LRS_REQUIRE(tokens > 0 && groups > 0 && max_count > 0 && heads > 0, "latent_attention_groups: bad sizes tokens=%d groups=%d max_count=%d heads=%d", tokens, groups, max_count, heads);
  LRS_REQUIRE(lrs_latent_attention_groups_takes(rank, width, page_size), "latent_attention_groups: rank=%d width=%d page=%d not taken (rank <= 512, width and page multiples of 8)",
              rank, width, page_size);
  LRS_REQUIRE((uintptr_t)queries % 16 == 0 && (uintptr_t)pages % 16 == 0 && (uintptr_t)value_pages % 16 == 0 && query_stride % 8 == 0, "latent_attention_groups: operands must be 16-byte aligned");
  LRS_REQUIRE((group_token0 == nullptr) == (group_count == nullptr), "latent_attention_groups: the groups' first tokens and counts come together");
  LRS_REQUIRE(splits >= 1 && splits <= 64 && (splits == 1 || (part_o && part_ml)), "latent_attention_groups: splits 1..64, with room for the parts");
  LRS_REQUIRE(window >= 0, "latent_attention_groups: window must be >= 0 (0 = none)");
  const int tiles = ((int64_t)max_count * heads + 63) / 64;
  LRS_REQUIRE(tiles <= 65535 && splits <= 65535, "latent_attention_groups: too many rows a group");
  const dim3 grid(groups, tiles, splits);
  hipStream_t s = (hipStream_t)stream;
#define LRS_LA(CT)                                                                                                                        \
  latent_attention_bf16_kernel<CT><<<grid, 256, 0, s>>>((bf16*)out, out_stride, part_o, part_ml, (const bf16*)queries, query_stride,      \
                                                        (const bf16*)pages, (const bf16*)value_pages, block_table, table_stride, token_request, \
                                                        positions, group_token0, group_count, sink, (const bf16*)gate, gate_stride, heads, rank, \
                                                        width, page_size, scale, window, splits)
  const int ct = (rank + 15) / 16;
  if (ct <= 2) LRS_LA(2);
  else if (ct <= 4) LRS_LA(4);
  else if (ct <= 6) LRS_LA(6);
  else if (ct <= 8) LRS_LA(8);
  else if (ct <= 12) LRS_LA(12);
  else if (ct <= 16) LRS_LA(16);
  else if (ct <= 24) LRS_LA(24);
  else LRS_LA(32);
#undef LRS_LA
  if (int rc = lrs_check_launch("latent_attention_groups")) return rc;
  if (splits > 1) {
    latent_merge_kernel<<<dim3(tokens, heads), 256, 0, s>>>((bf16*)out, out_stride, part_o, part_ml, sink, (const bf16*)gate, gate_stride, heads, rank, splits);
    return lrs_check_launch("latent_attention_groups merge");
  }
  return 0;
}
