// Gated delta rule: a linear-recurrent mixer whose state per head is a matrix S [dim, vdim] in float32.
//
// For every token, with q and k unit vectors of the head's key group, v the head's value, beta in (0, 1) the
// step size and g in (0, 1) the decay:
//     S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// so the read-out sees the token's own write.  Everything here is float32 whatever the run's dtype: only the
// projections that feed it and the output that leaves it may be bfloat16.
//
// Three kernels serve a step of any shape (prompt portions and single tokens side by side):
//   delta_prepare   per (token, head): the short causal convolution over time of the q, k and v channels
//                   (taps before the step's first token come from the request's state), silu, unit norm of
//                   q and k, and the two gates of the recurrence;
//   delta_conv_keep per (request, channel): the last taps-1 inputs of the convolution, for the next step;
//   delta_scan      per (request, head, 16 columns of S): walks the request's tokens in order with its part of S in
//                   registers, a column shared by the 16 lanes of a row of lanes;
//   delta_gate      per (token, head): the read-out divided by its root mean square over vdim, times the norm's
//                   weight, times silu of the output gate.
// A request's state row holds S for every head and then the convolution's inputs:
//   S of head h at h * rows * vdim * 16 floats, element (i, j) at ((i % rows) * vdim + j) * 16 + i / rows with
//   rows = 4, 8 or 16 (dim over the 16 lanes of a column, padded): the order in which the scan's threads hold it,
//   so that loading and storing it are whole lines; then [taps - 1, channels], oldest first.
#include "common.h"

namespace {

constexpr int SPLIT = 16;     // lanes that share a column of S (one row of lanes: their sums need no LDS)
constexpr int COLUMNS = 16;   // columns of S a workgroup of 256 threads owns
// tokens whose inputs are staged in LDS at a time: 16, or 8 for the widest keys (two buffers stay within 64 KB)

__device__ __forceinline__ float silu_f(float x) { return x / (1.f + expf(-x)); }

template <typename TP>
__global__ void delta_prepare_kernel(const TP* __restrict__ proj, int ld, const int* __restrict__ token_request,
                                     const int* __restrict__ cu, const int* __restrict__ slot_ids,
                                     float* __restrict__ state, int64_t state_stride, int64_t conv_offset,
                                     const float* __restrict__ conv_w, int taps, int G, int H, int d, int dv,
                                     const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                                     float* __restrict__ qkv, float* __restrict__ gates, int keep_inside) {
  // keep_inside: every request brings one token, so this wave alone reads and writes its channels' kept inputs of its
  // request: it moves them on itself (no delta_conv_keep launch)
  const int t = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
  const int channels = 2 * G * d + H * dv;
  const int r = token_request[t], start = cu[r], at = t - start;
  float* kept = state + (int64_t)slot_ids[r] * state_stride + conv_offset;
  const bool is_v = unit >= 2 * G;
  const int c0 = is_v ? 2 * G * d + (unit - 2 * G) * dv : unit * d, n = is_v ? dv : d;
  float* out = qkv + (int64_t)t * channels + c0;
  float ss = 0.f;
  for (int i = lane; i < n; i += WAVE) {
    const int c = c0 + i;
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int s = at - (taps - 1 - j);
      const float x = s >= 0 ? to_float(proj[(int64_t)(start + s) * ld + c]) : kept[(int64_t)(taps - 1 + s) * channels + c];
      acc = fmaf(conv_w[(int64_t)c * taps + j], x, acc);
      if (keep_inside && j > 0) kept[(int64_t)(j - 1) * channels + c] = x;      // input j of this token's window is entry j - 1 of the next one's
    }
    const float y = silu_f(acc);
    out[i] = y;
    ss = fmaf(y, y, ss);
  }
  if (!is_v) {
    ss = wave_sum(ss);
    // unit vectors; the queries also carry the 1 / sqrt(dim) of the scores
    const float scale = (unit < G ? 1.0f / sqrtf((float)d) : 1.0f) / sqrtf(ss + 1e-6f);
    for (int i = lane; i < n; i += WAVE) out[i] *= scale;
  } else if (lane == 0) {
    const int h = unit - 2 * G;
    const int64_t row = (int64_t)t * ld + channels + (int64_t)H * dv;
    const float b = to_float(proj[row + h]), a = to_float(proj[row + H + h]) + dt_bias[h];
    const float softplus = a > 20.f ? a : log1pf(expf(a));
    gates[(int64_t)t * 2 * H + h] = 1.f / (1.f + expf(-b));
    gates[(int64_t)t * 2 * H + H + h] = expf(-expf(a_log[h]) * softplus);
  }
}

template <typename TP>
__global__ void delta_conv_keep_kernel(const TP* __restrict__ proj, int ld, const int* __restrict__ cu,
                                       const int* __restrict__ slot_ids, float* __restrict__ state, int64_t state_stride,
                                       int64_t conv_offset, int taps, int channels) {
  const int r = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int start = cu[r], n = cu[r + 1] - start;
  float* kept = state + (int64_t)slot_ids[r] * state_stride + conv_offset;
  // entry j becomes the input n - (taps - 1) + j of this step, or the old entry j + n: read from further on only
  for (int j = 0; j < taps - 1; ++j) {
    const int s = n - (taps - 1) + j;
    kept[(int64_t)j * channels + c] = s >= 0 ? to_float(proj[(int64_t)(start + s) * ld + c]) : kept[(int64_t)(taps - 1 + s) * channels + c];
  }
}

// A 16-lane sum that every lane of the row gets: four adds whose second operand comes through the lanes' crossbar
// (quad swaps, then the row mirrored by halves and whole), no LDS.
template <int CTRL>
__device__ __forceinline__ float from_lane(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float row_sum16(float v) {
  v += from_lane<0xB1>(v);     // quad_perm [1, 0, 3, 2]
  v += from_lane<0x4E>(v);     // quad_perm [2, 3, 0, 1]
  v += from_lane<0x141>(v);    // row_half_mirror
  v += from_lane<0x140>(v);    // row_mirror
  return v;
}

// One workgroup of 256 threads owns 16 columns of one head's matrix for one request: thread (column c, part s) holds
// the ROWS rows s * rows .. of column c in registers, so a token costs each thread 4 * rows multiply-adds and two
// 16-lane sums, and a head of 128 columns is spread over eight compute units.  Both products with the old matrix are
// taken in one pass (the read-out of the new one follows from them: S'^T q = g S^T q + u (k . q)), then the matrix is
// updated.  The inputs of CHUNK tokens are staged in LDS, the next chunk's on their way into registers meanwhile.
template <int ROWS, int CHUNK>
__global__ __launch_bounds__(256) void delta_scan_kernel(const float* __restrict__ qkv, const float* __restrict__ gates,
                                                         const int* __restrict__ cu, const int* __restrict__ slot_ids,
                                                         float* __restrict__ state, int64_t state_stride, int G, int H, int d,
                                                         int dv, float* __restrict__ raw_out) {
  constexpr int K4 = ROWS / 4;                 // float4 pieces of a thread's slice of a key
  constexpr int rows = ROWS;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int r = blockIdx.x, h = blockIdx.y, block = blockIdx.z, tid = threadIdx.x;
  const int dpad = rows * SPLIT, channels = 2 * G * d + H * dv, hk = h / (H / G);
  const int per_buffer = CHUNK * (2 * dpad + COLUMNS + 4);
  const int c = tid / SPLIT, s = tid % SPLIT, column = block * COLUMNS + c;
  const bool mine = column < dv;
  const int start = cu[r], n = cu[r + 1] - start;
  float* st = state + (int64_t)slot_ids[r] * state_stride + (int64_t)h * rows * dv * SPLIT + (int64_t)block * COLUMNS * SPLIT;
  float S[ROWS];
#pragma unroll
  for (int i = 0; i < ROWS; ++i) S[i] = mine ? st[(int64_t)i * dv * SPLIT + tid] : 0.f;

  // what a thread brings in of a chunk: pieces of four values of the keys and queries (CHUNK * dpad / 4 pieces each,
  // at most KQ of them a thread), one value of the 16 columns' v, and the scalars of a token (step, decay, k . q)
  constexpr int KQ = (CHUNK * ROWS * SPLIT / 4 + 255) / 256;
  float4 k_reg[KQ], q_reg[KQ];
  float v_reg = 0.f, scalar_reg = 0.f;
  const int pieces = CHUNK * dpad / 4, row_pieces = dpad / 4;
  const bool d_whole = d % 4 == 0 && channels % 4 == 0;     // every piece of four is 16 bytes aligned
  auto fetch = [&](int c0) {
    const int count = min(CHUNK, n - c0);
#pragma unroll
    for (int p = 0; p < KQ; ++p) {
      const int e = tid + p * 256, tt = e / row_pieces, i = (e % row_pieces) * 4;
      k_reg[p] = q_reg[p] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (e < pieces && tt < count) {
        const float* row = qkv + (int64_t)(start + c0 + tt) * channels + hk * d + i;
        if (d_whole && i + 4 <= d) {
          q_reg[p] = *(const float4*)row;
          k_reg[p] = *(const float4*)(row + G * d);
        } else {
          float kq[8] = {};
          for (int x = 0; x < 4; ++x)
            if (i + x < d) {
              kq[x] = row[x];
              kq[4 + x] = row[G * d + x];
            }
          q_reg[p] = make_float4(kq[0], kq[1], kq[2], kq[3]);
          k_reg[p] = make_float4(kq[4], kq[5], kq[6], kq[7]);
        }
      }
    }
    const int tt = tid / COLUMNS, cc = tid % COLUMNS;
    v_reg = (tt < CHUNK && tt < count && block * COLUMNS + cc < dv) ? qkv[(int64_t)(start + c0 + tt) * channels + 2 * G * d + h * dv + block * COLUMNS + cc] : 0.f;
    scalar_reg = 0.f;
    if (tid < 2 * CHUNK && tid / 2 < count) scalar_reg = gates[(int64_t)(start + c0 + tid / 2) * 2 * H + (tid % 2) * H + h];
  };
  auto stage = [&](float* buf) {
    float* k_l = buf;
    float* q_l = buf + CHUNK * dpad;
#pragma unroll
    for (int p = 0; p < KQ; ++p) {
      const int e = tid + p * 256;
      if (e < pieces) {
        *(float4*)(k_l + e * 4) = k_reg[p];
        *(float4*)(q_l + e * 4) = q_reg[p];
      }
    }
    if (tid < CHUNK * COLUMNS) buf[2 * CHUNK * dpad + tid] = v_reg;      // [CHUNK][COLUMNS]
    if (tid < 2 * CHUNK) buf[2 * CHUNK * dpad + CHUNK * COLUMNS + (tid / 2) * 4 + tid % 2] = scalar_reg;
  };
  fetch(0);
  int turn = 0;
  for (int c0 = 0; c0 < n; c0 += CHUNK, turn ^= 1) {
    float* buf = lds + turn * per_buffer;
    stage(buf);
    __syncthreads();
    if (c0 + CHUNK < n) fetch(c0 + CHUNK);
    const int count = min(CHUNK, n - c0);
    const float* k_l = buf + s * rows;
    const float* q_l = buf + CHUNK * dpad + s * rows;
    const float* v_l = buf + 2 * CHUNK * dpad;
    const float* g_l = v_l + CHUNK * COLUMNS;
    for (int tt = 0; tt < count; ++tt) {
      float kk[ROWS], qq[ROWS];
#pragma unroll
      for (int p = 0; p < K4; ++p) {
        const float4 a = *(const float4*)(k_l + tt * dpad + 4 * p), b = *(const float4*)(q_l + tt * dpad + 4 * p);
        kk[4 * p] = a.x, kk[4 * p + 1] = a.y, kk[4 * p + 2] = a.z, kk[4 * p + 3] = a.w;
        qq[4 * p] = b.x, qq[4 * p + 1] = b.y, qq[4 * p + 2] = b.z, qq[4 * p + 3] = b.w;
      }
      float dk = 0.f, dq = 0.f, kq = 0.f;
#pragma unroll
      for (int i = 0; i < ROWS; ++i) {
        dk = fmaf(S[i], kk[i], dk);
        dq = fmaf(S[i], qq[i], dq);
        kq = fmaf(kk[i], qq[i], kq);
      }
      dk = row_sum16(dk);
      dq = row_sum16(dq);
      kq = row_sum16(kq);
      const float beta = g_l[4 * tt], g = g_l[4 * tt + 1];
      const float u = beta * (v_l[tt * COLUMNS + c] - g * dk);
#pragma unroll
      for (int i = 0; i < ROWS; ++i) S[i] = fmaf(kk[i], u, g * S[i]);
      if (s == 0 && mine) raw_out[(int64_t)(start + c0 + tt) * H * dv + h * dv + column] = fmaf(u, kq, g * dq);
    }
    // the other buffer is written next; this one again only after the barrier of the turn between
  }
  if (mine) {
#pragma unroll
    for (int i = 0; i < ROWS; ++i) st[(int64_t)i * dv * SPLIT + tid] = S[i];
  }
}

// The same for steps in which every request brings one token: nothing is staged, a thread reads its slices of the key
// and the query where the preparation left them, and as many workgroups as fit run side by side (no LDS holds them back).
template <int ROWS>
__global__ __launch_bounds__(256) void delta_scan_single_kernel(const float* __restrict__ qkv, const float* __restrict__ gates,
                                                                const int* __restrict__ slot_ids, float* __restrict__ state,
                                                                int64_t state_stride, int G, int H, int d, int dv, float* __restrict__ raw_out) {
  const int r = blockIdx.x, h = blockIdx.y, block = blockIdx.z, tid = threadIdx.x;
  const int channels = 2 * G * d + H * dv, hk = h / (H / G);
  const int c = tid / SPLIT, s = tid % SPLIT, column = block * COLUMNS + c;
  if (column >= dv) return;
  float* st = state + (int64_t)slot_ids[r] * state_stride + (int64_t)h * ROWS * dv * SPLIT + (int64_t)block * COLUMNS * SPLIT;
  const float* row = qkv + (int64_t)r * channels;
  float S[ROWS], kk[ROWS], qq[ROWS];
#pragma unroll
  for (int i = 0; i < ROWS; ++i) S[i] = st[(int64_t)i * dv * SPLIT + tid];
  if (d % 4 == 0 && channels % 4 == 0) {          // every piece of four values is 16 bytes aligned
#pragma unroll
    for (int p = 0; p < ROWS / 4; ++p) {
      const int at = s * ROWS + 4 * p;
      const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
      const float4 a = at < d ? *(const float4*)(row + hk * d + at) : zero, b = at < d ? *(const float4*)(row + G * d + hk * d + at) : zero;
      qq[4 * p] = a.x, qq[4 * p + 1] = a.y, qq[4 * p + 2] = a.z, qq[4 * p + 3] = a.w;
      kk[4 * p] = b.x, kk[4 * p + 1] = b.y, kk[4 * p + 2] = b.z, kk[4 * p + 3] = b.w;
    }
  } else {
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
      const int at = s * ROWS + i;
      qq[i] = at < d ? row[hk * d + at] : 0.f;
      kk[i] = at < d ? row[G * d + hk * d + at] : 0.f;
    }
  }
  const float v = row[2 * G * d + h * dv + column];
  const float beta = gates[(int64_t)r * 2 * H + h], g = gates[(int64_t)r * 2 * H + H + h];
  float dk = 0.f, dq = 0.f, kq = 0.f;
#pragma unroll
  for (int i = 0; i < ROWS; ++i) {
    dk = fmaf(S[i], kk[i], dk);
    dq = fmaf(S[i], qq[i], dq);
    kq = fmaf(kk[i], qq[i], kq);
  }
  dk = row_sum16(dk);
  dq = row_sum16(dq);
  kq = row_sum16(kq);
  const float u = beta * (v - g * dk);
#pragma unroll
  for (int i = 0; i < ROWS; ++i) st[(int64_t)i * dv * SPLIT + tid] = fmaf(kk[i], u, g * S[i]);
  if (s == 0) raw_out[(int64_t)r * H * dv + h * dv + column] = fmaf(u, kq, g * dq);
}

// The head's read-out divided by its root mean square over vdim, times the norm's weight, times silu(gate): a wave a
// (token, head).
template <typename TP, typename TO>
__global__ __launch_bounds__(256) void delta_gate_kernel(const float* __restrict__ raw_out, const TP* __restrict__ proj, int ld,
                                                         int gate_at, const float* __restrict__ norm_w, float eps, int tokens, int H,
                                                         int dv, TO* __restrict__ out) {
  const int64_t pair = (int64_t)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  if (pair >= (int64_t)tokens * H) return;
  const int64_t token = pair / H;
  const int h = (int)(pair % H);
  const float* o = raw_out + token * H * dv + (int64_t)h * dv;
  float ss = 0.f;
  for (int i = lane; i < dv; i += WAVE) ss = fmaf(o[i], o[i], ss);
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)dv + eps);
  for (int i = lane; i < dv; i += WAVE) {
    const float gate = to_float(proj[token * ld + gate_at + h * dv + i]);
    out[token * H * dv + (int64_t)h * dv + i] = from_float<TO>(o[i] * inv * norm_w[i] * silu_f(gate));
  }
}

}  // namespace

// Rows of a head's matrix that one lane holds: the key size over the 16 lanes of a column, to the next of 4, 8, 16.
LRS_API int lrs_delta_state_rows(int d) { return d <= 64 ? 4 : d <= 128 ? 8 : 16; }

// proj [tokens, ld]: columns q (G*d) | k (G*d) | v (H*dv) | output gate (H*dv) | step size (H) | decay input (H).
// qkv [tokens, 2*G*d + H*dv], gates [tokens, 2*H] and raw [tokens, H*dv] are float32 scratch; out [tokens, H*dv] in out_dtype.
LRS_API int lrs_delta_rule(void* out, int out_dtype, const void* proj, int proj_dtype, int ld, int tokens, int requests,
                           const int* token_request, const int* cu, const int* slot_ids, float* state, int64_t state_stride,
                           const float* conv_w, int taps, int G, int H, int d, int dv, const float* a_log,
                           const float* dt_bias, const float* norm_w, float eps, float* qkv, float* gates, float* raw, void* stream) {
  LRS_REQUIRE(tokens > 0 && requests > 0 && requests <= tokens, "delta_rule: bad sizes tokens=%d requests=%d", tokens, requests);
  LRS_REQUIRE(G > 0 && H > 0 && H % G == 0 && d > 0 && dv > 0 && taps >= 1, "delta_rule: bad sizes G=%d H=%d d=%d dv=%d taps=%d", G, H, d, dv, taps);
  LRS_REQUIRE(d <= 256, "delta_rule: takes keys of up to 256 values, got %d", d);
  const int rows = lrs_delta_state_rows(d), channels = 2 * G * d + H * dv;
  LRS_REQUIRE(ld >= channels + H * dv + 2 * H, "delta_rule: projection rows of %d hold fewer than the %d columns needed", ld, channels + H * dv + 2 * H);
  const int64_t conv_offset = (int64_t)H * rows * SPLIT * dv;
  LRS_REQUIRE(state_stride >= conv_offset + (int64_t)(taps - 1) * channels, "delta_rule: a state row of %lld floats is too short", (long long)state_stride);
  LRS_REQUIRE(eps > 0.f, "delta_rule: eps must be positive");
  LRS_REQUIRE(((uintptr_t)qkv % 16) == 0, "delta_rule: the scratch rows must be 16 bytes aligned");
  hipStream_t s = (hipStream_t)stream;
  dim3 pgrid(tokens, 2 * G + H), kgrid(requests, (channels + 255) / 256), sgrid(requests, H, (dv + COLUMNS - 1) / COLUMNS);
  const int chunk = rows == 16 ? 8 : 16;
  const size_t lds = (size_t)2 * chunk * (2 * rows * SPLIT + COLUMNS + 4) * sizeof(float);
  const int64_t pairs = (int64_t)tokens * H;
  const int gate_at = channels;
#define ALL(TP, TO)                                                                                                           \
  do {                                                                                                                        \
    delta_prepare_kernel<TP><<<pgrid, WAVE, 0, s>>>((const TP*)proj, ld, token_request, cu, slot_ids, state, state_stride,    \
                                                    conv_offset, conv_w, taps, G, H, d, dv, a_log, dt_bias, qkv, gates,       \
                                                    tokens == requests);                                                      \
    if (taps > 1 && tokens != requests)                                                                                       \
      delta_conv_keep_kernel<TP><<<kgrid, 256, 0, s>>>((const TP*)proj, ld, cu, slot_ids, state, state_stride, conv_offset,  \
                                                       taps, channels);                                                       \
    if (tokens == requests) {        /* one token each: token r is request r's */                                             \
      if (rows == 4) delta_scan_single_kernel<4><<<sgrid, 256, 0, s>>>(qkv, gates, slot_ids, state, state_stride, G, H, d, dv, raw);        \
      else if (rows == 8) delta_scan_single_kernel<8><<<sgrid, 256, 0, s>>>(qkv, gates, slot_ids, state, state_stride, G, H, d, dv, raw);   \
      else delta_scan_single_kernel<16><<<sgrid, 256, 0, s>>>(qkv, gates, slot_ids, state, state_stride, G, H, d, dv, raw);                 \
    } else if (rows == 4) delta_scan_kernel<4, 16><<<sgrid, 256, lds, s>>>(qkv, gates, cu, slot_ids, state, state_stride, G, H, d, dv, raw);       \
    else if (rows == 8) delta_scan_kernel<8, 16><<<sgrid, 256, lds, s>>>(qkv, gates, cu, slot_ids, state, state_stride, G, H, d, dv, raw);  \
    else delta_scan_kernel<16, 8><<<sgrid, 256, lds, s>>>(qkv, gates, cu, slot_ids, state, state_stride, G, H, d, dv, raw);                 \
    delta_gate_kernel<TP, TO><<<(unsigned)((pairs + 3) / 4), 256, 0, s>>>(raw, (const TP*)proj, ld, gate_at, norm_w, eps, tokens, H, dv, (TO*)out); \
  } while (0)
  if (proj_dtype == LRS_F32 && out_dtype == LRS_F32) ALL(float, float);
  else if (proj_dtype == LRS_F32 && out_dtype == LRS_BF16) ALL(float, bf16);
  else if (proj_dtype == LRS_BF16 && out_dtype == LRS_BF16) ALL(bf16, bf16);
  else return lrs_fail("delta_rule: projections in dtype %d with outputs in dtype %d are not served", proj_dtype, out_dtype);
#undef ALL
  return lrs_check_launch("delta_rule");
}
