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
//   delta_scan      per (request, head): walks the request's tokens in order with S in registers, a column of
//                   S shared by four neighbouring lanes, and finishes each token's output with the gated
//                   RMS norm over vdim.
// A request's state row holds S for every head and then the convolution's inputs:
//   S of head h at h * rows * vdim * 4 floats, element (i, j) at ((i % rows) * vdim + j) * 4 + i / rows with
//   rows = ceil(dim / 4): the order in which the scan's threads hold it, so that loading and storing it are
//   whole lines; then [taps - 1, channels], oldest first.
#include "common.h"

namespace {

constexpr int SPLIT = 4;      // lanes that share a column of S
constexpr int CHUNK = 16;     // tokens whose inputs are staged in LDS at a time

__device__ __forceinline__ float silu_f(float x) { return x / (1.f + expf(-x)); }

template <typename TP>
__global__ void delta_prepare_kernel(const TP* __restrict__ proj, int ld, const int* __restrict__ token_request,
                                     const int* __restrict__ cu, const int* __restrict__ slot_ids,
                                     const float* __restrict__ state, int64_t state_stride, int64_t conv_offset,
                                     const float* __restrict__ conv_w, int taps, int G, int H, int d, int dv,
                                     const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                                     float* __restrict__ qkv, float* __restrict__ gates) {
  const int t = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
  const int channels = 2 * G * d + H * dv;
  const int r = token_request[t], start = cu[r], at = t - start;
  const float* kept = state + (int64_t)slot_ids[r] * state_stride + conv_offset;
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

template <typename TP, typename TO, int ROWS>
__global__ __launch_bounds__(1024) void delta_scan_kernel(
    const float* __restrict__ qkv, const float* __restrict__ gates, const TP* __restrict__ proj, int ld,
    const int* __restrict__ cu, const int* __restrict__ slot_ids, float* __restrict__ state, int64_t state_stride,
    const float* __restrict__ norm_w, float eps, int G, int H, int d, int dv, int rows, TO* __restrict__ out) {
  extern __shared__ float lds[];
  const int r = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int dpad = rows * SPLIT, channels = 2 * G * d + H * dv, hk = h / (H / G);
  float* k_l = lds;                          // [CHUNK][dpad]
  float* q_l = k_l + CHUNK * dpad;           // [CHUNK][dpad]
  float* v_l = q_l + CHUNK * dpad;           // [CHUNK][dv]
  float* o_l = v_l + CHUNK * dv;             // [CHUNK][dv]
  float* g_l = o_l + CHUNK * dv;             // [CHUNK][2]: beta, decay
  const int j = tid / SPLIT, s = tid % SPLIT;
  const bool mine = j < dv;
  const int start = cu[r], n = cu[r + 1] - start;
  float* st = state + (int64_t)slot_ids[r] * state_stride + (int64_t)h * rows * dv * SPLIT;
  float S[ROWS];
#pragma unroll
  for (int i = 0; i < ROWS; ++i) S[i] = (mine && i < rows) ? st[(int64_t)i * dv * SPLIT + tid] : 0.f;
  const int waves = blockDim.x / WAVE, wave = tid / WAVE, lane = tid % WAVE;
  for (int c0 = 0; c0 < n; c0 += CHUNK) {
    const int count = min(CHUNK, n - c0);
    for (int e = tid; e < count * dpad; e += blockDim.x) {
      const int tt = e / dpad, i = e % dpad;
      const float* row = qkv + (int64_t)(start + c0 + tt) * channels;
      k_l[e] = i < d ? row[G * d + hk * d + i] : 0.f;
      q_l[e] = i < d ? row[hk * d + i] : 0.f;
    }
    for (int e = tid; e < count * dv; e += blockDim.x)
      v_l[e] = qkv[(int64_t)(start + c0 + e / dv) * channels + 2 * G * d + h * dv + e % dv];
    if (tid < count * 2) g_l[tid] = gates[(int64_t)(start + c0 + tid / 2) * 2 * H + (tid % 2) * H + h];
    __syncthreads();
    if (mine) {
      for (int tt = 0; tt < count; ++tt) {
        const float* kk = k_l + tt * dpad + s * rows;
        const float* qq = q_l + tt * dpad + s * rows;
        const float beta = g_l[2 * tt], g = g_l[2 * tt + 1];
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < ROWS; ++i)
          if (i < rows) dot = fmaf(S[i], kk[i], dot);
        dot += __shfl_xor(dot, 1, WAVE);
        dot += __shfl_xor(dot, 2, WAVE);
        const float u = beta * (v_l[tt * dv + j] - g * dot);
        float o = 0.f;
#pragma unroll
        for (int i = 0; i < ROWS; ++i)
          if (i < rows) {
            S[i] = fmaf(kk[i], u, g * S[i]);
            o = fmaf(S[i], qq[i], o);
          }
        o += __shfl_xor(o, 1, WAVE);
        o += __shfl_xor(o, 2, WAVE);
        if (s == 0) o_l[tt * dv + j] = o;
      }
    }
    __syncthreads();
    // the head's output: divided by its root mean square over vdim, times the norm's weight, times silu(gate)
    for (int tt = wave; tt < count; tt += waves) {
      float ss = 0.f;
      for (int i = lane; i < dv; i += WAVE) ss = fmaf(o_l[tt * dv + i], o_l[tt * dv + i], ss);
      ss = wave_sum(ss);
      const float inv = 1.0f / sqrtf(ss / (float)dv + eps);
      const int64_t token = start + c0 + tt;
      for (int i = lane; i < dv; i += WAVE) {
        const float gate = to_float(proj[token * ld + channels + h * dv + i]);
        out[token * (int64_t)H * dv + h * dv + i] = from_float<TO>(o_l[tt * dv + i] * inv * norm_w[i] * silu_f(gate));
      }
    }
    // the next chunk's loads touch k, q, v and the gates only; its scan, which writes the outputs' buffer, comes after a barrier
  }
  if (mine) {
#pragma unroll
    for (int i = 0; i < ROWS; ++i)
      if (i < rows) st[(int64_t)i * dv * SPLIT + tid] = S[i];
  }
}

}  // namespace

LRS_API int lrs_delta_state_rows(int d) { return (d + SPLIT - 1) / SPLIT; }

// proj [tokens, ld]: columns q (G*d) | k (G*d) | v (H*dv) | output gate (H*dv) | step size (H) | decay input (H).
// qkv [tokens, 2*G*d + H*dv] and gates [tokens, 2*H] are float32 scratch; out [tokens, H*dv] in out_dtype.
LRS_API int lrs_delta_rule(void* out, int out_dtype, const void* proj, int proj_dtype, int ld, int tokens, int requests,
                           const int* token_request, const int* cu, const int* slot_ids, float* state, int64_t state_stride,
                           const float* conv_w, int taps, int G, int H, int d, int dv, const float* a_log,
                           const float* dt_bias, const float* norm_w, float eps, float* qkv, float* gates, void* stream) {
  LRS_REQUIRE(tokens > 0 && requests > 0 && requests <= tokens, "delta_rule: bad sizes tokens=%d requests=%d", tokens, requests);
  LRS_REQUIRE(G > 0 && H > 0 && H % G == 0 && d > 0 && dv > 0 && taps >= 1, "delta_rule: bad sizes G=%d H=%d d=%d dv=%d taps=%d", G, H, d, dv, taps);
  const int rows = lrs_delta_state_rows(d), channels = 2 * G * d + H * dv;
  LRS_REQUIRE(rows <= 64 && dv * SPLIT <= 1024, "delta_rule: takes dim up to 256 and vdim up to 256, got %d and %d", d, dv);
  LRS_REQUIRE(ld >= channels + H * dv + 2 * H, "delta_rule: projection rows of %d hold fewer than the %d columns needed", ld, channels + H * dv + 2 * H);
  const int64_t conv_offset = (int64_t)H * rows * SPLIT * dv;
  LRS_REQUIRE(state_stride >= conv_offset + (int64_t)(taps - 1) * channels, "delta_rule: a state row of %lld floats is too short", (long long)state_stride);
  LRS_REQUIRE(eps > 0.f, "delta_rule: eps must be positive");
  hipStream_t s = (hipStream_t)stream;
  const int threads = ((dv * SPLIT + WAVE - 1) / WAVE) * WAVE;
  const size_t lds = (size_t)CHUNK * (2 * rows * SPLIT + 2 * dv + 2) * sizeof(float);
  LRS_REQUIRE(lds <= 64 * 1024, "delta_rule: %zu bytes of LDS are too many", lds);
  dim3 pgrid(tokens, 2 * G + H), kgrid(requests, (channels + 255) / 256), sgrid(requests, H);
#define SCAN(TP, TO, ROWS)                                                                                                   \
  delta_scan_kernel<TP, TO, ROWS><<<sgrid, threads, lds, s>>>(qkv, gates, (const TP*)proj, ld, cu, slot_ids, state, state_stride, \
                                                              norm_w, eps, G, H, d, dv, rows, (TO*)out)
#define SCAN_ROWS(TP, TO)          \
  do {                             \
    if (rows <= 8) SCAN(TP, TO, 8); \
    else if (rows <= 16) SCAN(TP, TO, 16); \
    else if (rows <= 32) SCAN(TP, TO, 32); \
    else SCAN(TP, TO, 64);         \
  } while (0)
#define ALL(TP, TO)                                                                                                           \
  do {                                                                                                                        \
    delta_prepare_kernel<TP><<<pgrid, WAVE, 0, s>>>((const TP*)proj, ld, token_request, cu, slot_ids, state, state_stride,    \
                                                    conv_offset, conv_w, taps, G, H, d, dv, a_log, dt_bias, qkv, gates);      \
    if (taps > 1)                                                                                                             \
      delta_conv_keep_kernel<TP><<<kgrid, 256, 0, s>>>((const TP*)proj, ld, cu, slot_ids, state, state_stride, conv_offset,  \
                                                       taps, channels);                                                       \
    SCAN_ROWS(TP, TO);                                                                                                        \
  } while (0)
  if (proj_dtype == LRS_F32 && out_dtype == LRS_F32) ALL(float, float);
  else if (proj_dtype == LRS_F32 && out_dtype == LRS_BF16) ALL(float, bf16);
  else if (proj_dtype == LRS_BF16 && out_dtype == LRS_BF16) ALL(bf16, bf16);
  else return lrs_fail("delta_rule: projections in dtype %d with outputs in dtype %d are not served", proj_dtype, out_dtype);
#undef ALL
#undef SCAN_ROWS
#undef SCAN
  return lrs_check_launch("delta_rule");
}
