// A gated delta rule: a matrix state per head that is corrected towards each new value, with a decay per key channel.
//
//   S <- diag(a_t) S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t
//
// per head and row, S being [key channels][value channels] 32-bit floats in the request's state line. Two kernels: the
// step before the walk (a short causal convolution with silu over the q, k and v columns of a 32-bit input product,
// unit q and k per head, beta) and the walk itself. Everything is 32-bit.
//
// A request's state line holds S [heads][dim][vdim] and, from float `conv_at` on, the convolution's last taps - 1
// inputs [taps - 1][channels], oldest first. Rows of the step are grouped by request: request s owns the rows
// [cu_rows[s], cu_rows[s + 1]) in order of position and the line seq_slots[s].
#include "common.h"

TIS_DEFINE_LAST_ERROR(tis_delta_rule)

static constexpr int DR_MAX_TAPS = 16;
static constexpr int DR_PER = 4;         // channels of a head a lane keeps in the step before the walk: dim <= 256

__device__ __forceinline__ float dr_sigmoid(float z) { return 1.f / (1.f + expf(-z)); }

// One convolved channel of row r: sum_j taps[ch][j] * input(i - (K - 1) + j), i the row's index among its request's rows
// of this step; inputs before the step's first row come from the state line, which is zero before a request's first row.
__device__ __forceinline__ float dr_conv(const float* __restrict__ proj, long ldp, int col, const float* __restrict__ taps,
                                         int K, int ch, int C, const float* __restrict__ line, long first_row, int i) {
  float acc = 0.f;
  for (int j = 0; j < K; ++j) {
    const int at = i - (K - 1) + j;
    const float x = at >= 0 ? proj[(first_row + at) * ldp + col] : line[(long)(i + j) * C + ch];
    acc += taps[(long)ch * K + j] * x;
  }
  return acc * dr_sigmoid(acc);
}

// grid (rows, units), one wave each. Units: the G query heads (unit vectors times dim^-1/2), the G key heads (unit
// vectors), blocks of 64 value channels, and one for the heads' beta = sigmoid(.). out: [rows][C + H], C = 2 G D + H V.
__global__ __launch_bounds__(TIS_WAVE) void delta_prepare_kernel(
    const float* __restrict__ proj, long ldp, int conv_off, int beta_off, const float* __restrict__ taps, int K,
    const float* __restrict__ state, long lds, int conv_at, const int* __restrict__ row_seq, const int* __restrict__ cu_rows,
    const int* __restrict__ seq_slots, float* __restrict__ out, long ldo, int H, int G, int D, int V) {
  const long r = blockIdx.x;
  const int unit = blockIdx.y, lane = threadIdx.x;
  const int C = 2 * G * D + H * V;
  const int s = row_seq[r];
  const long first_row = cu_rows[s];
  const int i = (int)(r - first_row);
  const float* line = state + (long)seq_slots[s] * lds + conv_at;
  if (unit < 2 * G) {
    float y[DR_PER];
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < DR_PER; ++u) {
      const int e = lane + u * TIS_WAVE;
      y[u] = 0.f;
      if (e < D) {
        const int ch = unit * D + e;
        y[u] = dr_conv(proj, ldp, conv_off + ch, taps, K, ch, C, line, first_row, i);
        ss += y[u] * y[u];
      }
    }
    ss = wave_sum(ss);
    const float mul = (unit < G ? 1.f / sqrtf((float)D) : 1.f) / sqrtf(ss + 1e-6f);
#pragma unroll
    for (int u = 0; u < DR_PER; ++u) {
      const int e = lane + u * TIS_WAVE;
      if (e < D) out[r * ldo + unit * D + e] = y[u] * mul;
    }
    return;
  }
  const int v_blocks = (H * V + TIS_WAVE - 1) / TIS_WAVE;
  if (unit < 2 * G + v_blocks) {
    const int e = (unit - 2 * G) * TIS_WAVE + lane;
    if (e < H * V) {
      const int ch = 2 * G * D + e;
      out[r * ldo + ch] = dr_conv(proj, ldp, conv_off + ch, taps, K, ch, C, line, first_row, i);
    }
    return;
  }
  for (int h = lane; h < H; h += TIS_WAVE) out[r * ldo + C + h] = dr_sigmoid(proj[r * ldp + beta_off + h]);
}

// The walk. grid (requests, heads, blocks of 16 value channels), 256 threads: thread (c, l) = (t / 16, t % 16) owns, for
// value channel c, the state's key channels [l * R, (l + 1) * R) in registers from the line before the first row to the
// line after the last. A token's two sums over the key channels (S^T k and S^T q) are R terms a lane and a butterfly over
// the 16 lanes of a column: every state element sees its rows strictly in order and every sum has one fixed order, so a
// row's result does not depend on how its prompt was cut or on what else is in the step, bit for bit. Rows come through
// LDS `tokens` at a time: [tokens][k: D | decay: D | q: D | v: 16 | beta: 1].
template <int R>
__global__ __launch_bounds__(256) void delta_scan_kernel(
    const float* __restrict__ u, long ldu, int q_off, int k_off, int v_off, int beta_off, const float* __restrict__ decay,
    long ldd, float* __restrict__ state, long lds, const int* __restrict__ cu_rows, const int* __restrict__ seq_slots,
    float* __restrict__ out, long ldo, int H, int G, int D, int V, int tokens) {
  extern __shared__ float dr_lds[];
  const int s = blockIdx.x, h = blockIdx.y, vb = blockIdx.z, t = threadIdx.x;
  const int first = cu_rows[s], n_rows = cu_rows[s + 1] - first;
  if (n_rows <= 0) return;
  const int c = vb * 16 + t / 16, l = t % 16;
  const bool live = c < V;
  const int hq = h / (H / G);
  const int Dp = 16 * R;                     // key channels as the lanes hold them (those from D on are zeros)
  const int stride = 3 * Dp + 17;
  float* S_line = state + (long)seq_slots[s] * lds + (long)h * D * V;
  float S[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int d = l * R + i;
    S[i] = (live && d < D) ? S_line[(long)d * V + c] : 0.f;
  }
  for (int r0 = 0; r0 < n_rows; r0 += tokens) {
    const int n = min(tokens, n_rows - r0);
    __syncthreads();
    for (int i = t; i < n * Dp; i += 256) {
      const int tt = i / Dp, d = i % Dp;
      const long row = first + r0 + tt;
      float* dst = dr_lds + tt * stride;
      dst[d] = d < D ? u[row * ldu + k_off + hq * D + d] : 0.f;
      dst[Dp + d] = d < D ? decay[row * ldd + h * D + d] : 0.f;
      dst[2 * Dp + d] = d < D ? u[row * ldu + q_off + hq * D + d] : 0.f;
    }
    for (int i = t; i < n * 17; i += 256) {
      const int tt = i / 17, j = i % 17;
      const long row = first + r0 + tt;
      const int cc = vb * 16 + j;
      dr_lds[tt * stride + 3 * Dp + j] = j == 16 ? u[row * ldu + beta_off + h] : (cc < V ? u[row * ldu + v_off + h * V + cc] : 0.f);
    }
    __syncthreads();
    for (int tt = 0; tt < n; ++tt) {
      const float* src = dr_lds + tt * stride;
      const float* kk = src + l * R;
      const float* aa = src + Dp + l * R;
      const float* qq = src + 2 * Dp + l * R;
      float kv[R];
      float dot = 0.f;
#pragma unroll
      for (int i = 0; i < R; ++i) {
        kv[i] = kk[i];
        S[i] *= aa[i];
        dot += S[i] * kv[i];
      }
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) dot += __shfl_xor(dot, o, TIS_WAVE);
      const float w = src[3 * Dp + 16] * (src[3 * Dp + t / 16] - dot);
      float res = 0.f;
#pragma unroll
      for (int i = 0; i < R; ++i) {
        S[i] += kv[i] * w;
        res += S[i] * qq[i];
      }
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) res += __shfl_xor(res, o, TIS_WAVE);
      if (live && l == 0) out[(long)(first + r0 + tt) * ldo + h * V + c] = res;
    }
  }
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int d = l * R + i;
    if (live && d < D) S_line[(long)d * V + c] = S[i];
  }
}

TIS_EXPORT int tis_delta_prepare(const float* proj, long ldp, int conv_off, int beta_off, const float* taps, int K,
                                 const float* state, long lds, int conv_at, const int* row_seq, const int* cu_rows,
                                 const int* seq_slots, float* out, long ldo, int rows, int H, int G, int D, int V,
                                 hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || H < 1 || G < 1 || H % G || D < 1 || D > DR_PER * TIS_WAVE || V < 1 || K < 1 || K > DR_MAX_TAPS)
    return tis_fail("delta_prepare: bad size rows=%d heads=%d qk_heads=%d dim=%d (at most %d) vdim=%d taps=%d (at most %d)",
                    rows, H, G, D, DR_PER * TIS_WAVE, V, K, DR_MAX_TAPS);
  const int units = 2 * G + (H * V + TIS_WAVE - 1) / TIS_WAVE + 1;
  if (units > 65535) return tis_fail("delta_prepare: %d units a row are too many", units);
  delta_prepare_kernel<<<dim3(rows, units), TIS_WAVE, 0, stream>>>(proj, ldp, conv_off, beta_off, taps, K, state, lds, conv_at,
                                                                   row_seq, cu_rows, seq_slots, out, ldo, H, G, D, V);
  return tis_launch_status("delta_prepare");
}

TIS_EXPORT int tis_delta_scan(const float* u, long ldu, int q_off, int k_off, int v_off, int beta_off, const float* decay,
                              long ldd, float* state, long lds, const int* cu_rows, const int* seq_slots, int n_seqs,
                              float* out, long ldo, int H, int G, int D, int V, hipStream_t stream) {
  if (n_seqs == 0) return 0;
  if (n_seqs < 0 || H < 1 || H > 65535 || G < 1 || H % G || D < 1 || D > 256 || V < 1 || (V + 15) / 16 > 65535)
    return tis_fail("delta_scan: bad size requests=%d heads=%d qk_heads=%d dim=%d (at most 256) vdim=%d", n_seqs, H, G, D, V);
  const int R = D <= 16 ? 1 : D <= 32 ? 2 : D <= 64 ? 4 : D <= 128 ? 8 : 16;
  const int tokens = R <= 8 ? 16 : 8;
  const size_t lds_bytes = (size_t)tokens * (3 * 16 * R + 17) * sizeof(float);
  dim3 grid(n_seqs, H, (V + 15) / 16);
#define DR_SCAN(RR)                                                                                                        \
  delta_scan_kernel<RR><<<grid, 256, lds_bytes, stream>>>(u, ldu, q_off, k_off, v_off, beta_off, decay, ldd, state, lds,   \
                                                          cu_rows, seq_slots, out, ldo, H, G, D, V, tokens)
  switch (R) {
    case 1: DR_SCAN(1); break;
    case 2: DR_SCAN(2); break;
    case 4: DR_SCAN(4); break;
    case 8: DR_SCAN(8); break;
    default: DR_SCAN(16); break;
  }
#undef DR_SCAN
  return tis_launch_status("delta_scan");
}
