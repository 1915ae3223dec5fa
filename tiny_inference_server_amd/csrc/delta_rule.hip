// A gated delta rule: a matrix state per head that is corrected towards each new value, with a decay per key channel.
//
//   S <- diag(a_t) S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t
//
// per head and row, S being 32-bit floats in the request's state line, laid out [head][block of 16 value channels]
// [key channel][16] (value channels rounded up to a multiple of 16; the channels beyond stay zero), so that the part
// of a line that one workgroup of the walk owns is one run of memory. Two kernels: the
// step before the walk (a short causal convolution with silu over the q, k and v columns of a 32-bit input product,
// unit q and k per head, beta) and the walk itself. Everything is 32-bit.
//
// A request's state line holds S and, from float `conv_at` on, the convolution's last taps - 1
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

// Sum over the 16 lanes of a row of lanes (lanes 16 r .. 16 r + 15), every lane gets it: four data-parallel moves
// inside the row (two inside quads, then the half row and the row mirrored), no trip through LDS. One fixed order.
__device__ __forceinline__ float dr_row_sum(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));    // quad_perm [1,0,3,2]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));    // quad_perm [2,3,0,1]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));   // row_half_mirror
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));   // row_mirror
  return v;
}

// The walk. grid (blocks of 16 value channels, heads, requests), 256 threads: thread (c, l) = (t / 16, t % 16) owns, for
// value channel c, the state's key channels [l * R, (l + 1) * R) in registers from the line before the first row to the
// line after the last (the line goes through LDS both ways, so that memory sees whole runs of 16 channels). With
// S' = diag(a) S, a token needs S'^T k for its write and (S' + k w^T)^T q = S'^T q + (k . q) w for its read: the three
// sums over the key channels (S'^T k, S'^T q, k . q) are R terms a lane each and then one pass over the 16 lanes of a
// column for all three together. Every state element sees its rows strictly in order and every sum has one fixed
// order, so a row's result does not depend on how its prompt was cut or on what else is in the step, bit for bit.
// Rows come through LDS 16 at a time (8 where a lane holds 16 key channels): [rows][k: Dp | decay: Dp | q: Dp | v: 16 | beta | 3 unused].
template <int R>
__global__ __launch_bounds__(256) void delta_scan_kernel(
    const float* __restrict__ u, long ldu, int q_off, int k_off, int v_off, int beta_off, const float* __restrict__ decay,
    long ldd, float* __restrict__ state, long lds, const int* __restrict__ cu_rows, const int* __restrict__ seq_slots,
    float* __restrict__ out, long ldo, int H, int G, int D, int V, int tokens) {
  extern __shared__ __attribute__((aligned(16))) float dr_lds[];
  const int s = blockIdx.z, h = blockIdx.y, vb = blockIdx.x, t = threadIdx.x;
  const int first = cu_rows[s], n_rows = cu_rows[s + 1] - first;
  if (n_rows <= 0) return;
  const int cl = t / 16, l = t % 16;
  const int c = vb * 16 + cl;
  const bool live = c < V;
  const int hq = h / (H / G);
  constexpr int Dp = 16 * R;                 // key channels as the lanes hold them (those from D on are zeros)
  constexpr int stride = 3 * Dp + 20;
  // this block's [D][16] part of the line: one run of memory, into LDS 16 bytes a lane, then each lane's own elements
  float* S_line = state + (long)seq_slots[s] * lds + ((long)h * gridDim.x + vb) * D * 16;
  for (int e = t; e < D * 4; e += 256)
    reinterpret_cast<float4*>(dr_lds)[e] = reinterpret_cast<const float4*>(S_line)[e];
  __syncthreads();
  float S[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int d = l * R + i;
    S[i] = d < D ? dr_lds[d * 16 + cl] : 0.f;
  }
  // Rows go through two LDS buffers: while one chunk of rows is walked, the next one's loads are in flight in registers
  // and are put into the other buffer afterwards, so one barrier a chunk and no wait for memory between chunks.
  constexpr int TOK = R <= 8 ? 16 : 8;       // rows a chunk (`tokens`)
  constexpr int NI = TOK * Dp / 256;         // k, decay and q elements a thread fetches for a chunk
  float pk[NI], pa[NI], pq[NI], pv[2];
  auto fetch = [&](int r0) {
    const int n = min(TOK, n_rows - r0);
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int i = t + 256 * j, tt = i / Dp, d = i % Dp;
      const long row = first + r0 + tt;
      const bool ok = tt < n && d < D;
      pk[j] = ok ? u[row * ldu + k_off + hq * D + d] : 0.f;
      pa[j] = ok ? decay[row * ldd + h * D + d] : 0.f;
      pq[j] = ok ? u[row * ldu + q_off + hq * D + d] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int i = t + 256 * j, tt = i / 17, e = i % 17;
      const long row = first + r0 + tt;
      const int cc = vb * 16 + e;
      pv[j] = tt < n ? (e == 16 ? u[row * ldu + beta_off + h] : (cc < V ? u[row * ldu + v_off + h * V + cc] : 0.f)) : 0.f;
    }
  };
  auto commit = [&](float* buf) {
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int i = t + 256 * j, tt = i / Dp, d = i % Dp;
      float* dst = buf + tt * stride;
      dst[d] = pk[j];
      dst[Dp + d] = pa[j];
      dst[2 * Dp + d] = pq[j];
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int i = t + 256 * j, tt = i / 17, e = i % 17;
      if (tt < TOK) buf[tt * stride + 3 * Dp + e] = pv[j];
    }
  };
  __syncthreads();               // every lane has taken its part of the line out of LDS
  fetch(0);
  commit(dr_lds);
  __syncthreads();
  int which = 0;
  for (int r0 = 0; r0 < n_rows; r0 += TOK, which ^= 1) {
    const int n = min(TOK, n_rows - r0);
    const bool more = r0 + TOK < n_rows;
    if (more) fetch(r0 + TOK);
    const float* rows_lds = dr_lds + which * (TOK * stride);
    for (int tt = 0; tt < n; ++tt) {
      const float* src = rows_lds + tt * stride;
      float kv[R], av[R], qv[R];
      if constexpr (R % 4 == 0) {
#pragma unroll
        for (int i = 0; i < R; i += 4) {
          const float4 a = *reinterpret_cast<const float4*>(src + l * R + i);
          const float4 b = *reinterpret_cast<const float4*>(src + Dp + l * R + i);
          const float4 q4 = *reinterpret_cast<const float4*>(src + 2 * Dp + l * R + i);
          kv[i] = a.x, kv[i + 1] = a.y, kv[i + 2] = a.z, kv[i + 3] = a.w;
          av[i] = b.x, av[i + 1] = b.y, av[i + 2] = b.z, av[i + 3] = b.w;
          qv[i] = q4.x, qv[i + 1] = q4.y, qv[i + 2] = q4.z, qv[i + 3] = q4.w;
        }
      } else {
#pragma unroll
        for (int i = 0; i < R; ++i) {
          kv[i] = src[l * R + i];
          av[i] = src[Dp + l * R + i];
          qv[i] = src[2 * Dp + l * R + i];
        }
      }
      float dk = 0.f, dq = 0.f, kq = 0.f;
#pragma unroll
      for (int i = 0; i < R; ++i) {
        S[i] *= av[i];
        dk += S[i] * kv[i];
        dq += S[i] * qv[i];
        kq += kv[i] * qv[i];
      }
      dk = dr_row_sum(dk);
      dq = dr_row_sum(dq);
      kq = dr_row_sum(kq);
      const float w = src[3 * Dp + 16] * (src[3 * Dp + cl] - dk);
#pragma unroll
      for (int i = 0; i < R; ++i) S[i] += kv[i] * w;
      if (live && l == 0) out[(long)(first + r0 + tt) * ldo + h * V + c] = dq + kq * w;
    }
    if (more) commit(dr_lds + (which ^ 1) * (TOK * stride));
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int d = l * R + i;
    if (d < D) dr_lds[d * 16 + cl] = S[i];
  }
  __syncthreads();
  // (channels beyond vdim have seen values of zero only and are still zero)
  for (int e = t; e < D * 4; e += 256)
    reinterpret_cast<float4*>(S_line)[e] = reinterpret_cast<const float4*>(dr_lds)[e];
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
  if (n_seqs < 0 || n_seqs > 65535 || H < 1 || H > 65535 || G < 1 || H % G || D < 1 || D > 256 || V < 1 || lds % 4 ||
      ((uintptr_t)state % 16))
    return tis_fail("delta_scan: bad size requests=%d heads=%d qk_heads=%d dim=%d (at most 256) vdim=%d, or state lines that are "
                    "not 16 bytes aligned", n_seqs, H, G, D, V);
  const int R = D <= 16 ? 1 : D <= 32 ? 2 : D <= 64 ? 4 : D <= 128 ? 8 : 16;
  const int tokens = R <= 8 ? 16 : 8;
  size_t lds_bytes = 2 * (size_t)tokens * (3 * 16 * R + 20) * sizeof(float);      // two buffers of rows
  if (lds_bytes < (size_t)D * 16 * sizeof(float)) lds_bytes = (size_t)D * 16 * sizeof(float);      // the line's way in and out
  dim3 grid((V + 15) / 16, H, n_seqs);
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
