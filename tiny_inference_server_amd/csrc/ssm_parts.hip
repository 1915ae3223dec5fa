// What stands around the scan of a selective state-space mixer (csrc/state_scan.hip walks the state itself):
//
//   conv_prepare       a short causal convolution per channel with silu over the columns [x | B | C] of the input
//                      product, the step size dt = softplus(dt_raw + dt_bias) per head, and from them what the scan
//                      reads: x * dt (the scan's values), exp(a * dt) (its decay, one per head and row), B (its keys)
//                      and C (its queries)
//   conv_state_update  the last taps - 1 inputs of every channel, kept per request beside the matrix state
//   gated_group_norm   (y + D * x) * silu(z), RMS-normed in equal parts of the row, times a gain
//
// A request's convolution state is [taps - 1][channels] 32-bit floats in its state line, oldest input first; a line
// taken anew is all zeros, which is what lies before a sequence's first token. A row reads the inputs of the rows
// before it from this step's rows where they are part of the step and from the state otherwise, so a result does not
// depend on where a prompt was cut. Everything is 32-bit; `T` is the compute type of the normed output.
#include "common.h"

TIS_DEFINE_LAST_ERROR(tis_ssm)

static constexpr int SSM_THREADS = 256;
static constexpr int SSM_MAX_TAPS = 16;

__device__ __forceinline__ float ssm_silu(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float ssm_softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// grid (rows * blocks of SSM_THREADS * per_thread channels, a row's blocks side by side): with few rows a thread has one
// channel of one row (per_thread 1), so that the step still fills the chip and no thread walks a chain of dependent
// loads; with many rows it has several, so that the grid is not made of crumbs. proj: a row's input product in 32-bit, the convolution's
// channels from xbc_off, dt_raw from dt_off. u (out) [rows][ldu]: [conv channels (x: H*P, then B and C) | x * dt: H*P |
// decay: H].
__global__ __launch_bounds__(SSM_THREADS) void conv_prepare_kernel(
    const float* __restrict__ proj, long ldp, int xbc_off, int dt_off, const float* __restrict__ taps,
    const float* __restrict__ tap_bias, const float* __restrict__ dt_bias, const float* __restrict__ neg_a,
    const float* __restrict__ state, long state_ld, int conv_at, const int* __restrict__ row_seq,
    const int* __restrict__ cu_rows, const int* __restrict__ seq_slots, float* __restrict__ u, long ldu, int C, int K,
    int H, int P, int row_blocks, int per_thread) {
  const long r = blockIdx.x / row_blocks;
  const int block = blockIdx.x % row_blocks;
  const int seq = row_seq[r];
  const int t = (int)(r - cu_rows[seq]);                    // rows of this request that the step brings before this one
  const float* old = state + (long)seq_slots[seq] * state_ld + conv_at;
  const float* row = proj + r * ldp;
  const int inner = H * P;
  for (int i = 0; i < per_thread; ++i) {
    const int c = (block * per_thread + i) * SSM_THREADS + threadIdx.x;
    if (c >= C) break;
    float acc = tap_bias ? tap_bias[c] : 0.f;
#pragma unroll 4
    for (int j = 0; j < K; ++j) {
      const int back = K - 1 - j;                           // the last tap weighs the row itself
      const float v = back <= t ? row[xbc_off + c - (long)back * ldp] : old[(long)(K - 1 + t - back) * C + c];
      acc += taps[(long)c * K + j] * v;
    }
    const float y = ssm_silu(acc);
    u[r * ldu + c] = y;
    if (c < inner) {
      const int h = c / P;
      u[r * ldu + C + c] = y * ssm_softplus(row[dt_off + h] + dt_bias[h]);
    }
  }
  if (block == 0)
    for (int h = threadIdx.x; h < H; h += SSM_THREADS)
      u[r * ldu + C + inner + h] = expf(neg_a[h] * ssm_softplus(row[dt_off + h] + dt_bias[h]));
}

// grid (requests of the step, blocks of SSM_THREADS channels). A thread owns one channel of one request: it reads the
// channel's old inputs before it writes the new.
__global__ __launch_bounds__(SSM_THREADS) void conv_state_update_kernel(const float* __restrict__ proj, long ldp, int xbc_off,
                                                                         float* __restrict__ state, long state_ld,
                                                                         int conv_at, const int* __restrict__ cu_rows,
                                                                         const int* __restrict__ seq_slots, int C, int K) {
  const int seq = blockIdx.x;
  const int r0 = cu_rows[seq], n = cu_rows[seq + 1] - r0;
  const int c = blockIdx.y * SSM_THREADS + threadIdx.x;
  if (n <= 0 || c >= C) return;
  float* line = state + (long)seq_slots[seq] * state_ld + conv_at;
  float next[SSM_MAX_TAPS];
#pragma unroll
  for (int k = 0; k < SSM_MAX_TAPS; ++k) {
    if (k >= K - 1) break;
    const int at = n - (K - 1) + k;                         // which row of the step becomes entry k (negative: an old one)
    next[k] = at >= 0 ? proj[(long)(r0 + at) * ldp + xbc_off + c] : line[(long)(k + n) * C + c];
  }
#pragma unroll
  for (int k = 0; k < SSM_MAX_TAPS; ++k) {
    if (k >= K - 1) break;
    line[(long)k * C + c] = next[k];
  }
}

// grid (rows, parts). v = (y + skip[head] * x) * silu(z) for the columns of one part of the row (width / parts
// each), then v / sqrt(mean(v^2) + eps) * gain. skip and z may be null. y, x, z are 32-bit (strided views are fine).
template <typename T>
__global__ __launch_bounds__(SSM_THREADS) void gated_group_norm_kernel(
    const float* __restrict__ y, long ldy, const float* __restrict__ x, long ldx, const float* __restrict__ skip, int P,
    const float* __restrict__ z, long ldz, const float* __restrict__ gain, float eps, T* __restrict__ out, long ldo,
    int part_width) {
  __shared__ float red[16];
  const long r = blockIdx.x;
  const int c0 = blockIdx.y * part_width;
  auto value = [&](int c) {
    float v = y[r * ldy + c];
    if (skip) v += skip[c / P] * x[r * ldx + c];
    if (z) v *= ssm_silu(z[r * ldz + c]);
    return v;
  };
  // a part of up to SSM_KEEP * SSM_THREADS columns stays in registers between the sum of squares and the division (its
  // loads are all in flight together); a wider one is read again
  constexpr int SSM_KEEP = 8;
  float kept[SSM_KEEP];
  float ss = 0.f;
  if (part_width <= SSM_KEEP * SSM_THREADS) {
#pragma unroll
    for (int i = 0; i < SSM_KEEP; ++i) {
      const int e = threadIdx.x + i * SSM_THREADS;
      kept[i] = e < part_width ? value(c0 + e) : 0.f;
    }
#pragma unroll
    for (int i = 0; i < SSM_KEEP; ++i) ss += kept[i] * kept[i];
    const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)part_width + eps);
#pragma unroll
    for (int i = 0; i < SSM_KEEP; ++i) {
      const int e = threadIdx.x + i * SSM_THREADS;
      if (e < part_width) out[r * ldo + c0 + e] = from_f<T>(kept[i] * inv * gain[c0 + e]);
    }
    return;
  }
  for (int e = threadIdx.x; e < part_width; e += SSM_THREADS) {
    const float v = value(c0 + e);
    ss += v * v;
  }
  const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)part_width + eps);
  for (int e = threadIdx.x; e < part_width; e += SSM_THREADS)
    out[r * ldo + c0 + e] = from_f<T>(value(c0 + e) * inv * gain[c0 + e]);
}

TIS_EXPORT int tis_conv_prepare(const float* proj, long ldp, int xbc_off, int dt_off, const float* taps,
                                const float* tap_bias, const float* dt_bias, const float* neg_a, const float* state,
                                long state_ld, int conv_at, const int* row_seq, const int* cu_rows, const int* seq_slots,
                                float* u, long ldu, int rows, int C, int K, int H, int P, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || C < 1 || K < 1 || K > SSM_MAX_TAPS || H < 1 || P < 1 || H * P > C || !taps || !dt_bias || !neg_a || !state)
    return tis_fail("conv_prepare: bad size rows=%d channels=%d taps=%d (at most %d) heads=%d of %d", rows, C, K,
                    SSM_MAX_TAPS, H, P);
  if (ldu < (long)C + (long)H * P + H || state_ld < (long)conv_at + (long)(K - 1) * C)
    return tis_fail("conv_prepare: rows of %ld floats for %ld, state lines of %ld for %ld", ldu, (long)C + (long)H * P + H,
                    state_ld, (long)conv_at + (long)(K - 1) * C);
  // as many channels a thread as keep the grid at about what the chip holds at once (a workgroup first finds its row's
  // request and state line, a chain of loads that further rounds of workgroups would pay again)
  const int blocks_a_row = (C + SSM_THREADS - 1) / SSM_THREADS;
  int per_thread = (int)(((long)rows * blocks_a_row + 2047) / 2048);
  per_thread = per_thread < 1 ? 1 : per_thread > blocks_a_row ? blocks_a_row : per_thread;
  const int row_blocks = (blocks_a_row + per_thread - 1) / per_thread;
  if ((long)rows * row_blocks > 0x7fffffffL) return tis_fail("conv_prepare: %d rows of %d channels in one call", rows, C);
  conv_prepare_kernel<<<rows * row_blocks, SSM_THREADS, 0, stream>>>(
      proj, ldp, xbc_off, dt_off, taps, tap_bias, dt_bias, neg_a, state, state_ld, conv_at, row_seq, cu_rows, seq_slots, u, ldu,
      C, K, H, P, row_blocks, per_thread);
  return tis_launch_status("conv_prepare");
}

TIS_EXPORT int tis_conv_state_update(const float* proj, long ldp, int xbc_off, float* state, long state_ld, int conv_at,
                                     const int* cu_rows, const int* seq_slots, int n_seqs, int C, int K,
                                     hipStream_t stream) {
  if (n_seqs == 0 || K == 1) return 0;
  if (n_seqs < 0 || C < 1 || K < 1 || K > SSM_MAX_TAPS || state_ld < (long)conv_at + (long)(K - 1) * C)
    return tis_fail("conv_state_update: bad size requests=%d channels=%d taps=%d state line=%ld", n_seqs, C, K, state_ld);
  conv_state_update_kernel<<<dim3(n_seqs, (C + SSM_THREADS - 1) / SSM_THREADS), SSM_THREADS, 0, stream>>>(proj, ldp, xbc_off, state, state_ld, conv_at, cu_rows,
                                                               seq_slots, C, K);
  return tis_launch_status("conv_state_update");
}

TIS_EXPORT int tis_gated_group_norm(int dtype, const float* y, long ldy, const float* x, long ldx, const float* skip, int P,
                                    const float* z, long ldz, const float* gain, float eps, void* out, long ldo, int rows,
                                    int width, int parts, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || width < 1 || parts < 1 || parts > 65535 || width % parts || !y || !gain || !out || (skip && (!x || P < 1)))
    return tis_fail("gated_group_norm: bad size rows=%d width=%d parts=%d", rows, width, parts);
  dim3 grid(rows, parts);
  if (dtype == TIS_F32)
    gated_group_norm_kernel<float><<<grid, SSM_THREADS, 0, stream>>>(y, ldy, x, ldx, skip, P, z, ldz, gain, eps, (float*)out,
                                                                      ldo, width / parts);
  else if (dtype == TIS_BF16)
    gated_group_norm_kernel<bf16><<<grid, SSM_THREADS, 0, stream>>>(y, ldy, x, ldx, skip, P, z, ldz, gain, eps, (bf16*)out,
                                                                     ldo, width / parts);
  else
    return tis_fail("unknown dtype code %d", dtype);
  return tis_launch_status("gated_group_norm");
}
