// Row-wise kernels for models whose residual stream is kept in 32-bit whatever the compute type: scaled embedding,
// the gated sum followed by an RMS norm (norm after the sum), the closing RMS norm, the per-head norm and output gate
// of recurrent mixers, and the low-rank decay of gated linear attention.
//
// The RMS norm here is x / sqrt(mean(x^2) + eps) * gain, eps under the root. Every sum is taken in 32-bit in an order
// that depends on the row's width alone. `T` is the compute type (float or bf16): what the next matrix product reads.
#include "common.h"

TIS_DEFINE_LAST_ERROR(tis_stream32)

static constexpr int S32_THREADS = 256;

__device__ __forceinline__ float sigmoid_f(float z) { return 1.f / (1.f + expf(-z)); }
__device__ __forceinline__ float log_sigmoid_f(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// x32[r] = table[token[r]] * scale, and the same rows in the compute type
template <typename T>
__global__ __launch_bounds__(S32_THREADS) void embed_scale_kernel(const T* __restrict__ table, const int* __restrict__ tokens,
                                                                   float scale, float* __restrict__ out32,
                                                                   T* __restrict__ outT, int D) {
  const long r = blockIdx.x;
  const T* src = table + (long)tokens[r] * D;
  for (int c = threadIdx.x; c < D; c += S32_THREADS) {
    const float v = to_f(src[c]) * scale;
    out32[r * D + c] = v;
    if (outT) outT[r * D + c] = from_f<T>(v);
  }
}

// r = alpha * x + sigmoid(gate + bias) * (s0 * y0 + s1 * y1);  out = r / sqrt(mean(r^2) + eps) * gain
// y1 and gate may be null (one branch; no gate).
template <typename T, int PER>      // PER: values a thread keeps in registers (width <= 256 * PER); 0: any width, through memory
__global__ __launch_bounds__(S32_THREADS) void gated_postnorm_kernel(
    const float* __restrict__ x, const float* __restrict__ y0, long ld0, float s0, const float* __restrict__ y1, long ld1,
    float s1, const float* __restrict__ gate, long ldg, const float* __restrict__ bias, float alpha,
    const float* __restrict__ gain, float eps, float* __restrict__ out32, T* __restrict__ outT, int D) {
  __shared__ float red[16];
  const long r = blockIdx.x;
  float ss = 0.f;
  float keep[PER > 0 ? PER : 1];
  auto summed = [&](int c) {
    float y = s0 * y0[r * ld0 + c];
    if (y1) y += s1 * y1[r * ld1 + c];
    if (gate) y *= sigmoid_f(gate[r * ldg + c] + (bias ? bias[c] : 0.f));
    return alpha * x[r * D + c] + y;
  };
  if (PER > 0) {
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int c = threadIdx.x + k * S32_THREADS;
      keep[k] = c < D ? summed(c) : 0.f;
      ss += keep[k] * keep[k];
    }
  } else {
    for (int c = threadIdx.x; c < D; c += S32_THREADS) {
      const float v = summed(c);
      out32[r * D + c] = v;
      ss += v * v;
    }
  }
  ss = block_sum(ss, red);      // (the order of this sum depends on the width alone, whichever way the values are kept)
  const float inv = 1.f / sqrtf(ss / (float)D + eps);
  if (PER > 0) {
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int c = threadIdx.x + k * S32_THREADS;
      if (c < D) {
        const float v = keep[k] * inv * gain[c];
        out32[r * D + c] = v;
        if (outT) outT[r * D + c] = from_f<T>(v);
      }
    }
  } else {
    for (int c = threadIdx.x; c < D; c += S32_THREADS) {
      const float v = out32[r * D + c] * inv * gain[c];
      out32[r * D + c] = v;
      if (outT) outT[r * D + c] = from_f<T>(v);
    }
  }
}

// out = x / sqrt(mean(x^2) + eps) * gain, from the 32-bit stream into the compute type
template <typename T>
__global__ __launch_bounds__(S32_THREADS) void rmsnorm32_kernel(const float* __restrict__ x, const float* __restrict__ gain,
                                                                 float eps, T* __restrict__ out, long ldo, int D) {
  __shared__ float red[16];
  const long r = blockIdx.x;
  float ss = 0.f;
  for (int c = threadIdx.x; c < D; c += S32_THREADS) {
    const float v = x[r * D + c];
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)D + eps);
  for (int c = threadIdx.x; c < D; c += S32_THREADS) out[r * ldo + c] = from_f<T>(x[r * D + c] * inv * gain[c]);
}

// One wave per (row, head): o / sqrt(mean_over_V(o^2) + eps) * gain * act(g). gain is [V] shared by the heads or
// [H * V]; act 0: g * sigmoid(g), 1: sigmoid(g).
template <typename T>
__global__ __launch_bounds__(TIS_WAVE) void head_norm_gate_kernel(const float* __restrict__ o, long ldo,
                                                                   const float* __restrict__ g, long ldg,
                                                                   const float* __restrict__ gain, int gain_per_head,
                                                                   int act, float eps, T* __restrict__ out, long ldout,
                                                                   int V) {
  const long r = blockIdx.x;
  const int h = blockIdx.y;
  const float* src = o + r * ldo + (long)h * V;
  float ss = 0.f;
  for (int j = threadIdx.x; j < V; j += TIS_WAVE) ss += src[j] * src[j];
  ss = wave_sum(ss);
  const float inv = 1.f / sqrtf(ss / (float)V + eps);
  for (int j = threadIdx.x; j < V; j += TIS_WAVE) {
    const float z = g[r * ldg + (long)h * V + j];
    const float a = act == 0 ? z * sigmoid_f(z) : sigmoid_f(z);
    out[r * ldout + (long)h * V + j] = from_f<T>(src[j] * inv * gain[gain_per_head ? h * V + j : j] * a);
  }
}

// decay[r][c] = sigmoid(z)^(1/tau) with z = sum_k low[r][k] * w2[c][k] + bias[c], as exp(log_sigmoid(z) / tau)
__global__ __launch_bounds__(S32_THREADS) void lowrank_decay_kernel(const float* __restrict__ low, long ldl, int rank,
                                                                     const float* __restrict__ w2,
                                                                     const float* __restrict__ bias, float tau,
                                                                     float* __restrict__ out, int C) {
  extern __shared__ float a[];
  const long r = blockIdx.x;
  for (int k = threadIdx.x; k < rank; k += S32_THREADS) a[k] = low[r * ldl + k];
  __syncthreads();
  for (int c = threadIdx.x; c < C; c += S32_THREADS) {
    float z = 0.f;
    const float* w = w2 + (long)c * rank;
    for (int k = 0; k < rank; ++k) z += a[k] * w[k];
    z += bias[c];
    out[r * C + c] = expf(log_sigmoid_f(z) / tau);
  }
}


// Layer norm of a 32-bit row into the compute type: (x - mean) / sqrt(var + eps) * gain + bias, the variance being the
// mean of the squared deviations (two passes over the row; bias may be null).
template <typename T>
__global__ __launch_bounds__(S32_THREADS) void layernorm32_kernel(const float* __restrict__ x, const float* __restrict__ gain,
                                                                   const float* __restrict__ bias, float eps,
                                                                   T* __restrict__ out, long ldo, int D) {
  __shared__ float red[16];
  const long r = blockIdx.x;
  float s = 0.f;
  for (int c = threadIdx.x; c < D; c += S32_THREADS) s += x[r * D + c];
  const float mean = block_sum(s, red) / (float)D;
  float ss = 0.f;
  for (int c = threadIdx.x; c < D; c += S32_THREADS) {
    const float d = x[r * D + c] - mean;
    ss += d * d;
  }
  const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)D + eps);
  for (int c = threadIdx.x; c < D; c += S32_THREADS)
    out[r * ldo + c] = from_f<T>((x[r * D + c] - mean) * inv * gain[c] + (bias ? bias[c] : 0.f));
}

// The residual sum of a 32-bit stream, with what usually follows it, in one pass over the row:
//   v = x + y                                  (y_gain null)
//   v = x + y / sqrt(mean(y^2) + y_eps) * y_gain   (an RMS norm on the branch before the sum)
// v goes to out32 (which may be x itself); `copy` (nullable) gets v in the compute type; `normed` (nullable) gets the
// norm of v in the compute type: kind 1 layer norm (gain, bias), kind 2 RMS norm (gain), eps under the root in both.
// Where the branch is a routed feed-forward's result that has not been summed yet: y then holds a line per (row, choice),
// and the branch's value at row r is sum_k weights[r][k] * (y[r * top + k] if ids[r][k] < n_experts else rows[r]): an
// id from n_experts on is an identity expert, whose result is the row it was given. ids null: y is the branch itself.
struct ChosenSum {
  const int* ids;
  const float* weights;
  int top, n_experts;
  const void* rows;      // [rows][ldr] in the compute type: what the feed-forward read
  long ldr;
  const float* extra = nullptr;        // [rows][lde]: what every row adds beside its choices (a shared expert's result),
  long lde = 0;                        // times sigmoid(extra_gate[row * ldg]); null: nothing
  const float* extra_gate = nullptr;
  long ldg = 0;
};

// PER: values a thread keeps in registers (width <= 256 * PER), so that the row is read once and the sums follow one
// another without a trip to memory between them; 0: any width, through out32.
template <typename T, int PER>
__global__ __launch_bounds__(S32_THREADS) void residual_norm_kernel(
    const float* __restrict__ x, const float* __restrict__ y_in, long ldy, const float* __restrict__ y_gain, float y_eps,
    float* __restrict__ out32, T* __restrict__ copy, long ldc, int norm_kind, const float* __restrict__ gain,
    const float* __restrict__ bias, float eps, T* __restrict__ normed, long ldn, int D, ChosenSum cs) {
  __shared__ float red[16];
  const long r = blockIdx.x;
  constexpr int P = PER > 0 ? PER : 1;
  const bool y = y_in != nullptr || cs.ids != nullptr;        // whether there is a branch at all
  // a row's choices and their weights, once for all its columns (up to 64 choices; beyond, from memory every time)
  __shared__ int chosen_id[64];
  __shared__ float chosen_w[64];
  const bool kept = cs.ids && cs.top <= 64;
  if (kept) {
    if (threadIdx.x < cs.top) {
      chosen_id[threadIdx.x] = cs.ids[r * cs.top + threadIdx.x];
      chosen_w[threadIdx.x] = cs.weights[r * cs.top + threadIdx.x];
    }
    __syncthreads();
  }
  auto y_at = [&](int c) {
    if (!cs.ids) return y_in[r * ldy + c];
    float v = 0.f;
    for (int k = 0; k < cs.top; ++k) {
      const int e = kept ? chosen_id[k] : cs.ids[r * cs.top + k];
      const float w = kept ? chosen_w[k] : cs.weights[r * cs.top + k];
      v += w * (e < cs.n_experts ? y_in[(r * cs.top + k) * ldy + c] : to_f(static_cast<const T*>(cs.rows)[r * cs.ldr + c]));
    }
    if (cs.extra) v += sigmoid_f(cs.extra_gate[r * cs.ldg]) * cs.extra[r * cs.lde + c];
    return v;
  };
  // (everything the row's columns need is asked for at once: the gains and the bias too, which are only used after
  // the sums, so that no trip to memory stands between two of them)
  float xv[P], yv[P], ygv[P], gv[P], bv[P];
  if (PER > 0) {
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int c = threadIdx.x + k * S32_THREADS;
      xv[k] = c < D ? x[r * D + c] : 0.f;
      yv[k] = (y && c < D) ? y_at(c) : 0.f;
      ygv[k] = (y && y_gain && c < D) ? y_gain[c] : 1.f;
      gv[k] = (norm_kind && c < D) ? gain[c] : 0.f;
      bv[k] = (norm_kind == 1 && bias && c < D) ? bias[c] : 0.f;
    }
  }
  float y_inv = 1.f;
  if (y && y_gain) {
    float ss = 0.f;
    if (PER > 0) {
#pragma unroll
      for (int k = 0; k < PER; ++k) ss += yv[k] * yv[k];
    } else {
      for (int c = threadIdx.x; c < D; c += S32_THREADS) {
        const float v = y_at(c);
        ss += v * v;
      }
    }
    y_inv = 1.f / sqrtf(block_sum(ss, red) / (float)D + y_eps);
  }
  float s = 0.f;
  if (PER > 0) {
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int c = threadIdx.x + k * S32_THREADS;
      if (c >= D) continue;
      float v = xv[k];
      if (y) v += y_gain ? yv[k] * y_inv * ygv[k] : yv[k];
      xv[k] = v;
      out32[r * D + c] = v;
      if (copy) copy[r * ldc + c] = from_f<T>(v);
      s += norm_kind == 2 ? v * v : v;
    }
  } else {
    for (int c = threadIdx.x; c < D; c += S32_THREADS) {
      float v = x[r * D + c];
      if (y) v += y_gain ? y_at(c) * y_inv * y_gain[c] : y_at(c);
      out32[r * D + c] = v;          // (each thread reads back only what it wrote itself)
      if (copy) copy[r * ldc + c] = from_f<T>(v);
      s += norm_kind == 2 ? v * v : v;
    }
  }
  if (!normed || norm_kind == 0) return;
  // every value of the row that this thread holds (with its gain and bias), from its registers or from memory
  auto each = [&](auto fn) {
    if (PER > 0) {
#pragma unroll
      for (int k = 0; k < P; ++k) {
        const int c = threadIdx.x + k * S32_THREADS;
        if (c < D) fn(xv[k], c, gv[k], bv[k]);
      }
    } else {
      for (int c = threadIdx.x; c < D; c += S32_THREADS) fn(out32[r * D + c], c, gain[c], (norm_kind == 1 && bias) ? bias[c] : 0.f);
    }
  };
  if (norm_kind == 2) {
    const float inv = 1.f / sqrtf(block_sum(s, red) / (float)D + eps);
    each([&](float v, int c, float g, float) { normed[r * ldn + c] = from_f<T>(v * inv * g); });
    return;
  }
  const float mean = block_sum(s, red) / (float)D;
  float ss = 0.f;
  each([&](float v, int, float, float) { ss += (v - mean) * (v - mean); });
  const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)D + eps);
  each([&](float v, int c, float g, float b) { normed[r * ldn + c] = from_f<T>((v - mean) * inv * g + b); });
}

__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// out[r][j] = act(z[r][j]) * table[token[r]][j]: a gate on a row of a per-token table. act 0: tanh-form gelu, 1: silu,
// 2: sigmoid. z is 32-bit (a strided view is fine), table and out are in the compute type.
template <typename T>
__global__ __launch_bounds__(S32_THREADS) void gate_table_kernel(const float* __restrict__ z, long ldz,
                                                                  const T* __restrict__ table, long ldt,
                                                                  const int* __restrict__ tokens, int act,
                                                                  T* __restrict__ out, long ldo, int rows, int W) {
  const long i = (long)blockIdx.x * S32_THREADS + threadIdx.x;
  if (i >= (long)rows * W) return;
  const long r = i / W;
  const int j = (int)(i % W);
  const float v = z[r * ldz + j];
  const float a = act == 0 ? gelu_tanh_f(v) : act == 1 ? v * sigmoid_f(v) : sigmoid_f(v);
  out[r * ldo + j] = from_f<T>(a * to_f(table[(long)tokens[r] * ldt + j]));
}

// In place on the columns [0, W) of 32-bit rows: act 1 silu, 2 sigmoid, 0 tanh-form gelu.
__global__ __launch_bounds__(S32_THREADS) void activate32_kernel(float* __restrict__ z, long ldz, int act, int rows, int W) {
  const long i = (long)blockIdx.x * S32_THREADS + threadIdx.x;
  if (i >= (long)rows * W) return;
  float* p = z + (i / W) * ldz + (i % W);
  const float v = *p;
  *p = act == 0 ? gelu_tanh_f(v) : act == 1 ? v * sigmoid_f(v) : sigmoid_f(v);
}

// x[r][h * V + j] *= sigmoid(gate[r][h]), in place
template <typename T>
__global__ __launch_bounds__(S32_THREADS) void head_gate_kernel(T* __restrict__ x, long ldx, const float* __restrict__ gate,
                                                                 long ldg, int rows, int H, int V) {
  const long i = (long)blockIdx.x * S32_THREADS + threadIdx.x;
  const long W = (long)H * V;
  if (i >= rows * W) return;
  const long r = i / W;
  const int c = (int)(i % W);
  x[r * ldx + c] = from_f<T>(to_f(x[r * ldx + c]) * sigmoid_f(gate[r * ldg + c / V]));
}

#define S32_DISPATCH(call_f32, call_bf16)                 \
  if (dtype == TIS_F32) { call_f32; }                     \
  else if (dtype == TIS_BF16) { call_bf16; }              \
  else return tis_fail("unknown dtype code %d", dtype);

TIS_EXPORT int tis_embed_scale(int dtype, const void* table, const int* tokens, float scale, float* out32, void* outT,
                               int rows, int D, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || D < 1) return tis_fail("embed_scale: bad size rows=%d width=%d", rows, D);
  S32_DISPATCH((embed_scale_kernel<float><<<rows, S32_THREADS, 0, stream>>>((const float*)table, tokens, scale, out32, (float*)outT, D)),
               (embed_scale_kernel<bf16><<<rows, S32_THREADS, 0, stream>>>((const bf16*)table, tokens, scale, out32, (bf16*)outT, D)))
  return tis_launch_status("embed_scale");
}

TIS_EXPORT int tis_gated_postnorm(int dtype, const float* x, const float* y0, long ld0, float s0, const float* y1, long ld1,
                                  float s1, const float* gate, long ldg, const float* bias, float alpha, const float* gain,
                                  float eps, float* out32, void* outT, int rows, int D, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || D < 1 || !x || !y0 || !gain || !out32) return tis_fail("gated_postnorm: bad arguments rows=%d width=%d", rows, D);
#define S32_POSTNORM(T, PER)                                                                                           \
  gated_postnorm_kernel<T, PER><<<rows, S32_THREADS, 0, stream>>>(x, y0, ld0, s0, y1, ld1, s1, gate, ldg, bias, alpha, gain, \
                                                                  eps, out32, (T*)outT, D)
#define S32_POSTNORM_BY_WIDTH(T)                         \
  if (D <= 4 * S32_THREADS) { S32_POSTNORM(T, 4); }      \
  else if (D <= 16 * S32_THREADS) { S32_POSTNORM(T, 16); } \
  else { S32_POSTNORM(T, 0); }
  S32_DISPATCH(S32_POSTNORM_BY_WIDTH(float), S32_POSTNORM_BY_WIDTH(bf16))
#undef S32_POSTNORM_BY_WIDTH
#undef S32_POSTNORM
  return tis_launch_status("gated_postnorm");
}

TIS_EXPORT int tis_rmsnorm32(int dtype, const float* x, const float* gain, float eps, void* out, long ldo, int rows, int D,
                             hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || D < 1) return tis_fail("rmsnorm32: bad size rows=%d width=%d", rows, D);
  S32_DISPATCH((rmsnorm32_kernel<float><<<rows, S32_THREADS, 0, stream>>>(x, gain, eps, (float*)out, ldo, D)),
               (rmsnorm32_kernel<bf16><<<rows, S32_THREADS, 0, stream>>>(x, gain, eps, (bf16*)out, ldo, D)))
  return tis_launch_status("rmsnorm32");
}

TIS_EXPORT int tis_head_norm_gate(int dtype, const float* o, long ldo, const float* g, long ldg, const float* gain,
                                  int gain_per_head, int act, float eps, void* out, long ldout, int rows, int H, int V,
                                  hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || H < 1 || H > 65535 || V < 1 || (act != 0 && act != 1))
    return tis_fail("head_norm_gate: bad size rows=%d heads=%d vdim=%d act=%d", rows, H, V, act);
  dim3 grid(rows, H);
  S32_DISPATCH((head_norm_gate_kernel<float><<<grid, TIS_WAVE, 0, stream>>>(o, ldo, g, ldg, gain, gain_per_head, act, eps, (float*)out, ldout, V)),
               (head_norm_gate_kernel<bf16><<<grid, TIS_WAVE, 0, stream>>>(o, ldo, g, ldg, gain, gain_per_head, act, eps, (bf16*)out, ldout, V)))
  return tis_launch_status("head_norm_gate");
}

TIS_EXPORT int tis_lowrank_decay(const float* low, long ldl, int rank, const float* w2, const float* bias, float tau,
                                 float* out, int rows, int C, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || rank < 1 || rank > 8192 || C < 1 || !(tau > 0.f))
    return tis_fail("lowrank_decay: bad size rows=%d rank=%d channels=%d tau=%g", rows, rank, C, (double)tau);
  lowrank_decay_kernel<<<rows, S32_THREADS, rank * sizeof(float), stream>>>(low, ldl, rank, w2, bias, tau, out, C);
  return tis_launch_status("lowrank_decay");
}

TIS_EXPORT int tis_layernorm32(int dtype, const float* x, const float* gain, const float* bias, float eps, void* out, long ldo,
                               int rows, int D, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || D < 1 || !x || !gain || !out) return tis_fail("layernorm32: bad arguments rows=%d width=%d", rows, D);
  S32_DISPATCH((layernorm32_kernel<float><<<rows, S32_THREADS, 0, stream>>>(x, gain, bias, eps, (float*)out, ldo, D)),
               (layernorm32_kernel<bf16><<<rows, S32_THREADS, 0, stream>>>(x, gain, bias, eps, (bf16*)out, ldo, D)))
  return tis_launch_status("layernorm32");
}

TIS_EXPORT int tis_residual_norm(int dtype, const float* x, const float* y, long ldy, const float* y_gain, float y_eps,
                                 float* out32, void* copy, long ldc, int norm_kind, const float* gain, const float* bias,
                                 float eps, void* normed, long ldn, int rows, int D, const int* ids, const float* weights,
                                 int top, int n_experts, const void* chosen_rows, long ldr, const float* extra, long lde,
                                 const float* extra_gate, long ldg, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || D < 1 || !x || !out32) return tis_fail("residual_norm: bad arguments rows=%d width=%d", rows, D);
  if (ids && (!weights || top < 1 || n_experts < 0 || (n_experts > 0 && !y) || !chosen_rows))
    return tis_fail("residual_norm: a sum over chosen experts needs ids, weights, the experts' results and the rows they read");
  if (extra && (!ids || !extra_gate)) return tis_fail("residual_norm: a shared term goes with chosen experts and has a gate");
  const ChosenSum cs{ids, weights, top, n_experts, chosen_rows, ldr, extra, lde, extra_gate, ldg};
  if (norm_kind < 0 || norm_kind > 2 || (norm_kind && (!gain || !normed)))
    return tis_fail("residual_norm: norm kind %d needs a gain and an output", norm_kind);
#define S32_RESIDUAL(T, PER)                                                                                              \
  residual_norm_kernel<T, PER><<<rows, S32_THREADS, 0, stream>>>(x, y, ldy, y_gain, y_eps, out32, (T*)copy, ldc, norm_kind, \
                                                                 gain, bias, eps, (T*)normed, ldn, D, cs)
#define S32_RESIDUAL_BY_WIDTH(T)                         \
  if (D <= 4 * S32_THREADS) { S32_RESIDUAL(T, 4); }      \
  else if (D <= 16 * S32_THREADS) { S32_RESIDUAL(T, 16); } \
  else { S32_RESIDUAL(T, 0); }
  S32_DISPATCH(S32_RESIDUAL_BY_WIDTH(float), S32_RESIDUAL_BY_WIDTH(bf16))
#undef S32_RESIDUAL_BY_WIDTH
#undef S32_RESIDUAL
  return tis_launch_status("residual_norm");
}

TIS_EXPORT int tis_gate_table(int dtype, const float* z, long ldz, const void* table, long ldt, const int* tokens, int act,
                              void* out, long ldo, int rows, int W, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || W < 1 || act < 0 || act > 2) return tis_fail("gate_table: bad size rows=%d width=%d act=%d", rows, W, act);
  const long blocks = ((long)rows * W + S32_THREADS - 1) / S32_THREADS;
  S32_DISPATCH((gate_table_kernel<float><<<blocks, S32_THREADS, 0, stream>>>(z, ldz, (const float*)table, ldt, tokens, act, (float*)out, ldo, rows, W)),
               (gate_table_kernel<bf16><<<blocks, S32_THREADS, 0, stream>>>(z, ldz, (const bf16*)table, ldt, tokens, act, (bf16*)out, ldo, rows, W)))
  return tis_launch_status("gate_table");
}

TIS_EXPORT int tis_activate32(float* z, long ldz, int act, int rows, int W, hipStream_t stream) {
  if (rows == 0 || W == 0) return 0;
  if (rows < 0 || W < 0 || act < 0 || act > 2) return tis_fail("activate32: bad size rows=%d width=%d act=%d", rows, W, act);
  const long blocks = ((long)rows * W + S32_THREADS - 1) / S32_THREADS;
  activate32_kernel<<<blocks, S32_THREADS, 0, stream>>>(z, ldz, act, rows, W);
  return tis_launch_status("activate32");
}

TIS_EXPORT int tis_head_gate(int dtype, void* x, long ldx, const float* gate, long ldg, int rows, int H, int V,
                             hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || H < 1 || V < 1) return tis_fail("head_gate: bad size rows=%d heads=%d vdim=%d", rows, H, V);
  const long blocks = ((long)rows * H * V + S32_THREADS - 1) / S32_THREADS;
  S32_DISPATCH((head_gate_kernel<float><<<blocks, S32_THREADS, 0, stream>>>((float*)x, ldx, gate, ldg, rows, H, V)),
               (head_gate_kernel<bf16><<<blocks, S32_THREADS, 0, stream>>>((bf16*)x, ldx, gate, ldg, rows, H, V)))
  return tis_launch_status("head_gate");
}

// ---- blocks whose sublayers all read one norm of the stream and are summed with a factor per channel ---------------

// Dynamic tanh: out = tanh(alpha * x) * gain + bias, element by element (no mean, no variance), in the compute type.
template <typename T>
__global__ __launch_bounds__(S32_THREADS) void dyt32_kernel(const float* __restrict__ x, float alpha,
                                                             const float* __restrict__ gain, const float* __restrict__ bias,
                                                             T* __restrict__ out, long ldo, int D, int row_blocks) {
  const long r = blockIdx.x / row_blocks;      // grid (rows * blocks of columns, a row's side by side): a few rows still fill the chip
  const int c = (blockIdx.x % row_blocks) * S32_THREADS + threadIdx.x;
  if (c < D) out[r * ldo + c] = from_f<T>(tanhf(alpha * x[r * D + c]) * gain[c] + (bias ? bias[c] : 0.f));
}

// One branch of a scaled sum: s[c] * (y[r][c] + b[c]); s and b may be null (1 and 0). With `cs.ids` the branch is the
// not yet summed result of a routed feed-forward (see ChosenSum; weights may be null: every choice counts once).
struct ScaledBranch {
  const float* y;
  long ld;
  const float* scale;
  const float* bias;
};

// x <- x + sum over the branches, in place or into out32; `normed` (nullable) gets the dynamic tanh of the new row in
// the compute type (the norm that the next block, or the model's end, reads the stream through). grid (rows * blocks of
// columns, a row's blocks side by side): every element is on its own, and a step of a few rows still spreads over the chip.
template <typename T>
__global__ __launch_bounds__(S32_THREADS) void scaled_sum_kernel(const float* __restrict__ x, ScaledBranch a, ScaledBranch b,
                                                                  ChosenSum cs, float* __restrict__ out32, int norm_kind,
                                                                  float alpha, const float* __restrict__ gain,
                                                                  const float* __restrict__ nbias, T* __restrict__ normed,
                                                                  long ldn, int D, int row_blocks) {
  const long r = blockIdx.x / row_blocks;
  __shared__ int chosen_id[64];
  __shared__ float chosen_w[64];
  const bool kept = cs.ids && cs.top <= 64;
  if (kept) {
    if (threadIdx.x < cs.top) {
      chosen_id[threadIdx.x] = cs.ids[r * cs.top + threadIdx.x];
      chosen_w[threadIdx.x] = cs.weights ? cs.weights[r * cs.top + threadIdx.x] : 1.f;
    }
    __syncthreads();
  }
  const int c = (blockIdx.x % row_blocks) * S32_THREADS + threadIdx.x;
  if (c < D) {
    float v = x[r * D + c];
    if (a.y) v += (a.scale ? a.scale[c] : 1.f) * (a.y[r * a.ld + c] + (a.bias ? a.bias[c] : 0.f));
    if (cs.ids) {
      float y = 0.f;
      for (int k = 0; k < cs.top; ++k) {
        const int e = kept ? chosen_id[k] : cs.ids[r * cs.top + k];
        const float w = kept ? chosen_w[k] : (cs.weights ? cs.weights[r * cs.top + k] : 1.f);
        y += w * (e < cs.n_experts ? b.y[(r * cs.top + k) * b.ld + c] : to_f(static_cast<const T*>(cs.rows)[r * cs.ldr + c]));
      }
      v += (b.scale ? b.scale[c] : 1.f) * (y + (b.bias ? b.bias[c] : 0.f));
    } else if (b.y) {
      v += (b.scale ? b.scale[c] : 1.f) * (b.y[r * b.ld + c] + (b.bias ? b.bias[c] : 0.f));
    }
    out32[r * D + c] = v;
    if (norm_kind == 3) normed[r * ldn + c] = from_f<T>(tanhf(alpha * v) * gain[c] + (nbias ? nbias[c] : 0.f));
  }
}

// out[r][j] = act(w_r * (z[r][j] + gb[j])) * (w_r * (z[r][F + j] + ub[j])): the gate of a gated feed-forward on a
// 32-bit product whose first F columns are the gate's and whose next F the other factor's. Biases and the factor per
// row (a router's weight on the row that an expert read) may be null. act 0: tanh-form gelu, 1: silu.
template <typename T>
__global__ __launch_bounds__(S32_THREADS) void gated_act_kernel(const float* __restrict__ z, long ldz, int F,
                                                                 const float* __restrict__ gb, const float* __restrict__ ub,
                                                                 const float* __restrict__ row_scale, int act,
                                                                 T* __restrict__ out, long ldo, int rows, float limit) {
  const long i = (long)blockIdx.x * S32_THREADS + threadIdx.x;
  if (i >= (long)rows * F) return;
  const long r = i / F;
  const int j = (int)(i % F);
  const float w = row_scale ? row_scale[r] : 1.f;
  float g = w * (z[r * ldz + j] + (gb ? gb[j] : 0.f)), u = w * (z[r * ldz + F + j] + (ub ? ub[j] : 0.f));
  if (act == 2) {      // g sigmoid(1.702 g) (u + 1) with g capped from above and u from both sides at `limit`
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    out[r * ldo + j] = from_f<T>(g * sigmoid_f(1.702f * g) * (u + 1.f));
    return;
  }
  out[r * ldo + j] = from_f<T>((act == 0 ? gelu_tanh_f(g) : g * sigmoid_f(g)) * u);
}

// z <- cap * tanh(z / cap) on 32-bit rows, in place
__global__ __launch_bounds__(S32_THREADS) void softcap_kernel(float* __restrict__ z, long ldz, float cap, int rows, int W) {
  const long i = (long)blockIdx.x * S32_THREADS + threadIdx.x;
  if (i >= (long)rows * W) return;
  float* p = z + (i / W) * ldz + (i % W);
  *p = cap * tanhf(*p / cap);
}

TIS_EXPORT int tis_dyt32(int dtype, const float* x, float alpha, const float* gain, const float* bias, void* out, long ldo,
                         int rows, int D, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || D < 1 || !x || !gain || !out) return tis_fail("dyt32: bad arguments rows=%d width=%d", rows, D);
  const int row_blocks = (D + S32_THREADS - 1) / S32_THREADS;
  if ((long)rows * row_blocks > 0x7fffffffL) return tis_fail("dyt32: %d rows of %d in one call", rows, D);
  S32_DISPATCH((dyt32_kernel<float><<<rows * row_blocks, S32_THREADS, 0, stream>>>(x, alpha, gain, bias, (float*)out, ldo, D, row_blocks)),
               (dyt32_kernel<bf16><<<rows * row_blocks, S32_THREADS, 0, stream>>>(x, alpha, gain, bias, (bf16*)out, ldo, D, row_blocks)))
  return tis_launch_status("dyt32");
}

TIS_EXPORT int tis_scaled_sum(int dtype, const float* x, const float* y0, long ld0, const float* s0, const float* b0,
                              const float* y1, long ld1, const float* s1, const float* b1, const int* ids,
                              const float* weights, int top, int n_experts, const void* chosen_rows, long ldr,
                              float* out32, int norm_kind, float alpha, const float* gain, const float* nbias, void* normed,
                              long ldn, int rows, int D, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || D < 1 || !x || !out32) return tis_fail("scaled_sum: bad arguments rows=%d width=%d", rows, D);
  if (ids && (top < 1 || n_experts < 0 || (n_experts > 0 && !y1) || !chosen_rows))
    return tis_fail("scaled_sum: a sum over chosen experts needs ids, the experts' results and the rows they read");
  if ((norm_kind != 0 && norm_kind != 3) || (norm_kind && (!gain || !normed)))
    return tis_fail("scaled_sum: norm kind %d (0: none, 3: dynamic tanh, with a gain and an output)", norm_kind);
  const ScaledBranch a{y0, ld0, s0, b0}, b{y1, ld1, s1, b1};
  const ChosenSum cs{ids, weights, top, n_experts, chosen_rows, ldr};
  const int row_blocks = (D + S32_THREADS - 1) / S32_THREADS;
  if ((long)rows * row_blocks > 0x7fffffffL) return tis_fail("scaled_sum: %d rows of %d in one call", rows, D);
  const int grid = rows * row_blocks;
  S32_DISPATCH((scaled_sum_kernel<float><<<grid, S32_THREADS, 0, stream>>>(x, a, b, cs, out32, norm_kind, alpha, gain, nbias, (float*)normed, ldn, D, row_blocks)),
               (scaled_sum_kernel<bf16><<<grid, S32_THREADS, 0, stream>>>(x, a, b, cs, out32, norm_kind, alpha, gain, nbias, (bf16*)normed, ldn, D, row_blocks)))
  return tis_launch_status("scaled_sum");
}

TIS_EXPORT int tis_gated_act(int dtype, const float* z, long ldz, int F, const float* gate_bias, const float* up_bias,
                             const float* row_scale, int act, void* out, long ldo, int rows, float limit, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || F < 1 || act < 0 || act > 2 || (act == 2 && !(limit > 0.f)))
    return tis_fail("gated_act: bad size rows=%d hidden=%d act=%d limit=%g", rows, F, act, (double)limit);
  const long blocks = ((long)rows * F + S32_THREADS - 1) / S32_THREADS;
  S32_DISPATCH((gated_act_kernel<float><<<blocks, S32_THREADS, 0, stream>>>(z, ldz, F, gate_bias, up_bias, row_scale, act, (float*)out, ldo, rows, limit)),
               (gated_act_kernel<bf16><<<blocks, S32_THREADS, 0, stream>>>(z, ldz, F, gate_bias, up_bias, row_scale, act, (bf16*)out, ldo, rows, limit)))
  return tis_launch_status("gated_act");
}

TIS_EXPORT int tis_softcap(float* z, long ldz, float cap, int rows, int W, hipStream_t stream) {
  if (rows == 0 || W == 0) return 0;
  if (rows < 0 || W < 0 || !(cap > 0.f)) return tis_fail("softcap: bad arguments rows=%d width=%d cap=%g", rows, W, (double)cap);
  const long blocks = ((long)rows * W + S32_THREADS - 1) / S32_THREADS;
  softcap_kernel<<<blocks, S32_THREADS, 0, stream>>>(z, ldz, cap, rows, W);
  return tis_launch_status("softcap");
}

// ---- blocks with a norm on both sides of a sublayer, several mixers side by side -----------------------------------

// out[r][c] = act(z) with z = sum_k low[r][k] * w2[c][k] + bias[c] (bias may be null): the second half of a low-rank
// projection, in 32-bit. kind 0: sigmoid(z)^(1/tau); 1: exp(-rate[c / group] * softplus(z)), a decay whose rate is one
// number per run of `group` channels; 2: z itself.
static constexpr int LR_ROWS = 8;      // rows a workgroup of lowrank_act takes: a channel's line of w2 is read once for them

__global__ __launch_bounds__(S32_THREADS) void lowrank_act_kernel(const float* __restrict__ low, long ldl, int rank,
                                                                   const float* __restrict__ w2,
                                                                   const float* __restrict__ bias, int kind, float tau,
                                                                   const float* __restrict__ rate, int group,
                                                                   float* __restrict__ out, int rows, int C, int col_blocks) {
  extern __shared__ float a[];                   // [LR_ROWS][rank]
  // grid (blocks of rows * blocks of channels, a row block's side by side): a few rows still fill the chip
  const long r0 = (long)(blockIdx.x / col_blocks) * LR_ROWS;
  const int n = (int)min((long)LR_ROWS, rows - r0);
  for (int i = threadIdx.x; i < n * rank; i += S32_THREADS) a[i] = low[(r0 + i / rank) * ldl + i % rank];
  __syncthreads();
  const int c = (blockIdx.x % col_blocks) * S32_THREADS + threadIdx.x;
  if (c >= C) return;
  float z[LR_ROWS];
#pragma unroll
  for (int r = 0; r < LR_ROWS; ++r) z[r] = 0.f;
  const float* w = w2 + (long)c * rank;
  for (int k = 0; k < rank; ++k) {
    const float wk = w[k];
#pragma unroll
    for (int r = 0; r < LR_ROWS; ++r) z[r] += a[(r < n ? r : 0) * rank + k] * wk;      // (k in rising order for every row)
  }
  const float b = bias ? bias[c] : 0.f;
  const float rt = kind == 1 ? rate[c / group] : 0.f;
#pragma unroll
  for (int r = 0; r < LR_ROWS; ++r) {
    if (r >= n) break;
    float v = z[r] + b;
    if (kind == 0) v = expf(log_sigmoid_f(v) / tau);
    else if (kind == 1) v = expf(-rt * (v > 20.f ? v : log1pf(expf(v))));
    out[(r0 + r) * C + c] = v;
  }
}

// out[r] = (1 / n) * sum_i y_i[r] / sqrt(mean(y_i[r]^2) + eps) * gain_i: the mean of one or two RMS-normed rows, 32-bit.
// One workgroup a row; the sums' order depends on the width alone.
__global__ __launch_bounds__(S32_THREADS) void normed_mean_kernel(const float* __restrict__ y0, long ld0,
                                                                   const float* __restrict__ g0,
                                                                   const float* __restrict__ y1, long ld1,
                                                                   const float* __restrict__ g1, float eps,
                                                                   float* __restrict__ out, int D) {
  __shared__ float red[16];
  const long r = blockIdx.x;
  float s0 = 0.f, s1 = 0.f;
  for (int c = threadIdx.x; c < D; c += S32_THREADS) {
    const float a = y0[r * ld0 + c];
    s0 += a * a;
    if (y1) {
      const float b = y1[r * ld1 + c];
      s1 += b * b;
    }
  }
  const float i0 = 1.f / sqrtf(block_sum(s0, red) / (float)D + eps);
  const float i1 = y1 ? 1.f / sqrtf(block_sum(s1, red) / (float)D + eps) : 0.f;
  const float share = y1 ? 0.5f : 1.f;
  for (int c = threadIdx.x; c < D; c += S32_THREADS) {
    float v = y0[r * ld0 + c] * i0 * g0[c];
    if (y1) v += y1[r * ld1 + c] * i1 * g1[c];
    out[r * D + c] = v * share;
  }
}

// out = act(z) in the compute type, z 32-bit (a strided view is fine). act 0: tanh-form gelu, 1: silu, 2: sigmoid,
// 3: the square of relu.
template <typename T>
__global__ __launch_bounds__(S32_THREADS) void activate_rows_kernel(const float* __restrict__ z, long ldz, int act,
                                                                     T* __restrict__ out, long ldo, int rows, int W) {
  const long i = (long)blockIdx.x * S32_THREADS + threadIdx.x;
  if (i >= (long)rows * W) return;
  const long r = i / W;
  const int j = (int)(i % W);
  const float v = z[r * ldz + j];
  const float p = fmaxf(v, 0.f);
  out[r * ldo + j] = from_f<T>(act == 0 ? gelu_tanh_f(v) : act == 1 ? v * sigmoid_f(v) : act == 2 ? sigmoid_f(v) : p * p);
}

TIS_EXPORT int tis_lowrank_act(const float* low, long ldl, int rank, const float* w2, const float* bias, int kind, float tau,
                               const float* rate, int group, float* out, int rows, int C, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || rank < 1 || rank > 8192 || C < 1 || kind < 0 || kind > 2 || (kind == 0 && !(tau > 0.f)) ||
      (kind == 1 && (!rate || group < 1)))
    return tis_fail("lowrank_act: bad arguments rows=%d rank=%d channels=%d kind=%d", rows, rank, C, kind);
  const int col_blocks = (C + S32_THREADS - 1) / S32_THREADS;
  const long row_blocks = ((long)rows + LR_ROWS - 1) / LR_ROWS;
  if (rank > 1024) return tis_fail("lowrank_act: rank %d (at most 1024)", rank);
  lowrank_act_kernel<<<row_blocks * col_blocks, S32_THREADS, LR_ROWS * rank * sizeof(float), stream>>>(
      low, ldl, rank, w2, bias, kind, tau, rate, group, out, rows, C, col_blocks);
  return tis_launch_status("lowrank_act");
}

TIS_EXPORT int tis_normed_mean(const float* y0, long ld0, const float* g0, const float* y1, long ld1, const float* g1, float eps,
                               float* out, int rows, int D, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || D < 1 || !y0 || !g0 || (y1 && !g1) || !out) return tis_fail("normed_mean: bad arguments rows=%d width=%d", rows, D);
  normed_mean_kernel<<<rows, S32_THREADS, 0, stream>>>(y0, ld0, g0, y1, ld1, g1, eps, out, D);
  return tis_launch_status("normed_mean");
}

TIS_EXPORT int tis_activate_rows(int dtype, const float* z, long ldz, int act, void* out, long ldo, int rows, int W,
                                 hipStream_t stream) {
  if (rows == 0 || W == 0) return 0;
  if (rows < 0 || W < 0 || act < 0 || act > 3) return tis_fail("activate_rows: bad size rows=%d width=%d act=%d", rows, W, act);
  const long blocks = ((long)rows * W + S32_THREADS - 1) / S32_THREADS;
  S32_DISPATCH((activate_rows_kernel<float><<<blocks, S32_THREADS, 0, stream>>>(z, ldz, act, (float*)out, ldo, rows, W)),
               (activate_rows_kernel<bf16><<<blocks, S32_THREADS, 0, stream>>>(z, ldz, act, (bf16*)out, ldo, rows, W)))
  return tis_launch_status("activate_rows");
}
