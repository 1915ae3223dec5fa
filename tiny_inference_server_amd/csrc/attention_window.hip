// Softmax attention whose keys and values differ in size, over a paged cache, with a sliding window: the step before
// it (biases, per-head RMS norm of queries and keys, rotation of the first channels in interleaved pairs, a factor per
// query head and one that grows with the position, unit-RMS values, the write into the pages: each optional), the same
// step for keys and values that are one shared latent, and the attention itself, with an optional sink in the softmax
// and an optional gate per head on the result.
//
// A page of `page_size` slots holds, for each key/value head, the keys as [slot][key size] and then, after the keys
// of all heads, the values transposed as [value size][slot]. With equal sizes that is the layout the other attention
// kernels read. The row at position p sees
// the keys at [max(0, p - window + 1), p] (window 0: all), and with chunk_size c > 0 only those from p - p % c on (the
// row's own chunk of positions, chunk edges at multiples of the size in the request), found through the request's block table; keys outside are
// never read, so what a reused page holds cannot reach a result.
// Norms, angles, scores, the softmax and the weighted sum are 32-bit; `T` is the type of queries and pages.
#include "common.h"

TIS_DEFINE_LAST_ERROR(tis_attention_window)

static constexpr int AW_THREADS = 256;
static constexpr int AW_CHUNK = 1024;
static constexpr int AW_MAX_DIM = 1024;
static constexpr int AW_PER = AW_MAX_DIM / AW_THREADS;   // value channels a thread may own

// What the step before attention may do beyond copying: every pointer may be null and every count zero.
struct PrepareArgs {
  const float* q_bias;     // [H * KD], added to the projections
  const float* k_bias;     // [G * KD]
  const float* v_bias;     // [G * VD]
  const float* q_gain;     // [KD]: RMS norm of every query head with this gain (null: no norm)
  const float* k_gain;     // [KD]
  const float* q_factor;   // [H]: a factor per query head
  const float* freqs;      // [rot_dims / 2]: angle = position * freqs[pair], pairs (2i, 2i+1) of the first rot_dims channels
  int rot_dims;
  float eps;
  int value_norm;          // values are divided by their root mean square
  float temp_coef;         // queries times 1 + temp_coef * ln(floor((position + 1) / temp_every) + 1); 0: none
  int temp_every;
  int whole_norm;          // the norms run over all heads of a row's queries (keys) at once, with gains of [H * KD] ([G * KD])
  int pair_half;           // rotated pairs are (i, i + rot_dims / 2) instead of (2i, 2i + 1)
};

// The norms may also run over all heads of a row at once (whole_norm), and the rotated pairs may be (i, i + rot_dims/2)
// (pair_half).
// One wave's work for unit u of row r: u < H is a query head, u < H + G a key head, else a value head. proj holds the
// projections of a row in 32-bit: queries at q_off, keys at k_off, values at v_off. whole_q, whole_k: with whole_norm,
// one over the root mean square of all of the row's queries (keys).
template <typename T>
__device__ __forceinline__ void prepare_unit(
    const float* __restrict__ proj, long ldp, int q_off, int k_off, int v_off, const int* __restrict__ positions,
    const int* __restrict__ write_slots, T* __restrict__ plane, T* __restrict__ q_out, long ldq, const PrepareArgs& a, int H,
    int G, int KD, int VD, int page_size, long r, int u, int lane, float whole_q, float whole_k) {
  const long page_stride = (long)G * page_size * (KD + VD);
  if (u < H + G) {
    const bool is_q = u < H;
    const int h = is_q ? u : u - H;
    if (!is_q && !write_slots) return;
    const float* src = proj + r * ldp + (is_q ? q_off : k_off) + (long)h * KD;
    const float* bias = is_q ? a.q_bias : a.k_bias;
    if (bias) bias += (long)h * KD;
    const float* gain = is_q ? a.q_gain : a.k_gain;
    float inv = 1.f;
    if (gain && a.whole_norm) {
      inv = is_q ? whole_q : whole_k;
      gain += (long)h * KD;
    } else if (gain) {
      float ss = 0.f;
      for (int e = lane; e < KD; e += TIS_WAVE) {
        const float v = src[e] + (bias ? bias[e] : 0.f);
        ss += v * v;
      }
      ss = wave_sum(ss);
      inv = 1.f / sqrtf(ss / (float)KD + a.eps);
    }
    float factor = is_q && a.q_factor ? a.q_factor[h] : 1.f;
    const int ipos = positions[r];
    if (is_q && a.temp_coef != 0.f) factor *= 1.f + a.temp_coef * logf((float)((ipos + 1) / a.temp_every) + 1.f);
    const float pos = (float)ipos;
    T* dst;
    if (is_q) {
      dst = q_out + r * ldq + (long)h * KD;
    } else {
      const int ws = write_slots[r];
      dst = plane + (long)(ws / page_size) * page_stride + ((long)h * page_size + ws % page_size) * KD;
    }
    if (a.pair_half) {
      const int half = a.rot_dims / 2;
      for (int p = lane; p < half; p += TIS_WAVE) {
        const int e0 = p, e1 = p + half;
        const float x = (src[e0] + (bias ? bias[e0] : 0.f)) * inv * (gain ? gain[e0] : 1.f);
        const float y = (src[e1] + (bias ? bias[e1] : 0.f)) * inv * (gain ? gain[e1] : 1.f);
        float sn, cs;
        sincosf(pos * a.freqs[p], &sn, &cs);
        dst[e0] = from_f<T>((x * cs - y * sn) * factor);
        dst[e1] = from_f<T>((y * cs + x * sn) * factor);
      }
      for (int e = a.rot_dims + lane; e < KD; e += TIS_WAVE)
        dst[e] = from_f<T>((src[e] + (bias ? bias[e] : 0.f)) * inv * (gain ? gain[e] : 1.f) * factor);
    } else
    for (int p = lane; 2 * p < KD; p += TIS_WAVE) {
      const int e0 = 2 * p, e1 = e0 + 1;
      float x = (src[e0] + (bias ? bias[e0] : 0.f)) * inv * (gain ? gain[e0] : 1.f);
      float y = e1 < KD ? (src[e1] + (bias ? bias[e1] : 0.f)) * inv * (gain ? gain[e1] : 1.f) : 0.f;
      if (e1 < a.rot_dims) {
        float sn, cs;
        sincosf(pos * a.freqs[p], &sn, &cs);
        const float rx = x * cs - y * sn, ry = y * cs + x * sn;
        x = rx;
        y = ry;
      }
      dst[e0] = from_f<T>(x * factor);
      if (e1 < KD) dst[e1] = from_f<T>(y * factor);
    }
  } else {
    if (!write_slots) return;
    const int h = u - H - G;
    const float* src = proj + r * ldp + v_off + (long)h * VD;
    const float* bias = a.v_bias ? a.v_bias + (long)h * VD : nullptr;
    float inv = 1.f;
    if (a.value_norm) {
      float ss = 0.f;
      for (int e = lane; e < VD; e += TIS_WAVE) {
        const float v = src[e] + (bias ? bias[e] : 0.f);
        ss += v * v;
      }
      ss = wave_sum(ss);
      inv = 1.f / sqrtf(ss / (float)VD + a.eps);
    }
    const int ws = write_slots[r];
    T* dst = plane + (long)(ws / page_size) * page_stride + (long)G * page_size * KD + (long)h * VD * page_size +
             ws % page_size;
    for (int e = lane; e < VD; e += TIS_WAVE) dst[(long)e * page_size] = from_f<T>((src[e] + (bias ? bias[e] : 0.f)) * inv);
  }
}

// grid (rows, H + 2 G), one wave each (norms per head or none).
template <typename T>
__global__ __launch_bounds__(TIS_WAVE) void attention_prepare_kernel(
    const float* __restrict__ proj, long ldp, int q_off, int k_off, int v_off, const int* __restrict__ positions,
    const int* __restrict__ write_slots, T* __restrict__ plane, T* __restrict__ q_out, long ldq, PrepareArgs a, int H, int G,
    int KD, int VD, int page_size) {
  prepare_unit<T>(proj, ldp, q_off, k_off, v_off, positions, write_slots, plane, q_out, ldq, a, H, G, KD, VD, page_size,
                  blockIdx.x, blockIdx.y, threadIdx.x, 1.f, 1.f);
}

// Norms over all heads of a row at once: grid (rows), 4 to 16 waves a row. The workgroup first sums the squares of
// the row's queries and of its keys (every element read once; the order of additions depends on the sizes alone), then
// its waves take the row's units in turn.
template <typename T>
__global__ __launch_bounds__(1024) void attention_prepare_row_kernel(
    const float* __restrict__ proj, long ldp, int q_off, int k_off, int v_off, const int* __restrict__ positions,
    const int* __restrict__ write_slots, T* __restrict__ plane, T* __restrict__ q_out, long ldq, PrepareArgs a, int H, int G,
    int KD, int VD, int page_size) {
  __shared__ float red[16];
  const long r = blockIdx.x;
  const int t = threadIdx.x, waves = blockDim.x / TIS_WAVE;
  // The first 256 threads sum, whatever the workgroup's size: a row's result is the same bit for bit in a step of few
  // rows (16 waves a row) and in one of many (4 waves a row).
  auto inverse_rms = [&](int off, int n, const float* bias) {
    const float* all = proj + r * ldp + off;
    float part[4] = {0.f, 0.f, 0.f, 0.f};        // four sums side by side, so that a thread's loads are in flight together
    if (t < 256)
      for (int e0 = t; e0 < n; e0 += 4 * 256) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int e = e0 + i * 256;
          const float v = e < n ? all[e] + (bias ? bias[e] : 0.f) : 0.f;
          part[i] += v * v;
        }
      }
    return 1.f / sqrtf(block_sum((part[0] + part[1]) + (part[2] + part[3]), red) / (float)n + a.eps);
  };
  const float whole_q = a.q_gain ? inverse_rms(q_off, H * KD, a.q_bias) : 1.f;
  const float whole_k = a.k_gain && write_slots ? inverse_rms(k_off, G * KD, a.k_bias) : 1.f;
  for (int u = t / TIS_WAVE; u < H + 2 * G; u += waves)
    prepare_unit<T>(proj, ldp, q_off, k_off, v_off, positions, write_slots, plane, q_out, ldq, a, H, G, KD, VD, page_size, r,
                    u, t % TIS_WAVE, whole_q, whole_k);
}

// The same step where all heads share one latent as keys and values. grid (rows, H + 1), one wave each.
// (A latent's pages are those of one key/value head with keys of C + R and values of C channels: the latent is kept
// twice, as the first channels of its key and transposed as its value.) Unit u < H, a query head: the head's R rotated channels (32-bit, at q_off + u * (D + R) + D of proj) are turned by
// the row's position and written to q_out[u * (C + R) + C ...]; its D unrotated channels go, in the compute type, to
// q_plain[u * D ...] (for the product that takes them into the latent's space, whose result belongs to
// q_out[u * (C + R) ...]). Unit H: the row's latent, C channels at c_off, RMS-normed with `gain`, then the R channels
// of the shared rotated key, turned alike; both go into the row's slot of the page's keys, and the latent also into
// its values.
template <typename T>
__global__ __launch_bounds__(TIS_WAVE) void latent_prepare_kernel(
    const float* __restrict__ proj, long ldp, int q_off, int c_off, const int* __restrict__ positions,
    const int* __restrict__ write_slots, T* __restrict__ plane, T* __restrict__ q_out, long ldq, T* __restrict__ q_plain,
    long ldqp, const float* __restrict__ gain, const float* __restrict__ freqs, int rot_dims, float eps, int H, int D,
    int R, int C, int page_size) {
  const long r = blockIdx.x;
  const int u = blockIdx.y, lane = threadIdx.x;
  const float pos = (float)positions[r];
  const float* src;
  T* dst;
  if (u < H) {
    src = proj + r * ldp + q_off + (long)u * (D + R);
    for (int e = lane; e < D; e += TIS_WAVE) q_plain[r * ldqp + (long)u * D + e] = from_f<T>(src[e]);
    src += D;
    dst = q_out + r * ldq + (long)u * (C + R) + C;
  } else {
    if (!write_slots) return;
    const int ws = write_slots[r];
    T* page = plane + (long)(ws / page_size) * page_size * (2 * C + R);
    T* key = page + (long)(ws % page_size) * (C + R);
    T* val = page + (long)page_size * (C + R) + ws % page_size;
    src = proj + r * ldp + c_off;
    float ss = 0.f;
    for (int e = lane; e < C; e += TIS_WAVE) ss += src[e] * src[e];
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / (float)C + eps);
    for (int e = lane; e < C; e += TIS_WAVE) {
      const T v = from_f<T>(src[e] * inv * gain[e]);
      key[e] = v;
      val[(long)e * page_size] = v;
    }
    src += C;
    dst = key + C;
  }
  for (int p = lane; 2 * p < R; p += TIS_WAVE) {
    const int e0 = 2 * p, e1 = e0 + 1;
    float x = src[e0], y = e1 < R ? src[e1] : 0.f;
    if (e1 < rot_dims) {
      float sn, cs;
      sincosf(pos * freqs[p], &sn, &cs);
      const float rx = x * cs - y * sn, ry = y * cs + x * sn;
      x = rx;
      y = ry;
    }
    dst[e0] = from_f<T>(x);
    if (e1 < R) dst[e1] = from_f<T>(y);
  }
}

// One workgroup per (row, query head). Keys are walked in chunks of AW_CHUNK with a running maximum; the order of
// every sum depends on the row's own position and window only. sink: the softmax's denominator also holds a key of
// score 0 that has no value. gate (nullable): the head's result is multiplied by sigmoid(gate[row * ldg + head]).
template <typename T>
__global__ __launch_bounds__(AW_THREADS) void attention_window_kernel(
    const T* __restrict__ q, long ldq, const T* __restrict__ plane, const int* __restrict__ block_tables, int bt_ld,
    const int* __restrict__ row_seq, const int* __restrict__ positions, T* __restrict__ out, long ldo, int group_size,
    int G, int KD, int VD, int page_size, int window, int chunk_size, float scale, int sink,
    const float* __restrict__ gate, long ldg) {
  __shared__ float qs[AW_MAX_DIM];
  __shared__ float sc[AW_CHUNK];
  __shared__ float red[16];
  __shared__ float accm[AW_PER][AW_THREADS];
  const long r = blockIdx.x;
  const int h = blockIdx.y, g = h / group_size, t = threadIdx.x;
  const int pos = positions[r];
  const int* bt = block_tables + (long)row_seq[r] * bt_ld;
  int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  if (chunk_size > 0) first = max(first, pos - pos % chunk_size);     // only keys of the row's own chunk of positions
  const int end = pos + 1;
  for (int d = t; d < KD; d += AW_THREADS) qs[d] = to_f(q[r * ldq + (long)h * KD + d]) * scale;
  __syncthreads();
  const long page_stride = (long)G * page_size * (KD + VD);
  const long k_off = (long)g * page_size * KD;
  const long v_off = (long)G * page_size * KD + (long)g * VD * page_size;
  // a thread owns `per` value channels, width apart; the threads that share a channel take every n-th key
  const int per = (VD + AW_THREADS - 1) / AW_THREADS;
  const int width = (VD + per - 1) / per;
  const int lanes_per_key = AW_THREADS / width;
  const int part = t / width, d = t % width;
  const bool pv = part < lanes_per_key;
  float m = sink ? 0.f : -INFINITY, l = sink ? 1.f : 0.f;
  float acc[AW_PER];
#pragma unroll
  for (int u = 0; u < AW_PER; ++u) acc[u] = 0.f;
  for (int c0 = first; c0 < end; c0 += AW_CHUNK) {
    const int n = min(AW_CHUNK, end - c0);
    float cmax = -INFINITY;
    for (int i = t; i < n; i += AW_THREADS) {
      const int j = c0 + i;
      const T* kp = plane + (long)bt[j / page_size] * page_stride + k_off + (long)(j % page_size) * KD;
      float s = 0.f;
      for (int e = 0; e < KD; ++e) s += qs[e] * to_f(kp[e]);
      sc[i] = s;
      cmax = fmaxf(cmax, s);
    }
    cmax = block_max(cmax, red);
    const float m_new = fmaxf(m, cmax);
    float csum = 0.f;
    for (int i = t; i < n; i += AW_THREADS) {
      const float p = expf(sc[i] - m_new);
      sc[i] = p;
      csum += p;
    }
    csum = block_sum(csum, red);      // its barriers also publish sc[]
    const float rescale = expf(m - m_new);
    l = l * rescale + csum;
#pragma unroll
    for (int u = 0; u < AW_PER; ++u) acc[u] *= rescale;
    m = m_new;
    if (pv) {
      for (int i = part; i < n; i += lanes_per_key) {
        const int j = c0 + i;
        const T* vp = plane + (long)bt[j / page_size] * page_stride + v_off + (j % page_size);
        const float p = sc[i];
#pragma unroll
        for (int u = 0; u < AW_PER; ++u)
          if (u < per && d + u * width < VD) acc[u] += p * to_f(vp[(long)(d + u * width) * page_size]);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int u = 0; u < AW_PER; ++u) accm[u][t] = pv ? acc[u] : 0.f;
  __syncthreads();
  const float mul = (gate ? 1.f / (1.f + expf(-gate[r * ldg + h])) : 1.f) / l;
  for (int c = t; c < VD; c += AW_THREADS) {
    const int u = c / width, dd = c % width;
    float o = 0.f;
    for (int p = 0; p < lanes_per_key; ++p) o += accm[u][p * width + dd];
    out[r * ldo + (long)h * VD + c] = from_f<T>(o * mul);
  }
}

TIS_EXPORT int tis_attention_prepare(int dtype, const float* proj, long ldp, int q_off, int k_off, int v_off,
                                     const int* positions, const int* write_slots, void* plane, void* q_out, long ldq,
                                     const float* q_bias, const float* k_bias, const float* v_bias, const float* q_gain,
                                     const float* k_gain, const float* q_factor, const float* freqs, int rot_dims, float eps,
                                     int value_norm, float temp_coef, int temp_every, int whole_norm, int pair_half, int rows,
                                     int H, int G, int KD, int VD, int page_size, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || H < 1 || G < 1 || KD < 1 || VD < 1 || page_size < 1 || H + 2 * G > 65535)
    return tis_fail("attention_prepare: bad size rows=%d heads=%d kv_heads=%d key=%d value=%d page=%d", rows, H, G, KD, VD,
                    page_size);
  if (rot_dims < 0 || rot_dims > KD || rot_dims % 2 || (rot_dims && !freqs))
    return tis_fail("attention_prepare: %d rotated channels of %d", rot_dims, KD);
  if (temp_coef != 0.f && temp_every < 1) return tis_fail("attention_prepare: a query factor every %d positions", temp_every);
  if (write_slots && !plane) return tis_fail("attention_prepare: write slots without pages");
  PrepareArgs a{q_bias, k_bias, v_bias, q_gain, k_gain, q_factor, freqs, rot_dims, eps, value_norm, temp_coef, temp_every,
                whole_norm, pair_half};
  if (whole_norm && (q_gain || k_gain)) {
    const int units = H + 2 * G;
    const int threads = rows >= 256 ? 256 : TIS_WAVE * (units < 4 ? 4 : units < 16 ? units : 16);
    if (dtype == TIS_F32)
      attention_prepare_row_kernel<float><<<rows, threads, 0, stream>>>(proj, ldp, q_off, k_off, v_off, positions, write_slots,
          (float*)plane, (float*)q_out, ldq, a, H, G, KD, VD, page_size);
    else if (dtype == TIS_BF16)
      attention_prepare_row_kernel<bf16><<<rows, threads, 0, stream>>>(proj, ldp, q_off, k_off, v_off, positions, write_slots,
          (bf16*)plane, (bf16*)q_out, ldq, a, H, G, KD, VD, page_size);
    else
      return tis_fail("unknown dtype code %d", dtype);
    return tis_launch_status("attention_prepare");
  }
  dim3 grid(rows, H + 2 * G);
  if (dtype == TIS_F32)
    attention_prepare_kernel<float><<<grid, TIS_WAVE, 0, stream>>>(proj, ldp, q_off, k_off, v_off, positions, write_slots,
        (float*)plane, (float*)q_out, ldq, a, H, G, KD, VD, page_size);
  else if (dtype == TIS_BF16)
    attention_prepare_kernel<bf16><<<grid, TIS_WAVE, 0, stream>>>(proj, ldp, q_off, k_off, v_off, positions, write_slots,
        (bf16*)plane, (bf16*)q_out, ldq, a, H, G, KD, VD, page_size);
  else
    return tis_fail("unknown dtype code %d", dtype);
  return tis_launch_status("attention_prepare");
}

TIS_EXPORT int tis_latent_prepare(int dtype, const float* proj, long ldp, int q_off, int c_off, const int* positions,
                                  const int* write_slots, void* plane, void* q_out, long ldq, void* q_plain, long ldqp,
                                  const float* gain, const float* freqs, int rot_dims, float eps, int rows, int H, int D,
                                  int R, int C, int page_size, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || H < 1 || H > 65534 || D < 0 || R < 0 || C < 1 || page_size < 1 || !gain || !q_out || (D && !q_plain))
    return tis_fail("latent_prepare: bad size rows=%d heads=%d dim=%d rotated=%d latent=%d page=%d", rows, H, D, R, C, page_size);
  if (rot_dims < 0 || rot_dims > R || rot_dims % 2 || (rot_dims && !freqs))
    return tis_fail("latent_prepare: %d rotated channels of %d", rot_dims, R);
  if (write_slots && !plane) return tis_fail("latent_prepare: write slots without pages");
  dim3 grid(rows, H + 1);
  if (dtype == TIS_F32)
    latent_prepare_kernel<float><<<grid, TIS_WAVE, 0, stream>>>(proj, ldp, q_off, c_off, positions, write_slots, (float*)plane,
        (float*)q_out, ldq, (float*)q_plain, ldqp, gain, freqs, rot_dims, eps, H, D, R, C, page_size);
  else if (dtype == TIS_BF16)
    latent_prepare_kernel<bf16><<<grid, TIS_WAVE, 0, stream>>>(proj, ldp, q_off, c_off, positions, write_slots, (bf16*)plane,
        (bf16*)q_out, ldq, (bf16*)q_plain, ldqp, gain, freqs, rot_dims, eps, H, D, R, C, page_size);
  else
    return tis_fail("unknown dtype code %d", dtype);
  return tis_launch_status("latent_prepare");
}

TIS_EXPORT int tis_attention_window(int dtype, const void* q, long ldq, const void* plane, const int* block_tables,
                                    int bt_ld, const int* row_seq, const int* positions, void* out, long ldo, int rows,
                                    int H, int G, int KD, int VD, int page_size, int window, int chunk_size, float scale,
                                    int sink, const float* gate, long ldg, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || H < 1 || G < 1 || H % G || page_size < 1 || window < 0 || chunk_size < 0 || H > 65535)
    return tis_fail("attention_window: bad size rows=%d heads=%d kv_heads=%d page=%d window=%d", rows, H, G, page_size, window);
  if (KD < 1 || KD > AW_MAX_DIM || VD < 1 || VD > AW_MAX_DIM)
    return tis_fail("attention_window: key size %d or value size %d is outside 1..%d", KD, VD, AW_MAX_DIM);
  dim3 grid(rows, H);
  if (dtype == TIS_F32)
    attention_window_kernel<float><<<grid, AW_THREADS, 0, stream>>>((const float*)q, ldq, (const float*)plane, block_tables,
        bt_ld, row_seq, positions, (float*)out, ldo, H / G, G, KD, VD, page_size, window, chunk_size, scale, sink, gate, ldg);
  else if (dtype == TIS_BF16)
    attention_window_kernel<bf16><<<grid, AW_THREADS, 0, stream>>>((const bf16*)q, ldq, (const bf16*)plane, block_tables,
        bt_ld, row_seq, positions, (bf16*)out, ldo, H / G, G, KD, VD, page_size, window, chunk_size, scale, sink, gate, ldg);
  else
    return tis_fail("unknown dtype code %d", dtype);
  return tis_launch_status("attention_window");
}

// ---- attention whose weights are sigmoids mixed across the heads ----------------------------------------------------
//
// For the row at position p and every key j it sees (j <= p, and with chunk_size c > 0 only j >= p - p % c):
//   s_g = q_g . k_kv(g) * scale;  s_g <- cap * tanh(s_g / cap) (cap 0: as it is);  w_g = sigmoid(s_g + head_bias[g]);
//   m_h = sum_g talk[h][g] * w_g;  out_h = sum_j m_h(j) * v_kv(h)(j).
// Nothing is normalised over the keys, so a row's result is a plain sum over its keys and may be cut anywhere: with
// n_splits > 1 workgroup (row, s) takes the key blocks s, s + n_splits, ... and leaves its part in `partial`
// [rows][n_splits][H * VD] (32-bit), which attention_mixed_merge_kernel adds up in the order of the splits.
//
// One workgroup per (row, split). A block of `block` keys at a time: every (head, key) score by one thread into LDS, the
// mixture of the heads' weights into LDS, then a thread per (head, value channel) adds the block's weighted values.
// LDS (floats): q of all heads [H * KD] | talk [H * H] | weights [H * block] | mixed [H * block].
static constexpr int AM_PER = 16;      // (head, value channel) outputs a thread may own: H * VD <= 16 * 256

template <typename T>
__global__ __launch_bounds__(AW_THREADS) void attention_mixed_kernel(
    const T* __restrict__ q, long ldq, const T* __restrict__ plane, const int* __restrict__ block_tables, int bt_ld,
    const int* __restrict__ row_seq, const int* __restrict__ positions, T* __restrict__ out, long ldo,
    float* __restrict__ partial, int n_splits, int H, int G, int KD, int VD, int page_size, int chunk_size, float scale,
    float softcap, const float* __restrict__ head_bias, const float* __restrict__ talk, int block) {
  extern __shared__ float am_lds[];
  float* qs = am_lds;
  float* tk = qs + H * KD;
  float* wr = tk + H * H;
  float* wm = wr + H * block;
  const long r = blockIdx.x;
  const int split = blockIdx.y, t = threadIdx.x;
  const int group_size = H / G;
  const int pos = positions[r];
  const int* bt = block_tables + (long)row_seq[r] * bt_ld;
  const int first = chunk_size > 0 ? pos - pos % chunk_size : 0;
  const int end = pos + 1;
  for (int d = t; d < H * KD; d += AW_THREADS) qs[d] = to_f(q[r * ldq + d]) * scale;
  for (int d = t; d < H * H; d += AW_THREADS) tk[d] = talk[d];
  __syncthreads();
  const long page_stride = (long)G * page_size * (KD + VD);
  const long v_base = (long)G * page_size * KD;
  const int n_out = H * VD;
  float acc[AM_PER];
#pragma unroll
  for (int u = 0; u < AM_PER; ++u) acc[u] = 0.f;
  const float inv_cap = softcap > 0.f ? 1.f / softcap : 0.f;
  for (int c0 = first + split * block; c0 < end; c0 += n_splits * block) {
    const int n = min(block, end - c0);
    for (int i = t; i < H * n; i += AW_THREADS) {
      const int g = i / n, k = i % n, j = c0 + k;
      const T* kp = plane + (long)bt[j / page_size] * page_stride + (long)(g / group_size) * page_size * KD +
                    (long)(j % page_size) * KD;
      const float* qg = qs + g * KD;
      float s = 0.f;
      for (int e = 0; e < KD; ++e) s += qg[e] * to_f(kp[e]);
      if (softcap > 0.f) s = softcap * tanhf(s * inv_cap);
      wr[g * block + k] = 1.f / (1.f + expf(-(s + head_bias[g])));
    }
    __syncthreads();
    for (int i = t; i < H * n; i += AW_THREADS) {
      const int h = i / n, k = i % n;
      float m = 0.f;
      for (int g = 0; g < H; ++g) m += tk[h * H + g] * wr[g * block + k];
      wm[h * block + k] = m;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < AM_PER; ++u) {
      const int o = t + u * AW_THREADS;
      if (o < n_out) {
        const int h = o / VD, c = o % VD;
        const long v_off = v_base + ((long)(h / group_size) * VD + c) * page_size;
        const float* w = wm + h * block;
        float a = acc[u];
        for (int k = 0; k < n; ++k) {
          const int j = c0 + k;
          a += w[k] * to_f(plane[(long)bt[j / page_size] * page_stride + v_off + (j % page_size)]);
        }
        acc[u] = a;
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int u = 0; u < AM_PER; ++u) {
    const int o = t + u * AW_THREADS;
    if (o < n_out) {
      if (n_splits > 1) partial[(r * n_splits + split) * n_out + o] = acc[u];
      else out[r * ldo + o] = from_f<T>(acc[u]);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(AW_THREADS) void attention_mixed_merge_kernel(const float* __restrict__ partial, int n_splits,
                                                                           T* __restrict__ out, long ldo, int rows,
                                                                           int n_out) {
  const long i = (long)blockIdx.x * AW_THREADS + threadIdx.x;
  if (i >= (long)rows * n_out) return;
  const long r = i / n_out;
  const int o = (int)(i % n_out);
  float a = 0.f;
  for (int s = 0; s < n_splits; ++s) a += partial[(r * n_splits + s) * n_out + o];
  out[r * ldo + o] = from_f<T>(a);
}

// block: keys a workgroup takes at a time (a multiple of 16 keeps a page's slots together; any value >= 1 is right).
// partial: [rows * n_splits * H * VD] floats where n_splits > 1.
TIS_EXPORT int tis_attention_mixed(int dtype, const void* q, long ldq, const void* plane, const int* block_tables, int bt_ld,
                                   const int* row_seq, const int* positions, void* out, long ldo, float* partial,
                                   int n_splits, int rows, int H, int G, int KD, int VD, int page_size, int chunk_size,
                                   float scale, float softcap, const float* head_bias, const float* talk, int block,
                                   hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || H < 1 || G < 1 || H % G || KD < 1 || VD < 1 || page_size < 1 || chunk_size < 0 || block < 1 ||
      n_splits < 1 || n_splits > 65535 || !head_bias || !talk || softcap < 0.f)
    return tis_fail("attention_mixed: bad size rows=%d heads=%d kv_heads=%d key=%d value=%d page=%d chunk=%d block=%d splits=%d",
                    rows, H, G, KD, VD, page_size, chunk_size, block, n_splits);
  if ((long)H * VD > (long)AM_PER * AW_THREADS)
    return tis_fail("attention_mixed: %d heads of %d value channels are more than %d outputs a row", H, VD, AM_PER * AW_THREADS);
  const long lds = ((long)H * KD + (long)H * H + 2L * H * block) * sizeof(float);
  if (lds > 64 * 1024) return tis_fail("attention_mixed: %ld bytes of LDS for %d heads of %d in blocks of %d keys", lds, H, KD, block);
  if (n_splits > 1 && !partial) return tis_fail("attention_mixed: key splits without a workspace");
  dim3 grid(rows, n_splits);
  const long merge_blocks = ((long)rows * H * VD + AW_THREADS - 1) / AW_THREADS;
  if (dtype == TIS_F32) {
    attention_mixed_kernel<float><<<grid, AW_THREADS, lds, stream>>>((const float*)q, ldq, (const float*)plane, block_tables,
        bt_ld, row_seq, positions, (float*)out, ldo, partial, n_splits, H, G, KD, VD, page_size, chunk_size, scale, softcap,
        head_bias, talk, block);
    if (n_splits > 1)
      attention_mixed_merge_kernel<float><<<merge_blocks, AW_THREADS, 0, stream>>>(partial, n_splits, (float*)out, ldo, rows, H * VD);
  } else if (dtype == TIS_BF16) {
    attention_mixed_kernel<bf16><<<grid, AW_THREADS, lds, stream>>>((const bf16*)q, ldq, (const bf16*)plane, block_tables,
        bt_ld, row_seq, positions, (bf16*)out, ldo, partial, n_splits, H, G, KD, VD, page_size, chunk_size, scale, softcap,
        head_bias, talk, block);
    if (n_splits > 1)
      attention_mixed_merge_kernel<bf16><<<merge_blocks, AW_THREADS, 0, stream>>>(partial, n_splits, (bf16*)out, ldo, rows, H * VD);
  } else {
    return tis_fail("unknown dtype code %d", dtype);
  }
  return tis_launch_status("attention_mixed");
}
