// Attention whose weights are sigmoids mixed across the heads, on the matrix cores (bfloat16, pages of 16 slots).
//
// For the row at position p and every key j it sees (j <= p, and with chunk c > 0 only j >= p - p % c):
//   s_g = q_g . k_kv(g) * scale;  s_g <- cap * tanh(s_g / cap) (cap 0: as it is);  w_g = sigmoid(s_g + head_bias[g]);
//   m_h = sum_g talk[h][g] * w_g;  out_h = sum_j m_h(j) * v_kv(h)(j).
// Nothing is normalised over the keys: a row's result is a plain sum over its keys and may be cut anywhere.
//
// A workgroup of four waves takes an item of up to 16 consecutive rows of one request, all heads, and every
// `n_splits`-th step of 32 keys (two pages). Wave w owns the heads [w * HPW, (w + 1) * HPW):
//   S^T[key, row] = K[key, :] . Q[row, :]     v_mfma_f32_16x16x32_bf16, A = keys straight from the page, B = the rows'
//                                              queries kept in registers; lane (c, g) = (lane % 16, lane / 16) gets the
//                                              keys g * 4 .. g * 4 + 3 of both pages for row c
//   w = sigmoid(cap(S * scale) + bias)         32-bit, masked by position; into LDS [head][lane][8]
//   m_h = sum_g talk[h][g] w_g                 every wave reads all heads' weights of its own lanes and mixes for its heads
//   O^T[channel, row] += V^T[channel, key] m_h^T[key, row]     the same instruction, A = transposed values from the page,
//                                              B = the lane's own eight mixed weights: they never leave its registers
// Scores, weights and the mixture are 32-bit; the mixture is rounded to bfloat16 only as the value product's operand.
// Slots past the item's last position and pages past its range are never weighted merely by zero: their values are set
// to zero before the product, so what a reused page holds there, finite or not, cannot reach a result.
//
// Built per (key size, value size, heads a wave): TIS_AMX = key * 100000 + value * 100 + heads_per_wave.
#include "common.h"

TIS_DEFINE_LAST_ERROR(tis_attention_mixed)

#ifndef TIS_AMX
#define TIS_AMX 12812804
#endif
static constexpr int KD = TIS_AMX / 100000;
static constexpr int VD = (TIS_AMX / 100) % 1000;
static constexpr int HPW = TIS_AMX % 100;
static_assert(KD >= 8 && KD % 8 == 0 && KD <= 512, "key size: a multiple of 8 up to 512");
static_assert(VD >= 16 && VD % 16 == 0 && VD <= 512, "value size: a multiple of 16 up to 512");
static_assert(HPW >= 1 && HPW <= 16, "heads a wave: 1 to 16");
static constexpr int DC = (KD + 31) / 32;      // steps of 32 key channels
static constexpr int DB = VD / 16;             // blocks of 16 value channels
static constexpr int PAGE = 16;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

__device__ __forceinline__ bf16x8 amx_load8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x4 amx_load4(const bf16* p) { return *reinterpret_cast<const bf16x4*>(p); }

// items: (first row, rows) pairs, or null: item i is row i alone. LDS (floats): talk [H * H, rounded up to 4] | weights [H][64][8].
__global__ __launch_bounds__(256) void attention_mixed_mfma_kernel(
    const bf16* __restrict__ q, long ldq, const bf16* __restrict__ plane, const int* __restrict__ block_tables, int bt_ld,
    const int* __restrict__ row_seq, const int* __restrict__ positions, const int* __restrict__ items,
    bf16* __restrict__ out, long ldo, float* __restrict__ partial, int n_splits, int H, int G, int chunk, float scale,
    float softcap, const float* __restrict__ head_bias, const float* __restrict__ talk) {
  extern __shared__ float amx_lds[];
  float* tk = amx_lds;
  float* wl = amx_lds + ((H * H + 3) & ~3);      // (16-byte reads and writes)
  const int item = blockIdx.x, split = blockIdx.y;
  const int wave = threadIdx.x / TIS_WAVE, lane = threadIdx.x % TIS_WAVE;
  const int c16 = lane % 16, g4 = lane / 16;
  const int first = items ? items[2 * item] : item;
  const int n_rows = items ? items[2 * item + 1] : 1;
  const int pos0 = positions[first];
  const int p_hi = pos0 + n_rows - 1;
  const int* bt = block_tables + (long)row_seq[first] * bt_ld;
  const int k_first = chunk > 0 ? pos0 - pos0 % chunk : 0;
  const int group_size = H / G;
  for (int i = threadIdx.x; i < H * H; i += 256) tk[i] = talk[i];
  // the lane's row: its position, its first visible key, whether it is a row at all
  const bool row_ok = c16 < n_rows;
  const int p_row = pos0 + (row_ok ? c16 : 0);
  const int lo_row = chunk > 0 ? p_row - p_row % chunk : 0;
  const bf16* q_row = q + (long)(first + (row_ok ? c16 : 0)) * ldq;
  // this wave's heads: queries as B operands, biases
  bf16x8 qb[HPW][DC];
  float hb[HPW];
#pragma unroll
  for (int u = 0; u < HPW; ++u) {
    const int h = wave * HPW + u;
    hb[u] = h < H ? head_bias[h] : 0.f;
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) {
      const int d = dc * 32 + g4 * 8;
      const bool ok = h < H && d < KD;
      const bf16x8 v = amx_load8(q_row + (long)(ok ? h : 0) * KD + (ok ? d : 0));
      qb[u][dc] = ok ? v : (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
    }
  }
  f32x4 o[HPW][DB];
#pragma unroll
  for (int u = 0; u < HPW; ++u)
#pragma unroll
    for (int db = 0; db < DB; ++db) o[u][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
  const long page_stride = (long)G * PAGE * (KD + VD);
  const long v_base = (long)G * PAGE * KD;
  const float inv_cap = softcap > 0.f ? 1.f / softcap : 0.f;
  const int s_first = k_first / 32, s_last = p_hi / 32;
  for (int s = s_first + split; s <= s_last; s += n_splits) {
    // the step's two pages; one past the item's last position is not looked up
    const bf16* base[2];
    bool page_ok[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int key0 = s * 32 + t * 16;
      page_ok[t] = key0 <= p_hi;
      base[t] = plane + (long)bt[(page_ok[t] ? key0 : p_hi) / PAGE] * page_stride;
    }
    // scores and weights of this wave's heads; the keys of a key/value head are fetched once for the heads that share it
    bf16x8 ka[2][DC];
    int kv_have = -1;
#pragma unroll
    for (int u = 0; u < HPW; ++u) {
      const int h = wave * HPW + u;
      if (h < H) {
        const int kv_head = h / group_size;
        if (kv_head != kv_have) {
          kv_have = kv_head;
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            const bf16* kp = base[t] + (long)kv_head * PAGE * KD + (long)c16 * KD;
#pragma unroll
            for (int dc = 0; dc < DC; ++dc) {
              const int d = dc * 32 + g4 * 8;
              const bool ok = d < KD;
              const bf16x8 kv = amx_load8(kp + (ok ? d : 0));
              ka[t][dc] = ok ? kv : (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
            }
          }
        }
        f32x4 st[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          st[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int dc = 0; dc < DC; ++dc) st[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[t][dc], qb[u][dc], st[t], 0, 0, 0);
        }
        float w[8];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int j = s * 32 + t * 16 + g4 * 4 + i;
            float x = st[t][i] * scale;
            // tanh(y) = 1 - 2 / (1 + exp(2 y)), on the fast exponential (|y| is capped so that exp stays finite)
            if (softcap > 0.f) x = softcap * (1.f - 2.f / (1.f + __expf(2.f * fminf(fmaxf(x * inv_cap, -15.f), 15.f))));
            const float sg = 1.f / (1.f + __expf(-(x + hb[u])));
            w[t * 4 + i] = (row_ok && j <= p_row && j >= lo_row) ? sg : 0.f;
          }
        float* dst = wl + ((long)h * TIS_WAVE + lane) * 8;
        *reinterpret_cast<f32x4*>(dst) = (f32x4){w[0], w[1], w[2], w[3]};
        *reinterpret_cast<f32x4*>(dst + 4) = (f32x4){w[4], w[5], w[6], w[7]};
      }
    }
    __syncthreads();
    // the mixture for this wave's heads, from all heads' weights of the lane's own keys and row
    float m[HPW][8];
#pragma unroll
    for (int u = 0; u < HPW; ++u)
#pragma unroll
      for (int e = 0; e < 8; ++e) m[u][e] = 0.f;
    for (int gg = 0; gg < H; ++gg) {
      const float* src = wl + ((long)gg * TIS_WAVE + lane) * 8;
      const f32x4 a = *reinterpret_cast<const f32x4*>(src), b = *reinterpret_cast<const f32x4*>(src + 4);
#pragma unroll
      for (int u = 0; u < HPW; ++u) {
        const int h = wave * HPW + u;
        const float tt = h < H ? tk[h * H + gg] : 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          m[u][e] += tt * a[e];
          m[u][4 + e] += tt * b[e];
        }
      }
    }
    // O^T += V^T . m^T
#pragma unroll
    for (int u = 0; u < HPW; ++u) {
      const int h = wave * HPW + u;
      if (h < H) {
        bf16x8 pb;
#pragma unroll
        for (int e = 0; e < 8; ++e) pb[e] = static_cast<__bf16>(m[u][e]);
        const long v_head = v_base + (long)(h / group_size) * VD * PAGE;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          bf16x8 va;
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            const bf16x4 x = amx_load4(base[t] + v_head + (long)(db * 16 + c16) * PAGE + g4 * 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const bool ok = page_ok[t] && s * 32 + t * 16 + g4 * 4 + e <= p_hi;
              va[t * 4 + e] = ok ? x[e] : static_cast<__bf16>(0.f);
            }
          }
          o[u][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pb, o[u][db], 0, 0, 0);
        }
      }
    }
    __syncthreads();      // the next step's weights overwrite this step's
  }
  // O^T[channel = db * 16 + g4 * 4 + i][row = c16]
  if (!row_ok) return;
  const long row = first + c16;
  const int n_out = H * VD;
#pragma unroll
  for (int u = 0; u < HPW; ++u) {
    const int h = wave * HPW + u;
    if (h >= H) continue;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int c = h * VD + db * 16 + g4 * 4;
      if (n_splits > 1) {
        *reinterpret_cast<f32x4*>(partial + (row * n_splits + split) * n_out + c) = o[u][db];
      } else {
        bf16x4 w;
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = static_cast<__bf16>(o[u][db][i]);
        *reinterpret_cast<bf16x4*>(out + row * ldo + c) = w;
      }
    }
  }
}

__global__ __launch_bounds__(256) void attention_mixed_sum_kernel(const float* __restrict__ partial, int n_splits,
                                                                  bf16* __restrict__ out, long ldo, int rows, int n_out) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long)rows * n_out) return;
  const long r = i / n_out;
  const int c = (int)(i % n_out);
  float a = 0.f;
  for (int s = 0; s < n_splits; ++s) a += partial[(r * n_splits + s) * n_out + c];
  out[r * ldo + c] = static_cast<bf16>(a);
}

TIS_EXPORT int tis_attention_mixed_sizes(int* kd, int* vd, int* hpw) {
  *kd = KD;
  *vd = VD;
  *hpw = HPW;
  return 0;
}

// items: n_items (first row, rows <= 16) pairs of consecutive rows of one request each, or null: every row by itself.
// partial: [rows * n_splits * H * VD] floats where n_splits > 1. q, out: bfloat16 with 16-byte aligned rows.
TIS_EXPORT int tis_attention_mixed_mfma(const void* q, long ldq, const void* plane, const int* block_tables, int bt_ld,
                                        const int* row_seq, const int* positions, const int* items, int n_items, void* out,
                                        long ldo, float* partial, int n_splits, int rows, int H, int G, int key_dim,
                                        int value_dim, int page_size, int chunk, float scale, float softcap,
                                        const float* head_bias, const float* talk, hipStream_t stream) {
  if (rows == 0 || n_items == 0) return 0;
  if (key_dim != KD || value_dim != VD || page_size != PAGE)
    return tis_fail("attention_mixed_mfma: built for keys of %d, values of %d and pages of %d, called with %d, %d, %d", KD, VD,
                    PAGE, key_dim, value_dim, page_size);
  if (rows < 0 || n_items < 0 || H < 1 || G < 1 || H % G || H > 4 * HPW || chunk < 0 || n_splits < 1 || n_splits > 65535 ||
      !head_bias || !talk || softcap < 0.f)
    return tis_fail("attention_mixed_mfma: bad size rows=%d items=%d heads=%d (at most %d) kv_heads=%d chunk=%d splits=%d", rows,
                    n_items, H, 4 * HPW, G, chunk, n_splits);
  if (ldq % 8 || ldo % 4 || ((uintptr_t)q % 16) || ((uintptr_t)out % 8))
    return tis_fail("attention_mixed_mfma: rows of q and out must be 16 and 8 bytes aligned");
  if (n_splits > 1 && (!partial || ((uintptr_t)partial % 16))) return tis_fail("attention_mixed_mfma: key splits without a workspace");
  const size_t lds = ((size_t)((H * H + 3) & ~3) + (size_t)H * TIS_WAVE * 8) * sizeof(float);
  if (lds > 64 * 1024) return tis_fail("attention_mixed_mfma: %d heads need %zu bytes of LDS", H, lds);
  attention_mixed_mfma_kernel<<<dim3(n_items, n_splits), 256, lds, stream>>>(
      (const bf16*)q, ldq, (const bf16*)plane, block_tables, bt_ld, row_seq, positions, items, (bf16*)out, ldo, partial, n_splits,
      H, G, chunk, scale, softcap, head_bias, talk);
  if (n_splits > 1) {
    const long blocks = ((long)rows * H * VD + 255) / 256;
    attention_mixed_sum_kernel<<<blocks, 256, 0, stream>>>(partial, n_splits, (bf16*)out, ldo, rows, H * VD);
  }
  return tis_launch_status("attention_mixed_mfma");
}
