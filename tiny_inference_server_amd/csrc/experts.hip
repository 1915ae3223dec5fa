// Routed feed-forwards (mixtures of experts) and other products that come in groups: the router's choice, the lists of
// rows per expert, a grouped product C_g = act(A_g . W_g^T), and the weighted sum of a row's chosen experts.
//
// Router: s = softmax(z) over all of a row's router outputs in 32-bit; the `top` outputs with the largest s + correction
// are chosen (the lower index wins a tie); a chosen output's weight is s * scale, taken without the correction and not
// renormalised. Outputs from n_experts on are identity experts: they have no matrices, their result is the row itself.
//
// An assignment is a (row, k-th choice) pair, numbered row * top + k. The lists kernel gives every expert the
// assignments that chose it, in rising order, in a line of `rows` entries of its own (an expert is chosen at most once
// a row), so nothing needs a prefix sum or an atomic and the order never depends on timing.
//
// The grouped product walks, for group g, tiles of 16 list entries against tiles of 64 output columns of the group's
// matrix W[g] ([N][K]). Entry e's input row is A + (e / a_div) * lda + g * a_group, its output row C + e * ldc +
// g * c_group: with a_div = top the input rows are the step's rows and the outputs lie by assignment (an expert's first
// product), with a_div = 1 both lie by assignment (its second); without lists every group takes all rows, and a_group /
// c_group move from one group's columns to the next (a product per head on a head's own columns). Sums are 32-bit in
// an order that depends on K alone, so a row's result does not depend on what else is in the step.
#include "common.h"

TIS_DEFINE_LAST_ERROR(tis_experts)

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

static constexpr int EX_MAX_PER_LANE = 16;      // router outputs a lane keeps: up to 1,024 outputs a row

__device__ __forceinline__ float gelu_erf_f(float z) { return 0.5f * z * (1.f + erff(z * 0.7071067811865476f)); }

// one wave per row
__global__ __launch_bounds__(TIS_WAVE) void route_topk_kernel(const float* __restrict__ z, long ldz,
                                                              const float* __restrict__ correction, float scale,
                                                              int n_out, int top, int score, int* __restrict__ ids,
                                                              float* __restrict__ weights, int n_groups, int keep,
                                                              int renorm) {
  const long r = blockIdx.x;
  const int lane = threadIdx.x;
  float s[EX_MAX_PER_LANE], c[EX_MAX_PER_LANE];
  float m = -INFINITY;
#pragma unroll
  for (int u = 0; u < EX_MAX_PER_LANE; ++u) {
    const int e = lane + u * TIS_WAVE;
    s[u] = e < n_out ? z[r * ldz + e] : -INFINITY;
    m = fmaxf(m, s[u]);
  }
  m = wave_max(m);
  float sum = 0.f;
#pragma unroll
  for (int u = 0; u < EX_MAX_PER_LANE; ++u) {
    const int e = lane + u * TIS_WAVE;
    if (score == 1) s[u] = e < n_out ? 1.f / (1.f + expf(-s[u])) : 0.f;      // a sigmoid per output, no sum over them
    else s[u] = e < n_out ? expf(s[u] - m) : 0.f;
    sum += s[u];
  }
  sum = wave_sum(sum);
  const float inv = score == 1 ? 1.f : 1.f / sum;
#pragma unroll
  for (int u = 0; u < EX_MAX_PER_LANE; ++u) {
    const int e = lane + u * TIS_WAVE;
    s[u] *= inv;
    c[u] = e < n_out ? s[u] + (correction ? correction[e] : 0.f) : -INFINITY;
  }
  if (n_groups > 1 && keep < n_groups) {
    // The outputs form n_groups equal runs of neighbours; a group's score is its largest c. Only outputs of the `keep`
    // best groups (the lower group keeps a tie) stay in the choice; the others' c become -inf. Up to 64 groups: lane g
    // holds group g's score.
    const int per = n_out / n_groups;
    float gs = -INFINITY;
    for (int g = 0; g < n_groups; ++g) {
      float m = -INFINITY;
#pragma unroll
      for (int u = 0; u < EX_MAX_PER_LANE; ++u) {
        const int e = lane + u * TIS_WAVE;
        if (e < n_out && e / per == g) m = fmaxf(m, c[u]);
      }
      m = wave_max(m);
      if (lane == g) gs = m;
    }
    // a group's rank: how many groups beat it
    int rank = 0;
    for (int g = 0; g < n_groups; ++g) {
      const float og = __shfl(gs, g, TIS_WAVE);
      if (og > gs || (og == gs && g < lane)) ++rank;
    }
    const unsigned long long kept = __ballot(lane < n_groups && rank < keep);
#pragma unroll
    for (int u = 0; u < EX_MAX_PER_LANE; ++u) {
      const int e = lane + u * TIS_WAVE;
      if (e < n_out && !((kept >> (e / per)) & 1ull)) c[u] = -INFINITY;
    }
  }
  float total = 0.f;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
#pragma unroll
    for (int u = 0; u < EX_MAX_PER_LANE; ++u) {
      const int e = lane + u * TIS_WAVE;
      if (e < n_out && c[u] > best) { best = c[u]; at = e; }       // rising e within a lane: the lower index keeps a tie
    }
#pragma unroll
    for (int o = TIS_WAVE / 2; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, TIS_WAVE);
      const int oa = __shfl_xor(at, o, TIS_WAVE);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    float w = 0.f;
#pragma unroll
    for (int u = 0; u < EX_MAX_PER_LANE; ++u) {
      if (lane + u * TIS_WAVE == at) { w = s[u]; c[u] = -INFINITY; }
    }
    w = wave_sum(w);          // only the owner's lane holds it
    total += w;
    if (lane == 0) {
      ids[r * top + k] = at;
      weights[r * top + k] = w * scale;
    }
  }
  // renorm: the chosen weights divided by their sum (lane 0 reads back what it wrote itself)
  if (renorm && lane == 0) {
    const float inv = 1.f / (total + 1e-20f);
    for (int k = 0; k < top; ++k) weights[r * top + k] *= inv;
  }
}

// one workgroup per expert: the assignments that chose it, in rising order
__global__ __launch_bounds__(256) void expert_lists_kernel(const int* __restrict__ ids, int n_assign, int line,
                                                           int* __restrict__ lists, int* __restrict__ counts) {
  __shared__ int wave_count[4];
  __shared__ int base;
  const int e = blockIdx.x, t = threadIdx.x, lane = t % TIS_WAVE, wave = t / TIS_WAVE;
  if (t == 0) base = 0;
  __syncthreads();
  for (int a0 = 0; a0 < n_assign; a0 += 256) {
    const int a = a0 + t;
    const bool mine = a < n_assign && ids[a] == e;
    const unsigned long long vote = __ballot(mine);
    const int before = __popcll(vote & ((1ull << lane) - 1ull));
    if (lane == 0) wave_count[wave] = __popcll(vote);
    __syncthreads();
    int off = base;
    for (int w = 0; w < wave; ++w) off += wave_count[w];
    if (mine) lists[(long)e * line + off + before] = a;
    __syncthreads();
    if (t == 0) base += wave_count[0] + wave_count[1] + wave_count[2] + wave_count[3];
    __syncthreads();
  }
  if (t == 0) counts[e] = base;
}

struct GroupedArgs {
  const int* lists;     // [groups][line] entries, or null: every group takes the entries 0 .. rows-1
  const int* counts;    // [groups], with lists
  int line, rows, a_div;
  long lda, a_group, ldc, c_group;
  int N, K, act;        // act 0: none, 1: erf-form gelu
};

// plain multiply-adds, any type and any alignment: 16 entries x 64 columns a workgroup, K in steps of 32 through LDS
template <typename TA, typename TO>
__global__ __launch_bounds__(256) void grouped_plain_kernel(const TA* __restrict__ A, const TA* __restrict__ W,
                                                            TO* __restrict__ C, GroupedArgs p) {
  __shared__ float As[16][33];
  __shared__ float Ws[64][33];
  __shared__ int entry[16];
  const int g = blockIdx.z, m0 = blockIdx.y * 16, n0 = blockIdx.x * 64, t = threadIdx.x;
  const int count = p.lists ? p.counts[g] : p.rows;
  if (m0 >= count) return;
  if (t < 16) entry[t] = m0 + t < count ? (p.lists ? p.lists[(long)g * p.line + m0 + t] : m0 + t) : -1;
  __syncthreads();
  const TA* Wg = W + (long)g * p.N * p.K;
  const int tx = t % 64, ty = t / 64;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < p.K; k0 += 32) {
    for (int i = t; i < 16 * 32; i += 256) {
      const int row = i / 32, kk = i % 32, e = entry[row];
      As[row][kk] = (e >= 0 && k0 + kk < p.K) ? to_f(A[(long)(e / p.a_div) * p.lda + (long)g * p.a_group + k0 + kk]) : 0.f;
    }
    for (int i = t; i < 64 * 32; i += 256) {
      const int col = i / 32, kk = i % 32;
      Ws[col][kk] = (n0 + col < p.N && k0 + kk < p.K) ? to_f(Wg[(long)(n0 + col) * p.K + k0 + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 32; ++kk) {
      const float w = Ws[tx][kk];
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] += As[ty * 4 + i][kk] * w;
    }
    __syncthreads();
  }
  if (n0 + tx >= p.N) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int e = entry[ty * 4 + i];
    if (e < 0) continue;
    const float v = p.act == 1 ? gelu_erf_f(acc[i]) : acc[i];
    C[(long)e * p.ldc + (long)g * p.c_group + n0 + tx] = from_f<TO>(v);
  }
}

// bfloat16 on the matrix cores. A workgroup of four waves, WM x WN of them, owns 16 RM WM entries x 16 RN WN columns; a
// wave owns RM x RN tiles of 16 x 16. A matrix row and an input row are the two operands of v_mfma_f32_16x16x32_bf16
// straight from memory, 16 bytes a lane (rows 16-byte aligned, K a multiple of 8); a wave's RM + RN loads of a step feed
// RM RN products, and what the waves of a workgroup share meets in the caches. Each result is one wave's sum over K in
// steps of 32. Two shapes are built: 16 entries x 64 columns for groups of a few rows (decoded tokens: the job is to
// stream the matrices once), 64 x 128 for groups of many.
template <typename TO, int WM, int WN, int RM, int RN>
__global__ __launch_bounds__(256) void grouped_mfma_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W,
                                                           TO* __restrict__ C, GroupedArgs p) {
  static_assert(WM * WN == 4, "four waves a workgroup");
  const int g = blockIdx.z, t = threadIdx.x, lane = t % 64, wave = t / 64;
  const int m0 = blockIdx.y * (16 * RM * WM) + (wave / WN) * (16 * RM);
  const int n0 = blockIdx.x * (16 * RN * WN) + (wave % WN) * (16 * RN);
  const int count = p.lists ? p.counts[g] : p.rows;
  if (m0 >= count || n0 >= p.N) return;
  const int c16 = lane & 15, kg = lane >> 4;
  int mine[RM];
  const bf16* arow[RM];
#pragma unroll
  for (int i = 0; i < RM; ++i) {
    const int m = m0 + i * 16 + c16;
    mine[i] = m < count ? (p.lists ? p.lists[(long)g * p.line + m] : m) : -1;
    arow[i] = A + (long)(mine[i] < 0 ? 0 : mine[i] / p.a_div) * p.lda + (long)g * p.a_group + kg * 8;
  }
  bool w_ok[RN];
  const bf16* wrow[RN];
#pragma unroll
  for (int j = 0; j < RN; ++j) {
    w_ok[j] = n0 + j * 16 + c16 < p.N;
    wrow[j] = W + ((long)g * p.N + (w_ok[j] ? n0 + j * 16 + c16 : 0)) * p.K + kg * 8;
  }
  f32x4 acc[RM][RN];
#pragma unroll
  for (int i = 0; i < RM; ++i)
#pragma unroll
    for (int j = 0; j < RN; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  // U steps of 32 at a time: all their loads are issued before the first product, so that a wave keeps several
  // steps' worth of requests in flight (the products of one step take far less time than its operands' way here)
  constexpr int U = 4;
  for (int k0 = 0; k0 < p.K; k0 += 32 * U) {
    bf16x8 av[U][RM], wv[U][RN];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = k0 + u * 32;
      const bool k_ok = k + kg * 8 < p.K;
#pragma unroll
      for (int i = 0; i < RM; ++i) av[u][i] = (mine[i] >= 0 && k_ok) ? *reinterpret_cast<const bf16x8*>(arow[i] + k) : zero;
#pragma unroll
      for (int j = 0; j < RN; ++j) wv[u][j] = (w_ok[j] && k_ok) ? *reinterpret_cast<const bf16x8*>(wrow[j] + k) : zero;
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int i = 0; i < RM; ++i)
#pragma unroll
        for (int j = 0; j < RN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[u][j], av[u][i], acc[i][j], 0, 0, 0);
  }
  // the lane holds, of tile (i, j), the columns n0 + 16 j + 4 kg + e of entry i * 16 + c16
#pragma unroll
  for (int i = 0; i < RM; ++i) {
    if (mine[i] < 0) continue;
#pragma unroll
    for (int j = 0; j < RN; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int n = n0 + j * 16 + 4 * kg + e;
        if (n >= p.N) continue;
        const float v = p.act == 1 ? gelu_erf_f(acc[i][j][e]) : acc[i][j][e];
        C[(long)mine[i] * p.ldc + (long)g * p.c_group + n] = from_f<TO>(v);
      }
  }
}

// Groups of many rows: the same product tiled in both directions on v_mfma_f32_32x32x16_bf16 with both operands
// through LDS, as the tiled product for many rows does it (gemm_tiles.hip: direct loads into LDS one step of 64 ahead,
// two buffers, a row's eight 16-byte pieces XORed by half the row's number against bank conflicts, the tile computed
// transposed so that a lane ends up with four consecutive columns). What differs: a tile's rows are list entries, each
// with an address of its own for reading and for writing, the matrix is the group's, a tile past the group's count
// leaves at once, and the epilogue may apply the activation. 128 entries x 128 columns, four waves.
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
static __device__ __attribute__((aligned(16))) unsigned char ex_zeros[16];

#pragma clang diagnostic ignored "-Winline-asm"   // M0 in a clobber list: meant
__device__ __forceinline__ void ex_copy16(const void* lane_src, unsigned lds_addr) {
  const unsigned base = (unsigned)__builtin_amdgcn_readfirstlane((int)lds_addr);
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(lane_src), "s"(base) : "memory", "m0");
}

template <typename TO>
__global__ __launch_bounds__(256) void grouped_tiles_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W,
                                                            TO* __restrict__ C, GroupedArgs p) {
  constexpr int BM = 128, BN = 128, WN = 2, BK = 64, PCS = 8, ROWS = BM + BN, WAVES = 4;
  constexpr int STAGE = ROWS * BK * 2;                  // bytes of a buffer: the entries' rows, then the matrix's
  constexpr int LPW = ROWS * PCS / 64 / WAVES;          // loads of a step that each wave issues, 8 rows each
  constexpr int TM = 2, TN = 2;                         // 32 x 32 result tiles of a wave
  __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * STAGE];
  const int g = blockIdx.z;
  const int count = p.lists ? p.counts[g] : p.rows;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  if (m0 >= count) return;
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, r32 = lane & 31, h = lane >> 5;
  const int wm = wave / WN, wn = wave % WN;
  const unsigned lds0 = (unsigned)(uintptr_t)(const __attribute__((address_space(3))) unsigned char*)lds;
  const bf16* Wg = W + (long)g * p.N * p.K;
  auto entry = [&](int m) {                             // the list entry of the tile's row m (the last one again past the count)
    const int e = min(m0 + m, count - 1);
    return p.lists ? p.lists[(long)g * p.line + e] : e;
  };
  const unsigned char* lane_src[LPW];                   // the lane's piece of its row at K offset 0
  int lane_piece[LPW];
#pragma unroll
  for (int j = 0; j < LPW; ++j) {
    const int row = (wave * LPW + j) * 8 + (lane >> 3);
    lane_piece[j] = (lane & 7) ^ ((row >> 1) & 7);
    const bf16* src = row < BM ? A + (long)(entry(row) / p.a_div) * p.lda + (long)g * p.a_group
                               : Wg + (long)min(p.N - 1, n0 + row - BM) * p.K;
    lane_src[j] = (const unsigned char*)src + lane_piece[j] * 16;
  }
  auto stage = [&](int k0, int buf) {
#pragma unroll
    for (int j = 0; j < LPW; ++j) {
      const bool inside = k0 + lane_piece[j] * 8 < p.K;
      ex_copy16(inside ? lane_src[j] + (long)k0 * 2 : ex_zeros, lds0 + buf * STAGE + (wave * LPW + j) * 1024);
    }
  };
  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  unsigned a_row[TM], b_row[TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) a_row[i] = wm * 64 + i * 32 + r32;
#pragma unroll
  for (int j = 0; j < TN; ++j) b_row[j] = BM + wn * 64 + j * 32 + r32;
  const int nk = (p.K + BK - 1) / BK;
  stage(0, 0);
  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");      // this wave's pieces of step kt are in LDS
    __builtin_amdgcn_s_barrier();                             // ... and everyone's; everyone has read step kt - 1
    if (kt + 1 < nk) stage((kt + 1) * BK, buf ^ 1);
    const unsigned char* st = lds + buf * STAGE;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      bf16x8 a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        a[i] = *(const bf16x8*)(st + (a_row[i] * PCS + ((2 * ks + h) ^ ((a_row[i] >> 1) & 7))) * 16);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        b[j] = *(const bf16x8*)(st + (b_row[j] * PCS + ((2 * ks + h) ^ ((b_row[j] >> 1) & 7))) * 16);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[j], a[i], acc[i][j], 0, 0, 0);
    }
  }
  // accumulator 4 q + e of block (i, j): entry wm * 64 + i * 32 + r32 of the tile, column n0 + wn * 64 + j * 32 + 8 q + 4 h + e
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = wm * 64 + i * 32 + r32;
    if (m0 + m >= count) continue;
    TO* dst = C + (long)entry(m) * p.ldc + (long)g * p.c_group;
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + wn * 64 + j * 32 + q * 8 + h * 4;
        if (n >= p.N) continue;               // (N is a multiple of 4: the four columns are inside or outside together)
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = p.act == 1 ? gelu_erf_f(acc[i][j][q * 4 + e]) : acc[i][j][q * 4 + e];
        if constexpr (sizeof(TO) == 4) {
          *(f32x4*)(dst + n) = (f32x4){v[0], v[1], v[2], v[3]};
        } else {
          bf16x4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = static_cast<__bf16>(v[e]);
          *(bf16x4*)(dst + n) = o;
        }
      }
  }
}

// out[r] = sum_k weight[r][k] * (y[r * top + k] if ids[r][k] < n_experts else x[r]), in 32-bit
template <typename T>
__global__ __launch_bounds__(256) void experts_combine_kernel(const float* __restrict__ y, long ldy, const T* __restrict__ x,
                                                              long ldx, const int* __restrict__ ids,
                                                              const float* __restrict__ weights, int top, int n_experts,
                                                              float* __restrict__ out, long ldo, int D) {
  const long r = blockIdx.x;
  for (int c = threadIdx.x; c < D; c += 256) {
    float v = 0.f;
    for (int k = 0; k < top; ++k) {
      const int e = ids[r * top + k];
      const float w = weights[r * top + k];
      v += w * (e < n_experts ? y[(r * top + k) * ldy + c] : to_f(x[r * ldx + c]));
    }
    out[r * ldo + c] = v;
  }
}

TIS_EXPORT int tis_route_topk(const float* z, long ldz, const float* correction, float scale, int rows, int n_out, int top, int score,
                              int* ids, float* weights, int n_groups, int keep, int renorm, hipStream_t stream) {
  if (rows == 0) return 0;
  if (n_groups < 1 || n_groups > TIS_WAVE || n_out % n_groups || keep < 1 || keep > n_groups || top > keep * (n_out / n_groups))
    return tis_fail("route_topk: %d outputs in %d groups (at most %d) of which %d are kept, top %d", n_out, n_groups, TIS_WAVE, keep, top);
  if (rows < 0 || n_out < 1 || n_out > EX_MAX_PER_LANE * TIS_WAVE || top < 1 || top > n_out)
    return tis_fail("route_topk: bad size rows=%d outputs=%d (at most %d) top=%d", rows, n_out, EX_MAX_PER_LANE * TIS_WAVE, top);
  if (score != 0 && score != 1) return tis_fail("route_topk: score kind %d (0: softmax, 1: sigmoid)", score);
  route_topk_kernel<<<rows, TIS_WAVE, 0, stream>>>(z, ldz, correction, scale, n_out, top, score, ids, weights, n_groups, keep, renorm);
  return tis_launch_status("route_topk");
}

TIS_EXPORT int tis_expert_lists(const int* ids, int n_assign, int n_experts, int line, int* lists, int* counts,
                                hipStream_t stream) {
  if (n_experts == 0) return 0;
  if (n_assign < 0 || n_experts < 0 || line < 1) return tis_fail("expert_lists: bad size assignments=%d experts=%d", n_assign, n_experts);
  expert_lists_kernel<<<n_experts, 256, 0, stream>>>(ids, n_assign, line, lists, counts);
  return tis_launch_status("expert_lists");
}

// in_dtype / out_dtype: 0 float, 1 bfloat16 (a bfloat16 input may give a 32-bit output). most_rows: the most entries a
// group can have (the grid's height).
TIS_EXPORT int tis_grouped_linear(int in_dtype, int out_dtype, const void* A, long lda, long a_group, int a_div, const void* W,
                                  void* C, long ldc, long c_group, const int* lists, const int* counts, int line,
                                  int groups, int most_rows, int N, int K, int act, hipStream_t stream) {
  if (groups == 0 || most_rows == 0) return 0;
  if (groups < 0 || groups > 65535 || most_rows < 0 || N < 1 || K < 1 || a_div < 1 || (act != 0 && act != 1))
    return tis_fail("grouped_linear: bad size groups=%d rows=%d N=%d K=%d", groups, most_rows, N, K);
  if ((lists == nullptr) != (counts == nullptr)) return tis_fail("grouped_linear: lists and counts go together");
  const int tiles_m = (most_rows + 15) / 16;
  if (tiles_m > 65535) return tis_fail("grouped_linear: %d rows are too many for one call", most_rows);
  GroupedArgs p{lists, counts, line, most_rows, a_div, lda, a_group, ldc, c_group, N, K, act};
  dim3 grid((N + 63) / 64, tiles_m, groups);
  if (in_dtype == TIS_BF16) {
    const bool aligned = K % 8 == 0 && lda % 8 == 0 && a_group % 8 == 0 && ((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0;
    // what a lane stores four columns at a time must be aligned for it
    const int oa = out_dtype == TIS_BF16 ? 8 : 16;
    const bool wide_ok = aligned && N % 4 == 0 && ldc % 4 == 0 && c_group % 4 == 0 && ((uintptr_t)C % oa) == 0 && K >= 64;
    if (wide_ok && most_rows >= 128 * (lists ? groups : 1)) {
      // groups of many rows (with lists: if the rows were spread evenly): 128 entries x 128 columns through LDS
      dim3 big((N + 127) / 128, (most_rows + 127) / 128, groups);
      if (big.y > 65535) return tis_fail("grouped_linear: %d rows are too many for one call", most_rows);
      if (out_dtype == TIS_BF16) grouped_tiles_kernel<bf16><<<big, 256, 0, stream>>>((const bf16*)A, (const bf16*)W, (bf16*)C, p);
      else grouped_tiles_kernel<float><<<big, 256, 0, stream>>>((const bf16*)A, (const bf16*)W, (float*)C, p);
    } else if (aligned && most_rows >= 64 * (lists ? groups : 1)) {
      // 64 entries x 128 columns a workgroup, operands straight from memory
      dim3 big((N + 127) / 128, (most_rows + 63) / 64, groups);
      if (out_dtype == TIS_BF16) grouped_mfma_kernel<bf16, 2, 2, 2, 4><<<big, 256, 0, stream>>>((const bf16*)A, (const bf16*)W, (bf16*)C, p);
      else grouped_mfma_kernel<float, 2, 2, 2, 4><<<big, 256, 0, stream>>>((const bf16*)A, (const bf16*)W, (float*)C, p);
    } else if (aligned) {
      if (out_dtype == TIS_BF16) grouped_mfma_kernel<bf16, 1, 4, 1, 1><<<grid, 256, 0, stream>>>((const bf16*)A, (const bf16*)W, (bf16*)C, p);
      else grouped_mfma_kernel<float, 1, 4, 1, 1><<<grid, 256, 0, stream>>>((const bf16*)A, (const bf16*)W, (float*)C, p);
    } else {
      if (out_dtype == TIS_BF16) grouped_plain_kernel<bf16, bf16><<<grid, 256, 0, stream>>>((const bf16*)A, (const bf16*)W, (bf16*)C, p);
      else grouped_plain_kernel<bf16, float><<<grid, 256, 0, stream>>>((const bf16*)A, (const bf16*)W, (float*)C, p);
    }
  } else if (in_dtype == TIS_F32 && out_dtype == TIS_F32) {
    grouped_plain_kernel<float, float><<<grid, 256, 0, stream>>>((const float*)A, (const float*)W, (float*)C, p);
  } else {
    return tis_fail("grouped_linear: dtype codes %d -> %d", in_dtype, out_dtype);
  }
  return tis_launch_status("grouped_linear");
}

TIS_EXPORT int tis_experts_combine(int dtype, const float* y, long ldy, const void* x, long ldx, const int* ids,
                                   const float* weights, int top, int n_experts, float* out, long ldo, int rows, int D,
                                   hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || D < 1 || top < 1) return tis_fail("experts_combine: bad size rows=%d width=%d top=%d", rows, D, top);
  if (dtype == TIS_F32)
    experts_combine_kernel<float><<<rows, 256, 0, stream>>>(y, ldy, (const float*)x, ldx, ids, weights, top, n_experts, out, ldo, D);
  else if (dtype == TIS_BF16)
    experts_combine_kernel<bf16><<<rows, 256, 0, stream>>>(y, ldy, (const bf16*)x, ldx, ids, weights, top, n_experts, out, ldo, D);
  else
    return tis_fail("unknown dtype code %d", dtype);
  return tis_launch_status("experts_combine");
}
