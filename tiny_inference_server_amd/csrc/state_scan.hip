// Recurrent mixers whose state is a matrix per head, S [key channels D][value channels V], walked token by token:
//
//   kind 0, decay per key channel:   S_t = diag(a_t) S_(t-1) + k_t v_t^T,                 o_t = S_t^T q_t
//   kind 1, scalar gates (log input gate i, log forget gate f) with a running maximum m that starts at 0:
//           m_t = max(f_t + m_(t-1), i_t);   S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T;
//           n_t the same with k_t alone;      o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6),
//           with i = cap tanh((x_i + b_i) / cap), f = log sigmoid(cap tanh((x_f + b_f) / cap)).
//
// One workgroup per (request of the step, head, block of 16 value channels). Thread (s, j) owns the state's column j
// for the NS key channels from s * NS on in registers (a token's q, k and decays lie in LDS rows of 16 * NS floats,
// zeros beyond the head's channels, so a thread reads its share in 16-byte pieces), from the request's state slot before the first token to
// the slot after the last. Tokens are taken in chunks: a chunk's q, k, v and gates go into LDS, the 16 threads of a
// column leave a partial o per token there, and one pass adds them up. Each state element sees its tokens strictly in
// order with nothing else mixed in, so the result of a token does not depend on how a prompt was cut into steps, on the
// chunk size or on what else is in the batch, bit for bit. State, gates and sums are 32-bit. Kind 1 keeps n and m once
// per block of value channels (every block needs them, none may read what another has already advanced).
//
// Long portions of prompts are cut into segments of `seg_len` tokens that run side by side (`segments` > 0): the same
// kernel walks every segment from an empty state and leaves the segment's own state, its outputs as if nothing had
// come before, and what ties them to the past (kind 0: the product of the decays from the segment's start to each
// token; kind 1: the running maximum, the sum of log forget gates and n . q from the segment's start). A second kernel
// then walks the segments of a request in order, element by element, to the state at every segment's start and the
// request's new state; a third adds to every token's output what the state at its segment's start contributes:
//   kind 0: o_t += (q_t * decay product to t)^T S_start
//   kind 1: m_t = max(m'_t, F_t + m_start); numerator and n . q are sums of the segment's own part scaled by
//           exp(m'_t - m_t) and the start's part scaled by exp(F_t + m_start - m_t); o_t as above.
// Everything is still 32-bit; only the order of additions differs from the token-by-token walk.
#include "common.h"

TIS_DEFINE_LAST_ERROR(tis_state_scan)

static constexpr int SC_THREADS = 256;
static constexpr int SC_VB = 16;       // value channels of a workgroup
static constexpr int SC_R = 16;        // threads that share a column
static constexpr int SC_LDS_BYTES = 60 * 1024;

__device__ __forceinline__ float sc_log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// Workspace of a segmented call, per (request, segment) pair v and head h:
//   seg_state [v][h][D*V + D + 2]   the segment's own S, n and m (kernel 1); kernel 2 puts the S and n at the segment's
//                                   start in their place and the m at its start into the last float
//   cum       [row][H*D]            kind 0: product of the decays from the segment's start to the row
//   aux       [row][H][3]           kind 1: m', F and n . q of the segment alone
// Where a head finds its columns: `qk_group` consecutive heads share one set of query and key columns (1: every head
// has its own); head h's decay for key channel i lies at h * decay_hs + i * decay_cs of a row's decays (D and 1: one per
// key channel; 1 and 0: one per head).
// With one decay per head (decay_cs 0) a row's decays are one number a head: the walk reads that one number from LDS
// instead of a line of equal ones, keeps one running product instead of one per key channel, and the workspace's
// `cum` holds [row][H] numbers instead of [row][H*D].
struct ScanLayout {
  int qk_group, decay_hs, decay_cs;
};
__device__ __forceinline__ long cum_at(const ScanLayout& lay, long row, int H, int D, int h, int i) {
  return lay.decay_cs ? (row * H + h) * D + i : row * H + h;
}

struct SegArgs {
  int segments;      // most segments of one request in this call; 0: not segmented
  int seg_len;
  float* seg_state;
  float* cum;
  float* aux;
};

// VB value channels a workgroup, R = 256 / VB threads a column. A request's state line keeps n and m once per 16 value
// channels, so the walk in order runs with VB = 16; segments keep n and m once per head and may take 64 channels a
// workgroup, which loads a head's q, k and decays a quarter as often.
template <int KIND, int NS, bool SEG, int VB>
__global__ __launch_bounds__(SC_THREADS) void state_scan_kernel(
    const float* __restrict__ proj, long ldp, int q_off, int k_off, int v_off, float q_scale,
    const float* __restrict__ decay, long ldd, int i_off, int f_off, const float* __restrict__ bias_i,
    const float* __restrict__ bias_f, float cap, float* __restrict__ state, long state_ld,
    const int* __restrict__ cu_rows, const int* __restrict__ seq_slots, float* __restrict__ out, long ldo, int H, int D,
    int V, int n_vb, int chunk, SegArgs sg, ScanLayout lay) {
  static_assert(SEG || VB == SC_VB, "a state line keeps n and m per 16 value channels");
  constexpr int R = SC_THREADS / VB;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int DP = R * NS;                         // a token's row in LDS: the head's channels, then zeros
  float* sq = lds;                                   // [chunk][DP]
  float* sk = sq + chunk * DP;                       // [chunk][DP]
  float* sa = sk + chunk * DP;                       // kind 0: [chunk][DP] decays; kind 1: [chunk][4] gates i, f and m
  float* sv = sa + (KIND == 0 ? chunk * DP : chunk * 4);  // [chunk][VB]
  float* part = sv + chunk * VB;                     // [chunk][R][VB + 1]

  const int seq = SEG ? blockIdx.x / sg.segments : blockIdx.x, h = blockIdx.y, vb = blockIdx.z, t = threadIdx.x;
  int r0 = cu_rows[seq], r1 = cu_rows[seq + 1];
  if (SEG) {
    r0 += (blockIdx.x % sg.segments) * sg.seg_len;
    r1 = min(r1, r0 + sg.seg_len);
  }
  if (r0 >= r1) return;
  float* st = SEG ? sg.seg_state + ((long)blockIdx.x * H) * ((long)D * V + D + 2) : state + (long)seq_slots[seq] * state_ld;
  float* S = st + (long)h * (SEG ? (long)D * V + D + 2 : (long)D * V);
  // kind 1: n [D], then m; once per block of value channels in a request's state line, once per head in a segment's
  float* nm = SEG ? S + (long)D * V : st + (long)H * D * V + ((long)h * n_vb + vb) * (D + 1);
  const int j = t % VB, s = t / VB;
  const int col = vb * VB + j;
  const bool col_ok = col < V;

  const bool per_head = KIND == 0 && lay.decay_cs == 0;
  float Sreg[NS], nreg[NS], creg[NS];
  float m = SEG ? -INFINITY : 0.f, fsum = 0.f, cprod = 1.f;
#pragma unroll
  for (int e = 0; e < NS; ++e) {
    const int i = s * NS + e;
    Sreg[e] = (!SEG && i < D && col_ok) ? S[(long)i * V + col] : 0.f;
    nreg[e] = (!SEG && KIND == 1 && i < D) ? nm[i] : 0.f;
    creg[e] = 1.f;
  }
  if (!SEG && KIND == 1) m = nm[D];

  for (int c0 = r0; c0 < r1; c0 += chunk) {
    const int nc = min(chunk, r1 - c0);
    __syncthreads();
    for (int idx = t; idx < nc * DP; idx += SC_THREADS) {
      const int c = idx / DP, i = idx - c * DP;
      const float* row = proj + (long)(c0 + c) * ldp;
      const bool in = i < D;
      sq[idx] = in ? row[q_off + (h / lay.qk_group) * D + i] * q_scale : 0.f;
      sk[idx] = in ? row[k_off + (h / lay.qk_group) * D + i] : 0.f;
      if (KIND == 0 && (!per_head || i == 0))
        sa[idx] = in ? decay[(long)(c0 + c) * ldd + h * lay.decay_hs + i * lay.decay_cs] : 0.f;
    }
    for (int idx = t; idx < nc * VB; idx += SC_THREADS) {
      const int c = idx / VB, jj = idx - c * VB;
      sv[idx] = (vb * VB + jj < V) ? proj[(long)(c0 + c) * ldp + v_off + h * V + vb * VB + jj] : 0.f;
    }
    if (KIND == 1 && t < nc) {
      const float* row = proj + (long)(c0 + t) * ldp;
      const float xi = row[i_off + h] + bias_i[h], xf = row[f_off + h] + bias_f[h];
      sa[t * 4] = cap * tanhf(xi / cap);
      sa[t * 4 + 1] = sc_log_sigmoid(cap * tanhf(xf / cap));
    }
    __syncthreads();
    for (int c = 0; c < nc; ++c) {
      float keep = 1.f, take = 1.f;
      if (KIND == 1) {
        const float gi = sa[c * 4], gf = sa[c * 4 + 1];
        const float m_new = fmaxf(gf + m, gi);
        keep = expf(gf + m - m_new);      // (an empty segment's m is -inf: nothing is kept of nothing)
        take = expf(gi - m_new);
        m = m_new;
        fsum += gf;
      }
      const float vj = sv[c * VB + j];
      float acc = 0.f, nq = 0.f;
      const int at = c * DP + s * NS;
      // (channels beyond the head's are zeros in k and q: their state stays zero and adds nothing)
      constexpr int STEP = NS % 4 == 0 ? 4 : 1;      // a thread reads its channels in 16-byte pieces where they allow
      if (per_head) {
        const float a = sa[c * DP];                  // the head's one decay of this token
        cprod *= a;
#pragma unroll
        for (int e0 = 0; e0 < NS; e0 += STEP) {
          float kk[STEP], qq[STEP];
          if (STEP == 4) {
            *reinterpret_cast<float4*>(kk) = *reinterpret_cast<const float4*>(sk + at + e0);
            *reinterpret_cast<float4*>(qq) = *reinterpret_cast<const float4*>(sq + at + e0);
          } else {
            kk[0] = sk[at + e0];
            qq[0] = sq[at + e0];
          }
#pragma unroll
          for (int u = 0; u < STEP; ++u) {
            const int e = e0 + u;
            Sreg[e] = a * Sreg[e] + kk[u] * vj;
            acc += Sreg[e] * qq[u];
          }
        }
        if (SEG && vb == 0 && t == 0) sg.cum[cum_at(lay, c0 + c, H, D, h, 0)] = cprod;
      } else {
#pragma unroll
        for (int e0 = 0; e0 < NS; e0 += STEP) {
          float kk[STEP], qq[STEP], aa[STEP];
          if (STEP == 4) {
            *reinterpret_cast<float4*>(kk) = *reinterpret_cast<const float4*>(sk + at + e0);
            *reinterpret_cast<float4*>(qq) = *reinterpret_cast<const float4*>(sq + at + e0);
            if (KIND == 0) *reinterpret_cast<float4*>(aa) = *reinterpret_cast<const float4*>(sa + at + e0);
          } else {
            kk[0] = sk[at + e0];
            qq[0] = sq[at + e0];
            if (KIND == 0) aa[0] = sa[at + e0];
          }
#pragma unroll
          for (int u = 0; u < STEP; ++u) {
            const int e = e0 + u;
            if (KIND == 0) {
              Sreg[e] = aa[u] * Sreg[e] + kk[u] * vj;
              if (SEG) creg[e] *= aa[u];
            } else {
              Sreg[e] = keep * Sreg[e] + take * (kk[u] * vj);
              nreg[e] = keep * nreg[e] + take * kk[u];
              nq += nreg[e] * qq[u];
            }
            acc += Sreg[e] * qq[u];
          }
        }
        if (KIND == 0 && SEG && vb == 0 && j == 0) {
#pragma unroll
          for (int e = 0; e < NS; ++e)
            if (s * NS + e < D) sg.cum[cum_at(lay, c0 + c, H, D, h, s * NS + e)] = creg[e];
        }
      }
      part[(c * R + s) * (VB + 1) + j] = acc;
      if (KIND == 1) {
        if (j == 0) part[(c * R + s) * (VB + 1) + VB] = nq;
        if (t == 0) sa[c * 4 + 2] = m;
        if (SEG && t == 0 && vb == 0) sg.aux[((long)(c0 + c) * H + h) * 3 + 1] = fsum;
      }
    }
    __syncthreads();
    for (int idx = t; idx < nc * VB; idx += SC_THREADS) {
      const int c = idx / VB, jj = idx - c * VB;
      float o = 0.f, nq = 0.f;
      for (int ss = 0; ss < R; ++ss) {
        o += part[(c * R + ss) * (VB + 1) + jj];
        if (KIND == 1) nq += part[(c * R + ss) * (VB + 1) + VB];
      }
      if (KIND == 1 && !SEG) o /= fmaxf(fabsf(nq), expf(-sa[c * 4 + 2])) + 1e-6f;
      if (KIND == 1 && SEG && vb == 0 && jj == 0) {
        sg.aux[((long)(c0 + c) * H + h) * 3] = sa[c * 4 + 2];
        sg.aux[((long)(c0 + c) * H + h) * 3 + 2] = nq;
      }
      if (vb * VB + jj < V) out[(long)(c0 + c) * ldo + h * V + vb * VB + jj] = o;
    }
  }
#pragma unroll
  for (int e = 0; e < NS; ++e) {
    const int i = s * NS + e;
    if (i < D && col_ok) S[(long)i * V + col] = Sreg[e];
    if (KIND == 1 && j == 0 && i < D && (!SEG || vb == 0)) nm[i] = nreg[e];
  }
  if (KIND == 1 && t == 0 && (!SEG || vb == 0)) nm[D] = m;
}

// Kernel 2 of a segmented call: one thread per element of a head's S (and of n), segment after segment in order. What
// the first kernel left as a segment's own state is replaced by the state at the segment's start; the request's state
// line receives the state after its last row.
template <int KIND>
__global__ __launch_bounds__(SC_THREADS) void segment_states_kernel(float* __restrict__ state, long state_ld,
                                                                    const int* __restrict__ cu_rows,
                                                                    const int* __restrict__ seq_slots, int H, int D,
                                                                    int V, int n_vb, SegArgs sg, ScanLayout lay) {
  const int seq = blockIdx.x, h = blockIdx.y;
  const int r0 = cu_rows[seq], r1 = cu_rows[seq + 1];
  if (r0 >= r1) return;
  const int el = blockIdx.z * SC_THREADS + threadIdx.x;      // [0, D*V): S; [D*V, D*V + D): n
  if (el >= D * V + (KIND == 1 ? D : 0)) return;
  const bool is_n = el >= D * V;
  const int i = is_n ? el - D * V : el / V;
  float* st = state + (long)seq_slots[seq] * state_ld;
  const long per = (long)D * V + D + 2;
  float x = is_n ? st[(long)H * D * V + (long)h * n_vb * (D + 1) + i] : st[(long)h * D * V + el];
  float m = KIND == 1 ? st[(long)H * D * V + (long)h * n_vb * (D + 1) + D] : 0.f;
  const int n_seg = (r1 - r0 + sg.seg_len - 1) / sg.seg_len;
  for (int g = 0; g < n_seg; ++g) {
    float* own = sg.seg_state + (((long)seq * sg.segments + g) * H + h) * per;
    const int last = min(r1, r0 + (g + 1) * sg.seg_len) - 1;
    const float mine = own[el];
    float next, m_next = 0.f;
    if (KIND == 0) {
      next = sg.cum[cum_at(lay, last, H, D, h, i)] * x + mine;
    } else {
      const float m_own = own[per - 2], f_all = sg.aux[((long)last * H + h) * 3 + 1];
      m_next = fmaxf(f_all + m, m_own);
      next = expf(f_all + m - m_next) * x + expf(m_own - m_next) * mine;
    }
    own[el] = x;
    if (KIND == 1 && el == 0) own[per - 1] = m;
    x = next;
    m = m_next;
  }
  if (is_n) {
    for (int b = 0; b < n_vb; ++b) st[(long)H * D * V + ((long)h * n_vb + b) * (D + 1) + i] = x;
  } else {
    st[(long)h * D * V + el] = x;
  }
  if (KIND == 1 && el == 0)
    for (int b = 0; b < n_vb; ++b) st[(long)H * D * V + ((long)h * n_vb + b) * (D + 1) + D] = m;
}

// Kernel 3 of a segmented call: what the state at a segment's start adds to its rows. One workgroup per (request and
// segment, head, 64 value channels); rows in tiles of 32, a thread owns one channel for 8 rows.
static constexpr int SG_COLS = 64, SG_ROWS = 32;

template <int KIND>
__global__ __launch_bounds__(SC_THREADS) void segment_outputs_kernel(const float* __restrict__ proj, long ldp, int q_off,
                                                                     float q_scale, const int* __restrict__ cu_rows,
                                                                     float* __restrict__ out, long ldo, int H, int D,
                                                                     int V, SegArgs sg, ScanLayout lay) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* s0 = lds;                       // [D][SG_COLS]
  float* qt = s0 + D * SG_COLS;          // [SG_ROWS][D + 1]
  float* qn = qt + SG_ROWS * (D + 1);    // [SG_ROWS] kind 1: q . n_start
  const int seq = blockIdx.x / sg.segments, g = blockIdx.x % sg.segments, h = blockIdx.y, t = threadIdx.x;
  const int r0 = cu_rows[seq] + g * sg.seg_len, r1 = min(cu_rows[seq + 1], r0 + sg.seg_len);
  if (r0 >= r1) return;
  const long per = (long)D * V + D + 2;
  const float* start = sg.seg_state + ((long)blockIdx.x * H + h) * per;
  const int c0 = blockIdx.z * SG_COLS, cg = t % 16, rg = t / 16;      // columns cg*4 .. cg*4+3, rows rg*2, rg*2+1
  for (int idx = t; idx < D * SG_COLS; idx += SC_THREADS) {
    const int i = idx / SG_COLS, cc = idx - i * SG_COLS;
    s0[idx] = c0 + cc < V ? start[(long)i * V + c0 + cc] : 0.f;
  }
  const float m0 = KIND == 1 ? start[per - 1] : 0.f;
  for (int t0 = r0; t0 < r1; t0 += SG_ROWS) {
    const int nr = min(SG_ROWS, r1 - t0);
    __syncthreads();
    for (int idx = t; idx < nr * D; idx += SC_THREADS) {
      const int r = idx / D, i = idx - r * D;
      float q = proj[(long)(t0 + r) * ldp + q_off + (h / lay.qk_group) * D + i] * q_scale;
      if (KIND == 0) q *= sg.cum[cum_at(lay, t0 + r, H, D, h, i)];
      qt[r * (D + 1) + i] = q;
    }
    __syncthreads();
    if (KIND == 1 && t < nr) {
      float a = 0.f;
      for (int i = 0; i < D; ++i) a += qt[t * (D + 1) + i] * start[(long)D * V + i];
      qn[t] = a;
    }
    float acc[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) acc[k] = 0.f;
    for (int i = 0; i < D; ++i) {
      const float4 sv = *reinterpret_cast<const float4*>(s0 + i * SG_COLS + cg * 4);
      const float qa = qt[(rg * 2) * (D + 1) + i], qb = qt[(rg * 2 + 1) * (D + 1) + i];
      acc[0] += qa * sv.x; acc[1] += qa * sv.y; acc[2] += qa * sv.z; acc[3] += qa * sv.w;
      acc[4] += qb * sv.x; acc[5] += qb * sv.y; acc[6] += qb * sv.z; acc[7] += qb * sv.w;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int r = rg * 2 + k / 4, col = cg * 4 + k % 4;
      if (r < nr && c0 + col < V) {
        float* o = out + (long)(t0 + r) * ldo + h * V + c0 + col;
        if (KIND == 0) {
          *o += acc[k];
        } else {
          const float* a = sg.aux + ((long)(t0 + r) * H + h) * 3;
          const float m_own = a[0], m_t = fmaxf(m_own, a[1] + m0);
          const float w_own = expf(m_own - m_t), w_start = expf(a[1] + m0 - m_t);
          const float nq = w_own * a[2] + w_start * qn[r];
          *o = (w_own * *o + w_start * acc[k]) / (fmaxf(fabsf(nq), expf(-m_t)) + 1e-6f);
        }
      }
    }
  }
}

static constexpr int SC_WIDE_VB = 64;      // value channels of a workgroup that walks a segment, where the sizes allow

template <int KIND>
static int launch_scan(bool wide, int ns, dim3 grid, size_t lds, hipStream_t stream, const float* proj, long ldp, int q_off, int k_off,
                       int v_off, float q_scale, const float* decay, long ldd, int i_off, int f_off, const float* bias_i,
                       const float* bias_f, float cap, float* state, long state_ld, const int* cu_rows,
                       const int* seq_slots, float* out, long ldo, int H, int D, int V, int n_vb, int chunk, SegArgs sg,
                       ScanLayout lay) {
#define SC_LAUNCH(NS)                                                                                                   \
  if (sg.segments)                                                                                                      \
    state_scan_kernel<KIND, NS, true, SC_VB><<<grid, SC_THREADS, lds, stream>>>(                                        \
        proj, ldp, q_off, k_off, v_off, q_scale, decay, ldd, i_off, f_off, bias_i, bias_f, cap, state, state_ld,        \
        cu_rows, seq_slots, out, ldo, H, D, V, n_vb, chunk, sg, lay);                                                   \
  else                                                                                                                  \
    state_scan_kernel<KIND, NS, false, SC_VB><<<grid, SC_THREADS, lds, stream>>>(                                       \
        proj, ldp, q_off, k_off, v_off, q_scale, decay, ldd, i_off, f_off, bias_i, bias_f, cap, state, state_ld,        \
        cu_rows, seq_slots, out, ldo, H, D, V, n_vb, chunk, sg, lay)
#define SC_LAUNCH_WIDE(NS)                                                                                              \
  state_scan_kernel<KIND, NS, true, SC_WIDE_VB><<<grid, SC_THREADS, lds, stream>>>(                                     \
      proj, ldp, q_off, k_off, v_off, q_scale, decay, ldd, i_off, f_off, bias_i, bias_f, cap, state, state_ld, cu_rows, \
      seq_slots, out, ldo, H, D, V, n_vb, chunk, sg, lay)
  if (wide) {
    if (ns <= 8) { SC_LAUNCH_WIDE(8); }
    else if (ns <= 16) { SC_LAUNCH_WIDE(16); }
    else { SC_LAUNCH_WIDE(32); }
  } else
  if (ns <= 1) { SC_LAUNCH(1); }
  else if (ns <= 2) { SC_LAUNCH(2); }
  else if (ns <= 4) { SC_LAUNCH(4); }
  else if (ns <= 8) { SC_LAUNCH(8); }
  else { SC_LAUNCH(16); }
#undef SC_LAUNCH_WIDE
#undef SC_LAUNCH
  if (tis_launch_status("state_scan")) return -1;
  if (!sg.segments) return 0;
  const int n_seqs = grid.x / sg.segments;
  const int elems = D * V + (KIND == 1 ? D : 0);
  segment_states_kernel<KIND><<<dim3(n_seqs, H, (elems + SC_THREADS - 1) / SC_THREADS), SC_THREADS, 0, stream>>>(
      state, state_ld, cu_rows, seq_slots, H, D, V, n_vb, sg, lay);
  if (tis_launch_status("segment_states")) return -1;
  const size_t lds3 = sizeof(float) * ((size_t)D * SG_COLS + (size_t)SG_ROWS * (D + 1) + SG_ROWS);
  segment_outputs_kernel<KIND><<<dim3(grid.x, H, (V + SG_COLS - 1) / SG_COLS), SC_THREADS, lds3, stream>>>(
      proj, ldp, q_off, q_scale, cu_rows, out, ldo, H, D, V, sg, lay);
  return tis_launch_status("segment_outputs");
}

// Whether heads of D key channels can be run in segments (the third kernel keeps 64 columns of a state in LDS).
TIS_EXPORT int tis_state_scan_segmentable(int D) {
  return sizeof(float) * ((size_t)D * SG_COLS + (size_t)SG_ROWS * (D + 1) + SG_ROWS) <= 64 * 1024;
}

// 32-bit floats of the workspace a segmented call needs: the states, then `rows` lines of decay products or gate sums.
TIS_EXPORT long tis_state_scan_workspace(int kind, int n_seqs, int segments, int rows, int H, int D, int V) {
  return (long)n_seqs * segments * H * ((long)D * V + D + 2) + (kind == 0 ? (long)rows * H * D : (long)rows * H * 3);
}

// Floats of one request's state: S for every head, and for kind 1 also n and m per head and block of value channels.
TIS_EXPORT long tis_state_scan_floats(int kind, int H, int D, int V) {
  const long n_vb = (V + SC_VB - 1) / SC_VB;
  return (long)H * D * V + (kind == 1 ? (long)H * n_vb * (D + 1) : 0);
}

TIS_EXPORT int tis_state_scan(int kind, const float* proj, long ldp, int q_off, int k_off, int v_off, float q_scale,
                              const float* decay, long ldd, int i_off, int f_off, const float* bias_i,
                              const float* bias_f, float cap, float* state, long state_ld, const int* cu_rows,
                              const int* seq_slots, int n_seqs, float* out, long ldo, int H, int D, int V,
                              int segments, int seg_len, int rows, float* workspace, int qk_group, int decay_per_head,
                              hipStream_t stream) {
  if (n_seqs == 0) return 0;
  if (qk_group < 1 || H % qk_group) return tis_fail("state_scan: %d heads in groups of %d", H, qk_group);
  const ScanLayout lay = {qk_group, decay_per_head ? 1 : D, decay_per_head ? 0 : 1};
  if (n_seqs < 0 || H < 1 || H > 65535 || D < 1 || D > SC_R * 16 || V < 1)
    return tis_fail("state_scan: bad size requests=%d heads=%d key channels=%d (at most %d) value channels=%d", n_seqs, H,
                    D, SC_R * 16, V);
  if (kind != 0 && kind != 1) return tis_fail("state_scan: unknown kind %d", kind);
  if (kind == 0 && !decay) return tis_fail("state_scan: kind 0 needs the decays");
  if (kind == 1 && (!bias_i || !bias_f || !(cap > 0.f))) return tis_fail("state_scan: kind 1 needs gate biases and a cap");
  const int n_vb = (V + SC_VB - 1) / SC_VB;
  if (n_vb > 65535) return tis_fail("state_scan: %d value channels exceed the grid", V);
  if (state_ld < tis_state_scan_floats(kind, H, D, V))
    return tis_fail("state_scan: a state line of %ld floats is too short for %ld", state_ld, tis_state_scan_floats(kind, H, D, V));
  // segments of heads with up to 128 key channels and whole blocks of 64 value channels: 64 channels a workgroup
  const bool wide = segments > 0 && V % SC_WIDE_VB == 0 && D <= 32 * (SC_THREADS / SC_WIDE_VB);
  const int vb_cols = wide ? SC_WIDE_VB : SC_VB, col_threads = SC_THREADS / vb_cols;
  int chunk = 16;
  const int ns_need = (D + col_threads - 1) / col_threads;
  const int ns_built = wide ? (ns_need <= 8 ? 8 : ns_need <= 16 ? 16 : 32) : (D + SC_R - 1) / SC_R <= 1 ? 1 : (D + SC_R - 1) / SC_R <= 2 ? 2 : (D + SC_R - 1) / SC_R <= 4 ? 4
                       : (D + SC_R - 1) / SC_R <= 8 ? 8 : 16;
  const size_t dp = (size_t)col_threads * ns_built;      // a token's row in LDS (see the kernel)
  auto bytes = [&](int c) {
    return sizeof(float) * ((size_t)c * dp * 2 + (kind == 0 ? (size_t)c * dp : (size_t)c * 4) + (size_t)c * vb_cols +
                            (size_t)c * col_threads * (vb_cols + 1));
  };
  while (chunk > 1 && bytes(chunk) > SC_LDS_BYTES) chunk /= 2;
  if (bytes(chunk) > SC_LDS_BYTES) return tis_fail("state_scan: %d key channels do not fit the chunk buffers", D);
  SegArgs sg = {0, 0, nullptr, nullptr, nullptr};
  if (segments > 0) {
    if (seg_len < 1 || rows < 1 || !workspace || (long)n_seqs * segments > 0x7fffffffL)
      return tis_fail("state_scan: %d segments of %d rows need a workspace", segments, seg_len);
    sg.segments = segments;
    sg.seg_len = seg_len;
    sg.seg_state = workspace;
    float* lines = workspace + (long)n_seqs * segments * H * ((long)D * V + D + 2);
    sg.cum = kind == 0 ? lines : nullptr;
    sg.aux = kind == 1 ? lines : nullptr;
    if (sizeof(float) * ((size_t)D * SG_COLS + (size_t)SG_ROWS * (D + 1) + SG_ROWS) > 64 * 1024)
      return tis_fail("state_scan: %d key channels do not fit the segment kernels (see tis_state_scan_segmentable)", D);
  }
  dim3 grid(segments > 0 ? n_seqs * segments : n_seqs, H, (V + vb_cols - 1) / vb_cols);
  const int ns = ns_need;
  if (kind == 0)
    return launch_scan<0>(wide, ns, grid, bytes(chunk), stream, proj, ldp, q_off, k_off, v_off, q_scale, decay, ldd, i_off, f_off,
                          bias_i, bias_f, cap, state, state_ld, cu_rows, seq_slots, out, ldo, H, D, V, n_vb, chunk, sg, lay);
  return launch_scan<1>(wide, ns, grid, bytes(chunk), stream, proj, ldp, q_off, k_off, v_off, q_scale, decay, ldd, i_off, f_off,
                        bias_i, bias_f, cap, state, state_ld, cu_rows, seq_slots, out, ldo, H, D, V, n_vb, chunk, sg, lay);
}
