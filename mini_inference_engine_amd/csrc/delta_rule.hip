// The delta-rule recurrence over a step's rows, with the request's state in its slot; everything is 32-bit.
//
// Per head a state S [d, d] (key channel i, value channel j):
//     S <- diag(decay) S - (a * u) (u^T S) + k v^T   (both terms of the old S),   o = S^T r.
// delta_prepare: a workgroup a token, from the projection's float32 sums: decay = exp(-decay_scale *
//     sigmoid(W tanh(inner) + bias)) (the product over the inner size in FMAs, ascending), a = sigmoid(a + bias),
//     the unit key u = k / sqrt(sum(k^2) + 1e-6) of each head -> prep [T, 3, H d] = decay, a * u, u.
// delta_scan: a workgroup a (row, chunk, head), thread j owns column j of S in registers (every term of the update of
//     column j reads that column only), tokens in order.  What all columns share (decay, a * u, u, k, r of a token) comes
//     in through the LDS, eight tokens at a time, the next eight on their way meanwhile.  The head's output is divided by
//     its root mean square, times the weight and the sigmoid of the output gate, and rounded once.
//
// Rows run whole (one chunk: S from state[slot], left there afterwards), or, long rows, in chunks of L tokens side by
// side in three passes, since a chunk acts on the state it starts from as S_end = P S_start + B with P and B of the
// chunk's own tokens:  (1) every chunk but a row's last computes P (the recurrence without k v^T on the identity) and
// B (the recurrence on zero), a thread carrying the same column of both;  (2) per row and head, chunk after chunk, S_start(c + 1) = P_c S_start(c) + B_c from
// state[slot] (16 columns a workgroup; columns do not mix);  (3) every chunk runs its tokens from its S_start and writes
// the outputs, a row's last chunk leaves state[slot].  The two ways differ by the rounding of pass 2 alone.
#include "common.hpp"

constexpr int PT_MAX = 16;       // most tokens a workgroup of delta_prepare takes: a channel's row of the decay matrix is read once for all of them

// RMAX > 0: inner sizes up to RMAX, the channel's row of the matrix in registers; 0: any inner size, the row read from memory
template <int RMAX>
__global__ void __launch_bounds__(256)
delta_prepare_kernel(const float* __restrict__ sums, long ld, int k_col, int a_col, int w_col, const float* __restrict__ w_decay,
                     int rank, const float* __restrict__ decay_bias, float decay_scale, const float* __restrict__ removal_bias,
                     float* __restrict__ prep, int tokens, int H, int d, int heads_here, int PT) {
  extern __shared__ __align__(16) float prep_lds[];
  const int rank4 = RMAX > 0 ? RMAX : (rank + 3) & ~3;
  float* inner = prep_lds;                       // [PT][rank4]: the decay's inner activations after their tanh
  float* ssq = prep_lds + (size_t)PT * rank4;    // [PT][heads_here]: sum of squares of the keys of the heads this workgroup touches
  const int t0 = blockIdx.x * PT, n = H * d;
  const int nt = tokens - t0 < PT ? tokens - t0 : PT;
  const int c0 = blockIdx.y * 256, h0 = c0 / d;
  for (int e = threadIdx.x; e < nt * rank4; e += blockDim.x) {
    const int tt = e / rank4, j = e % rank4;
    inner[e] = j < rank ? tanhf(sums[(size_t)(t0 + tt) * ld + w_col + j]) : 0.f;
  }
  for (int e = threadIdx.x; e < nt * heads_here; e += blockDim.x) {
    const int tt = e / heads_here, h = h0 + e % heads_here;
    float s = 0.f;
    if (h < H) {
      const float* kh = sums + (size_t)(t0 + tt) * ld + k_col + (size_t)h * d;
      if ((d & 3) == 0 && (((uintptr_t)kh) & 15) == 0) {          // the same order whatever the step holds, either way
#pragma unroll 4
        for (int i = 0; i < d; i += 4) {
          const float4 v = *reinterpret_cast<const float4*>(kh + i);
          s = fmaf(v.x, v.x, s);
          s = fmaf(v.y, v.y, s);
          s = fmaf(v.z, v.z, s);
          s = fmaf(v.w, v.w, s);
        }
      } else {
        for (int i = 0; i < d; ++i) s = fmaf(kh[i], kh[i], s);
      }
    }
    ssq[e] = s;
  }
  __syncthreads();
  const int c = c0 + threadIdx.x;                // a thread a channel
  if (c >= n) return;
  const float* w = w_decay + (size_t)c * rank;
  const float zb = decay_bias[c], rb = removal_bias[c];
  const int hl = c / d - h0;
  const bool vec = (rank & 3) == 0 && (((uintptr_t)w_decay) & 15) == 0;
  float wreg[RMAX > 0 ? RMAX : 1];
  if (RMAX > 0) {
#pragma unroll
    for (int j = 0; j < RMAX; ++j) wreg[j] = j < rank ? w[j] : 0.f;
  }
  for (int tt = 0; tt < nt; ++tt) {
    float z = zb;
    const float* in = inner + (size_t)tt * rank4;
    if (RMAX > 0) {
#pragma unroll
      for (int j = 0; j < RMAX; j += 4) {          // inner is zero beyond the inner size
        const float4 iv = *reinterpret_cast<const float4*>(in + j);
        z = fmaf(wreg[j], iv.x, z);
        z = fmaf(wreg[j + 1], iv.y, z);
        z = fmaf(wreg[j + 2], iv.z, z);
        z = fmaf(wreg[j + 3], iv.w, z);
      }
    } else if (vec) {
      for (int j = 0; j < rank; j += 4) {        // the row of the matrix stays in the cache nearest this thread over the tokens
        const float4 wv = *reinterpret_cast<const float4*>(w + j);
        const float4 iv = *reinterpret_cast<const float4*>(in + j);
        z = fmaf(wv.x, iv.x, z);
        z = fmaf(wv.y, iv.y, z);
        z = fmaf(wv.z, iv.z, z);
        z = fmaf(wv.w, iv.w, z);
      }
    } else {
      for (int j = 0; j < rank; ++j) z = fmaf(w[j], in[j], z);
    }
    const float* row = sums + (size_t)(t0 + tt) * ld;
    const float a = mie_sigmoid(row[a_col + c] + rb);
    const float u = row[k_col + c] / sqrtf(ssq[tt * heads_here + hl] + 1e-6f);
    float* out = prep + (size_t)(t0 + tt) * 3 * n;
    out[c] = expf(-decay_scale * mie_sigmoid(z));
    out[n + c] = a * u;
    out[2 * n + c] = u;
  }
}

enum { SCAN_WHOLE = 0, SCAN_SUMMARY = 1, SCAN_FROM_START = 2 };
constexpr int TB = 8;            // tokens a block of the LDS
constexpr int NV = 6;            // vectors a token: decay, a * u, u, k, r, v

struct ScanArgs {
  const float* sums; long ld; int r_col, k_col, v_col, g_col;
  const float* prep; const float* norm_weight; float eps;
  float* state; const int* row_start; const int* slots; void* out;
  float* summaries;      // [rows * max_chunks, H, 2, d, d]: B, P of a chunk
  float* starts;         // [rows * max_chunks, H, d, d]: the state a chunk starts from
  int H, d, L, max_chunks, mode;
};

template <int DMAX, typename TO, bool SUMMARY>
__global__ void __launch_bounds__(DMAX < 64 ? 64 : DMAX)
delta_scan_kernel(ScanArgs a) {
  constexpr int NT = DMAX < 64 ? 64 : DMAX;
  __shared__ float scratch[16];
  __shared__ __align__(16) float stage[TB][NV][DMAX];   // channels beyond the head's size hold zeros
  const int row = blockIdx.x / a.max_chunks, chunk = blockIdx.x % a.max_chunks, h = blockIdx.y, j = threadIdx.x;
  const int d = a.d, n = a.H * d;
  const int row_end = a.row_start[row + 1];
  const int t0 = a.row_start[row] + chunk * a.L;
  if (t0 >= row_end) return;                                   // the whole workgroup: this row has no such chunk
  const int t1 = t0 + a.L < row_end ? t0 + a.L : row_end;
  const bool last = t1 == row_end;
  constexpr bool summary = SUMMARY;                            // one thread carries column j of B (in S) and of P (in Q)
  if (summary && last) return;                                 // nobody starts from the end of a row's last chunk
  const bool live = j < d;
  const int jj = live ? j : 0;
  float* sp = a.state + ((size_t)a.slots[row] * a.H + h) * d * d;
  const size_t ch = (size_t)blockIdx.x * a.H + h;
  float S[DMAX];
  float Q[SUMMARY ? DMAX : 1];
  if (summary) {
#pragma unroll
    for (int i = 0; i < DMAX; ++i) S[i] = 0.f;
#pragma unroll
    for (int i = 0; i < (SUMMARY ? DMAX : 1); ++i) Q[i] = live && i == j ? 1.f : 0.f;
  } else {
    const float* from = a.mode == SCAN_FROM_START ? a.starts + ch * d * d : sp;
#pragma unroll
    for (int i = 0; i < DMAX; ++i) S[i] = i < d ? from[(size_t)i * d + jj] : 0.f;
  }
  const float nw = a.norm_weight[h * d + jj];
  int lane0;
  asm volatile("v_mov_b32 %0, 0" : "=v"(lane0));
  // thread j brings channel j of a token's six vectors in, for TB tokens at a time (zeros beyond the head's size and
  // beyond the chunk, so that the loops below need no bounds: a channel that is not there keeps S at zero)
  constexpr int PER = TB * NV;
  float nxt[PER];
  const size_t hj = (size_t)h * d + jj;
  auto fetch = [&](int tb) {
#pragma unroll
    for (int tt = 0; tt < TB; ++tt) {
      const int t = tb + tt < t1 ? tb + tt : t1 - 1;            // clamped: what is read beyond the chunk is not used
      const bool ok = live && tb + tt < t1;
      const float* prow = a.prep + (size_t)t * 3 * n + hj;
      const float* srow = a.sums + (size_t)t * a.ld + hj;
      nxt[tt * NV + 0] = ok ? prow[0] : 0.f;
      nxt[tt * NV + 1] = ok ? prow[n] : 0.f;
      nxt[tt * NV + 2] = ok ? prow[2 * n] : 0.f;
      nxt[tt * NV + 3] = ok ? srow[a.k_col] : 0.f;
      nxt[tt * NV + 4] = ok ? srow[a.r_col] : 0.f;
      nxt[tt * NV + 5] = ok ? srow[a.v_col] : 0.f;
    }
  };
  fetch(t0);
  TO* out = (TO*)a.out;
  for (int tb = t0; tb < t1; tb += TB) {
    __syncthreads();                                           // the block before is used up
    if (j < DMAX) {
#pragma unroll
      for (int p = 0; p < PER; ++p) stage[p / NV][p % NV][j] = nxt[p];
    }
    __syncthreads();
    if (tb + TB < t1) fetch(tb + TB);
    const int nt = t1 - tb < TB ? t1 - tb : TB;
    for (int tt = 0; tt < nt; ++tt) {
      // What every column shares is read by every lane from the same LDS address.  ``lane0`` is a zero the compiler
      // cannot see through: without it the values count as uniform, are moved to scalar registers, and those run out.
      const float* decay = stage[tt][0] + lane0;
      const float* au = stage[tt][1] + lane0;
      const float* u = stage[tt][2] + lane0;
      const float* k = stage[tt][3] + lane0;
      const float* r = stage[tt][4] + lane0;
      const float v = stage[tt][5][jj];
      float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f, q0 = 0.f, q1 = 0.f, q2 = 0.f, q3 = 0.f;
#pragma unroll
      for (int i = 0; i < DMAX; i += 4) {
        s0 = fmaf(u[i], S[i], s0);
        s1 = fmaf(u[i + 1], S[i + 1], s1);
        s2 = fmaf(u[i + 2], S[i + 2], s2);
        s3 = fmaf(u[i + 3], S[i + 3], s3);
        if (summary) {
          q0 = fmaf(u[i], Q[i], q0);
          q1 = fmaf(u[i + 1], Q[i + 1], q1);
          q2 = fmaf(u[i + 2], Q[i + 2], q2);
          q3 = fmaf(u[i + 3], Q[i + 3], q3);
        }
      }
      const float seen = (s0 + s1) + (s2 + s3), seen_q = (q0 + q1) + (q2 + q3);
      float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
#pragma unroll
      for (int i = 0; i < DMAX; i += 4) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          S[i + e] = fmaf(k[i + e], v, fmaf(-au[i + e], seen, decay[i + e] * S[i + e]));
          if (summary) Q[i + e] = fmaf(-au[i + e], seen_q, decay[i + e] * Q[i + e]);       // no k v^T: what the start state becomes
        }
        if (!summary) {
          o0 = fmaf(S[i], r[i], o0);
          o1 = fmaf(S[i + 1], r[i + 1], o1);
          o2 = fmaf(S[i + 2], r[i + 2], o2);
          o3 = fmaf(S[i + 3], r[i + 3], o3);
        }
      }
      if (!summary) {
        const float o = (o0 + o1) + (o2 + o3);
        const float sq = live ? o * o : 0.f;
        const float total = DMAX <= 64 ? wave_sum(sq) : block_sum(sq, scratch);
        const float rstd = 1.0f / sqrtf(total / (float)d + a.eps);
        const int t = tb + tt;
        if (live)
          out[(size_t)t * n + h * d + j] = from_float<TO>(o * rstd * nw * mie_sigmoid(a.sums[(size_t)t * a.ld + a.g_col + h * d + j]));
      }
    }
  }
  if (!live) return;
  float* to = summary ? a.summaries + ch * 2 * d * d : sp;
  if (summary || last) {
#pragma unroll
    for (int i = 0; i < DMAX; ++i)
      if (i < d) to[(size_t)i * d + j] = S[i];
  }
  if (summary) {
#pragma unroll
    for (int i = 0; i < (SUMMARY ? DMAX : 1); ++i)
      if (i < d) to[(size_t)(d + i) * d + j] = Q[i];
  }
}

// Pass 2: per (row, head, block of 16 columns), chunk after chunk: start(c + 1) = P_c start(c) + B_c, start(0) = state[slot].
// The column block of start(c) and the whole of P_c sit in the LDS; a thread makes four neighbouring columns of a row.
__global__ void __launch_bounds__(256)
delta_fold_kernel(const float* __restrict__ summaries, float* __restrict__ starts, const float* __restrict__ state,
                  const int* __restrict__ row_start, const int* __restrict__ slots, int H, int d, int L, int max_chunks) {
  extern __shared__ __align__(16) float fold_lds[];
  float* col = fold_lds;                         // [d][16]
  float* pm = fold_lds + (size_t)d * 16;         // [d][d + 1]
  const int row = blockIdx.x, h = blockIdx.y, j0 = blockIdx.z * 16;
  const int tokens = row_start[row + 1] - row_start[row];
  const int chunks = (tokens + L - 1) / L;
  const float* sp = state + ((size_t)slots[row] * H + h) * d * d;
  for (int e = threadIdx.x; e < d * 16; e += blockDim.x) {
    const int i = e / 16, jl = e % 16;
    col[e] = j0 + jl < d ? sp[(size_t)i * d + j0 + jl] : 0.f;
  }
  __syncthreads();
  // P of a chunk comes in through registers while the chunk before is folded (d * d / 256 numbers a thread)
  const int per = (d * d + 255) / 256;
  float pre[16];                                 // the first 16 of them; the rest, for d > 64, is read when needed
  auto ask = [&](int c) {
    const float* P = summaries + ((((size_t)row * max_chunks + c) * H + h) * 2 + 1) * d * d;
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int e = threadIdx.x + k * 256;
      pre[k] = (k < per && e < d * d) ? P[e] : 0.f;
    }
  };
  if (chunks > 1) ask(0);
  for (int c = 0; c < chunks; ++c) {
    const size_t ch = ((size_t)row * max_chunks + c) * H + h;
    float* st = starts + ch * d * d;
    for (int e = threadIdx.x; e < d * 16; e += blockDim.x)
      if (j0 + e % 16 < d) st[(size_t)(e / 16) * d + j0 + e % 16] = col[e];
    if (c + 1 == chunks) break;
    const float* B = summaries + ch * 2 * d * d;
    const float* P = B + (size_t)d * d;
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int e = threadIdx.x + k * 256;
      if (k < per && e < d * d) pm[(e / d) * (d + 1) + e % d] = pre[k];
    }
    for (int e = threadIdx.x + 16 * 256; e < d * d; e += blockDim.x) pm[(e / d) * (d + 1) + e % d] = P[e];
    __syncthreads();
    if (c + 2 < chunks) ask(c + 1);
    // every thread's new values first (up to four quads of columns at d = 256), then all of them into the LDS
    float4 fresh[4];
#pragma unroll
    for (int cnt = 0; cnt < 4; ++cnt) {
      const int q = threadIdx.x + cnt * 256;
      if (q >= d * 4) break;
      const int i = q / 4, jq = (q % 4) * 4;
      float4 acc;
      acc.x = j0 + jq < d ? B[(size_t)i * d + j0 + jq] : 0.f;
      acc.y = j0 + jq + 1 < d ? B[(size_t)i * d + j0 + jq + 1] : 0.f;
      acc.z = j0 + jq + 2 < d ? B[(size_t)i * d + j0 + jq + 2] : 0.f;
      acc.w = j0 + jq + 3 < d ? B[(size_t)i * d + j0 + jq + 3] : 0.f;
      const float* pr = pm + (size_t)i * (d + 1);
      for (int m = 0; m < d; ++m) {
        const float p = pr[m];
        const float4 sv = *reinterpret_cast<const float4*>(col + m * 16 + jq);
        acc.x = fmaf(p, sv.x, acc.x);
        acc.y = fmaf(p, sv.y, acc.y);
        acc.z = fmaf(p, sv.z, acc.z);
        acc.w = fmaf(p, sv.w, acc.w);
      }
      fresh[cnt] = acc;
    }
    __syncthreads();
#pragma unroll
    for (int cnt = 0; cnt < 4; ++cnt) {
      const int q = threadIdx.x + cnt * 256;
      if (q < d * 4) *reinterpret_cast<float4*>(col + (q / 4) * 16 + (q % 4) * 4) = fresh[cnt];
    }
    __syncthreads();
  }
}

MIE_EXPORT const char* delta_rule_last_error() { return g_mie_error; }

// prep: scratch of tokens * 3 * H * d floats.  chunk_tokens 0: rows run whole.  Else rows run in chunks of that many
// tokens, at most max_chunks a row, with scratch summaries [rows * max_chunks * H * 2 * d * d] and starts
// [rows * max_chunks * H * d * d] floats.
MIE_EXPORT int mie_delta_rule(const float* sums, long ld, int r_col, int k_col, int v_col, int g_col, int a_col, int w_col,
                              const float* w_decay, int rank, const float* decay_bias, float decay_scale,
                              const float* removal_bias, const float* norm_weight, float eps, float* state,
                              const int* row_start, const int* slots, float* prep, void* out, int out_dtype, int tokens,
                              int rows, int H, int d, int chunk_tokens, int max_chunks, float* summaries, float* starts,
                              hipStream_t s) {
  if (tokens <= 0 || rows <= 0) return 0;
  if (H <= 0 || d <= 0 || d > 256 || rank <= 0) MIE_FAIL("delta_rule: %d heads of %d, inner size %d (heads up to 256)", H, d, rank);
  if (H > 65535) MIE_FAIL("delta_rule: %d heads is beyond the grid", H);
  if (chunk_tokens > 0 && d > 128) MIE_FAIL("delta_rule: heads of %d run whole, not in chunks (up to 128)", d);
  if (chunk_tokens < 0 || (chunk_tokens > 0 && (max_chunks < 1 || !summaries || !starts)))
    MIE_FAIL("delta_rule: chunks of %d tokens, %d a row, need their scratch", chunk_tokens, max_chunks);
  const int heads_here = 255 / d + 2;           // heads a workgroup's 256 channels can touch
  // few tokens: a workgroup a token; many: up to PT_MAX tokens a workgroup, the matrix read once for them
  const int pt = tokens <= 64 ? 1 : tokens < 64 * PT_MAX ? (tokens + 63) / 64 : PT_MAX;
  const int rmax = rank <= 16 ? 16 : rank <= 64 ? 64 : 0;
  const size_t lds = ((size_t)pt * (rmax ? rmax : (rank + 3) & ~3) + (size_t)pt * heads_here) * sizeof(float);
  if (lds > 60 * 1024) MIE_FAIL("delta_rule: an inner size of %d does not fit the LDS", rank);
  if ((H * d + 255) / 256 > 65535) MIE_FAIL("delta_rule: %d channels is beyond the grid", H * d);
#define DP_LAUNCH(RMAX_)                                                                                                     \
  hipLaunchKernelGGL(delta_prepare_kernel<RMAX_>, dim3((tokens + pt - 1) / pt, (H * d + 255) / 256), dim3(256), lds, s, sums, ld, \
                     k_col, a_col, w_col, w_decay, rank, decay_bias, decay_scale, removal_bias, prep, tokens, H, d, heads_here, pt)
  if (rmax == 16) DP_LAUNCH(16);
  else if (rmax == 64) DP_LAUNCH(64);
  else DP_LAUNCH(0);
#undef DP_LAUNCH
  MIE_CHECK_LAUNCH("delta_rule (prepare)");
  ScanArgs a{sums, ld, r_col, k_col, v_col, g_col, prep, norm_weight, eps, state, row_start, slots, out, summaries, starts,
             H, d, chunk_tokens > 0 ? chunk_tokens : 1 << 30, chunk_tokens > 0 ? max_chunks : 1, SCAN_WHOLE};
#define DR_LAUNCH(DMAX_, TO_, GRID_, SUM_) \
  hipLaunchKernelGGL((delta_scan_kernel<DMAX_, TO_, SUM_>), GRID_, dim3(DMAX_ < 64 ? 64 : DMAX_), 0, s, a)
#define DR_SIZES(TO_, GRID_, SUM_)                      \
  if (d <= 16) DR_LAUNCH(16, TO_, GRID_, SUM_);         \
  else if (d <= 32) DR_LAUNCH(32, TO_, GRID_, SUM_);    \
  else if (d <= 64) DR_LAUNCH(64, TO_, GRID_, SUM_);    \
  else if (d <= 128) DR_LAUNCH(128, TO_, GRID_, SUM_);  \
  else DR_LAUNCH(256, TO_, GRID_, SUM_)
#define DR_DTYPES(GRID_, SUM_)                                   \
  if (out_dtype == MIE_F32) { DR_SIZES(float, GRID_, SUM_); }    \
  else if (out_dtype == MIE_BF16) { DR_SIZES(bf16, GRID_, SUM_); } \
  else MIE_FAIL("delta_rule: out dtype code %d", out_dtype)
  if (chunk_tokens == 0) {
    DR_DTYPES(dim3(rows, H), false);
    MIE_CHECK_LAUNCH("delta_rule (scan)");
    return 0;
  }
  if ((long)rows * max_chunks > 2147483647L) MIE_FAIL("delta_rule: %d rows of %d chunks is beyond the grid", rows, max_chunks);
  a.mode = SCAN_SUMMARY;
  DR_SIZES(float, dim3(rows * max_chunks, H), true);              // writes no outputs: one instantiation serves both dtypes
  MIE_CHECK_LAUNCH("delta_rule (chunk summaries)");
  const size_t fold_lds = ((size_t)d * 16 + (size_t)d * (d + 1)) * sizeof(float);
  if (fold_lds > 64 * 1024) {
    static bool allowed = false;
    if (!allowed) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(delta_fold_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)fold_lds);
      if (e != hipSuccess) MIE_FAIL("delta_rule: %zu bytes of LDS refused: %s", fold_lds, hipGetErrorString(e));
      allowed = true;
    }
  }
  hipLaunchKernelGGL(delta_fold_kernel, dim3(rows, H, (d + 15) / 16), dim3(256), fold_lds, s, summaries,
                     starts, state, row_start, slots, H, d, chunk_tokens, max_chunks);
  MIE_CHECK_LAUNCH("delta_rule (fold)");
  a.mode = SCAN_FROM_START;
  DR_DTYPES(dim3(rows * max_chunks, H), false);
  MIE_CHECK_LAUNCH("delta_rule (chunks)");
  return 0;
#undef DR_DTYPES
#undef DR_SIZES
#undef DR_LAUNCH
}
