// The delta-rule recurrence over a step's rows, with the request's state in its slot; everything is 32-bit.
//
// Per head a state S [d, d] (key channel i, value channel j):
//     S <- diag(decay) S - (a * u) (u^T S) + k v^T   (both terms of the old S),   o = S^T r.
// delta_prepare: a workgroup a token, from the projection's float32 sums: decay = exp(-decay_scale *
//     sigmoid(W tanh(inner) + bias)) (the product over the inner size in FMAs, ascending), a = sigmoid(a + bias),
//     the unit key u = k / sqrt(sum(k^2) + 1e-6) of each head -> prep [T, 3, H d] = decay, a * u, u.
// delta_scan: a workgroup a (row, head), thread j owns column j of S in registers, tokens in order; every term of
//     the update of column j reads that column only.  The head's output is divided by its root mean square, times
//     the weight and the sigmoid of the output gate, and rounded once.  S comes from state[slot] and is left there.
#include "common.hpp"

__global__ void __launch_bounds__(256)
delta_prepare_kernel(const float* __restrict__ sums, long ld, int k_col, int a_col, int w_col, const float* __restrict__ w_decay,
                     int rank, const float* __restrict__ decay_bias, float decay_scale, const float* __restrict__ removal_bias,
                     float* __restrict__ prep, int H, int d) {
  extern __shared__ float lds[];          // inner [rank], head sums [H]
  float* inner = lds;
  float* ss = lds + rank;
  const int t = blockIdx.x, n = H * d;
  const float* row = sums + (size_t)t * ld;
  for (int j = threadIdx.x; j < rank; j += blockDim.x) inner[j] = tanhf(row[w_col + j]);
  for (int h = threadIdx.x; h < H; h += blockDim.x) {
    float s = 0.f;
    for (int i = 0; i < d; ++i) s = fmaf(row[k_col + h * d + i], row[k_col + h * d + i], s);
    ss[h] = s;
  }
  __syncthreads();
  float* out = prep + (size_t)t * 3 * n;
  for (int c = threadIdx.x; c < n; c += blockDim.x) {
    float z = decay_bias[c];
    const float* w = w_decay + (size_t)c * rank;
    for (int j = 0; j < rank; ++j) z = fmaf(w[j], inner[j], z);
    const float a = mie_sigmoid(row[a_col + c] + removal_bias[c]);
    const float u = row[k_col + c] / sqrtf(ss[c / d] + 1e-6f);
    out[c] = expf(-decay_scale * mie_sigmoid(z));
    out[n + c] = a * u;
    out[2 * n + c] = u;
  }
}

template <int DMAX, typename TO>
__global__ void __launch_bounds__(DMAX < 64 ? 64 : DMAX)
delta_scan_kernel(const float* __restrict__ sums, long ld, int r_col, int k_col, int v_col, int g_col,
                  const float* __restrict__ prep, const float* __restrict__ norm_weight, float eps, float* __restrict__ state,
                  const int* __restrict__ row_start, const int* __restrict__ slots, TO* __restrict__ out, int H, int d) {
  __shared__ float scratch[16];
  const int row = blockIdx.x, h = blockIdx.y, j = threadIdx.x;
  const int n = H * d;
  const bool live = j < d;
  const int jj = live ? j : 0;
  const int t0 = row_start[row], t1 = row_start[row + 1];
  float* sp = state + ((size_t)slots[row] * H + h) * d * d;
  float S[DMAX];
#pragma unroll
  for (int i = 0; i < DMAX; ++i) S[i] = i < d ? sp[(size_t)i * d + jj] : 0.f;
  const float nw = norm_weight[h * d + jj];
  for (int t = t0; t < t1; ++t) {
    const float* srow = sums + (size_t)t * ld;
    const float* decay = prep + (size_t)t * 3 * n + h * d;
    const float* au = decay + n;
    const float* u = decay + 2 * n;
    const float* k = srow + k_col + h * d;
    const float* r = srow + r_col + h * d;
    const float v = srow[v_col + h * d + jj];
    float seen = 0.f;
#pragma unroll
    for (int i = 0; i < DMAX; ++i)
      if (i < d) seen = fmaf(u[i], S[i], seen);
    float o = 0.f;
#pragma unroll
    for (int i = 0; i < DMAX; ++i)
      if (i < d) {
        S[i] = fmaf(decay[i], S[i], fmaf(-au[i], seen, k[i] * v));
        o = fmaf(S[i], r[i], o);
      }
    const float sq = live ? o * o : 0.f;
    const float total = DMAX <= 64 ? wave_sum(sq) : block_sum(sq, scratch);
    const float rstd = 1.0f / sqrtf(total / (float)d + eps);
    if (live) out[(size_t)t * n + h * d + j] = from_float<TO>(o * rstd * nw * mie_sigmoid(srow[g_col + h * d + j]));
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < DMAX; ++i)
      if (i < d) sp[(size_t)i * d + j] = S[i];
  }
}

MIE_EXPORT const char* delta_rule_last_error() { return g_mie_error; }

// prep: scratch of tokens * 3 * H * d floats
MIE_EXPORT int mie_delta_rule(const float* sums, long ld, int r_col, int k_col, int v_col, int g_col, int a_col, int w_col,
                              const float* w_decay, int rank, const float* decay_bias, float decay_scale,
                              const float* removal_bias, const float* norm_weight, float eps, float* state,
                              const int* row_start, const int* slots, float* prep, void* out, int out_dtype, int tokens,
                              int rows, int H, int d, hipStream_t s) {
  if (tokens <= 0 || rows <= 0) return 0;
  if (H <= 0 || d <= 0 || d > 256 || rank <= 0) MIE_FAIL("delta_rule: %d heads of %d, inner size %d (heads up to 256)", H, d, rank);
  if (H > 65535) MIE_FAIL("delta_rule: %d heads is beyond the grid", H);
  const size_t lds = (size_t)(rank + H) * sizeof(float);
  if (lds > 60 * 1024) MIE_FAIL("delta_rule: inner size %d and %d heads do not fit the LDS", rank, H);
  hipLaunchKernelGGL(delta_prepare_kernel, dim3(tokens), dim3(256), lds, s, sums, ld, k_col, a_col, w_col, w_decay, rank,
                     decay_bias, decay_scale, removal_bias, prep, H, d);
  MIE_CHECK_LAUNCH("delta_rule (prepare)");
#define DR_LAUNCH(DMAX_, TO_)                                                                                             \
  hipLaunchKernelGGL((delta_scan_kernel<DMAX_, TO_>), dim3(rows, H), dim3(DMAX_ < 64 ? 64 : DMAX_), 0, s, sums, ld, r_col,  \
                     k_col, v_col, g_col, prep, norm_weight, eps, state, row_start, slots, (TO_*)out, H, d)
#define DR_SIZES(TO_)                       \
  if (d <= 16) DR_LAUNCH(16, TO_);          \
  else if (d <= 32) DR_LAUNCH(32, TO_);     \
  else if (d <= 64) DR_LAUNCH(64, TO_);     \
  else if (d <= 128) DR_LAUNCH(128, TO_);   \
  else DR_LAUNCH(256, TO_)
  if (out_dtype == MIE_F32) { DR_SIZES(float); }
  else if (out_dtype == MIE_BF16) { DR_SIZES(bf16); }
  else MIE_FAIL("delta_rule: out dtype code %d", out_dtype);
#undef DR_SIZES
#undef DR_LAUNCH
  MIE_CHECK_LAUNCH("delta_rule (scan)");
  return 0;
}
