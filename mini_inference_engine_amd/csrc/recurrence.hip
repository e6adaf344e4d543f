// The gated linear recurrence of the recurrent mixer and the short causal convolution before it, over a step's
// rows (a request's next tokens), with the request's state in its slot.  Everything is 32-bit.
//
// causal_conv:  u[t, c] = conv_bias[c] + sum_k taps[c, k] in(t - (K - 1 - k), c),  in(t, c) = x[t, c] + in_bias[c];
//               inputs before the row's first token come from tail[slot] (the request's last K - 1 inputs, zeros at
//               its start).  One thread a (token, channel); the tail is only read.
// rglru_scan:   per (row, channel) thread, tokens in order:
//                 r = sigmoid(gates[t, c]), i = sigmoid(gates[t, C + c]), a = exp(-decay_scale r softplus(lam[c])),
//                 S = a S + sqrt(1 - a^2) i u[t, c];  out[t, c] = S gelu_tanh(y[t, c] + y_bias[c]);
//               S starts from state[slot] and is left there; then the row's inputs are shifted into tail[slot].
#include "common.hpp"

__global__ void __launch_bounds__(256)
causal_conv_kernel(const float* __restrict__ x, long ldx, const float* __restrict__ in_bias, const float* __restrict__ taps,
                   const float* __restrict__ conv_bias, const float* __restrict__ tail, const int* __restrict__ token_row,
                   const int* __restrict__ row_start, const int* __restrict__ slots, float* __restrict__ u, int C, int K) {
  const int t = blockIdx.x;
  const int r = token_row[t], j = t - row_start[r];
  const float* tl = tail + (size_t)slots[r] * (K > 1 ? K - 1 : 1) * C;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
    float acc = conv_bias[c];
    const float b = in_bias[c];
    for (int k = 0; k < K; ++k) {
      const int back = K - 1 - k;              // how many tokens before t
      const float v = back <= j ? x[(size_t)(t - back) * ldx + c] + b : tl[(size_t)(K - 1 + j - back) * C + c];
      acc = fmaf(taps[(size_t)c * K + k], v, acc);
    }
    u[(size_t)t * C + c] = acc;
  }
}

// residual_conv: y[t, c] = h[t, c] + sum_k taps[c, k] h[t - (K - 1 - k), c], no bias; inputs before the row's first
// token come from tail[slot], which is only read here.  conv_tail_update, launched after it: the row's last K - 1
// inputs (old tail, then this step's), oldest first, into tail[slot]; a thread a (row, channel), reads ahead of writes.
template <typename TO>
__global__ void __launch_bounds__(256)
residual_conv_kernel(const float* __restrict__ h, const float* __restrict__ taps, const float* __restrict__ tail,
                     const int* __restrict__ token_row, const int* __restrict__ row_start, const int* __restrict__ slots,
                     TO* __restrict__ y, int C, int K) {
  const int t = blockIdx.x;
  const int r = token_row[t], j = t - row_start[r];
  const float* tl = tail + (size_t)slots[r] * (K > 1 ? K - 1 : 1) * C;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
    float acc = h[(size_t)t * C + c];
    for (int k = 0; k < K; ++k) {
      const int back = K - 1 - k;
      const float v = back <= j ? h[(size_t)(t - back) * C + c] : tl[(size_t)(K - 1 + j - back) * C + c];
      acc = fmaf(taps[(size_t)c * K + k], v, acc);
    }
    y[(size_t)t * C + c] = from_float<TO>(acc);
  }
}

__global__ void __launch_bounds__(256)
conv_tail_update_kernel(const float* __restrict__ h, float* __restrict__ tail, const int* __restrict__ row_start,
                        const int* __restrict__ slots, int C, int K) {
  const int r = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int a0 = row_start[r], n = row_start[r + 1] - a0, keep = K - 1;
  float* tl = tail + (size_t)slots[r] * keep * C;
  for (int i = 0; i < keep; ++i) {
    const int src = n + i;                     // place in the joined sequence of keep + n inputs
    tl[(size_t)i * C + c] = src < keep ? tl[(size_t)src * C + c] : h[(size_t)(a0 + src - keep) * C + c];
  }
}

template <typename TO>
__global__ void __launch_bounds__(256)
rglru_scan_kernel(const float* __restrict__ u, const float* __restrict__ gates, const float* __restrict__ lam,
                  const float* __restrict__ y, long ldy, const float* __restrict__ y_bias, const float* __restrict__ x,
                  long ldx, const float* __restrict__ x_bias, float* __restrict__ state, float* __restrict__ tail,
                  const int* __restrict__ row_start, const int* __restrict__ slots, TO* __restrict__ out, int C, int K,
                  float decay_scale) {
  const int r = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int a0 = row_start[r], b0 = row_start[r + 1], slot = slots[r];
  const float lm = lam[c];
  const float sp = decay_scale * (lm > 20.f ? lm : log1pf(expf(lm)));
  const float yb = y_bias[c];
  float S = state[(size_t)slot * C + c];
  for (int t = a0; t < b0; ++t) {
    const float rg = mie_sigmoid(gates[(size_t)t * 2 * C + c]);
    const float ig = mie_sigmoid(gates[(size_t)t * 2 * C + C + c]);
    const float log_a = -sp * rg;
    const float a = expf(log_a);
    // 1 - a^2 as -expm1(2 log a): no cancellation where a is close to 1
    S = fmaf(a, S, sqrtf(-expm1f(2.0f * log_a)) * ig * u[(size_t)t * C + c]);
    out[(size_t)t * C + c] = from_float<TO>(S * mie_gelu_tanh(y[(size_t)t * ldy + c] + yb));
  }
  state[(size_t)slot * C + c] = S;
  // the last K - 1 of (old tail, this row's inputs), oldest first; reads run ahead of writes
  const int n = b0 - a0, keep = K - 1;
  float* tl = tail + (size_t)slot * (keep > 0 ? keep : 1) * C;
  const float xb = x_bias[c];
  for (int i = 0; i < keep; ++i) {
    const int src = n + i;                     // place in the joined sequence of keep + n inputs
    tl[(size_t)i * C + c] = src < keep ? tl[(size_t)src * C + c] : x[(size_t)(a0 + src - keep) * ldx + c] + xb;
  }
}

// Rows of many tokens: the same recurrence in chunks of L tokens that run side by side.  S_t = a_t S_{t-1} + b_t is
// linear in S, so a chunk is summed up by (A, B) with S_end = A S_start + B.  Pass 1: every (row, chunk, channel)
// computes its A and B (and chunk 0 notes the state the row starts from); pass 2: every chunk folds the
// summaries of the chunks before it, in order, onto the start state and runs its tokens from there; the last
// chunk of a row leaves the state and the convolution's tail.  Each value comes out of the same chain of
// operations as in the one-pass kernel except for the fold over whole chunks.
struct ScanArgs {
  const float* u; const float* gates; const float* lam; const float* y; long ldy; const float* y_bias; const float* x; long ldx;
  const float* x_bias; float* state; float* tail; const int* row_start; const int* slots; void* out; float* chunk_a;
  float* chunk_b; float* start; int C, K, L, max_chunks; float decay_scale;
};

__device__ __forceinline__ void rglru_step(const ScanArgs& p, int t, int c, float sp, float& a, float& b) {
  const float rg = mie_sigmoid(p.gates[(size_t)t * 2 * p.C + c]);
  const float ig = mie_sigmoid(p.gates[(size_t)t * 2 * p.C + p.C + c]);
  const float log_a = -sp * rg;
  a = expf(log_a);
  b = sqrtf(-expm1f(2.0f * log_a)) * ig * p.u[(size_t)t * p.C + c];
}

template <int PASS, typename TO>
__global__ void __launch_bounds__(256)
rglru_chunk_kernel(ScanArgs p) {
  const int r = blockIdx.x / p.max_chunks, j = blockIdx.x - r * p.max_chunks, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= p.C) return;
  const int a0 = p.row_start[r], b0 = p.row_start[r + 1], slot = p.slots[r];
  const int t0 = a0 + j * p.L;
  if (t0 >= b0) return;
  const int t1 = t0 + p.L < b0 ? t0 + p.L : b0;
  const float lm = p.lam[c];
  const float sp = p.decay_scale * (lm > 20.f ? lm : log1pf(expf(lm)));
  const size_t at = ((size_t)r * p.max_chunks + j) * p.C + c;
  if (PASS == 1) {
    float A = 1.f, B = 0.f;
    for (int t = t0; t < t1; ++t) {
      float a, b;
      rglru_step(p, t, c, sp, a, b);
      B = fmaf(a, B, b);
      A *= a;
    }
    p.chunk_a[at] = A;
    p.chunk_b[at] = B;
    if (j == 0) p.start[(size_t)r * p.C + c] = p.state[(size_t)slot * p.C + c];
    return;
  }
  float S = p.start[(size_t)r * p.C + c];
  for (int i = 0; i < j; ++i) {
    const size_t e = ((size_t)r * p.max_chunks + i) * p.C + c;
    S = fmaf(p.chunk_a[e], S, p.chunk_b[e]);
  }
  const float yb = p.y_bias[c];
  TO* out = (TO*)p.out;
  for (int t = t0; t < t1; ++t) {
    float a, b;
    rglru_step(p, t, c, sp, a, b);
    S = fmaf(a, S, b);
    out[(size_t)t * p.C + c] = from_float<TO>(S * mie_gelu_tanh(p.y[(size_t)t * p.ldy + c] + yb));
  }
  if (t1 != b0) return;
  p.state[(size_t)slot * p.C + c] = S;
  const int n = b0 - a0, keep = p.K - 1;
  float* tl = p.tail + (size_t)slot * (keep > 0 ? keep : 1) * p.C;
  const float xb = p.x_bias[c];
  for (int i = 0; i < keep; ++i) {
    const int src = n + i;
    tl[(size_t)i * p.C + c] = src < keep ? tl[(size_t)src * p.C + c] : p.x[(size_t)(a0 + src - keep) * p.ldx + c] + xb;
  }
}

MIE_EXPORT const char* recurrence_last_error() { return g_mie_error; }

// The chunked form for steps whose longest row has max_row_tokens tokens: chunk_a, chunk_b [rows, max_chunks, C] and
// start [rows, C] are scratch, max_chunks = ceil(max_row_tokens / chunk).
MIE_EXPORT int mie_rglru_scan_chunked(const float* u, const float* gates, const float* lam, const float* y, long ldy,
                                      const float* y_bias, const float* x, long ldx, const float* x_bias, float* state,
                                      float* tail, const int* row_start, const int* slots, void* out, int out_dtype, int rows,
                                      int C, int K, float decay_scale, int chunk, int max_chunks, float* chunk_a, float* chunk_b,
                                      float* start, hipStream_t s) {
  if (rows <= 0) return 0;
  if (C <= 0 || K <= 0 || ldy < C || ldx < C || chunk <= 0 || max_chunks <= 0)
    MIE_FAIL("rglru_scan_chunked: %d channels, %d taps, row strides %ld, %ld, chunks of %d x %d", C, K, ldy, ldx, chunk, max_chunks);
  if (!u || !gates || !lam || !y || !y_bias || !x || !x_bias || !state || !tail || !row_start || !slots || !out || !chunk_a ||
      !chunk_b || !start)
    MIE_FAIL("rglru_scan_chunked: operands");
  if ((long)rows * max_chunks > 2000000000L) MIE_FAIL("rglru_scan_chunked: %d rows of %d chunks are beyond the grid", rows, max_chunks);
  if (out_dtype != MIE_F32 && out_dtype != MIE_BF16) MIE_FAIL("rglru_scan_chunked: output dtype code %d", out_dtype);
  ScanArgs p = {u, gates, lam, y, ldy, y_bias, x, ldx, x_bias, state, tail, row_start, slots, out, chunk_a, chunk_b, start,
                C, K, chunk, max_chunks, decay_scale};
  dim3 grid(rows * max_chunks, (C + 255) / 256);
  hipLaunchKernelGGL((rglru_chunk_kernel<1, float>), grid, dim3(256), 0, s, p);
  if (out_dtype == MIE_F32)
    hipLaunchKernelGGL((rglru_chunk_kernel<2, float>), grid, dim3(256), 0, s, p);
  else
    hipLaunchKernelGGL((rglru_chunk_kernel<2, bf16>), grid, dim3(256), 0, s, p);
  MIE_CHECK_LAUNCH("rglru_scan_chunked");
  return 0;
}

// x points at the first of the C input columns (rows ldx floats apart); taps [C, K]; tail [slots, max(1, K - 1), C].
MIE_EXPORT int mie_causal_conv(const float* x, long ldx, const float* in_bias, const float* taps, const float* conv_bias,
                               const float* tail, const int* token_row, const int* row_start, const int* slots, float* u,
                               int tokens, int C, int K, hipStream_t s) {
  if (tokens <= 0) return 0;
  if (C <= 0 || K <= 0 || ldx < C) MIE_FAIL("causal_conv: %d channels, %d taps, row stride %ld", C, K, ldx);
  if (!x || !in_bias || !taps || !conv_bias || !tail || !token_row || !row_start || !slots || !u) MIE_FAIL("causal_conv: operands");
  const int by = (C + 255) / 256;
  hipLaunchKernelGGL(causal_conv_kernel, dim3(tokens, by > 64 ? 64 : by), dim3(256), 0, s, x, ldx, in_bias, taps, conv_bias, tail,
                     token_row, row_start, slots, u, C, K);
  MIE_CHECK_LAUNCH("causal_conv");
  return 0;
}

// u [tokens, C], gates [tokens, 2 C] contiguous; y, x point at their first column; out [tokens, C] of out_dtype.
MIE_EXPORT int mie_rglru_scan(const float* u, const float* gates, const float* lam, const float* y, long ldy,
                              const float* y_bias, const float* x, long ldx, const float* x_bias, float* state, float* tail,
                              const int* row_start, const int* slots, void* out, int out_dtype, int rows, int C, int K,
                              float decay_scale, hipStream_t s) {
  if (rows <= 0) return 0;
  if (C <= 0 || K <= 0 || ldy < C || ldx < C) MIE_FAIL("rglru_scan: %d channels, %d taps, row strides %ld, %ld", C, K, ldy, ldx);
  if (!u || !gates || !lam || !y || !y_bias || !x || !x_bias || !state || !tail || !row_start || !slots || !out)
    MIE_FAIL("rglru_scan: operands");
  dim3 grid(rows, (C + 255) / 256);
  if (out_dtype == MIE_F32)
    hipLaunchKernelGGL(rglru_scan_kernel<float>, grid, dim3(256), 0, s, u, gates, lam, y, ldy, y_bias, x, ldx, x_bias, state, tail,
                       row_start, slots, (float*)out, C, K, decay_scale);
  else if (out_dtype == MIE_BF16)
    hipLaunchKernelGGL(rglru_scan_kernel<bf16>, grid, dim3(256), 0, s, u, gates, lam, y, ldy, y_bias, x, ldx, x_bias, state, tail,
                       row_start, slots, (bf16*)out, C, K, decay_scale);
  else
    MIE_FAIL("rglru_scan: output dtype code %d", out_dtype);
  MIE_CHECK_LAUNCH("rglru_scan");
  return 0;
}

// h [tokens, C] float32 contiguous; y [tokens, C] of y_dtype; tail [slots, max(1, K - 1), C] float32, read, then moved on.
MIE_EXPORT int mie_residual_conv(const float* h, const float* taps, float* tail, const int* token_row, const int* row_start,
                                 const int* slots, void* y, int y_dtype, int tokens, int rows, int C, int K, hipStream_t s) {
  if (tokens <= 0 || rows <= 0) return 0;
  if (C <= 0 || K < 1 || K > 64) MIE_FAIL("residual_conv: %d channels, %d taps (1 to 64)", C, K);
  const int by = (C + 255) / 256 < 64 ? (C + 255) / 256 : 64;
  if (y_dtype == MIE_F32)
    hipLaunchKernelGGL(residual_conv_kernel<float>, dim3(tokens, by), dim3(256), 0, s, h, taps, tail, token_row, row_start,
                       slots, (float*)y, C, K);
  else if (y_dtype == MIE_BF16)
    hipLaunchKernelGGL(residual_conv_kernel<bf16>, dim3(tokens, by), dim3(256), 0, s, h, taps, tail, token_row, row_start,
                       slots, (bf16*)y, C, K);
  else MIE_FAIL("residual_conv: out dtype code %d", y_dtype);
  MIE_CHECK_LAUNCH("residual_conv");
  if (K > 1) {
    hipLaunchKernelGGL(conv_tail_update_kernel, dim3(rows, (C + 255) / 256), dim3(256), 0, s, h, tail, row_start, slots, C, K);
    MIE_CHECK_LAUNCH("residual_conv (tail)");
  }
  return 0;
}
