// Many small products in one launch, and the kernels around routed experts.
//
// grouped_linear: group g of G computes C_g = A_g W_g^T (+ bias_g), A_g [M_g, K], W_g [N, K], in one of two shapes:
//   columns   every group takes all M rows; its operands are column blocks: A + (g % a_mod) * a_group, W + g * w_group,
//             C + g * c_group (heads of an attention layer, the diagonal blocks of a block-diagonal matrix);
//   rows      group g takes rows offs[g] .. offs[g + 1] of a list sorted by group (experts): row r of the list reads
//             A row gather[r] / gather_div (or r) and writes C row r; offs lives on the device, so nothing waits for
//             the host to learn how many rows a group got.
// Epilogues: bias, an activation, or times sigmoid(gate[m, g N + n]).  Accumulation is one 32-bit FMA chain per
// output in increasing k whatever the tile, so a row's result does not depend on the rows beside it.
//
// route_topk, moe_align, moe_combine: choose a token's experts and their shares, sort (token, choice) pairs by
// expert, and add a token's expert outputs back together in the order of its choices.
#include "common.hpp"

#define GG_T 64
#define GG_K 16
#define GG_PAD 4

struct GroupedArgs {
  const void* A; long lda; long a_group; int a_mod;
  const void* W; long ldw; long w_group;
  void* C; long ldc; long c_group;
  const float* bias;            // [G, N] or null
  const float* gate; long ldg;  // gate[m * ldg + g * N + n] before its sigmoid, or null
  const int* offs;              // rows shape: [G + 1]; null: columns shape
  const int* gather; int gather_div;
  int M, N, K, G, act;
};

template <typename TA, typename TW, typename TC>
__global__ void __launch_bounds__(256)
grouped_gemm_kernel(GroupedArgs p) {
  __shared__ float As[GG_K][GG_T + GG_PAD];
  __shared__ float Ws[GG_K][GG_T + GG_PAD];
  __shared__ int a_rows[GG_T];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int n0 = blockIdx.x * GG_T;
  int g, m0, m_end, c_row0;
  if (p.offs) {
    int tile = blockIdx.y, start = 0, cnt = 0;
    for (g = 0; g < p.G; ++g) {
      start = p.offs[g];
      cnt = p.offs[g + 1] - start;
      const int nt = (cnt + GG_T - 1) / GG_T;
      if (tile < nt) break;
      tile -= nt;
    }
    if (g == p.G) return;
    m0 = tile * GG_T;
    m_end = cnt;
    c_row0 = start;
    if (tid < GG_T) {
      const int r = m0 + tid;
      a_rows[tid] = r < cnt ? (p.gather ? p.gather[start + r] / p.gather_div : start + r) : -1;
    }
  } else {
    g = blockIdx.z;
    m0 = blockIdx.y * GG_T;
    m_end = p.M;
    c_row0 = 0;
    if (tid < GG_T) a_rows[tid] = m0 + tid < p.M ? m0 + tid : -1;
  }
  __syncthreads();
  const TA* A = (const TA*)p.A + (size_t)(g % p.a_mod) * p.a_group;
  const TW* W = (const TW*)p.W + (size_t)g * p.w_group;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  for (int k0 = 0; k0 < p.K; k0 += GG_K) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = tid + i * 256;
      const int r = idx >> 4, c = idx & 15, k = k0 + c;
      float a = 0.f, w = 0.f;
      if (k < p.K) {
        const int ar = a_rows[r];
        if (ar >= 0) a = to_float(A[(size_t)ar * p.lda + k]);
        if (n0 + r < p.N) w = to_float(W[(size_t)(n0 + r) * p.ldw + k]);
      }
      As[c][r] = a;
      Ws[c][r] = w;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GG_K; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
  TC* C = (TC*)p.C + (size_t)g * p.c_group;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= m_end) continue;
    const size_t crow = (size_t)(c_row0 + m);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= p.N) continue;
      float v = acc[i][j];
      if (p.bias) v += p.bias[(size_t)g * p.N + n];
      v = mie_act(v, p.act);
      if (p.gate) v *= mie_sigmoid(p.gate[crow * p.ldg + (size_t)g * p.N + n]);
      C[crow * p.ldc + n] = from_float<TC>(v);
    }
  }
}

// The same product for bfloat16 operands on the matrix cores (v_mfma_f32_16x16x32_bf16).  A workgroup of 4 waves
// owns a 64 x 64 tile of C; a k-step of 32 brings 64 rows x 32 k of A and of W into the LDS in 16-byte pieces
// (row r, k-block b at slot 4 r + (b ^ (r / 4) % 4), which spreads the fragment reads over the banks) while the
// next k-step's pieces are already on their way into registers; wave w multiplies the four 16-row tiles of A
// with its own 16 weight rows.  Every output is the same chain of matrix instructions in increasing k wherever
// its tile lies, so a row's result does not depend on the rows beside it.  K, the row strides and the group
// offsets are multiples of 8 and the operands 16-byte aligned (checked by the caller).
typedef __bf16 gg_bf16x8 __attribute__((ext_vector_type(8)));
typedef float gg_f32x4 __attribute__((ext_vector_type(4)));
union GGFrag {
  gg_bf16x8 v;
  uint4 q;
};

template <typename TC>
__global__ void __launch_bounds__(256)
grouped_gemm_mfma_kernel(GroupedArgs p) {
  __shared__ uint4 As[256];
  __shared__ uint4 Ws[256];
  __shared__ int a_rows[GG_T];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * GG_T;
  int g, m0, m_end, c_row0;
  if (p.offs) {
    int tile = blockIdx.y, start = 0, cnt = 0;
    for (g = 0; g < p.G; ++g) {
      start = p.offs[g];
      cnt = p.offs[g + 1] - start;
      const int nt = (cnt + GG_T - 1) / GG_T;
      if (tile < nt) break;
      tile -= nt;
    }
    if (g == p.G) return;
    m0 = tile * GG_T;
    m_end = cnt;
    c_row0 = start;
    if (tid < GG_T) {
      const int r = m0 + tid;
      a_rows[tid] = r < cnt ? (p.gather ? p.gather[start + r] / p.gather_div : start + r) : -1;
    }
  } else {
    g = blockIdx.z;
    m0 = blockIdx.y * GG_T;
    m_end = p.M;
    c_row0 = 0;
    if (tid < GG_T) a_rows[tid] = m0 + tid < p.M ? m0 + tid : -1;
  }
  __syncthreads();
  const bf16* A = (const bf16*)p.A + (size_t)(g % p.a_mod) * p.a_group;
  const bf16* W = (const bf16*)p.W + (size_t)g * p.w_group;
  // the piece this thread brings in: row tid / 4, k-block tid % 4
  const int lrow = tid >> 2, lkb = tid & 3;
  const int ar = a_rows[lrow];
  const bf16* a_src = ar >= 0 ? A + (size_t)ar * p.lda + lkb * 8 : nullptr;
  const bf16* w_src = n0 + lrow < p.N ? W + (size_t)(n0 + lrow) * p.ldw + lkb * 8 : nullptr;
  const int put = lrow * 4 + (lkb ^ ((lrow >> 2) & 3));
  const uint4 zero = make_uint4(0, 0, 0, 0);
  auto fetch = [&](const bf16* src, int k0) { return src && k0 + lkb * 8 < p.K ? *reinterpret_cast<const uint4*>(src + k0) : zero; };
  const int col = lane & 15, kb = lane >> 4;
  const int wr = wave * 16 + col;
  const int w_get = wr * 4 + (kb ^ ((wr >> 2) & 3));
  gg_f32x4 acc[4];
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) acc[mt] = gg_f32x4{0.f, 0.f, 0.f, 0.f};
  uint4 ra = fetch(a_src, 0), rw = fetch(w_src, 0);
  for (int k0 = 0; k0 < p.K; k0 += 32) {
    As[put] = ra;
    Ws[put] = rw;
    __syncthreads();
    if (k0 + 32 < p.K) {
      ra = fetch(a_src, k0 + 32);
      rw = fetch(w_src, k0 + 32);
    }
    GGFrag b;
    b.q = Ws[w_get];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
      const int r = mt * 16 + col;
      GGFrag a;
      a.q = As[r * 4 + (kb ^ ((r >> 2) & 3))];
      acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, acc[mt], 0, 0, 0);
    }
    __syncthreads();
  }
  TC* C = (TC*)p.C + (size_t)g * p.c_group;
  const int n = n0 + wave * 16 + col;
  if (n >= p.N) return;
  const float bias = p.bias ? p.bias[(size_t)g * p.N + n] : 0.f;
#pragma unroll
  for (int mt = 0; mt < 4; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m0 + mt * 16 + kb * 4 + i;
      if (m >= m_end) continue;
      const size_t crow = (size_t)(c_row0 + m);
      float v = mie_act(acc[mt][i] + bias, p.act);
      if (p.gate) v *= mie_sigmoid(p.gate[crow * p.ldg + (size_t)g * p.N + n]);
      C[crow * p.ldc + n] = from_float<TC>(v);
    }
}

MIE_EXPORT const char* grouped_gemm_last_error() { return g_mie_error; }

template <typename TA, typename TW>
static int launch_grouped(const GroupedArgs& p, int c_dtype, dim3 grid, hipStream_t s) {
  if (c_dtype == MIE_F32)
    hipLaunchKernelGGL((grouped_gemm_kernel<TA, TW, float>), grid, dim3(256), 0, s, p);
  else if (c_dtype == MIE_BF16)
    hipLaunchKernelGGL((grouped_gemm_kernel<TA, TW, bf16>), grid, dim3(256), 0, s, p);
  else
    MIE_FAIL("grouped_linear: output dtype code %d", c_dtype);
  MIE_CHECK_LAUNCH("grouped_linear");
  return 0;
}

// Strides and group offsets are in elements.  Rows shape: offs non-null, M = the length of the sorted list (an upper
// bound of any group's rows), a_group / c_group / a_mod unused.
MIE_EXPORT int mie_grouped_linear(const void* A, int a_dtype, long lda, long a_group, int a_mod, const void* W, int w_dtype,
                                  long ldw, long w_group, void* C, int c_dtype, long ldc, long c_group, const float* bias,
                                  const float* gate, long ldg, const int* offs, const int* gather, int gather_div, int M,
                                  int N, int K, int G, int act, hipStream_t s) {
  if (M <= 0 || N <= 0 || G <= 0) return 0;
  if (K <= 0 || !A || !W || !C) MIE_FAIL("grouped_linear: K %d or a null operand", K);
  if (lda < K && !offs && a_group == 0) MIE_FAIL("grouped_linear: A row stride %ld < K %d", lda, K);
  if (ldw < K || ldc < N) MIE_FAIL("grouped_linear: strides %ld, %ld for K %d, N %d", ldw, ldc, K, N);
  if (a_mod <= 0) a_mod = G;
  if (gather && gather_div <= 0) MIE_FAIL("grouped_linear: gather divisor %d", gather_div);
  if (act < MIE_ACT_NONE || act > MIE_ACT_RELU2) MIE_FAIL("grouped_linear: activation code %d", act);
  GroupedArgs p = {A, lda, offs ? 0 : a_group, offs ? 1 : a_mod, W, ldw, w_group, C, ldc, offs ? 0 : c_group, bias, gate, ldg,
                   offs, gather, gather_div, M, N, K, G, act};
  const long mt = (M + GG_T - 1) / GG_T + (offs ? G : 0);
  if (mt > 65535 || G > 65535) MIE_FAIL("grouped_linear: %ld row tiles, %d groups are beyond the grid", mt, G);
  dim3 grid((N + GG_T - 1) / GG_T, (unsigned)mt, offs ? 1 : G);
  // bfloat16 operands that the matrix-core kernel's 16-byte loads can take
  if (a_dtype == MIE_BF16 && w_dtype == MIE_BF16 && (c_dtype == MIE_BF16 || c_dtype == MIE_F32) && K % 8 == 0 && lda % 8 == 0 &&
      ldw % 8 == 0 && p.a_group % 8 == 0 && w_group % 8 == 0 && (((uintptr_t)A | (uintptr_t)W) & 15) == 0) {
    if (c_dtype == MIE_BF16)
      hipLaunchKernelGGL(grouped_gemm_mfma_kernel<bf16>, grid, dim3(256), 0, s, p);
    else
      hipLaunchKernelGGL(grouped_gemm_mfma_kernel<float>, grid, dim3(256), 0, s, p);
    MIE_CHECK_LAUNCH("grouped_linear");
    return 0;
  }
  if (a_dtype == MIE_F32 && w_dtype == MIE_F32) return launch_grouped<float, float>(p, c_dtype, grid, s);
  if (a_dtype == MIE_F32 && w_dtype == MIE_BF16) return launch_grouped<float, bf16>(p, c_dtype, grid, s);
  if (a_dtype == MIE_BF16 && w_dtype == MIE_F32) return launch_grouped<bf16, float>(p, c_dtype, grid, s);
  if (a_dtype == MIE_BF16 && w_dtype == MIE_BF16) return launch_grouped<bf16, bf16>(p, c_dtype, grid, s);
  MIE_FAIL("grouped_linear: dtype codes A %d, W %d", a_dtype, w_dtype);
}

// ---- router: the `top` largest of logits[t, :] + bias (lowest index first among equals), in falling order, and
// the softmax over those alone.  One thread a token.
#define ROUTE_MAX_TOP 16
__global__ void route_topk_kernel(const float* __restrict__ logits, long ld, const float* __restrict__ bias,
                                  int* __restrict__ experts, float* __restrict__ shares, int T, int E, int top) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  const float* z = logits + (size_t)t * ld;
  int chosen[ROUTE_MAX_TOP];
  float val[ROUTE_MAX_TOP];
  for (int j = 0; j < top; ++j) {
    int best = -1;
    float bv = 0.f;
    for (int e = 0; e < E; ++e) {
      bool taken = false;
      for (int i = 0; i < j; ++i) taken |= chosen[i] == e;
      if (taken) continue;
      const float v = z[e] + (bias ? bias[e] : 0.f);
      if (best < 0 || v > bv) { best = e; bv = v; }
    }
    chosen[j] = best;
    val[j] = bv;
  }
  float sum = 0.f;
  const float largest = val[0];
  for (int j = 0; j < top; ++j) { val[j] = expf(val[j] - largest); sum += val[j]; }
  for (int j = 0; j < top; ++j) {
    experts[(size_t)t * top + j] = chosen[j];
    shares[(size_t)t * top + j] = val[j] / sum;
  }
}

MIE_EXPORT int mie_route_topk(const float* logits, long ld, const float* bias, int* experts, float* shares, int T, int E,
                              int top, hipStream_t s) {
  if (T <= 0) return 0;
  if (E <= 0 || top <= 0 || top > E || top > ROUTE_MAX_TOP) MIE_FAIL("route_topk: top %d of %d experts (at most %d)", top, E, ROUTE_MAX_TOP);
  if (ld < E) MIE_FAIL("route_topk: row stride %ld < %d", ld, E);
  hipLaunchKernelGGL(route_topk_kernel, dim3((T + 63) / 64), dim3(64), 0, s, logits, ld, bias, experts, shares, T, E, top);
  MIE_CHECK_LAUNCH("route_topk");
  return 0;
}

// ---- sort the n = T * top (token, choice) pairs by expert: offs [E + 1] (where each expert's pairs start in the
// sorted list), sorted [n] (the pair at each place), place [n] (the place of each pair).  One workgroup; the order
// of pairs inside an expert is whatever the counters gave, which no result depends on.
#define ALIGN_THREADS 1024
#define ALIGN_MAX_EXPERTS 1024
__global__ void __launch_bounds__(ALIGN_THREADS)
moe_align_kernel(const int* __restrict__ experts, int n, int E, int* __restrict__ offs, int* __restrict__ sorted,
                 int* __restrict__ place) {
  __shared__ int count[ALIGN_MAX_EXPERTS];
  __shared__ int start[ALIGN_MAX_EXPERTS + 1];
  for (int e = threadIdx.x; e < E; e += ALIGN_THREADS) count[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += ALIGN_THREADS) {
    int e = experts[i];
    e = e < 0 ? 0 : (e >= E ? E - 1 : e);
    place[i] = atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) { start[e] = run; run += count[e]; }
    start[E] = run;
  }
  __syncthreads();
  for (int e = threadIdx.x; e <= E; e += ALIGN_THREADS) offs[e] = start[e];
  for (int i = threadIdx.x; i < n; i += ALIGN_THREADS) {
    int e = experts[i];
    e = e < 0 ? 0 : (e >= E ? E - 1 : e);
    const int at = start[e] + place[i];
    place[i] = at;
    sorted[at] = i;
  }
}

MIE_EXPORT int mie_moe_align(const int* experts, int n, int E, int* offs, int* sorted, int* place, hipStream_t s) {
  if (n <= 0) return 0;
  if (E <= 0 || E > ALIGN_MAX_EXPERTS) MIE_FAIL("moe_align: %d experts (at most %d)", E, ALIGN_MAX_EXPERTS);
  hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(ALIGN_THREADS), 0, s, experts, n, E, offs, sorted, place);
  MIE_CHECK_LAUNCH("moe_align");
  return 0;
}

// ---- out[t, :] = sum over a token's choices j, in order, of shares[t, j] * y[place[t * top + j], :]
__global__ void moe_combine_kernel(const float* __restrict__ y, const int* __restrict__ place, const float* __restrict__ shares,
                                   float* __restrict__ out, int width, int top) {
  const int t = blockIdx.x;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < width; c += gridDim.y * blockDim.x) {
    float acc = 0.f;
    for (int j = 0; j < top; ++j)
      acc = fmaf(shares[(size_t)t * top + j], y[(size_t)place[(size_t)t * top + j] * width + c], acc);
    out[(size_t)t * width + c] = acc;
  }
}

MIE_EXPORT int mie_moe_combine(const float* y, const int* place, const float* shares, float* out, int T, int width, int top,
                               hipStream_t s) {
  if (T <= 0 || width <= 0) return 0;
  if (top <= 0) MIE_FAIL("moe_combine: top %d", top);
  int by = (width + 255) / 256;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(T, by > 16 ? 16 : by), dim3(256), 0, s, y, place, shares, out, width, top);
  MIE_CHECK_LAUNCH("moe_combine");
  return 0;
}
