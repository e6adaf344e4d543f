// Between a q/k/v projection's float32 sums and attention, for mixers that want more than a rotation there:
// an RMS norm over a token's whole query (key) projection, the rotation of the first numbers of every head by
// angles computed here in 32-bit (adjacent pairs or the two halves of the turned part), a temperature a query
// head, values that are the keys as projected, and heads kept in the cache at a padded size.
//
// qkv_finish: one workgroup a token.  Queries go out as [T, Hq, P], keys to k_cache [pages, Hkv, page, P], values
// to v_cache [pages, Hkv, P, page] (transposed within a page), zeros beyond dim / vdim.  Everything is computed in
// 32-bit from the sums and rounded once on the way out.
// head_gate:  o[t, h, :] *= sigmoid(gate[t, h]).
#include "common.hpp"

enum { LAYOUT_INTERLEAVED = 0, LAYOUT_HALF = 1 };

// element d of a head whose first 2 * nf numbers turn: the pair's angle index, the partner's place, and whether d
// is the pair's first member
__device__ __forceinline__ void pair_of(int d, int nf, int layout, int& i, int& partner, bool& first) {
  if (layout == LAYOUT_INTERLEAVED) {
    i = d >> 1;
    partner = d ^ 1;
    first = (d & 1) == 0;
  } else {
    first = d < nf;
    i = first ? d : d - nf;
    partner = first ? d + nf : d - nf;
  }
}

struct FinishArgs {
  const float* sums; long ld; int q_col, k_col, v_col;      // v_col < 0: the values are the keys as projected
  const float* q_norm; const float* k_norm; float eps;
  const float* inv_freq; int nf, layout;
  const float* q_head_scale;
  const int* positions; const int* slots;
  void* q_out; void* k_cache; void* v_cache;
  int Hq, Hkv, dim, vdim, P, page;
};

template <typename TO>
__global__ void __launch_bounds__(256)
qkv_finish_kernel(FinishArgs a) {
  __shared__ float scratch[16];
  // blockIdx.y: which share of the token's numbers this workgroup makes (every one takes the norms' sums itself)
  const int t = blockIdx.x, first = blockIdx.y * blockDim.x + threadIdx.x, stride = gridDim.y * blockDim.x;
  const float* __restrict__ row = a.sums + (size_t)t * a.ld;
  const float* __restrict__ q = row + a.q_col;
  const float* __restrict__ k = row + a.k_col;
  const int nq = a.Hq * a.dim, nk = a.Hkv * a.dim;
  float rq = 1.f, rk = 1.f;
  if (a.q_norm) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < nq; i += blockDim.x) ss = fmaf(q[i], q[i], ss);
    rq = 1.0f / sqrtf(block_sum(ss, scratch) / (float)nq + a.eps);
  }
  if (a.k_norm) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < nk; i += blockDim.x) ss = fmaf(k[i], k[i], ss);
    rk = 1.0f / sqrtf(block_sum(ss, scratch) / (float)nk + a.eps);
  }
  // the angles' cosines and sines once a token: every head turns by the same ones
  extern __shared__ float cs[];                 // cos [nf], sin [nf]
  const float pos = (float)a.positions[t];
  for (int i = threadIdx.x; i < a.nf; i += blockDim.x) sincosf(pos * a.inv_freq[i], &cs[a.nf + i], &cs[i]);
  __syncthreads();
  const int turned = 2 * a.nf;
  auto value = [&](const float* x, const float* w, float r, int h, int d) -> float {
    auto normed = [&](int e) { return w ? x[h * a.dim + e] * r * w[h * a.dim + e] : x[h * a.dim + e]; };
    const float own = normed(d);
    if (d >= turned) return own;
    int i, partner;
    bool first;
    pair_of(d, a.nf, a.layout, i, partner, first);
    const float other = normed(partner);
    const float c = cs[i], s = cs[a.nf + i];
    float o1, o2;
    if (first) {
      rotate_pair(own, other, c, s, o1, o2);
      return o1;
    }
    rotate_pair(other, own, c, s, o1, o2);
    return o2;
  };
  TO* __restrict__ qo = (TO*)a.q_out + (size_t)t * a.Hq * a.P;
  for (int e = first; e < a.Hq * a.P; e += stride) {
    const int h = e / a.P, d = e - h * a.P;
    float v = 0.f;
    if (d < a.dim) {
      v = value(q, a.q_norm, rq, h, d);
      if (a.q_head_scale) v *= a.q_head_scale[h];
    }
    qo[e] = from_float<TO>(v);
  }
  const int slot = a.slots[t];
  const size_t pg = slot / a.page, off = slot % a.page;
  TO* __restrict__ kc = (TO*)a.k_cache;
  TO* __restrict__ vc = (TO*)a.v_cache;
  const float* __restrict__ vals = a.v_col < 0 ? k : row + a.v_col;
  for (int e = first; e < a.Hkv * a.P; e += stride) {
    const int g = e / a.P, d = e - g * a.P;
    const float kv = d < a.dim ? value(k, a.k_norm, rk, g, d) : 0.f;
    kc[((pg * a.Hkv + g) * a.page + off) * a.P + d] = from_float<TO>(kv);
    const float vv = d < a.vdim ? vals[g * a.vdim + d] : 0.f;
    vc[((pg * a.Hkv + g) * a.P + d) * a.page + off] = from_float<TO>(vv);
  }
}

MIE_EXPORT const char* attention_prep_last_error() { return g_mie_error; }

MIE_EXPORT int mie_qkv_finish(const float* sums, long ld, int q_col, int k_col, int v_col, const float* q_norm,
                              const float* k_norm, float eps, const float* inv_freq, int nf, int layout,
                              const float* q_head_scale, const int* positions, const int* slots, void* q_out, void* k_cache,
                              void* v_cache, int dtype, int tokens, int Hq, int Hkv, int dim, int vdim, int P, int page,
                              hipStream_t s) {
  if (tokens <= 0) return 0;
  if (Hq <= 0 || Hkv <= 0 || dim <= 0 || vdim <= 0 || P < dim || P < vdim || page <= 0)
    MIE_FAIL("qkv_finish: %d / %d heads of %d (values %d) in %d, page %d", Hq, Hkv, dim, vdim, P, page);
  if (2 * nf > dim || nf < 0 || (nf > 0 && !inv_freq)) MIE_FAIL("qkv_finish: %d turned pairs in heads of %d", nf, dim);
  if (layout != LAYOUT_INTERLEAVED && layout != LAYOUT_HALF) MIE_FAIL("qkv_finish: layout code %d", layout);
  if (v_col < 0 && vdim != dim) MIE_FAIL("qkv_finish: values that are the keys have their size");
  FinishArgs a{sums, ld, q_col, k_col, v_col, q_norm, k_norm, eps, inv_freq, nf, layout, q_head_scale, positions, slots,
               q_out, k_cache, v_cache, Hq, Hkv, dim, vdim, P, page};
  const size_t lds = (size_t)2 * (nf > 0 ? nf : 1) * sizeof(float);
  // few tokens: several workgroups a token, so that a decode step's few rows are spread over the GPU
  const long numbers = (long)(Hq + Hkv) * P;
  int parts = tokens >= 256 ? 1 : (int)((numbers + 511) / 512);
  parts = parts < 1 ? 1 : parts > 8 ? 8 : parts;
  if (dtype == MIE_F32) hipLaunchKernelGGL(qkv_finish_kernel<float>, dim3(tokens, parts), dim3(256), lds, s, a);
  else if (dtype == MIE_BF16) hipLaunchKernelGGL(qkv_finish_kernel<bf16>, dim3(tokens, parts), dim3(256), lds, s, a);
  else MIE_FAIL("qkv_finish: dtype code %d", dtype);
  MIE_CHECK_LAUNCH("qkv_finish");
  return 0;
}

template <typename T>
__global__ void __launch_bounds__(256)
head_gate_kernel(T* __restrict__ o, const float* __restrict__ gate, long ldg, int H, int D) {
  const int t = blockIdx.x;
  T* row = o + (size_t)t * H * D;
  for (int e = threadIdx.x; e < H * D; e += blockDim.x)
    row[e] = from_float<T>(to_float(row[e]) * mie_sigmoid(gate[(size_t)t * ldg + e / D]));
}

// gate points at the first gate column; rows are ldg floats apart
MIE_EXPORT int mie_head_gate(void* o, int dtype, const float* gate, long ldg, int tokens, int H, int D, hipStream_t s) {
  if (tokens <= 0) return 0;
  if (H <= 0 || D <= 0 || ldg < H) MIE_FAIL("head_gate: %d heads of %d, gate rows %ld apart", H, D, ldg);
  if (dtype == MIE_F32) hipLaunchKernelGGL(head_gate_kernel<float>, dim3(tokens), dim3(256), 0, s, (float*)o, gate, ldg, H, D);
  else if (dtype == MIE_BF16) hipLaunchKernelGGL(head_gate_kernel<bf16>, dim3(tokens), dim3(256), 0, s, (bf16*)o, gate, ldg, H, D);
  else MIE_FAIL("head_gate: dtype code %d", dtype);
  MIE_CHECK_LAUNCH("head_gate");
  return 0;
}
