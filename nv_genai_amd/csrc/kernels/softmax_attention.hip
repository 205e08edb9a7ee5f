// Softmax attention with head maps over row-major pages, and the projection-side kernel that
// feeds it.
//
//   headnorm_cache     per token row [q: nq heads of dk | k: nk heads of dk | v: nv heads of dv]:
//                      bias, RMS norm of every q head and every k head over its dk elements
//                      (weight per element, shared by the heads), query temperature
//                      1 + coef * ln(floor((p + 1) / every) + 1), q / k / v written back in
//                      place, k and v into the token's page slot
//   softmax_attention  one wave per (token row, head), prompt portions and single-token rows
//                      alike: keys by lane for q.k, value columns by lane for w.V, running
//                      maximum and sum per map (fp32)
//
// Pages: K [blocks, G * maps, 64, dk], V [blocks, G, 64, dv] (T = bf16 or fp32). A head has
// `maps` score maps (1 or 2) that share its values: q head (h, m) is column block h * maps + m,
// its keys are k head (h / (H / G)) * maps + m. Two maps combine as a_0 - lam * a_1
// (differential attention). Optional: unit RMS of the head output (eps inside the root) times
// out_scale, and a per-head sigmoid gate. Visible keys of the query at position i: j <= i, and
// i - j < window when window > 0.
#include <cstdlib>

#include "common.h"
#include "kernels.h"

namespace nga {

namespace {

constexpr int BS = 64;   // tokens per page

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }

// q . k over dk elements, q in LDS (fp32), k a page row; 16-byte loads when vec
__device__ __forceinline__ float dot_row(const float* qs, const uint16_t* kr, int dk, bool vec) {
  float s = 0.f;
  if (vec) {
    for (int d = 0; d < dk; d += 8) {
      const u16x8 k8 = load8(kr + d);
#pragma unroll
      for (int j = 0; j < 8; ++j) s += qs[d + j] * bf2f(k8[j]);
    }
  } else {
    for (int d = 0; d < dk; ++d) s += qs[d] * bf2f(kr[d]);
  }
  return s;
}
__device__ __forceinline__ float dot_row(const float* qs, const float* kr, int dk, bool vec) {
  float s = 0.f;
  if (vec) {
    for (int d = 0; d < dk; d += 4) {
      const float4 k4 = *reinterpret_cast<const float4*>(kr + d);
      s += qs[d] * k4.x + qs[d + 1] * k4.y + qs[d + 2] * k4.z + qs[d + 3] * k4.w;
    }
  } else {
    for (int d = 0; d < dk; ++d) s += qs[d] * kr[d];
  }
  return s;
}

template <typename T>
__global__ void __launch_bounds__(256) headnorm_cache_kernel(
    T* __restrict__ proj, int64_t stride, const int32_t* __restrict__ slots, T* __restrict__ kc, T* __restrict__ vc,
    int nq, int nk, int dk, int nv, int dv, float eps, const float* __restrict__ qw, const float* __restrict__ kw,
    const float* __restrict__ bias, const int32_t* __restrict__ pos, float coef, int every) {
  const int64_t row = blockIdx.x;
  T* pr = proj + row * stride;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float temp = 1.0f;
  if (coef != 0.f && nq > 0) {
    const int p = pos[row] < 0 ? 0 : pos[row];
    temp = 1.0f + coef * logf((float)((p + 1) / every + 1));
  }
  const int slot = slots[row];
  const int64_t page = slot >= 0 ? slot / BS : 0;
  const int off = slot >= 0 ? slot % BS : 0;
  for (int u = wave; u < nq + nk; u += 4) {
    const bool isq = u < nq;
    const float* w = isq ? qw : kw;
    const int base = u * dk;
    float r = 1.0f;
    if (w) {
      float ss = 0.f;
      for (int c = lane; c < dk; c += 64) {
        const float v = ldf(pr + base + c) + (bias ? bias[base + c] : 0.f);
        ss += v * v;
      }
      ss = wave_sum(ss);
      r = 1.0f / sqrtf(ss / (float)dk + eps);
    }
    T* kdst = (!isq && slot >= 0) ? kc + ((page * nk + (u - nq)) * BS + off) * (int64_t)dk : nullptr;
    for (int c = lane; c < dk; c += 64) {
      float v = ldf(pr + base + c) + (bias ? bias[base + c] : 0.f);
      if (w) v = v * r * w[c];
      if (isq) v *= temp;
      stf(pr + base + c, v);
      if (kdst) stf(kdst + c, v);
    }
  }
  const int vb = (nq + nk) * dk;
  for (int c = threadIdx.x; c < nv * dv; c += blockDim.x) {
    const float v = ldf(pr + vb + c) + (bias ? bias[vb + c] : 0.f);
    stf(pr + vb + c, v);
    if (slot >= 0) {
      const int hh = c / dv, d = c - hh * dv;
      stf(vc + ((page * nv + hh) * BS + off) * (int64_t)dv + d, v);
    }
  }
}

// One wave per (token row, head). q: row stride q_stride, head (h, m) at (h * maps + m) * dk.
// gate: row stride g_stride, one pre-sigmoid value per head (nullptr: no gate). out [T, H * dv].
template <typename T>
__global__ void __launch_bounds__(64) softmax_attention_kernel(
    T* __restrict__ out, const T* __restrict__ q, int64_t q_stride, const T* __restrict__ gate, int64_t g_stride,
    const T* __restrict__ kc, const T* __restrict__ vc, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ pos, int H, int G, int dk, int dv, float scale,
    int window, int maps, float lam, float unit_eps, float out_scale) {
  extern __shared__ float smem[];
  float* qs = smem;                 // [maps * dk]
  float* ws = smem + maps * dk;     // [64]
  const int64_t row = blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x;
  const int i = pos[row];
  T* orow = out + row * (int64_t)H * dv + (int64_t)h * dv;
  if (i < 0) {   // padding row
    for (int d = lane; d < dv; d += 64) stf(orow + d, 0.f);
    return;
  }
  const int seq = tok_seq[row];
  const int g = h / (H / G);
  const int32_t* bt = block_tables + (int64_t)seq * max_blocks;
  for (int d = lane; d < maps * dk; d += 64) qs[d] = ldf(q + row * q_stride + (int64_t)h * maps * dk + d);
  constexpr int MAXV = 8;   // dv <= 512
  float res[MAXV] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, acc[MAXV];
  const int lo = window > 0 && i - window + 1 > 0 ? i - window + 1 : 0;
  const int p_lo = lo / BS, p_hi = i / BS;
  const bool vec = (dk % (16 / (int)sizeof(T))) == 0;
  __syncthreads();
  for (int m = 0; m < maps; ++m) {
    const int kh = g * maps + m;
    float mx = -INFINITY, l = 0.f;
#pragma unroll
    for (int u = 0; u < MAXV; ++u) acc[u] = 0.f;
    for (int p = p_lo; p <= p_hi; ++p) {
      const int j = p * BS + lane;
      const bool vis = j >= lo && j <= i;
      const int64_t page = bt[p];
      float s = -INFINITY;
      if (vis) s = dot_row(qs + m * dk, kc + ((page * G * maps + kh) * BS + lane) * (int64_t)dk, dk, vec) * scale;
      const float nmx = fmaxf(mx, wave_max(s));   // every visited page holds a visible key
      const float corr = expf(mx - nmx);          // 0 on the first page (mx = -inf)
      const float w = vis ? expf(s - nmx) : 0.f;
      l = l * corr + wave_sum(w);
      mx = nmx;
      ws[lane] = w;
      __syncthreads();
      const unsigned long long any = __ballot(vis);
      const int j0 = __builtin_ctzll(any), j1 = 63 - __builtin_clzll(any);
      const T* vp = vc + ((page * G + g) * BS) * (int64_t)dv;
#pragma unroll
      for (int u = 0; u < MAXV; ++u) {
        const int d = lane + u * 64;
        if (d < dv) {
          float a = acc[u] * corr;
          for (int jj = j0; jj <= j1; ++jj) a += ws[jj] * ldf(vp + (int64_t)jj * dv + d);
          acc[u] = a;
        }
      }
      __syncthreads();
    }
    const float inv = 1.0f / l;
#pragma unroll
    for (int u = 0; u < MAXV; ++u) res[u] = m == 0 ? acc[u] * inv : res[u] - lam * (acc[u] * inv);
  }
  float r = 1.0f;
  if (unit_eps >= 0.f) {
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < MAXV; ++u)
      if (lane + u * 64 < dv) ss += res[u] * res[u];
    ss = wave_sum(ss);
    r = out_scale / sqrtf(ss / (float)dv + unit_eps);
  }
  if (gate) r *= sigmoidf_(ldf(gate + row * g_stride + h));
#pragma unroll
  for (int u = 0; u < MAXV; ++u) {
    const int d = lane + u * 64;
    if (d < dv) stf(orow + d, res[u] * r);
  }
}

}  // namespace

void launch_headnorm_cache(void* proj, int64_t stride, const int32_t* slots, void* kc, void* vc, int64_t T, int nq,
                           int nk, int dk, int nv, int dv, float eps, const float* qw, const float* kw,
                           const float* bias, const int32_t* pos, float coef, int every, bool f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32)
    headnorm_cache_kernel<float><<<dim3((unsigned)T), 256, 0, stream>>>((float*)proj, stride, slots, (float*)kc,
                                                                       (float*)vc, nq, nk, dk, nv, dv, eps, qw, kw,
                                                                       bias, pos, coef, every);
  else
    headnorm_cache_kernel<uint16_t><<<dim3((unsigned)T), 256, 0, stream>>>((uint16_t*)proj, stride, slots,
                                                                          (uint16_t*)kc, (uint16_t*)vc, nq, nk, dk, nv,
                                                                          dv, eps, qw, kw, bias, pos, coef, every);
}

void launch_softmax_attention(void* out, const void* q, int64_t q_stride, const void* gate, int64_t g_stride,
                              const void* kc, const void* vc, const int32_t* block_tables, int max_blocks,
                              const int32_t* tok_seq, const int32_t* pos, int64_t T, int H, int G, int dk, int dv,
                              float scale, int window, int maps, float lam, float unit_eps, float out_scale, bool f32,
                              hipStream_t stream) {
  if (T == 0) return;
  const dim3 grid((unsigned)T, (unsigned)H);
  const size_t smem = (size_t)(maps * dk + 64) * sizeof(float);
  if (f32)
    softmax_attention_kernel<float><<<grid, 64, smem, stream>>>(
        (float*)out, (const float*)q, q_stride, (const float*)gate, g_stride, (const float*)kc, (const float*)vc,
        block_tables, max_blocks, tok_seq, pos, H, G, dk, dv, scale, window, maps, lam, unit_eps, out_scale);
  else
    softmax_attention_kernel<uint16_t><<<grid, 64, smem, stream>>>(
        (uint16_t*)out, (const uint16_t*)q, q_stride, (const uint16_t*)gate, g_stride, (const uint16_t*)kc,
        (const uint16_t*)vc, block_tables, max_blocks, tok_seq, pos, H, G, dk, dv, scale, window, maps, lam, unit_eps,
        out_scale);
}

}  // namespace nga
