// Gated sigmoid attention over a paged KV cache: un-normalised attention whose weight of a
// visible key is sigmoid(q.k * scale - r1 * ln(1 + r2 * (i - j)) + pb) (r1, r2, pb per query
// head), with a sliding window that also keeps the first tokens of the sequence:
//
//     j visible to i  <=>  j <= i  and  (i - j < window  or  j < keep_first)
//
// and an output gate sigmoid(g) on the concatenated heads. No softmax: no running maximum and
// no normaliser, so key tiles simply accumulate and split sequences need no rescaling.
//
//   qk_norm_cache      per token: RMS-normalise the whole q projection and the whole k
//                      projection (one statistic over all heads, weight per element), write q
//                      back in place and k / v into the token's page slot
//   sigmoid_attention  one wave per (token row, query head), prompt portions and decode rows
//                      alike: keys by lane for q.k, value columns by lane for w.V
//   sigmoid_attention_mfma (bf16)  one workgroup per (64-row block of a sequence, query head):
//                      MFMA q.k and w.V tiles over the pages the block can see
//
// Pages: K [blocks, Hkv, 64, dk], V^T [blocks, Hkv, dv, 64] (T = bf16 or fp32). Scores, the
// distance term, the sigmoid and the accumulation are fp32 in every form.
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

// proj row: [q (Hq*dk) | k (Hkv*dk) | v (Hkv*dv) | ...]; slot < 0: no cache write
template <typename T>
__global__ void __launch_bounds__(256) qk_norm_cache_kernel(T* __restrict__ proj, int64_t stride,
                                                            const float* __restrict__ qw, const float* __restrict__ kw,
                                                            float eps, const int32_t* __restrict__ slots,
                                                            T* __restrict__ kc, T* __restrict__ vc, int Hq, int Hkv,
                                                            int dk, int dv) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  T* pr = proj + row * stride;
  const int nq = Hq * dk, nk = Hkv * dk, nv = Hkv * dv;
  float sq = 0.f, sk = 0.f;
  for (int c = threadIdx.x; c < nq; c += blockDim.x) {
    const float v = ldf(pr + c);
    sq += v * v;
  }
  for (int c = threadIdx.x; c < nk; c += blockDim.x) {
    const float v = ldf(pr + nq + c);
    sk += v * v;
  }
  sq = block_sum(sq, red);
  sk = block_sum(sk, red);
  const float rq = 1.0f / sqrtf(sq / (float)nq + eps);
  const float rk = 1.0f / sqrtf(sk / (float)nk + eps);
  for (int c = threadIdx.x; c < nq; c += blockDim.x) stf(pr + c, ldf(pr + c) * rq * qw[c]);
  const int slot = slots[row];
  if (slot < 0) return;
  const int64_t page = slot / BS;
  const int off = slot % BS;
  for (int c = threadIdx.x; c < nk; c += blockDim.x) {
    const int hh = c / dk, d = c - hh * dk;
    stf(kc + ((page * Hkv + hh) * BS + off) * dk + d, ldf(pr + nq + c) * rk * kw[c]);
  }
  for (int c = threadIdx.x; c < nv; c += blockDim.x) {
    const int hh = c / dv, d = c - hh * dv;
    vc[((page * Hkv + hh) * dv + d) * BS + off] = pr[nq + nk + c];
  }
}

// One wave per (token row, head). q: row stride q_stride, head h at h*dk. gate: row stride
// g_stride, head h at h*dv (nullptr: no gate). out [T, Hq*dv].
template <typename T>
__global__ void __launch_bounds__(64) sigmoid_attention_kernel(
    T* __restrict__ out, const T* __restrict__ q, int64_t q_stride, const T* __restrict__ gate, int64_t g_stride,
    const T* __restrict__ kc, const T* __restrict__ vc, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ pos, int Hq, int Hkv, int dk, int dv,
    float scale, int window, int keep_first, const float* __restrict__ r1, const float* __restrict__ r2,
    const float* __restrict__ pb) {
  extern __shared__ float smem[];
  float* qs = smem;            // [dk]
  float* ws = smem + dk;       // [64]
  const int64_t row = blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x;
  const int i = pos[row];
  T* orow = out + row * (int64_t)Hq * dv + (int64_t)h * dv;
  if (i < 0) {   // padding row
    for (int d = lane; d < dv; d += 64) stf(orow + d, 0.f);
    return;
  }
  const int seq = tok_seq[row];
  const int kvh = h / (Hq / Hkv);
  const int32_t* bt = block_tables + (int64_t)seq * max_blocks;
  for (int d = lane; d < dk; d += 64) qs[d] = ldf(q + row * q_stride + (int64_t)h * dk + d);
  const float a1 = r1[h], a2 = r2[h], b = pb[h];
  constexpr int MAXV = 4;   // dv <= 256
  float acc[MAXV] = {0.f, 0.f, 0.f, 0.f};
  const int lo = i - window + 1 > 0 ? i - window + 1 : 0;   // first key inside the window
  const int keep = keep_first < lo ? keep_first : lo;        // kept keys [0, keep) below the window
  const int p_keep_end = (keep + BS - 1) / BS;               // pages [0, p_keep_end) hold kept keys
  const int p_lo = lo / BS, p_hi = i / BS;
  __syncthreads();
  for (int p = 0; p <= p_hi; ++p) {
    if (p >= p_keep_end && p < p_lo) {
      p = p_lo - 1;
      continue;
    }
    const int j = p * BS + lane;
    const bool vis = j <= i && (j >= lo || j < keep_first);
    const int64_t page = bt[p];
    float w = 0.f;
    if (vis) {
      const T* kr = kc + ((page * Hkv + kvh) * BS + lane) * dk;
      float s = 0.f;
      for (int d = 0; d < dk; ++d) s += qs[d] * ldf(kr + d);
      s = s * scale - a1 * log1pf(a2 * (float)(i - j));
      w = sigmoidf_(s + b);
    }
    const unsigned long long any = __ballot(vis);
    ws[lane] = w;
    __syncthreads();
    if (any) {
      const int j0 = __builtin_ctzll(any), j1 = 63 - __builtin_clzll(any);
#pragma unroll
      for (int u = 0; u < MAXV; ++u) {
        const int d = lane + u * 64;
        if (d < dv) {
          const T* vr = vc + ((page * Hkv + kvh) * dv + d) * BS;
          float a = acc[u];
          for (int jj = j0; jj <= j1; ++jj) a += ws[jj] * ldf(vr + jj);
          acc[u] = a;
        }
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int u = 0; u < MAXV; ++u) {
    const int d = lane + u * 64;
    if (d < dv) {
      float o = acc[u];
      if (gate) o *= sigmoidf_(ldf(gate + row * g_stride + (int64_t)h * dv + d));
      stf(orow + d, o);
    }
  }
}

}  // namespace

void launch_qk_norm_cache(void* proj, int64_t stride, const float* qw, const float* kw, float eps,
                          const int32_t* slots, void* kc, void* vc, int64_t T, int Hq, int Hkv, int dk, int dv,
                          bool f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32)
    qk_norm_cache_kernel<float><<<dim3((unsigned)T), 256, 0, stream>>>((float*)proj, stride, qw, kw, eps, slots,
                                                                      (float*)kc, (float*)vc, Hq, Hkv, dk, dv);
  else
    qk_norm_cache_kernel<uint16_t><<<dim3((unsigned)T), 256, 0, stream>>>((uint16_t*)proj, stride, qw, kw, eps, slots,
                                                                         (uint16_t*)kc, (uint16_t*)vc, Hq, Hkv, dk,
                                                                         dv);
}

void launch_sigmoid_attention(void* out, const void* q, int64_t q_stride, const void* gate, int64_t g_stride,
                              const void* kc, const void* vc, const int32_t* block_tables, int max_blocks,
                              const int32_t* tok_seq, const int32_t* pos, int64_t T, int Hq, int Hkv, int dk, int dv,
                              float scale, int window, int keep_first, const float* r1, const float* r2,
                              const float* pb, bool f32, hipStream_t stream) {
  if (T == 0) return;
  const dim3 grid((unsigned)T, (unsigned)Hq);
  const size_t lds = (size_t)(dk + 64) * sizeof(float);
  if (f32)
    sigmoid_attention_kernel<float><<<grid, 64, lds, stream>>>(
        (float*)out, (const float*)q, q_stride, (const float*)gate, g_stride, (const float*)kc, (const float*)vc,
        block_tables, max_blocks, tok_seq, pos, Hq, Hkv, dk, dv, scale, window, keep_first, r1, r2, pb);
  else
    sigmoid_attention_kernel<uint16_t><<<grid, 64, lds, stream>>>(
        (uint16_t*)out, (const uint16_t*)q, q_stride, (const uint16_t*)gate, g_stride, (const uint16_t*)kc,
        (const uint16_t*)vc, block_tables, max_blocks, tok_seq, pos, Hq, Hkv, dk, dv, scale, window, keep_first, r1,
        r2, pb);
}

}  // namespace nga
