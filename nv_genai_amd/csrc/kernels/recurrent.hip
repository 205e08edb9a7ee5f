// Gated linear recurrences with a matrix state per head, carried across steps in state slots.
//
//   hgrn2_scan   per head S <- diag(f) S + (1 - f) v^T, o = S^T q over the rows of a segment
//                (a prompt portion, or a single decode row), with q = silu(q_pre) and
//                f = lower + (1 - lower) * sigmoid(f_pre + f_bias) formed in fp32 in the kernel.
//
// A workgroup owns (segment, head, tile of VT value columns): thread (rg, j) keeps the state
// elements S[rg + RG * k][j] in registers for the whole segment, so the state is read from its
// slot once and written back once. Rows are staged through LDS TC at a time (activations
// applied while staging); per row every thread updates its NR state elements and adds its part of
// o, the RG parts are summed through LDS for all TC rows at once. State, gates and sums are fp32
// whatever the activation type.
#include "common.h"
#include "kernels.h"

namespace nga {

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }

constexpr int TC = 8;   // rows staged per pass

// proj row: [q_pre (H*d) | f_pre (H*d) | v (H*dv) | ...]. cu == nullptr: segment b is row b.
template <typename T, int NR>
__global__ void __launch_bounds__(256) hgrn2_scan_kernel(float* __restrict__ out, const T* __restrict__ proj,
                                                         int64_t stride, const float* __restrict__ f_bias,
                                                         const float* __restrict__ lower, float* __restrict__ state,
                                                         int H, int d, int dv, const int32_t* __restrict__ cu,
                                                         const int32_t* __restrict__ slots,
                                                         const int32_t* __restrict__ pos, int VT) {
  extern __shared__ float smem[];
  const int RG = 256 / VT;
  float* qs = smem;                  // [TC][d]
  float* fs = qs + TC * d;           // [TC][d]
  float* vs = fs + TC * d;           // [TC][VT]
  float* part = vs + TC * VT;        // [TC][RG][VT] = [TC][256]
  const int vt = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int t0 = cu ? cu[b] : b, t1 = cu ? cu[b + 1] : b + 1;
  if (t1 <= t0) return;
  const int slot = slots[b];
  const bool fresh = slot < 0 || pos[t0] == 0;
  const int tid = threadIdx.x;
  const int j = tid % VT, rg = tid / VT;
  const int col = vt * VT + j;
  const bool colok = col < dv;
  float* sp = slot >= 0 ? state + ((int64_t)slot * H + h) * (int64_t)d * dv : nullptr;
  float S[NR];
#pragma unroll
  for (int k = 0; k < NR; ++k) {
    const int i = rg + RG * k;
    S[k] = (!fresh && colok && i < d) ? sp[(int64_t)i * dv + col] : 0.f;
  }
  const int qoff = h * d, foff = H * d + h * d, voff = 2 * H * d + h * dv + vt * VT;
  for (int tc = t0; tc < t1; tc += TC) {
    const int nt = t1 - tc < TC ? t1 - tc : TC;
    for (int e = tid; e < nt * d; e += 256) {
      const int tt = e / d, i = e - tt * d;
      const T* pr = proj + (int64_t)(tc + tt) * stride;
      const float qv = ldf(pr + qoff + i);
      qs[e] = qv / (1.0f + expf(-qv));
      const float lw = lower[qoff + i];
      const float fv = ldf(pr + foff + i) + f_bias[qoff + i];
      fs[e] = lw + (1.0f - lw) * (1.0f / (1.0f + expf(-fv)));
    }
    for (int e = tid; e < nt * VT; e += 256) {
      const int tt = e / VT, jj = e - tt * VT;
      vs[e] = vt * VT + jj < dv ? ldf(proj + (int64_t)(tc + tt) * stride + voff + jj) : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float vv = vs[tt * VT + j];
      const float* fr = fs + tt * d;
      const float* qr = qs + tt * d;
      float p = 0.f;
#pragma unroll
      for (int k = 0; k < NR; ++k) {
        const int i = rg + RG * k;
        if (i < d) {
          const float f = fr[i];
          S[k] = f * S[k] + (1.0f - f) * vv;
          p += S[k] * qr[i];
        }
      }
      part[tt * 256 + tid] = p;
    }
    __syncthreads();
    for (int e = tid; e < nt * VT; e += 256) {
      const int tt = e / VT, jj = e - tt * VT;
      if (vt * VT + jj < dv) {
        float s = 0.f;
        for (int r = 0; r < RG; ++r) s += part[tt * 256 + r * VT + jj];
        out[(int64_t)(tc + tt) * H * dv + h * dv + vt * VT + jj] = s;
      }
    }
    __syncthreads();
  }
  if (sp && colok) {
#pragma unroll
    for (int k = 0; k < NR; ++k) {
      const int i = rg + RG * k;
      if (i < d) sp[(int64_t)i * dv + col] = S[k];
    }
  }
}

template <typename T>
bool launch_hgrn2_t(float* out, const T* proj, int64_t stride, const float* f_bias, const float* lower, float* state,
                    int H, int d, int dv, const int32_t* cu, const int32_t* slots, const int32_t* pos, int n_seg,
                    hipStream_t stream) {
  const int VT = dv >= 64 ? 64 : (dv >= 32 ? 32 : 16);
  const int RG = 256 / VT;
  const int nr = (d + RG - 1) / RG;
  const dim3 grid((unsigned)((dv + VT - 1) / VT), (unsigned)H, (unsigned)n_seg);
  const size_t smem = (size_t)TC * (2 * d + VT + 256) * sizeof(float);
#define NGA_HGRN2_CASE(N)                                                                                             \
  if (nr <= N) {                                                                                                      \
    hgrn2_scan_kernel<T, N><<<grid, 256, smem, stream>>>(out, proj, stride, f_bias, lower, state, H, d, dv, cu, slots, \
                                                         pos, VT);                                                    \
    return true;                                                                                                      \
  }
  NGA_HGRN2_CASE(2)
  NGA_HGRN2_CASE(4)
  NGA_HGRN2_CASE(8)
  NGA_HGRN2_CASE(16)
  NGA_HGRN2_CASE(32)
  NGA_HGRN2_CASE(64)
#undef NGA_HGRN2_CASE
  return false;
}

}  // namespace

int hgrn2_max_dim(int dv) { return 64 * (256 / (dv >= 64 ? 64 : (dv >= 32 ? 32 : 16))); }

bool launch_hgrn2_scan(float* out, const void* proj, int64_t stride, const float* f_bias, const float* lower,
                       float* state, int H, int d, int dv, const int32_t* cu, const int32_t* slots, const int32_t* pos,
                       int n_seg, bool f32, hipStream_t stream) {
  if (n_seg == 0) return true;
  if (f32)
    return launch_hgrn2_t<float>(out, (const float*)proj, stride, f_bias, lower, state, H, d, dv, cu, slots, pos, n_seg,
                                 stream);
  return launch_hgrn2_t<uint16_t>(out, (const uint16_t*)proj, stride, f_bias, lower, state, H, d, dv, cu, slots, pos,
                                  n_seg, stream);
}

}  // namespace nga
