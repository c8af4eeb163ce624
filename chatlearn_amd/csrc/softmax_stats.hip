// Softmax statistics (logprob, entropy, lse) from materialised logits and the
// matching d(logits), for call sites that already hold [R, V] logits.
// One 256-thread block per row; the row is streamed once for the statistics
// (online max / sum / weighted sum, fp32) and, in the backward, once more to
// write d(logits).  HBM-bound: V*sizeof(dtype) bytes per row read (+ written).
#include "common.hpp"

namespace clgrpo {

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<__bf16>(__bf16 v) { return (float)v; }

struct RowStats { float m, s, u; };

__device__ __forceinline__ void rs_merge(RowStats& a, const RowStats& b) {
  const float nm = fmaxf(a.m, b.m);
  const float fa = (a.m == nm) ? 1.f : expf(a.m - nm);
  const float fb = (b.m == nm) ? 1.f : expf(b.m - nm);
  a.s = a.s * fa + b.s * fb;
  a.u = a.u * fa + b.u * fb;
  a.m = nm;
}

template <typename T>
__device__ RowStats row_stats(const T* row, int64_t V) {
  RowStats st{-INFINITY, 0.f, 0.f};
  for (int64_t v = threadIdx.x; v < V; v += 256) {
    const float z = to_f32<T>(row[v]);
    if (z > st.m) {
      const float f = expf(st.m - z);   // st.m = -inf -> 0
      st.s = st.s * f + 1.f;
      st.u = st.u * f + z;
      st.m = z;
    } else {
      const float e = expf(z - st.m);
      st.s += e;
      st.u = fmaf(e, z, st.u);
    }
  }
  for (int off = 32; off > 0; off >>= 1) {
    RowStats o{__shfl_xor(st.m, off), __shfl_xor(st.s, off), __shfl_xor(st.u, off)};
    rs_merge(st, o);
  }
  __shared__ RowStats sh[4];
  if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = st;
  __syncthreads();
  RowStats t = sh[0];
  rs_merge(t, sh[1]);
  rs_merge(t, sh[2]);
  rs_merge(t, sh[3]);
  __syncthreads();
  return t;
}

template <typename T>
__global__ __launch_bounds__(256) void softmax_stats_kernel(clgrpo_softmax_stats_args a) {
  const int64_t r = blockIdx.x;
  const T* row = static_cast<const T*>(a.logits) + r * a.ld;
  const RowStats st = row_stats<T>(row, a.V);
  if (threadIdx.x == 0) {
    const float lse = st.m + logf(st.s);
    if (a.lse) a.lse[r] = lse;
    if (a.entropy) a.entropy[r] = lse - st.u / st.s;
    if (a.logprob) {
      const int64_t y = a.labels[r];
      a.logprob[r] = (y >= 0 && y < a.V) ? to_f32<T>(row[y]) - lse : NAN;
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void softmax_stats_bwd_kernel(clgrpo_softmax_stats_bwd_args a) {
  const int64_t r = blockIdx.x;
  const T* row = static_cast<const T*>(a.logits) + r * a.ld;
  T* out = static_cast<T*>(a.dlogits) + r * a.V;
  const RowStats st = row_stats<T>(row, a.V);
  const float lse = st.m + logf(st.s);
  const float ent = lse - st.u / st.s;
  const float glp = a.g_logprob ? a.g_logprob[r] : 0.f;
  const float gen = a.g_entropy ? a.g_entropy[r] : 0.f;
  const int64_t y = a.g_logprob ? a.labels[r] : -1;
  for (int64_t v = threadIdx.x; v < a.V; v += 256) {
    const float z = to_f32<T>(row[v]);
    const float logp = z - lse;
    const float p = expf(logp);
    float d = -p * (glp + gen * (logp + ent));
    if (v == y) d += glp;
    out[v] = (T)d;
  }
}

}  // namespace clgrpo

using namespace clgrpo;

extern "C" int clgrpo_softmax_stats(const clgrpo_softmax_stats_args* a, void* stream) {
  CLGRPO_REQUIRE_PTR(a, "args");
  if (a->dtype != CLGRPO_BF16 && a->dtype != CLGRPO_F32) return fail(CLGRPO_EDTYPE, "clgrpo_softmax_stats: dtype %d", a->dtype);
  if (a->R < 0 || a->V <= 0 || a->ld < a->V) return fail(CLGRPO_EINVAL, "clgrpo_softmax_stats: R=%lld V=%lld ld=%lld",
                                                         (long long)a->R, (long long)a->V, (long long)a->ld);
  if (a->R == 0) return CLGRPO_OK;
  CLGRPO_REQUIRE_PTR(a->logits, "logits");
  if (a->logprob) CLGRPO_REQUIRE_PTR(a->labels, "labels");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (a->dtype == CLGRPO_BF16) hipLaunchKernelGGL(softmax_stats_kernel<__bf16>, dim3((unsigned)a->R), dim3(256), 0, s, *a);
  else hipLaunchKernelGGL(softmax_stats_kernel<float>, dim3((unsigned)a->R), dim3(256), 0, s, *a);
  return check_launch("softmax_stats_kernel");
}

extern "C" int clgrpo_softmax_stats_bwd(const clgrpo_softmax_stats_bwd_args* a, void* stream) {
  CLGRPO_REQUIRE_PTR(a, "args");
  if (a->dtype != CLGRPO_BF16 && a->dtype != CLGRPO_F32) return fail(CLGRPO_EDTYPE, "clgrpo_softmax_stats_bwd: dtype %d", a->dtype);
  if (a->R < 0 || a->V <= 0 || a->ld < a->V) return fail(CLGRPO_EINVAL, "clgrpo_softmax_stats_bwd: bad sizes");
  if (a->R == 0) return CLGRPO_OK;
  CLGRPO_REQUIRE_PTR(a->logits, "logits");
  CLGRPO_REQUIRE_PTR(a->dlogits, "dlogits");
  if (a->g_logprob) CLGRPO_REQUIRE_PTR(a->labels, "labels");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (a->dtype == CLGRPO_BF16) hipLaunchKernelGGL(softmax_stats_bwd_kernel<__bf16>, dim3((unsigned)a->R), dim3(256), 0, s, *a);
  else hipLaunchKernelGGL(softmax_stats_bwd_kernel<float>, dim3((unsigned)a->R), dim3(256), 0, s, *a);
  return check_launch("softmax_stats_bwd_kernel");
}
