// Softmax statistics (logprob, entropy, lse) from materialised logits and the
// matching d(logits), for call sites that already hold [R, V] logits.
// One 256-thread block per row, 16 bytes per lane and four loads in flight per thread; the row is
// streamed once for the statistics (online max / sum / weighted sum, fp32).  The backward reads
// it once more and writes d(logits), taking lse / entropy from the forward when the caller kept
// them.  HBM-bound: V*sizeof(dtype) bytes per row read (+ the same written).
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

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// 16 bytes of a row as floats.
template <typename T> struct Vec16 {
  static constexpr int N = 16 / (int)sizeof(T);
  __device__ static __forceinline__ void unpack(const u32x4_t& raw, float (&z)[N]) {
    const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
    for (int k = 0; k < N; ++k) z[k] = to_f32<T>(e[k]);
  }
  __device__ static __forceinline__ u32x4_t pack(const float (&d)[N]) {
    alignas(16) T e[N];
#pragma unroll
    for (int k = 0; k < N; ++k) e[k] = (T)d[k];
    return *reinterpret_cast<const u32x4_t*>(e);
  }
};

// Online (max, sum e^{z-max}, sum e^{z-max} z) update with N new values: one rescale, then N exponentials
// against a fixed maximum (no per-element branch).
template <int N>
__device__ __forceinline__ void rs_update(RowStats& st, const float (&z)[N]) {
  float vmax = z[0];
#pragma unroll
  for (int k = 1; k < N; ++k) vmax = fmaxf(vmax, z[k]);
  constexpr float kLog2e = 1.4426950408889634f;
  if (vmax > st.m) {
    const float f = __builtin_amdgcn_exp2f((st.m - vmax) * kLog2e);   // st.m = -inf -> 0
    st.s *= f;
    st.u *= f;
    st.m = vmax;
  }
  const float nb = (st.m == -INFINITY) ? 0.f : -st.m * kLog2e;   // only -inf so far (masked entries): every term is 0
#pragma unroll
  for (int k = 0; k < N; ++k) {
    const float e = __builtin_amdgcn_exp2f(fmaf(z[k], kLog2e, nb));   // one hardware exp2 per element
    st.s += e;
    st.u = fmaf(e, z[k], st.u);
  }
}

// Rows whose start and length are multiples of 16 bytes are streamed 16 bytes per lane, four
// independent loads in flight per thread; other rows element by element.
template <typename T>
__device__ __forceinline__ bool rows_vectorizable(const void* base, int64_t ld, int64_t V) {
  constexpr int N = Vec16<T>::N;
  return (reinterpret_cast<uintptr_t>(base) % 16 == 0) && (ld % N == 0) && (V % N == 0);
}

template <typename T>
__device__ RowStats row_stats(const T* row, int64_t V, bool vec) {
  constexpr int N = Vec16<T>::N;
  RowStats st{-INFINITY, 0.f, 0.f};
  if (vec) {
    const u32x4_t* rv = reinterpret_cast<const u32x4_t*>(row);
    const int64_t nvec = V / N;
    int64_t i = threadIdx.x;
    // two independent running states per thread (merged below): the update is a dependent chain
    RowStats st2{-INFINITY, 0.f, 0.f};
    for (; i + 3 * 256 < nvec; i += 4 * 256) {
      const u32x4_t r0 = rv[i], r1 = rv[i + 256], r2 = rv[i + 512], r3 = rv[i + 768];
      float z[N], y[N];
      Vec16<T>::unpack(r0, z); Vec16<T>::unpack(r1, y);
      rs_update<N>(st, z); rs_update<N>(st2, y);
      Vec16<T>::unpack(r2, z); Vec16<T>::unpack(r3, y);
      rs_update<N>(st, z); rs_update<N>(st2, y);
    }
    rs_merge(st, st2);
    for (; i < nvec; i += 256) {
      float z[N];
      Vec16<T>::unpack(rv[i], z);
      rs_update<N>(st, z);
    }
  } else {
    for (int64_t v = threadIdx.x; v < V; v += 256) {
      const float z[1] = {to_f32<T>(row[v])};
      rs_update<1>(st, z);
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
  const RowStats st = row_stats<T>(row, a.V, rows_vectorizable<T>(a.logits, a.ld, a.V));
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

// d(logits) of one row: with the row's lse (and entropy, when it carries a gradient) from the forward the
// row is read once and written once; without them the statistics are rebuilt by one more pass over it.
template <typename T>
__global__ __launch_bounds__(256) void softmax_stats_bwd_kernel(clgrpo_softmax_stats_bwd_args a) {
  constexpr int N = Vec16<T>::N;
  const int64_t r = blockIdx.x;
  const T* row = static_cast<const T*>(a.logits) + r * a.ld;
  T* out = static_cast<T*>(a.dlogits) + r * a.V;
  const bool vec = rows_vectorizable<T>(a.logits, a.ld, a.V) && (reinterpret_cast<uintptr_t>(a.dlogits) % 16 == 0);
  float lse, ent;
  if (a.lse != nullptr && (a.g_entropy == nullptr || a.entropy != nullptr)) {
    lse = a.lse[r];
    ent = a.g_entropy ? a.entropy[r] : 0.f;
  } else {
    const RowStats st = row_stats<T>(row, a.V, vec);
    lse = st.m + logf(st.s);
    ent = lse - st.u / st.s;
  }
  const float glp = a.g_logprob ? a.g_logprob[r] : 0.f;
  const float gen = a.g_entropy ? a.g_entropy[r] : 0.f;
  const int64_t y = a.g_logprob ? a.labels[r] : -1;
  auto dz = [&](float z, int64_t v) {
    const float logp = z - lse;
    const float p = __builtin_amdgcn_exp2f(logp * 1.4426950408889634f);
    float d = -p * (glp + gen * (logp + ent));
    if (v == y) d += glp;
    return d;
  };
  if (vec) {
    const u32x4_t* rv = reinterpret_cast<const u32x4_t*>(row);
    u32x4_t* ov = reinterpret_cast<u32x4_t*>(out);
    const int64_t nvec = a.V / N;
    auto one = [&](const u32x4_t& raw, int64_t i) {
      float z[N], d[N];
      Vec16<T>::unpack(raw, z);
#pragma unroll
      for (int k = 0; k < N; ++k) d[k] = dz(z[k], i * N + k);
      ov[i] = Vec16<T>::pack(d);
    };
    int64_t i = threadIdx.x;
    for (; i + 3 * 256 < nvec; i += 4 * 256) {
      const u32x4_t r0 = rv[i], r1 = rv[i + 256], r2 = rv[i + 512], r3 = rv[i + 768];
      one(r0, i); one(r1, i + 256); one(r2, i + 512); one(r3, i + 768);
    }
    for (; i < nvec; i += 256) one(rv[i], i);
  } else {
    for (int64_t v = threadIdx.x; v < a.V; v += 256) out[v] = (T)dz(to_f32<T>(row[v]), v);
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
