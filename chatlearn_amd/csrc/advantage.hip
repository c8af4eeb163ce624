// Group-wise reward -> advantage normalisation in float64.
//
// One thread per sample walks the pooled rewards of the sample's group (a group
// is the 8-32 responses of one prompt, so the pool sits in L2).  Sums follow
// numpy's pairwise scheme for blocks of up to 128 values (eight running sums,
// then a fixed tree), and this file is compiled with -ffp-contract=off so no add is fused with
// a multiply; the result is numpy.mean / numpy.std bit for
// bit for pools of at most 128 rewards and differs only by summation order above.
#include "common.hpp"

namespace clgrpo {

template <bool SQ>
__device__ double np_block_sum(const double* x, int n, double mean) {
  // value(i) = SQ ? (x[i]-mean)^2 : x[i]
  auto val = [&](int i) -> double {
    if (!SQ) return x[i];
    const double d = __dsub_rn(x[i], mean);
    return __dmul_rn(d, d);
  };
  if (n < 8) {
    double r = 0.0;
    for (int i = 0; i < n; ++i) r = __dadd_rn(r, val(i));
    return r;
  }
  double acc[8];
  for (int j = 0; j < 8; ++j) acc[j] = val(j);
  int i = 8;
  for (; i + 8 <= n; i += 8)
    for (int j = 0; j < 8; ++j) acc[j] = __dadd_rn(acc[j], val(i + j));
  double r = __dadd_rn(__dadd_rn(__dadd_rn(acc[0], acc[1]), __dadd_rn(acc[2], acc[3])),
                       __dadd_rn(__dadd_rn(acc[4], acc[5]), __dadd_rn(acc[6], acc[7])));
  for (; i < n; ++i) r = __dadd_rn(r, val(i));
  return r;
}

template <bool SQ>
__device__ double np_pairwise_sum(const double* x, int n, double mean) {
  if (n <= 128) return np_block_sum<SQ>(x, n, mean);
  // numpy halves with the split rounded down to a multiple of 8
  int n2 = n / 2;
  n2 -= n2 % 8;
  return __dadd_rn(np_pairwise_sum<SQ>(x, n2, mean), np_pairwise_sum<SQ>(x + n2, n - n2, mean));
}

__global__ void group_advantage_kernel(clgrpo_group_advantage_args a) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= a.n_samples) return;
  const int g = a.group_of[i];
  if (g < 0 || g >= a.n_groups) {
    // a sample that names no group: NaN marks it instead of reading outside pool_offsets
    a.advantages[i] = __longlong_as_double(0x7ff8000000000000LL);
    if (a.all_zeros) a.all_zeros[i] = 0;
    if (a.all_ones) a.all_ones[i] = 0;
    return;
  }
  const int lo = a.pool_offsets[g], hi = a.pool_offsets[g + 1];
  const double* x = a.pool + lo;
  const int n = hi - lo;
  const double mean = __ddiv_rn(np_pairwise_sum<false>(x, n, 0.0), (double)n);
  const double var = __ddiv_rn(np_pairwise_sum<true>(x, n, mean), (double)n);
  const double sd = __dsqrt_rn(var);
  a.advantages[i] = __ddiv_rn(__dsub_rn(a.rewards[i], mean), __dadd_rn(sd, a.eps));
  bool z = true, o = true;
  for (int k = 0; k < n; ++k) { z &= (x[k] == 0.0); o &= (x[k] == 1.0); }
  if (a.all_zeros) a.all_zeros[i] = z;
  if (a.all_ones) a.all_ones[i] = o;
}

}  // namespace clgrpo

using namespace clgrpo;

extern "C" int clgrpo_group_advantage(const clgrpo_group_advantage_args* a, void* stream) {
  CLGRPO_REQUIRE_PTR(a, "args");
  if (a->n_samples < 0 || a->n_groups < 0) return fail(CLGRPO_EINVAL, "clgrpo_group_advantage: negative size");
  if (a->n_samples == 0) return CLGRPO_OK;
  CLGRPO_REQUIRE_PTR(a->rewards, "rewards");
  CLGRPO_REQUIRE_PTR(a->group_of, "group_of");
  CLGRPO_REQUIRE_PTR(a->pool, "pool");
  CLGRPO_REQUIRE_PTR(a->pool_offsets, "pool_offsets");
  CLGRPO_REQUIRE_PTR(a->advantages, "advantages");
  const int threads = 128;
  hipLaunchKernelGGL(group_advantage_kernel, dim3((unsigned)((a->n_samples + threads - 1) / threads)), dim3(threads), 0,
                     static_cast<hipStream_t>(stream), *a);
  return check_launch("group_advantage_kernel");
}
