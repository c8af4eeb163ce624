// Clipped importance-ratio policy loss (GRPO token-level, GSPO sequence-level),
// k3 KL estimator, masked sums and the per-token upstream gradients, for padded
// [B,S] or cu_seqlens-packed batches.  Memory-bound: each token is read once
// (logprob, old, ref, entropy, mask: 20 B) and written once (loss, dloss, kl,
// g_logprob, g_entropy: <= 24 B); reductions are wavefront shuffles + one LDS
// step per block + a fixed-order pass over the per-block partials, so the sums
// are reproducible run to run.
//
// dtype rules follow what torch does in the reference: logprob arithmetic,
// exp, clamp and the KL stay fp32; the product with the advantages (and the
// final cap) is carried in the advantages' dtype, fp32 or fp64.
#include "common.hpp"

namespace clgrpo {

constexpr int kLossThreads = 256;
constexpr int kMaxLossBlocks = 1024;
constexpr int kNumSums = 8;

struct LossParams {
  int mode;
  int64_t n, B, S, token_offset;
  const int32_t* cu_seqlens;
  const float* logprob;
  const float* old_logprob;
  const float* ref_logprob;
  const float* entropy;
  const int32_t* loss_mask;
  const void* advantages;
  float diff_clip, lo, hi;   // fp32-rounded clamp bounds
  double final_clip;
  double kl_coef, entropy_coef, grad_scale;
  void* loss;
  void* dloss;
  float* kl;
  uint8_t* is_pos;
  uint8_t* is_neg;
  uint8_t* is_clip;
  float* g_logprob;
  float* g_entropy;
  int32_t* flags;
  float* seq_mean;     // workspace [B] (GSPO)
  double* partials;    // workspace [blocks][kNumSums]
};

__device__ __forceinline__ int seq_of_token(const LossParams& p, int64_t i) {
  if (p.cu_seqlens == nullptr) return (int)(i / p.S);
  i += p.token_offset;
  // largest b with cu_seqlens[b] <= i; tokens at or past cu_seqlens[B] belong to no sequence
  if (i >= p.cu_seqlens[p.B] || i < p.cu_seqlens[0]) return -1;
  int lo = 0, hi = (int)p.B;  // invariant: cu[lo] <= i < cu[hi]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (p.cu_seqlens[mid] <= i) lo = mid; else hi = mid;
  }
  return lo;
}

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  return v;
}

// GSPO: per-sequence mean of (logprob - old) over masked positions, as the
// reference forms it: sum(where(mask, d, 0) * mask) / (sum(mask) + 1e-8), fp32.
__global__ __launch_bounds__(kLossThreads) void gspo_seq_mean_kernel(LossParams p) {
  const int b = blockIdx.x;
  int64_t begin, end;
  if (p.cu_seqlens) {
    // positions relative to this call's first token; a sequence outside the window contributes nothing
    begin = (int64_t)p.cu_seqlens[b] - p.token_offset;
    end = (int64_t)p.cu_seqlens[b + 1] - p.token_offset;
    if (begin < 0) begin = 0;
    if (end > p.n) end = p.n;
  } else { begin = (int64_t)b * p.S; end = begin + p.S; }
  double num = 0.0, den = 0.0;
  for (int64_t i = begin + threadIdx.x; i < end; i += kLossThreads) {
    const int mk = p.loss_mask ? p.loss_mask[i] : 1;
    if (mk != 0) {
      const float d = p.logprob[i] - p.old_logprob[i];
      num += (double)(d * (float)mk);
      den += (double)mk;
    }
  }
  __shared__ double sh[2][kLossThreads / 64];
  num = wave_sum(num);
  den = wave_sum(den);
  if ((threadIdx.x & 63) == 0) { sh[0][threadIdx.x >> 6] = num; sh[1][threadIdx.x >> 6] = den; }
  __syncthreads();
  if (threadIdx.x == 0) {
    double a = 0, c = 0;
    for (int w = 0; w < kLossThreads / 64; ++w) { a += sh[0][w]; c += sh[1][w]; }
    p.seq_mean[b] = (float)a / ((float)c + 1e-8f);
  }
}

template <typename CT>
__global__ __launch_bounds__(kLossThreads) void policy_loss_kernel(LossParams p) {
  const CT* adv = static_cast<const CT*>(p.advantages);
  CT* loss_out = static_cast<CT*>(p.loss);
  CT* dloss_out = static_cast<CT*>(p.dloss);
  double acc[kNumSums];
#pragma unroll
  for (int k = 0; k < kNumSums; ++k) acc[k] = 0.0;
  int flag = 0;
  const CT cap = (CT)p.final_clip;

  for (int64_t i = (int64_t)blockIdx.x * kLossThreads + threadIdx.x; i < p.n;
       i += (int64_t)gridDim.x * kLossThreads) {
    const int b = seq_of_token(p, i);
    if (b < 0) {
      // Trailing slots of a packed row that belong to no sequence: defined zeros, no statistics.
      loss_out[i] = (CT)0;
      if (dloss_out) dloss_out[i] = (CT)0;
      if (p.kl) p.kl[i] = 0.f;
      if (p.is_pos) p.is_pos[i] = 0;
      if (p.is_neg) p.is_neg[i] = 0;
      if (p.is_clip) p.is_clip[i] = 0;
      if (p.g_logprob) p.g_logprob[i] = 0.f;
      if (p.g_entropy) p.g_entropy[i] = 0.f;
      continue;
    }
    const int mk = p.loss_mask ? p.loss_mask[i] : 1;
    const CT A = adv[b];
    const float lp = p.logprob[i];
    const float delta = (p.mode == CLGRPO_LOSS_GSPO) ? p.seq_mean[b] : (lp - p.old_logprob[i]);
    // clamp(delta, max=diff_clip): NaN stays NaN
    const float dcl = (delta > p.diff_clip) ? p.diff_clip : delta;
    const float ratio = expf(dcl);
    const float rcl = (ratio < p.lo) ? p.lo : ((ratio > p.hi) ? p.hi : ratio);
    const CT l1 = -A * (CT)ratio;
    const CT l2 = -A * (CT)rcl;
    // torch.max / torch.min propagate NaN
    const CT lc = (l1 != l1 || l2 != l2) ? (CT)NAN : (l1 > l2 ? l1 : l2);
    const CT L = (lc != lc) ? lc : (lc < cap ? lc : cap);
    if (L != L) flag |= 1;
    loss_out[i] = L;

    // d L / d logprob with torch's sub-gradient conventions (ties split in halves,
    // clamp passes the gradient on the closed interval).
    const CT w1 = (l1 > l2) ? (CT)1 : ((l1 == l2) ? (CT)0.5 : (CT)0);
    const CT w2 = (l2 > l1) ? (CT)1 : ((l1 == l2) ? (CT)0.5 : (CT)0);
    const CT gmin = (lc < cap) ? (CT)1 : ((lc == cap) ? (CT)0.5 : (CT)0);
    const CT in_clip = (ratio >= p.lo && ratio <= p.hi) ? (CT)1 : (CT)0;
    const CT pass = (delta <= p.diff_clip) ? (CT)1 : (CT)0;
    const CT dL = gmin * (w1 + w2 * in_clip) * (-A * (CT)ratio) * pass;
    if (dloss_out) dloss_out[i] = dL;

    const bool pos = (ratio > p.hi) && (A > (CT)0);
    const bool neg = (ratio < p.lo) && (A < (CT)0);
    const bool clp = l2 > l1;
    if (p.is_pos) p.is_pos[i] = pos;
    if (p.is_neg) p.is_neg[i] = neg;
    if (p.is_clip) p.is_clip[i] = clp;

    float klv = 0.f, dkl = 0.f;
    if (p.ref_logprob) {
      const float k = p.ref_logprob[i] - lp;
      float rk = expf(k);
      if (mk == 0) rk = 1.f;
      else {
        if (isinf(rk)) flag |= 2;
        if (rk != rk) flag |= 4;
      }
      const float kld = rk - k - 1.f;
      klv = (kld < -10.f) ? -10.f : ((kld > 10.f) ? 10.f : kld);
      dkl = (kld >= -10.f && kld <= 10.f) ? (1.f - rk) : 0.f;
      if (p.kl) p.kl[i] = klv;
    }
    const double w = (double)mk;
    if (p.g_logprob)
      p.g_logprob[i] = (mk != 0) ? (float)(p.grad_scale * w * ((double)dL + p.kl_coef * (double)dkl)) : 0.f;
    if (p.g_entropy)
      p.g_entropy[i] = (mk != 0) ? (float)(-p.entropy_coef * p.grad_scale * w) : 0.f;
    if (mk != 0) {
      acc[0] += w * (double)L;
      acc[1] += w * (double)klv;
      if (p.entropy) acc[2] += w * (double)p.entropy[i];
      acc[3] += w;
      acc[4] += w * (double)pos;
      acc[5] += w * (double)neg;
      acc[6] += w * (double)clp;
    }
  }

  __shared__ double sh[kLossThreads / 64][kNumSums];
#pragma unroll
  for (int k = 0; k < kNumSums; ++k) acc[k] = wave_sum(acc[k]);
  if ((threadIdx.x & 63) == 0) {
#pragma unroll
    for (int k = 0; k < kNumSums; ++k) sh[threadIdx.x >> 6][k] = acc[k];
  }
  __syncthreads();
  if (threadIdx.x < kNumSums) {
    double t = 0;
    for (int w = 0; w < kLossThreads / 64; ++w) t += sh[w][threadIdx.x];
    p.partials[(int64_t)blockIdx.x * kNumSums + threadIdx.x] = t;
  }
  if (flag) atomicOr(p.flags, flag);
}

__global__ void policy_loss_finalize_kernel(const double* partials, int n_blocks, double* sums) {
  const int k = threadIdx.x;
  if (k >= kNumSums) return;
  double t = 0;
  for (int b = 0; b < n_blocks; ++b) t += partials[(int64_t)b * kNumSums + k];
  sums[k] = t;
}

__global__ void zero_flags_kernel(int32_t* flags) { flags[0] = 0; }

static int loss_blocks(int64_t n) {
  int64_t b = (n + kLossThreads - 1) / kLossThreads;
  if (b > kMaxLossBlocks) b = kMaxLossBlocks;
  if (b < 1) b = 1;
  return (int)b;
}

}  // namespace clgrpo

using namespace clgrpo;

extern "C" size_t clgrpo_policy_loss_workspace_bytes(int64_t n, int64_t B) {
  if (n < 0 || B < 0) return 0;
  return align_up((size_t)B * sizeof(float), 256) + (size_t)kMaxLossBlocks * kNumSums * sizeof(double);
}

extern "C" int clgrpo_policy_loss(const clgrpo_policy_loss_args* a, void* stream) {
  CLGRPO_REQUIRE_PTR(a, "args");
  if (a->mode != CLGRPO_LOSS_GRPO && a->mode != CLGRPO_LOSS_GSPO)
    return fail(CLGRPO_EINVAL, "clgrpo_policy_loss: mode %d", a->mode);
  if (a->compute_dtype != CLGRPO_F32 && a->compute_dtype != CLGRPO_F64)
    return fail(CLGRPO_EDTYPE, "clgrpo_policy_loss: compute_dtype %d", a->compute_dtype);
  if (a->token_offset < 0) return fail(CLGRPO_EINVAL, "clgrpo_policy_loss: token_offset=%lld", (long long)a->token_offset);
  if (a->n < 0 || a->B <= 0) return fail(CLGRPO_EINVAL, "clgrpo_policy_loss: n=%lld B=%lld", (long long)a->n, (long long)a->B);
  if (a->cu_seqlens == nullptr) {
    if (a->S <= 0 || a->B * a->S != a->n)
      return fail(CLGRPO_ESHAPE, "clgrpo_policy_loss: padded layout needs n == B*S (n=%lld B=%lld S=%lld)",
                  (long long)a->n, (long long)a->B, (long long)a->S);
  }
  CLGRPO_REQUIRE_PTR(a->logprob, "logprob");
  CLGRPO_REQUIRE_PTR(a->old_logprob, "old_logprob");
  CLGRPO_REQUIRE_PTR(a->advantages, "advantages");
  CLGRPO_REQUIRE_PTR(a->loss, "loss");
  CLGRPO_REQUIRE_PTR(a->sums, "sums");
  CLGRPO_REQUIRE_PTR(a->flags, "flags");
  CLGRPO_REQUIRE_PTR(a->workspace, "workspace");
  if (a->kl != nullptr) CLGRPO_REQUIRE_PTR(a->ref_logprob, "ref_logprob");
  const size_t need = clgrpo_policy_loss_workspace_bytes(a->n, a->B);
  if (a->workspace_bytes < need)
    return fail(CLGRPO_EWORKSPACE, "clgrpo_policy_loss: workspace %zu < %zu bytes", a->workspace_bytes, need);
  hipStream_t s = static_cast<hipStream_t>(stream);

  LossParams p;
  p.mode = a->mode;
  p.n = a->n; p.B = a->B; p.S = a->S;
  p.token_offset = a->cu_seqlens ? a->token_offset : 0;
  p.cu_seqlens = a->cu_seqlens;
  p.logprob = a->logprob; p.old_logprob = a->old_logprob; p.ref_logprob = a->ref_logprob;
  p.entropy = a->entropy; p.loss_mask = a->loss_mask; p.advantages = a->advantages;
  p.diff_clip = (float)a->diff_clip_ratio;
  p.lo = (float)(1.0 - a->neg_clip_ratio);
  p.hi = (float)(1.0 + a->pos_clip_ratio);
  p.final_clip = a->compute_dtype == CLGRPO_F32 ? (double)(float)a->final_clip_ratio : a->final_clip_ratio;
  p.kl_coef = a->kl_coef; p.entropy_coef = a->entropy_coef; p.grad_scale = a->grad_scale;
  p.loss = a->loss; p.dloss = a->dloss_dlogprob; p.kl = a->kl;
  p.is_pos = a->is_positive_clipped; p.is_neg = a->is_negative_clipped; p.is_clip = a->is_clipped;
  p.g_logprob = a->g_logprob; p.g_entropy = a->g_entropy; p.flags = a->flags;
  char* ws = static_cast<char*>(a->workspace);
  p.seq_mean = reinterpret_cast<float*>(ws);
  p.partials = reinterpret_cast<double*>(ws + align_up((size_t)a->B * sizeof(float), 256));

  hipLaunchKernelGGL(zero_flags_kernel, dim3(1), dim3(1), 0, s, a->flags);
  if (a->mode == CLGRPO_LOSS_GSPO) {
    hipLaunchKernelGGL(gspo_seq_mean_kernel, dim3((unsigned)a->B), dim3(kLossThreads), 0, s, p);
    int rc = check_launch("gspo_seq_mean_kernel");
    if (rc) return rc;
  }
  const int blocks = loss_blocks(a->n);
  if (a->compute_dtype == CLGRPO_F32)
    hipLaunchKernelGGL(policy_loss_kernel<float>, dim3(blocks), dim3(kLossThreads), 0, s, p);
  else
    hipLaunchKernelGGL(policy_loss_kernel<double>, dim3(blocks), dim3(kLossThreads), 0, s, p);
  int rc = check_launch("policy_loss_kernel");
  if (rc) return rc;
  hipLaunchKernelGGL(policy_loss_finalize_kernel, dim3(1), dim3(64), 0, s, p.partials, blocks, a->sums);
  return check_launch("policy_loss_finalize_kernel");
}
