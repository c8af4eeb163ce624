// Clipped importance-ratio policy loss (GRPO token-level, GSPO sequence-level),
// k3 KL estimator, masked sums and the per-token upstream gradients, for padded
// [B,S] or cu_seqlens-packed batches.  Memory-bound: each token is read once
// (logprob, old, ref, entropy, mask: 20 B) and written once (loss, dloss, kl,
// g_logprob, g_entropy: <= 24 B); reductions are wavefront shuffles + one LDS
// step per block (+ a fixed-order pass over the per-block partials when more
// than one block runs), so the sums are reproducible run to run.
//
// Up to 4096 tokens go through ONE launch of one 1024-thread workgroup: sequence
// means (GSPO), per-token work, the reductions and the flag word.  Larger inputs
// take the multi-block kernels: (sequence means,) the per-token pass, which leaves
// per-block partial sums and flag bits, and a finalize pass that reduces them in a
// fixed order - two launches (three for GSPO), nothing to zero beforehand.  The
// work is a few hundred KB per micro-batch, so launch latency is what it costs.
//
// dtype rules follow what torch does in the reference: logprob arithmetic,
// exp, clamp and the KL stay fp32; the product with the advantages (and the
// final cap) is carried in the advantages' dtype, fp32 or fp64.
#include "common.hpp"
#include <mutex>

namespace clgrpo {

constexpr int kLossThreads = 256;
constexpr int kMaxLossBlocks = 1024;
constexpr int kNumSums = 8;
constexpr int kOneWgThreads = 1024;
constexpr int64_t kOneWgMaxTokens = 4096;   // above this the multi-block kernels take over

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
  double* sums;        // [kNumSums] out (written directly by the one-workgroup kernel)
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

// Token range [begin, end) of sequence b inside this call's window.
__device__ __forceinline__ void seq_range(const LossParams& p, int64_t b, int64_t& begin, int64_t& end) {
  if (p.cu_seqlens) {
    // positions relative to this call's first token; a sequence outside the window contributes nothing
    begin = (int64_t)p.cu_seqlens[b] - p.token_offset;
    end = (int64_t)p.cu_seqlens[b + 1] - p.token_offset;
    if (begin < 0) begin = 0;
    if (end > p.n) end = p.n;
  } else { begin = b * p.S; end = begin + p.S; }
}

// GSPO: this thread's share (positions begin + first, + stride, ...) of the masked sum of
// (logprob - old) and of the mask count of one sequence.
__device__ __forceinline__ void seq_mean_partial(const LossParams& p, int64_t begin, int64_t end, int first, int stride,
                                                 double& num, double& den) {
  num = 0.0; den = 0.0;
  for (int64_t i = begin + first; i < end; i += stride) {
    const int mk = p.loss_mask ? p.loss_mask[i] : 1;
    if (mk != 0) {
      const float d = p.logprob[i] - p.old_logprob[i];
      num += (double)(d * (float)mk);
      den += (double)mk;
    }
  }
}

// GSPO: per-sequence mean of (logprob - old) over masked positions, as the
// reference forms it: sum(where(mask, d, 0) * mask) / (sum(mask) + 1e-8), fp32.
__global__ __launch_bounds__(kLossThreads) void gspo_seq_mean_kernel(LossParams p) {
  const int b = blockIdx.x;
  int64_t begin, end;
  seq_range(p, b, begin, end);
  double num, den;
  seq_mean_partial(p, begin, end, threadIdx.x, kLossThreads, num, den);
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

// One token: surrogate, clip flags, k3 KL, upstream gradients; adds its masked terms to `acc`.
template <typename CT>
__device__ __forceinline__ void loss_token(const LossParams& p, int64_t i, double (&acc)[kNumSums], int& flag) {
  const CT* adv = static_cast<const CT*>(p.advantages);
  CT* loss_out = static_cast<CT*>(p.loss);
  CT* dloss_out = static_cast<CT*>(p.dloss);
  const CT cap = (CT)p.final_clip;
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
    return;
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

template <typename CT>
__global__ __launch_bounds__(kLossThreads) void policy_loss_kernel(LossParams p) {
  double acc[kNumSums];
#pragma unroll
  for (int k = 0; k < kNumSums; ++k) acc[k] = 0.0;
  int flag = 0;
  for (int64_t i = (int64_t)blockIdx.x * kLossThreads + threadIdx.x; i < p.n;
       i += (int64_t)gridDim.x * kLossThreads)
    loss_token<CT>(p, i, acc, flag);

  __shared__ double sh[kLossThreads / 64][kNumSums];
#pragma unroll
  for (int k = 0; k < kNumSums; ++k) acc[k] = wave_sum(acc[k]);
  if ((threadIdx.x & 63) == 0) {
#pragma unroll
    for (int k = 0; k < kNumSums; ++k) sh[threadIdx.x >> 6][k] = acc[k];
  }
  __syncthreads();
  __shared__ int sh_flag[kLossThreads / 64];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) flag |= __shfl_xor(flag, off);
  if ((threadIdx.x & 63) == 0) sh_flag[threadIdx.x >> 6] = flag;
  __syncthreads();
  if (threadIdx.x < kNumSums - 1) {
    double t = 0;
    for (int w = 0; w < kLossThreads / 64; ++w) t += sh[w][threadIdx.x];
    p.partials[(int64_t)blockIdx.x * kNumSums + threadIdx.x] = t;
  }
  if (threadIdx.x == kNumSums - 1) {
    // the last slot (always zero in the sums) carries this block's flag bits to the finalize pass
    int f = 0;
    for (int w = 0; w < kLossThreads / 64; ++w) f |= sh_flag[w];
    p.partials[(int64_t)blockIdx.x * kNumSums + threadIdx.x] = (double)f;
  }
}


// The whole call in one workgroup: sequence means (one wavefront per sequence), a barrier, the
// per-token pass, the reductions, sums and flag word.  Nothing has to be zeroed beforehand and the
// summation order is fixed.
template <typename CT>
__global__ __launch_bounds__(kOneWgThreads) void policy_loss_onewg_kernel(LossParams p) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (p.mode == CLGRPO_LOSS_GSPO) {
    for (int64_t b = wave; b < p.B; b += kOneWgThreads / 64) {
      int64_t begin, end;
      seq_range(p, b, begin, end);
      double num, den;
      seq_mean_partial(p, begin, end, lane, 64, num, den);
      num = wave_sum(num);
      den = wave_sum(den);
      if (lane == 0) p.seq_mean[b] = (float)num / ((float)den + 1e-8f);
    }
    __threadfence();     // the means are read back by other wavefronts of this workgroup
    __syncthreads();
  }
  double acc[kNumSums];
#pragma unroll
  for (int k = 0; k < kNumSums; ++k) acc[k] = 0.0;
  int flag = 0;
  for (int64_t i = threadIdx.x; i < p.n; i += kOneWgThreads) loss_token<CT>(p, i, acc, flag);

  __shared__ double sh[kOneWgThreads / 64][kNumSums];
  __shared__ int sh_flag[kOneWgThreads / 64];
#pragma unroll
  for (int k = 0; k < kNumSums; ++k) acc[k] = wave_sum(acc[k]);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) flag |= __shfl_xor(flag, off);
  if (lane == 0) {
#pragma unroll
    for (int k = 0; k < kNumSums; ++k) sh[wave][k] = acc[k];
    sh_flag[wave] = flag;
  }
  __syncthreads();
  if (threadIdx.x < kNumSums) {
    double t = 0;
    for (int w = 0; w < kOneWgThreads / 64; ++w) t += sh[w][threadIdx.x];
    p.sums[threadIdx.x] = t;
  }
  if (threadIdx.x == kNumSums) {
    int f = 0;
    for (int w = 0; w < kOneWgThreads / 64; ++w) f |= sh_flag[w];
    p.flags[0] = f;
  }
}

// Fixed-order pass over the per-block partials: one wavefront per sum (lane l adds blocks l, l + 64, ...,
// then a shuffle tree), and the flag word OR-ed from the blocks' flag slots.  Launched with kNumSums * 64 threads.
__global__ void policy_loss_finalize_kernel(const double* partials, int n_blocks, double* sums, int32_t* flags) {
  const int k = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (k >= kNumSums) return;
  if (k == kNumSums - 1) {
    int f = 0;
    for (int b = lane; b < n_blocks; b += 64) f |= (int)partials[(int64_t)b * kNumSums + k];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) f |= __shfl_xor(f, off);
    if (lane == 0) { flags[0] = f; sums[k] = 0.0; }
    return;
  }
  double t = 0;
  for (int b = lane; b < n_blocks; b += 64) t += partials[(int64_t)b * kNumSums + k];
  t = wave_sum(t);
  if (lane == 0) sums[k] = t;
}

// Masked sums of up to kMaxMaskedSums per-token tensors in one launch of one workgroup (fixed
// summation order): out[j] = sum_i float(src_j[i]) * mask[i], divided by (1e-5 + sum(mask)) where
// average[j] is set; count = sum(mask).  fp64 accumulation, fp32 results.
constexpr int kMaxMaskedSums = 16;
struct MaskedSumsParams {
  int64_t n;
  int k;
  const void* src[kMaxMaskedSums];
  int32_t dtype[kMaxMaskedSums];
  int32_t average[kMaxMaskedSums];
  const int32_t* mask;
  float* out;
  int32_t* count;
};

__device__ __forceinline__ float load_as_float(const void* base, int32_t dtype, int64_t i) {
  if (dtype == CLGRPO_F32) return static_cast<const float*>(base)[i];
  if (dtype == CLGRPO_F64) return (float)static_cast<const double*>(base)[i];
  return (float)static_cast<const uint8_t*>(base)[i];
}

__global__ __launch_bounds__(kOneWgThreads) void masked_sums_kernel(MaskedSumsParams p) {
  double acc[kMaxMaskedSums + 1];
#pragma unroll
  for (int j = 0; j <= kMaxMaskedSums; ++j) acc[j] = 0.0;
  for (int64_t i = threadIdx.x; i < p.n; i += kOneWgThreads) {
    const float mk = (float)p.mask[i];
    if (mk == 0.f) continue;
    acc[kMaxMaskedSums] += (double)mk;
#pragma unroll
    for (int j = 0; j < kMaxMaskedSums; ++j)
      if (j < p.k) acc[j] += (double)(load_as_float(p.src[j], p.dtype[j], i) * mk);
  }
  __shared__ double sh[kOneWgThreads / 64][kMaxMaskedSums + 1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int j = 0; j <= kMaxMaskedSums; ++j) {
    const double t = wave_sum(acc[j]);
    if (lane == 0) sh[wave][j] = t;
  }
  __syncthreads();
  if (threadIdx.x <= kMaxMaskedSums) {
    double cnt = 0, t = 0;
    for (int w = 0; w < kOneWgThreads / 64; ++w) { cnt += sh[w][kMaxMaskedSums]; t += sh[w][threadIdx.x]; }
    if (threadIdx.x == kMaxMaskedSums) p.count[0] = (int32_t)cnt;
    else if (threadIdx.x < p.k) p.out[threadIdx.x] = p.average[threadIdx.x] ? (float)t / (1e-5f + (float)cnt) : (float)t;
  }
}

// d/dsrc of one masked sum: dst[i] = g[0] * mask[i] in the source's dtype (g is a device scalar).
template <typename CT>
__global__ void masked_sums_bwd_kernel(int64_t n, const float* g, const int32_t* mask, CT* dst) {
  const float gv = g[0];
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = (CT)(gv * (float)mask[i]);
}

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

// Validation and launches shared by the entry points; `ws` is the scratch memory they differ in.
static int run_policy_loss(const char* who, const clgrpo_policy_loss_args* a, void* ws_ptr, size_t ws_bytes, void* stream) {
  CLGRPO_REQUIRE_PTR(a, "args");
  if (a->mode != CLGRPO_LOSS_GRPO && a->mode != CLGRPO_LOSS_GSPO)
    return fail(CLGRPO_EINVAL, "%s: mode %d", who, a->mode);
  if (a->compute_dtype != CLGRPO_F32 && a->compute_dtype != CLGRPO_F64)
    return fail(CLGRPO_EDTYPE, "%s: compute_dtype %d", who, a->compute_dtype);
  if (a->token_offset < 0) return fail(CLGRPO_EINVAL, "%s: token_offset=%lld", who, (long long)a->token_offset);
  if (a->n < 0 || a->B <= 0) return fail(CLGRPO_EINVAL, "%s: n=%lld B=%lld", who, (long long)a->n, (long long)a->B);
  if (a->cu_seqlens == nullptr) {
    if (a->S <= 0 || a->B * a->S != a->n)
      return fail(CLGRPO_ESHAPE, "%s: padded layout needs n == B*S (n=%lld B=%lld S=%lld)", who,
                  (long long)a->n, (long long)a->B, (long long)a->S);
  }
  CLGRPO_REQUIRE_PTR(a->logprob, "logprob");
  CLGRPO_REQUIRE_PTR(a->old_logprob, "old_logprob");
  CLGRPO_REQUIRE_PTR(a->advantages, "advantages");
  CLGRPO_REQUIRE_PTR(a->loss, "loss");
  CLGRPO_REQUIRE_PTR(a->sums, "sums");
  CLGRPO_REQUIRE_PTR(a->flags, "flags");
  CLGRPO_REQUIRE_PTR(ws_ptr, "workspace");
  if (a->kl != nullptr) CLGRPO_REQUIRE_PTR(a->ref_logprob, "ref_logprob");
  const size_t need = clgrpo_policy_loss_workspace_bytes(a->n, a->B);
  if (ws_bytes < need)
    return fail(CLGRPO_EWORKSPACE, "%s: workspace %zu < %zu bytes", who, ws_bytes, need);
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
  p.sums = a->sums;
  char* ws = static_cast<char*>(ws_ptr);
  p.seq_mean = reinterpret_cast<float*>(ws);
  p.partials = reinterpret_cast<double*>(ws + align_up((size_t)a->B * sizeof(float), 256));

  if (a->n <= kOneWgMaxTokens) {
    // one launch: sequence means, per-token pass, sums and flag word in a single workgroup
    if (a->compute_dtype == CLGRPO_F32)
      hipLaunchKernelGGL(policy_loss_onewg_kernel<float>, dim3(1), dim3(kOneWgThreads), 0, s, p);
    else
      hipLaunchKernelGGL(policy_loss_onewg_kernel<double>, dim3(1), dim3(kOneWgThreads), 0, s, p);
    return check_launch("policy_loss_onewg_kernel");
  }
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
  hipLaunchKernelGGL(policy_loss_finalize_kernel, dim3(1), dim3(kNumSums * 64), 0, s, p.partials, blocks, a->sums, a->flags);
  return check_launch("policy_loss_finalize_kernel");
}

extern "C" int clgrpo_policy_loss(const clgrpo_policy_loss_args* a, void* stream) {
  CLGRPO_REQUIRE_PTR(a, "args");
  return run_policy_loss("clgrpo_policy_loss", a, a->workspace, a->workspace_bytes, stream);
}

// ---- the entry point that allocates nothing ---------------------------------------------------
// Scratch memory of clgrpo_policy_loss_static: what the other entry point takes from the caller's
// workspace (sequence means for up to kStaticMaxSeqs sequences, then the per-block partial sums).
// Each device the library runs on holds its own copy of this array until the process ends.  Nothing
// in it has to start at zero: every call writes the means of all its sequences and the partials of
// all its blocks before reading them.  Calls that overlap on one device share it and race.
constexpr int64_t kStaticMaxSeqs = 65536;
constexpr size_t kStaticScratchBytes = (size_t)kStaticMaxSeqs * sizeof(float) + (size_t)kMaxLossBlocks * kNumSums * sizeof(double);
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Device address of `scratch` on the current device, looked up once per device (the array's name is
// only a host-side handle of the symbol, not an address a kernel could use).
static int static_scratch_address(void** out) {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static void* address[kMaxDevices];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(CLGRPO_ELAUNCH, "clgrpo_policy_loss_static: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(CLGRPO_EINVAL, "clgrpo_policy_loss_static: device %d out of range", dev);
  std::lock_guard<std::mutex> lock(mu);
  if (address[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr)
      return fail(CLGRPO_ELAUNCH, "clgrpo_policy_loss_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    address[dev] = ptr;
  }
  *out = address[dev];
  return CLGRPO_OK;
}

extern "C" int64_t clgrpo_policy_loss_static_max_sequences(void) { return kStaticMaxSeqs; }

extern "C" int clgrpo_policy_loss_static(const clgrpo_policy_loss_args* a, void* stream) {
  CLGRPO_REQUIRE_PTR(a, "args");
  if (a->B > kStaticMaxSeqs)
    return fail(CLGRPO_EWORKSPACE, "clgrpo_policy_loss_static: B=%lld sequences exceed the built-in scratch (at most %lld); "
                "use clgrpo_policy_loss with a workspace", (long long)a->B, (long long)kStaticMaxSeqs);
  void* ptr = nullptr;
  int rc = static_scratch_address(&ptr);
  if (rc) return rc;
  return run_policy_loss("clgrpo_policy_loss_static", a, ptr, kStaticScratchBytes, stream);
}

extern "C" int clgrpo_policy_loss_launches(int64_t n, int32_t mode) {
  if (n <= kOneWgMaxTokens) return 1;
  return mode == CLGRPO_LOSS_GSPO ? 3 : 2;
}

extern "C" int clgrpo_masked_sums(const clgrpo_masked_sums_args* a, void* stream) {
  CLGRPO_REQUIRE_PTR(a, "args");
  if (a->n < 0 || a->k <= 0 || a->k > kMaxMaskedSums)
    return fail(CLGRPO_EINVAL, "clgrpo_masked_sums: n=%lld k=%d (at most %d tensors)", (long long)a->n, a->k, kMaxMaskedSums);
  CLGRPO_REQUIRE_PTR(a->mask, "mask");
  CLGRPO_REQUIRE_PTR(a->out, "out");
  CLGRPO_REQUIRE_PTR(a->count, "count");
  MaskedSumsParams p;
  p.n = a->n; p.k = a->k; p.mask = a->mask; p.out = a->out; p.count = a->count;
  for (int j = 0; j < kMaxMaskedSums; ++j) {
    p.src[j] = j < a->k ? a->src[j] : nullptr;
    p.dtype[j] = j < a->k ? a->dtype[j] : CLGRPO_F32;
    p.average[j] = j < a->k ? a->average[j] : 0;
    if (j < a->k) {
      CLGRPO_REQUIRE_PTR(a->src[j], "src[j]");
      if (a->dtype[j] != CLGRPO_F32 && a->dtype[j] != CLGRPO_F64 && a->dtype[j] != CLGRPO_U8)
        return fail(CLGRPO_EDTYPE, "clgrpo_masked_sums: dtype[%d] = %d", j, a->dtype[j]);
    }
  }
  hipLaunchKernelGGL(masked_sums_kernel, dim3(1), dim3(kOneWgThreads), 0, static_cast<hipStream_t>(stream), p);
  return check_launch("masked_sums_kernel");
}

extern "C" int clgrpo_masked_sums_bwd(int64_t n, const float* g, const int32_t* mask, void* dst, int32_t dtype,
                                      void* stream) {
  CLGRPO_REQUIRE_PTR(g, "g");
  CLGRPO_REQUIRE_PTR(mask, "mask");
  CLGRPO_REQUIRE_PTR(dst, "dst");
  if (n < 0) return fail(CLGRPO_EINVAL, "clgrpo_masked_sums_bwd: n=%lld", (long long)n);
  if (dtype != CLGRPO_F32 && dtype != CLGRPO_F64) return fail(CLGRPO_EDTYPE, "clgrpo_masked_sums_bwd: dtype %d", dtype);
  if (n == 0) return CLGRPO_OK;
  const int blocks = (int)((n + 255) / 256 < 1024 ? (n + 255) / 256 : 1024);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == CLGRPO_F32)
    hipLaunchKernelGGL(masked_sums_bwd_kernel<float>, dim3(blocks), dim3(256), 0, s, n, g, mask, static_cast<float*>(dst));
  else
    hipLaunchKernelGGL(masked_sums_bwd_kernel<double>, dim3(blocks), dim3(256), 0, s, n, g, mask, static_cast<double*>(dst));
  return check_launch("masked_sums_bwd_kernel");
}
