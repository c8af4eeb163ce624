// Mask / index builders for padded <-> packed batches.  Integer work, bit-exact.
// All kernels are bandwidth-bound streaming passes; each element of a [B,S]
// array is read or written once with consecutive lanes on consecutive addresses.
#include "common.hpp"

namespace clgrpo {

__global__ void build_masks_kernel(int64_t B, int64_t S, const int32_t* __restrict__ plen,
                                   const int32_t* __restrict__ rlen, int32_t* __restrict__ attn,
                                   int32_t* __restrict__ loss, int64_t* __restrict__ pos) {
  const int64_t n = B * S;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t b = i / S, s = i - b * S;
    const int64_t p = plen[b], e = (int64_t)plen[b] + rlen[b];
    attn[i] = (s < e) ? 1 : 0;
    loss[i] = (s >= p && s < e) ? 1 : 0;
    if (pos) pos[i] = s;
  }
}

__global__ void shift_labels_kernel(int64_t B, int64_t S, const int64_t* __restrict__ tokens,
                                    const int32_t* __restrict__ mask, int64_t* __restrict__ labels,
                                    int32_t* __restrict__ shifted, int zero_last) {
  const int64_t n = B * S;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t b = i / S, s = i - b * S;
    const int64_t src = b * S + ((s + 1 == S) ? 0 : s + 1);
    if (tokens) labels[i] = tokens[src];
    if (mask) shifted[i] = (zero_last && s + 1 == S) ? 0 : mask[src];
  }
}

// Row statistics: seqlens[b] = sum of mask values (int32), nnz[b] = count of nonzeros.
__global__ __launch_bounds__(256) void unpad_row_stats_kernel(int64_t S, const int32_t* __restrict__ mask,
                                                              int32_t* __restrict__ seqlens, int32_t* __restrict__ nnz) {
  const int64_t b = blockIdx.x;
  int sum = 0, cnt = 0;
  for (int64_t s = threadIdx.x; s < S; s += 256) {
    const int v = mask[b * S + s];
    sum += v;
    cnt += (v != 0);
  }
  __shared__ int sh[2][4];
  for (int off = 32; off > 0; off >>= 1) { sum += __shfl_xor(sum, off); cnt += __shfl_xor(cnt, off); }
  if ((threadIdx.x & 63) == 0) { sh[0][threadIdx.x >> 6] = sum; sh[1][threadIdx.x >> 6] = cnt; }
  __syncthreads();
  if (threadIdx.x == 0) {
    seqlens[b] = sh[0][0] + sh[0][1] + sh[0][2] + sh[0][3];
    nnz[b + 1] = sh[1][0] + sh[1][1] + sh[1][2] + sh[1][3];
  }
}

// One block: cu_seqlens = [0, cumsum(seqlens)], row_offsets = exclusive scan of nnz, totals.
__global__ __launch_bounds__(256) void unpad_scan_kernel(int64_t B, const int32_t* __restrict__ seqlens,
                                                         int32_t* __restrict__ cu, int32_t* __restrict__ row_off,
                                                         int32_t* __restrict__ total) {
  __shared__ int sh_a[256], sh_b[256], sh_m[256];
  __shared__ int carry_a, carry_b, carry_m;
  if (threadIdx.x == 0) { carry_a = 0; carry_b = 0; carry_m = INT32_MIN; cu[0] = 0; row_off[0] = 0; }
  __syncthreads();
  for (int64_t base = 0; base < B; base += 256) {
    const int64_t b = base + threadIdx.x;
    const int a = (b < B) ? seqlens[b] : 0;
    const int c = (b < B) ? row_off[b + 1] : 0;   // holds nnz[b] until overwritten below
    sh_a[threadIdx.x] = a; sh_b[threadIdx.x] = c; sh_m[threadIdx.x] = (b < B) ? a : INT32_MIN;
    __syncthreads();
    for (int off = 1; off < 256; off <<= 1) {
      int ta = 0, tb = 0, tm = INT32_MIN;
      if ((int)threadIdx.x >= off) { ta = sh_a[threadIdx.x - off]; tb = sh_b[threadIdx.x - off]; tm = sh_m[threadIdx.x - off]; }
      __syncthreads();
      sh_a[threadIdx.x] += ta; sh_b[threadIdx.x] += tb;
      sh_m[threadIdx.x] = sh_m[threadIdx.x] > tm ? sh_m[threadIdx.x] : tm;
      __syncthreads();
    }
    if (b < B) { cu[b + 1] = carry_a + sh_a[threadIdx.x]; row_off[b + 1] = carry_b + sh_b[threadIdx.x]; }
    __syncthreads();
    if (threadIdx.x == 255) {
      carry_a += sh_a[255]; carry_b += sh_b[255];
      carry_m = carry_m > sh_m[255] ? carry_m : sh_m[255];
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) { total[0] = carry_b; total[1] = carry_m; }
}

// Ordered compaction of one row: indices[row_off[b] + rank] = b*S + s for mask != 0.
__global__ __launch_bounds__(256) void unpad_compact_kernel(int64_t S, const int32_t* __restrict__ mask,
                                                            const int32_t* __restrict__ row_off,
                                                            int64_t* __restrict__ indices) {
  const int64_t b = blockIdx.x;
  __shared__ int wave_cnt[4];
  __shared__ int base_sh;
  if (threadIdx.x == 0) base_sh = row_off[b];
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int64_t s0 = 0; s0 < S; s0 += 256) {
    const int64_t s = s0 + threadIdx.x;
    const bool on = (s < S) && (mask[b * S + s] != 0);
    const unsigned long long bal = __ballot(on);
    if (lane == 0) wave_cnt[wave] = __popcll(bal);
    __syncthreads();
    int before = 0;
    for (int w = 0; w < wave; ++w) before += wave_cnt[w];
    const int rank = before + __popcll(bal & ((1ull << lane) - 1ull));
    if (on) indices[(int64_t)base_sh + rank] = b * S + s;
    __syncthreads();
    if (threadIdx.x == 0) base_sh += wave_cnt[0] + wave_cnt[1] + wave_cnt[2] + wave_cnt[3];
    __syncthreads();
  }
}

template <typename U>
__global__ void gather_rows_kernel(const U* __restrict__ src, U* __restrict__ dst, const int64_t* __restrict__ idx,
                                   int64_t n_idx, int64_t units, int64_t n_rows, int scatter) {
  const int64_t n = n_idx * units;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / units, u = i - r * units;
    const int64_t j = idx[r];
    if (j < 0 || j >= n_rows) continue;   // out-of-range index: skipped, never dereferenced
    if (scatter) dst[j * units + u] = src[i];
    else dst[i] = src[j * units + u];
  }
}

__global__ void fill_zero_kernel(uint32_t* __restrict__ p, int64_t n_words, uint8_t* __restrict__ tail, int n_tail) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_words; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0u;
  if (blockIdx.x == 0 && (int)threadIdx.x < n_tail) tail[threadIdx.x] = 0;
}

static int grid_for(int64_t n, int threads) {
  int64_t g = (n + threads - 1) / threads;
  if (g > 65536) g = 65536;
  if (g < 1) g = 1;
  return (int)g;
}

static int rows_dispatch(const clgrpo_rows_args* a, hipStream_t s, int scatter) {
  const uintptr_t al = reinterpret_cast<uintptr_t>(a->src) | reinterpret_cast<uintptr_t>(a->dst) | (uintptr_t)a->row_bytes;
  const int64_t total = a->n_idx * a->row_bytes;
  if (total == 0) return CLGRPO_OK;
#define CLGRPO_ROWS(U)                                                                                      \
  hipLaunchKernelGGL(gather_rows_kernel<U>, dim3(grid_for(total / (int64_t)sizeof(U), 256)), dim3(256), 0, s, \
                     static_cast<const U*>(a->src), static_cast<U*>(a->dst), a->indices, a->n_idx,           \
                     a->row_bytes / (int64_t)sizeof(U), a->n_rows, scatter)
  if (al % 16 == 0) CLGRPO_ROWS(uint4);
  else if (al % 8 == 0) CLGRPO_ROWS(uint2);
  else if (al % 4 == 0) CLGRPO_ROWS(uint32_t);
  else if (al % 2 == 0) CLGRPO_ROWS(uint16_t);
  else CLGRPO_ROWS(uint8_t);
#undef CLGRPO_ROWS
  return check_launch("gather_rows_kernel");
}


// ---------------------------------------------------------------------------------------------
// Packed (THD) micro-batch from per-sample lengths.

// One workgroup: padded lengths, their exclusive scan, totals and the consistency word.
__global__ __launch_bounds__(256) void thd_offsets_kernel(int64_t B, int64_t S, const int32_t* __restrict__ plen,
                                                          const int32_t* __restrict__ rlen, int align, int cp_size,
                                                          int64_t total_expected, int32_t* __restrict__ cu,
                                                          int32_t* __restrict__ seqlens, int32_t* __restrict__ padded,
                                                          int32_t* __restrict__ stats, int32_t* __restrict__ status) {
  __shared__ int64_t part[256];
  __shared__ int32_t pmax[256];
  __shared__ int32_t bad[256];
  const int tid = threadIdx.x;
  const int64_t per = (B + 255) / 256;
  const int64_t lo = tid * per, hi = (lo + per) < B ? (lo + per) : B;
  int64_t sum = 0;
  int32_t mx = 0, flag = 0;
  for (int64_t b = lo; b < hi; ++b) {
    const int64_t len = (int64_t)plen[b] + rlen[b];
    const int64_t pad = (len + align - 1) / align * align;
    seqlens[b] = (int32_t)len;
    padded[b] = (int32_t)pad;
    if (len > S || len < 0) flag |= 2;
    if (cp_size > 1 && pad % (2 * cp_size) != 0) flag |= 4;   // one rank keeps everything: any length will do
    sum += pad;
    mx = pad > mx ? (int32_t)pad : mx;
  }
  part[tid] = sum;
  pmax[tid] = mx;
  bad[tid] = flag;
  __syncthreads();
  if (tid == 0) {
    int64_t run = 0;
    int32_t m = 0, f = 0;
    for (int i = 0; i < 256; ++i) {
      const int64_t v = part[i];
      part[i] = run;
      run += v;
      m = pmax[i] > m ? pmax[i] : m;
      f |= bad[i];
    }
    if (run != total_expected) f |= 1;
    cu[B] = (int32_t)run;
    stats[0] = (int32_t)run;
    stats[1] = m;
    stats[2] = 0;
    status[0] = f;
  }
  __syncthreads();
  int64_t run = part[tid];
  for (int64_t b = lo; b < hi; ++b) {
    cu[b] = (int32_t)run;
    run += padded[b];
  }
}

// Largest i with cu[i] <= pos (cu ascending, cu[0] = 0, pos < cu[B]; empty segments are skipped).
__device__ __forceinline__ int thd_find_seq(const int32_t* __restrict__ cu, int B, int64_t pos) {
  int lo = 0, hi = B;   // invariant: cu[lo] <= pos < cu[hi]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cu[mid] <= pos) lo = mid; else hi = mid;
  }
  return lo;
}

struct ThdFill {
  int64_t B, S, total, per_rank;
  const int64_t* tokens;
  const int32_t* plen;
  const int32_t* rlen;
  const int32_t* cu;
  const int32_t* seqlens;
  const int32_t* status;
  int32_t* stats;
  int cp_size, cp_rank;
  int64_t pad_token;
  int64_t* indices;
  int64_t* seq_indices;
  int64_t* out_tokens;
  int64_t* out_labels;
  int32_t* out_loss_mask;
  int64_t* out_position_ids;
};

__device__ __forceinline__ void thd_at(const ThdFill& p, int64_t pos, int64_t& token, int& in_loss, int& seq, int64_t& j) {
  seq = thd_find_seq(p.cu, (int)p.B, pos);
  j = pos - p.cu[seq];
  token = j < p.seqlens[seq] ? p.tokens[(int64_t)seq * p.S + j] : p.pad_token;
  const int64_t pl = p.plen[seq];
  in_loss = (j >= pl && j < pl + p.rlen[seq]) ? 1 : 0;
}

__global__ __launch_bounds__(256) void thd_fill_kernel(ThdFill p) {
  if (p.status[0] != 0) return;   // inconsistent sizes: leave the outputs alone, the host raises
  const int max_padded = p.stats[1];
  int ones = 0;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < p.total; i += (int64_t)gridDim.x * blockDim.x) {
    int64_t token, j;
    int in_loss, seq;
    thd_at(p, i, token, in_loss, seq, j);
    p.indices[i] = (int64_t)seq * max_padded + j;
    if (i < p.per_rank) {
      // i-th entry of this rank: position `src` of the packed row
      const int sq = thd_find_seq(p.cu, (int)p.B, i * p.cp_size);   // the rank's share keeps the order of the sequences
      const int64_t start_r = p.cu[sq] / p.cp_size;
      const int64_t len_r = (p.cu[sq + 1] - p.cu[sq]) / p.cp_size;
      const int64_t k = i - start_r;
      const int64_t half = len_r / 2;
      const int64_t chunk = k < half ? p.cp_rank : 2 * (p.cp_size - 1) - p.cp_rank;
      const int64_t src = (int64_t)p.cu[sq] + k + half * chunk;
      p.seq_indices[i] = src;
      int64_t tk, nj;
      int il, ns;
      thd_at(p, src, tk, il, ns, nj);
      p.out_tokens[i] = tk;
      if (p.out_position_ids) p.out_position_ids[i] = nj;
      thd_at(p, src + 1 == p.total ? 0 : src + 1, tk, il, ns, nj);
      p.out_labels[i] = tk;
      if (p.out_loss_mask) p.out_loss_mask[i] = il;
      ones += il;
    }
  }
  // number of loss positions on this rank: wave reduction, one atomic per wave
  for (int off = 32; off > 0; off >>= 1) ones += __shfl_down(ones, off, 64);
  if ((threadIdx.x & 63) == 0 && ones) atomicAdd(&p.stats[2], ones);
}

}  // namespace clgrpo

using namespace clgrpo;

extern "C" int clgrpo_build_masks(const clgrpo_build_masks_args* a, void* stream) {
  CLGRPO_REQUIRE_PTR(a, "args");
  if (a->B < 0 || a->S < 0) return fail(CLGRPO_EINVAL, "clgrpo_build_masks: B=%lld S=%lld", (long long)a->B, (long long)a->S);
  if (a->B * a->S == 0) return CLGRPO_OK;
  CLGRPO_REQUIRE_PTR(a->prompt_len, "prompt_len");
  CLGRPO_REQUIRE_PTR(a->response_len, "response_len");
  CLGRPO_REQUIRE_PTR(a->attn_mask, "attn_mask");
  CLGRPO_REQUIRE_PTR(a->loss_mask, "loss_mask");
  hipLaunchKernelGGL(build_masks_kernel, dim3(grid_for(a->B * a->S, 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     a->B, a->S, a->prompt_len, a->response_len, a->attn_mask, a->loss_mask, a->position_ids);
  return check_launch("build_masks_kernel");
}

extern "C" int clgrpo_shift_labels(const clgrpo_shift_labels_args* a, void* stream) {
  CLGRPO_REQUIRE_PTR(a, "args");
  if (a->B < 0 || a->S < 0) return fail(CLGRPO_EINVAL, "clgrpo_shift_labels: B=%lld S=%lld", (long long)a->B, (long long)a->S);
  if (a->B * a->S == 0) return CLGRPO_OK;
  if (a->tokens) CLGRPO_REQUIRE_PTR(a->labels, "labels");
  if (a->loss_mask) CLGRPO_REQUIRE_PTR(a->shifted_mask, "shifted_mask");
  if (!a->tokens && !a->loss_mask) return fail(CLGRPO_ENULL, "clgrpo_shift_labels: tokens and loss_mask both NULL");
  hipLaunchKernelGGL(shift_labels_kernel, dim3(grid_for(a->B * a->S, 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     a->B, a->S, a->tokens, a->loss_mask, a->labels, a->shifted_mask, a->zero_last);
  return check_launch("shift_labels_kernel");
}

extern "C" int clgrpo_unpad_indices(const clgrpo_unpad_indices_args* a, void* stream) {
  CLGRPO_REQUIRE_PTR(a, "args");
  if (a->B <= 0 || a->S <= 0) return fail(CLGRPO_EINVAL, "clgrpo_unpad_indices: B=%lld S=%lld", (long long)a->B, (long long)a->S);
  if (a->B * a->S >= (1LL << 31)) return fail(CLGRPO_ESHAPE, "clgrpo_unpad_indices: B*S must fit int32 counts");
  CLGRPO_REQUIRE_PTR(a->attn_mask, "attn_mask");
  CLGRPO_REQUIRE_PTR(a->indices, "indices");
  CLGRPO_REQUIRE_PTR(a->cu_seqlens, "cu_seqlens");
  CLGRPO_REQUIRE_PTR(a->seqlens, "seqlens");
  CLGRPO_REQUIRE_PTR(a->total, "total");
  CLGRPO_REQUIRE_PTR(a->row_offsets, "row_offsets");
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(unpad_row_stats_kernel, dim3((unsigned)a->B), dim3(256), 0, s, a->S, a->attn_mask, a->seqlens, a->row_offsets);
  int rc = check_launch("unpad_row_stats_kernel");
  if (rc) return rc;
  hipLaunchKernelGGL(unpad_scan_kernel, dim3(1), dim3(256), 0, s, a->B, a->seqlens, a->cu_seqlens, a->row_offsets, a->total);
  rc = check_launch("unpad_scan_kernel");
  if (rc) return rc;
  hipLaunchKernelGGL(unpad_compact_kernel, dim3((unsigned)a->B), dim3(256), 0, s, a->S, a->attn_mask, a->row_offsets, a->indices);
  return check_launch("unpad_compact_kernel");
}

static int rows_validate(const clgrpo_rows_args* a, const char* who) {
  if (a == nullptr) return fail(CLGRPO_ENULL, "%s: args is NULL", who);
  if (a->n_idx < 0 || a->row_bytes < 0 || a->n_rows < 0) return fail(CLGRPO_EINVAL, "%s: negative size", who);
  if (a->n_idx * a->row_bytes == 0) return CLGRPO_OK;
  if (!a->src || !a->dst || !a->indices) return fail(CLGRPO_ENULL, "%s: NULL pointer", who);
  return CLGRPO_OK;
}

extern "C" int clgrpo_gather_rows(const clgrpo_rows_args* a, void* stream) {
  int rc = rows_validate(a, "clgrpo_gather_rows");
  if (rc) return rc;
  return rows_dispatch(a, static_cast<hipStream_t>(stream), 0);
}

extern "C" int clgrpo_scatter_rows(const clgrpo_rows_args* a, void* stream) {
  int rc = rows_validate(a, "clgrpo_scatter_rows");
  if (rc) return rc;
  if (a->dst == nullptr && a->n_rows * a->row_bytes > 0) return fail(CLGRPO_ENULL, "clgrpo_scatter_rows: dst is NULL");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t bytes = a->n_rows * a->row_bytes;
  if (bytes > 0) {
    // dst comes from an allocator, so it is at least 4-byte aligned; the tail handles odd sizes.
    if (reinterpret_cast<uintptr_t>(a->dst) % 4 != 0) return fail(CLGRPO_EINVAL, "clgrpo_scatter_rows: dst must be 4-byte aligned");
    const int64_t words = bytes / 4;
    hipLaunchKernelGGL(fill_zero_kernel, dim3(grid_for(words, 256)), dim3(256), 0, s, static_cast<uint32_t*>(a->dst), words,
                       static_cast<uint8_t*>(a->dst) + words * 4, (int)(bytes - words * 4));
    rc = check_launch("fill_zero_kernel");
    if (rc) return rc;
  }
  return rows_dispatch(a, s, 1);
}

extern "C" int clgrpo_thd_pack(const clgrpo_thd_pack_args* a, void* stream) {
  CLGRPO_REQUIRE_PTR(a, "args");
  if (a->B <= 0 || a->S <= 0) return fail(CLGRPO_EINVAL, "clgrpo_thd_pack: B=%lld S=%lld", (long long)a->B, (long long)a->S);
  if (a->align <= 0 || a->cp_size <= 0 || a->cp_rank < 0 || a->cp_rank >= a->cp_size)
    return fail(CLGRPO_EINVAL, "clgrpo_thd_pack: align=%d cp_size=%d cp_rank=%d", a->align, a->cp_size, a->cp_rank);
  if (a->total_padded <= 0 || a->total_padded >= (1LL << 31) || a->total_padded % a->cp_size != 0)
    return fail(CLGRPO_EINVAL, "clgrpo_thd_pack: total_padded=%lld must be positive, fit int32 and divide by cp_size",
                (long long)a->total_padded);
  if (a->B >= (1LL << 24)) return fail(CLGRPO_ESHAPE, "clgrpo_thd_pack: B too large");
  CLGRPO_REQUIRE_PTR(a->tokens, "tokens");
  CLGRPO_REQUIRE_PTR(a->prompt_len, "prompt_len");
  CLGRPO_REQUIRE_PTR(a->response_len, "response_len");
  CLGRPO_REQUIRE_PTR(a->cu_seqlens_padded, "cu_seqlens_padded");
  CLGRPO_REQUIRE_PTR(a->seqlens, "seqlens");
  CLGRPO_REQUIRE_PTR(a->seqlens_padded, "seqlens_padded");
  CLGRPO_REQUIRE_PTR(a->stats, "stats");
  CLGRPO_REQUIRE_PTR(a->status, "status");
  CLGRPO_REQUIRE_PTR(a->indices, "indices");
  CLGRPO_REQUIRE_PTR(a->seq_indices, "seq_indices");
  CLGRPO_REQUIRE_PTR(a->out_tokens, "out_tokens");
  CLGRPO_REQUIRE_PTR(a->out_labels, "out_labels");
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(thd_offsets_kernel, dim3(1), dim3(256), 0, s, a->B, a->S, a->prompt_len, a->response_len, a->align,
                     a->cp_size, a->total_padded, a->cu_seqlens_padded, a->seqlens, a->seqlens_padded, a->stats, a->status);
  int rc = check_launch("thd_offsets_kernel");
  if (rc) return rc;
  ThdFill f;
  f.B = a->B;
  f.S = a->S;
  f.total = a->total_padded;
  f.per_rank = a->total_padded / a->cp_size;
  f.tokens = a->tokens;
  f.plen = a->prompt_len;
  f.rlen = a->response_len;
  f.cu = a->cu_seqlens_padded;
  f.seqlens = a->seqlens;
  f.status = a->status;
  f.stats = a->stats;
  f.cp_size = a->cp_size;
  f.cp_rank = a->cp_rank;
  f.pad_token = a->pad_token;
  f.indices = a->indices;
  f.seq_indices = a->seq_indices;
  f.out_tokens = a->out_tokens;
  f.out_labels = a->out_labels;
  f.out_loss_mask = a->out_loss_mask;
  f.out_position_ids = a->out_position_ids;
  hipLaunchKernelGGL(thd_fill_kernel, dim3(grid_for(a->total_padded, 256)), dim3(256), 0, s, f);
  return check_launch("thd_fill_kernel");
}
