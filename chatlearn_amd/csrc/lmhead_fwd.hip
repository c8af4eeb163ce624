// Fused lm_head projection + online log-softmax statistics (forward).
//
// z^T tile [256 vocab x 256 tokens] = W tile * hidden tile^T on the matrix cores;
// the vocabulary runs along the accumulator registers, the tokens along the
// lanes, so each lane keeps a running (max, sum e^{z-max}, sum e^{z-max} z,
// target logit) for its own tokens across all vocabulary tiles of its split.
// A workgroup owns one block of 256 tokens and one contiguous range of
// vocabulary tiles ("split"); a second small kernel merges the splits with an
// exact rescale and writes logprob / entropy / rowmax / lse.  Logits go to
// memory only when the caller asks for a chunk's raw logits to be kept for the
// backward; they then leave straight from the accumulators, 16 bytes per lane,
// in the accumulators' own order (see ZNative).
//
// Algorithmic work: 2*T*H*V flop; bytes 2*T*H + 2*V*H (bf16) + 16*T.
#include "common.hpp"
#include "gemm_core.hpp"

namespace clgrpo {

constexpr int kFwdBM = 256, kFwdBN = 256;
constexpr float kLog2e = 1.4426950408889634f;
constexpr int kMaxFwdSplits = 64;   // most vocabulary splits a forward launch uses

struct FwdParams {
  const void* hidden;
  const void* weight;
  const int64_t* labels;
  int64_t label_offset;  // first vocabulary id of `weight` (0 unless this is a vocabulary shard)
  int T, H, V;
  int n_tb, n_split, tiles_per_split, n_vt;
  float c;  // inv_temperature * log2(e)
  void* z_out;   // optional raw logits, z-native layout (see ZNative): rows x ldz entries of KeptLogit<T>
  int64_t ldz;
  const int32_t* z_row_map;  // optional [T]: destination row per token, < 0: not stored
  int z_rows;                // rows of z_out; mapped rows outside [0, z_rows) are not stored
  float4* part;  // [n_split][T]: (max raw, sum 2^{(z-max) c}, sum 2^{(z-max) c} z raw, target raw)
  int xcd_wgs;   // > 0: launch of several rounds, see xcd_round_remap
};

// 16 bytes of kept logits from consecutive accumulator registers.
template <typename ZT> __device__ __forceinline__ u32x4 pack_piece(const f32x16& a, int first);
template <> __device__ __forceinline__ u32x4 pack_piece<float>(const f32x16& a, int first) {
  f32x4 v = {a[first], a[first + 1], a[first + 2], a[first + 3]};
  return __builtin_bit_cast(u32x4, v);
}
template <> __device__ __forceinline__ u32x4 pack_piece<_Float16>(const f32x16& a, int first) {
  typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
  f16x8 v;
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = (_Float16)a[first + e];     // round to nearest even
  return __builtin_bit_cast(u32x4, v);
}

__device__ __forceinline__ void merge_state(float& m, float& s, float& u, float om, float os,
                                            float ou, float c) {
  const float nm = fmaxf(m, om);
  const float a = (m == nm) ? 1.f : exp2f((m - nm) * c);
  const float b = (om == nm) ? 1.f : exp2f((om - nm) * c);
  s = s * a + os * b;
  u = u * a + ou * b;
  m = nm;
}

template <typename T, bool STORE_Z>
__global__ __launch_bounds__(kHeadThreads) void lmhead_fwd_kernel(FwdParams p) {
  using Tile = HeadTile<T>;
  constexpr int MI = Tile::MI, NI = Tile::NI, WM = Tile::WM, WN = Tile::WN;
  extern __shared__ __align__(16) char lds[];

  const int item = work_item(p.xcd_wgs);
  if (item >= p.n_tb * p.n_split) return;
  int vs, tb;
  grouped_tile(item, p.n_split, p.n_tb, 4, vs, tb);
  if (STORE_Z && sizeof(typename KeptLogit<T>::type) == 2) {
    // Kept logits are IEEE half: a raw logit beyond the half range must stay finite (the largest half),
    // or the softmax the backward rebuilds from it would be inf/NaN.  The wave's FP16_OVFL mode bit
    // (MODE register, bit 23) makes every conversion to half clamp instead of overflowing to infinity.
    __builtin_amdgcn_s_setreg(1 | (23 << 6) | (0 << 11), 1);
  }

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave % 2, wn = wave / 2;
  const int t0 = tb * kFwdBN;
  const int b_rows = (p.T - t0) < kFwdBN ? (p.T - t0) : kFwdBN;
  const T* hidden = static_cast<const T*>(p.hidden) + (int64_t)t0 * p.H;
  const T* weight = static_cast<const T*>(p.weight);
  const float c = p.c;

  int lab[NI], zrow[NI];
  float m[NI], s[NI], u[NI], zt[NI];
#pragma unroll
  for (int ni = 0; ni < NI; ++ni) {
    const int tok = t0 + wn * WN + ni * 32 + (lane & 31);
    lab[ni] = -1;
    if (p.labels != nullptr && tok < p.T) {
      const int64_t rel = p.labels[tok] - p.label_offset;   // a label outside these rows matches nothing
      if (rel >= 0 && rel < p.V) lab[ni] = (int)rel;
    }
    zrow[ni] = (STORE_Z && tok < p.T) ? (p.z_row_map ? p.z_row_map[tok] : tok) : -1;
    if (zrow[ni] >= p.z_rows) zrow[ni] = -1;
    m[ni] = -INFINITY;
    s[ni] = 0.f;
    u[ni] = 0.f;
    zt[ni] = 0.f;
  }

  typename Tile::Stream st;
  const int vt_begin = vs * p.tiles_per_split;
  const int vt_end = (vt_begin + p.tiles_per_split) < p.n_vt ? (vt_begin + p.tiles_per_split) : p.n_vt;
  for (int vt = vt_begin; vt < vt_end; ++vt) {
    const int v0 = vt * kFwdBM;
    const int a_rows = (p.V - v0) < kFwdBM ? (p.V - v0) : kFwdBM;
    f32x16 acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.f;

    // The K loop requests the first slabs of the next vocabulary tile during its last two slab periods.
    const bool has_next = vt + 1 < vt_end;
    const int v1 = v0 + kFwdBM;
    const int next_rows = (p.V - v1) < kFwdBM ? (p.V - v1) : kFwdBM;
    const T* next_w = weight + (int64_t)v1 * p.H;
    Tile::run(acc, Tile::Operand::row_major(weight + (int64_t)v0 * p.H, p.H, a_rows),
              Tile::Operand::row_major(hidden, p.H, b_rows), p.H, lds, st, has_next ? next_w : nullptr, next_rows, true);

    if (STORE_Z) {
      // Raw logits for the backward, straight from the accumulators: per 32x32 block a lane stores its
      // 16 values as 16-byte pieces, each piece of the 64 lanes one contiguous KB (z-native layout).
      // Vocabulary rows past V hold zeros already (the operand loads are range-checked), and the
      // backward ignores whatever the padding columns hold.
      typedef typename KeptLogit<T>::type ZT;
      typedef ZNative<ZT> ZL;
      char* z = static_cast<char*>(p.z_out);
      const int64_t n_kslab = p.ldz / ZL::kSlabElems;
#pragma unroll
      for (int ni = 0; ni < NI; ++ni) {
        // The row is the same for every vocabulary tile, so the compiler would keep the 64-bit addresses it
        // forms from it alive across the K loops, where registers are scarcest, spill them, and reload them
        // between the stores (a reload waits for the stores issued before it).  Re-deriving them from the
        // 32-bit row costs a handful of instructions per tile.
        int row = zrow[ni];
        asm volatile("" : "+v"(row));
        if (row < 0) continue;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
          const int v_blk = v0 + wm * WM + mi * 32;
          if (v_blk >= p.ldz) continue;
#pragma unroll
          for (int j = 0; j < ZL::PIECES; ++j)
            *reinterpret_cast<u32x4*>(z + ZL::piece_offset(row, v_blk >> 5, n_kslab, lane >> 5, j)) =
                pack_piece<ZT>(acc[mi][ni], j * ZL::kPerPiece);
        }
      }
    }

    if (a_rows == kFwdBM) {
#pragma unroll
      for (int ni = 0; ni < NI; ++ni) {
        float tmax = acc[0][ni][0];
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
          for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, acc[mi][ni][r]);
        const float nm = fmaxf(m[ni], tmax);
        const float scale = exp2f((m[ni] - nm) * c);  // m = -inf on the first tile -> 0
        const float nb = -nm * c;
        float ls = 0.f, lu = 0.f;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float v = acc[mi][ni][r];
            const float e = __builtin_amdgcn_exp2f(fmaf(v, c, nb));
            ls += e;
            lu = fmaf(e, v, lu);
          }
        s[ni] = fmaf(s[ni], scale, ls);
        u[ni] = fmaf(u[ni], scale, lu);
        m[ni] = nm;
      }
    } else {
      // Last, partial vocabulary tile: rows >= a_rows are clamped duplicates and must not count.
#pragma unroll
      for (int ni = 0; ni < NI; ++ni) {
        float tmax = -INFINITY;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int row = wm * WM + mi * 32 + acc_row(r, lane);
            if (row < a_rows) tmax = fmaxf(tmax, acc[mi][ni][r]);
          }
        const float nm = fmaxf(m[ni], tmax);
        if (nm == -INFINITY) continue;  // this lane has seen no valid row yet
        const float scale = exp2f((m[ni] - nm) * c);
        const float nb = -nm * c;
        float ls = 0.f, lu = 0.f;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int row = wm * WM + mi * 32 + acc_row(r, lane);
            if (row < a_rows) {
              const float v = acc[mi][ni][r];
              const float e = __builtin_amdgcn_exp2f(fmaf(v, c, nb));
              ls += e;
              lu = fmaf(e, v, lu);
            }
          }
        s[ni] = fmaf(s[ni], scale, ls);
        u[ni] = fmaf(u[ni], scale, lu);
        m[ni] = nm;
      }
    }

    // Target logit: only the wave whose 128 vocabulary rows hold the label looks for it.
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) {
      const int rel = lab[ni] - (v0 + wm * WM);
      const bool in = (unsigned)rel < (unsigned)WM && (lab[ni] < p.V);
      if (__any(in)) {
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (rel == mi * 32 + acc_row(r, lane)) zt[ni] = acc[mi][ni][r];
      }
    }
  }

  // Merge the two lane halves (same tokens, different vocabulary rows).
#pragma unroll
  for (int ni = 0; ni < NI; ++ni) {
    const float om = __shfl_xor(m[ni], 32);
    const float os = __shfl_xor(s[ni], 32);
    const float ou = __shfl_xor(u[ni], 32);
    const float oz = __shfl_xor(zt[ni], 32);
    merge_state(m[ni], s[ni], u[ni], om, os, ou, c);
    zt[ni] += oz;
  }
  // Merge the two waves that share these tokens (wm = 0, 1) through LDS.
  float4* xch = reinterpret_cast<float4*>(lds);
  if (wm == 1 && lane < 32) {
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
      xch[wn * WN + ni * 32 + lane] = make_float4(m[ni], s[ni], u[ni], zt[ni]);
  }
  __syncthreads();
  if (wm == 0 && lane < 32) {
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) {
      const float4 o = xch[wn * WN + ni * 32 + lane];
      merge_state(m[ni], s[ni], u[ni], o.x, o.y, o.z, c);
      zt[ni] += o.w;
      const int tok = t0 + wn * WN + ni * 32 + lane;
      if (tok < p.T) p.part[(int64_t)vs * p.T + tok] = make_float4(m[ni], s[ni], u[ni], zt[ni]);
    }
  }
}

struct FinalizeParams {
  const float4* part;
  const int64_t* labels;
  int T, V, n_split;
  float c, inv_temperature;
  float* logprob;
  float* entropy;
  float* rowmax;
  float* lse;
  float4* record;   // non-null: only the merged (max, sum, sum*z, target) record is written
};

__global__ void lmhead_fwd_finalize_kernel(FinalizeParams p) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= p.T) return;
  float m = -INFINITY, s = 0.f, u = 0.f, zt = 0.f;
  for (int k = 0; k < p.n_split; ++k) {
    const float4 o = p.part[(int64_t)k * p.T + t];
    merge_state(m, s, u, o.x, o.y, o.z, p.c);
    zt += o.w;
  }
  if (p.record) {
    p.record[t] = make_float4(m, s, u, zt);
    return;
  }
  const float mx = m * p.inv_temperature;
  const float lse = mx + logf(s);
  p.lse[t] = lse;
  if (p.rowmax) p.rowmax[t] = mx;
  if (p.entropy) p.entropy[t] = lse - p.inv_temperature * u / s;
  if (p.logprob) {
    const int64_t lab = p.labels[t];
    // A label outside [0, V) has no logit; NaN marks it instead of a silent wrong number.
    p.logprob[t] = (lab >= 0 && lab < p.V) ? (zt * p.inv_temperature - lse) : NAN;
  }
}

// Split of the vocabulary tiles over workgroups.  A workgroup walks ceil(n_vt / n_split) tiles for
// one block of 256 tokens; with each CU holding one workgroup a launch takes
// ceil(n_tb * n_split / CUs) rounds, so its cost in tile periods is rounds * tiles-per-workgroup.
// Many splits and several rounds are fine (65 token blocks: 35 splits of 17 tiles, 9 rounds = 153 tile
// periods against the ideal 151), so the plan stays within a few per cent of n_tb * n_vt / CUs tile periods
// from about 7 token blocks on.  Two smaller terms, both measured on launches of equal tile periods:
//  - the splits are handed out in groups of 4 (the workgroups of an XCD then form a block of 4 splits x
//    CUs/32 token blocks that shares operand slabs in the XCD's L2: 4 + 8 = 12 slabs per step for 32 tiles).
//    A last group of w < 4 splits makes blocks of w x 32/w, w + 32/w slabs per step; the time grows by about
//    0.11 of that excess (65536 tokens at H = 4096: 5 splits 63.4 ms, 2 splits 64.2 ms, 6 splits 61.3 ms
//    against 60.6 ms with 4 or 60.9 ms with 8);
//  - every run of tiles starts with a K loop whose first slabs nothing has requested in advance and ends
//    with its partial record: 0.3 tile periods (32768 tokens at H = 7168: 22 splits x 23 tiles 45.2 ms, 4
//    x 127 or 8 x 64 tiles 44.3 - 44.6 ms).
// Returns the launch's cost in sixteenths of a tile period.  `cus` <= 0 plans for a 256-CU device.
static long fwd_single_cost(int n_tb, int n_vt, int cus, int& n_split, int& tiles_per_split) {
  if (cus <= 0) cus = 256;
  const double xcd_wgs = cus / 8.0, full_block = 4.0 + xcd_wgs / 4.0;
  int best = 1;
  double best_cost = -1.0;
  for (int sp = 1; sp <= kMaxFwdSplits && sp <= n_vt; ++sp) {
    const int tps = (n_vt + sp - 1) / sp;
    const int eff_sp = (n_vt + tps - 1) / tps;
    const long rounds = ((long)n_tb * eff_sp + cus - 1) / cus;
    const int rem = eff_sp % 4;
    const double excess = rem ? (double)rem / eff_sp * ((rem + xcd_wgs / rem) / full_block - 1.0) : 0.0;
    const double cost = (double)rounds * (tps + 0.3) * 16.0 * (1.0 + 0.11 * excess) + eff_sp * 0.01;
    if (best_cost < 0 || cost < best_cost) { best_cost = cost; best = sp; }
  }
  tiles_per_split = (n_vt + best - 1) / best;
  n_split = (n_vt + tiles_per_split - 1) / tiles_per_split;
  return (long)(best_cost + 0.5);
}

template <typename T, bool STORE_Z>
static int launch_fwd(const clgrpo_lmhead_fwd_args* a, hipStream_t stream, int64_t label_offset, float4* record) {
  using Tile = HeadTile<T>;
  FwdParams p;
  p.hidden = a->hidden;
  p.weight = a->weight;
  p.labels = a->labels;
  p.label_offset = label_offset;
  p.T = (int)a->T;
  p.H = (int)a->H;
  p.V = (int)a->V;
  p.n_tb = (int)((a->T + kFwdBN - 1) / kFwdBN);
  p.n_vt = (int)((a->V + kFwdBM - 1) / kFwdBM);
  fwd_single_cost(p.n_tb, p.n_vt, device_cu_count(), p.n_split, p.tiles_per_split);
  p.c = a->inv_temperature * kLog2e;
  p.part = static_cast<float4*>(a->workspace);
  p.z_out = a->saved_logits;
  p.ldz = a->ld_saved;
  p.z_row_map = a->saved_row_map;
  p.z_rows = (int)a->saved_rows;
  constexpr int lds_bytes = Tile::kLdsBytes;
  int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(&lmhead_fwd_kernel<T, STORE_Z>), lds_bytes, "lmhead_fwd_kernel");
  if (rc) return rc;
  const ItemGrid ig = item_grid(p.n_tb * p.n_split, device_cu_count());
  p.xcd_wgs = ig.xcd_wgs;
  hipLaunchKernelGGL((lmhead_fwd_kernel<T, STORE_Z>), dim3(ig.grid), dim3(Tile::kThreads), lds_bytes, stream, p);
  rc = check_launch("lmhead_fwd_kernel");
  if (rc) return rc;
  FinalizeParams f;
  f.part = p.part;
  f.labels = a->labels;
  f.T = p.T;
  f.V = p.V;
  f.n_split = p.n_split;
  f.c = p.c;
  f.inv_temperature = a->inv_temperature;
  f.logprob = a->labels ? a->logprob : nullptr;
  f.entropy = a->entropy;
  f.rowmax = a->rowmax;
  f.lse = a->lse;
  f.record = record;
  hipLaunchKernelGGL(lmhead_fwd_finalize_kernel, dim3((p.T + 255) / 256), dim3(256), 0, stream, f);
  return check_launch("lmhead_fwd_finalize_kernel");
}

int validate_head_shape(const char* who, int64_t T, int64_t H, int64_t V, int32_t dtype) {
  if (dtype != CLGRPO_BF16 && dtype != CLGRPO_F32) return fail(CLGRPO_EDTYPE, "%s: dtype %d unsupported", who, dtype);
  if (T <= 0 || H <= 0 || V <= 0) return fail(CLGRPO_EINVAL, "%s: T, H, V must be positive (got %lld, %lld, %lld)", who,
                                             (long long)T, (long long)H, (long long)V);
  const int slab = dtype == CLGRPO_BF16 ? 64 : 32;
  if (H % slab != 0) return fail(CLGRPO_ESHAPE, "%s: H=%lld must be a multiple of %d", who, (long long)H, slab);
  // 256 rows of H elements must stay below 2^31 bytes (32-bit offsets of the buffer loads)
  if (T >= (1LL << 30) || V >= (1LL << 30) || H > (1LL << 20)) return fail(CLGRPO_ESHAPE, "%s: size too large", who);
  return CLGRPO_OK;
}

}  // namespace clgrpo

using namespace clgrpo;

extern "C" int64_t clgrpo_saved_logits_ld(int64_t V) { return V <= 0 ? 0 : round_up64(V, 64); }

extern "C" int clgrpo_lmhead_fwd_launch_plan(int64_t T, int64_t V, int32_t cus, int32_t* out) {
  if (T <= 0 || V <= 0 || out == nullptr) return CLGRPO_EINVAL;
  const int n_tb = (int)((T + kFwdBN - 1) / kFwdBN), n_vt = (int)((V + kFwdBM - 1) / kFwdBM);
  int n_split, tps;
  fwd_single_cost(n_tb, n_vt, cus, n_split, tps);
  out[0] = n_tb;
  out[1] = n_split;
  out[2] = tps;
  return CLGRPO_OK;
}

extern "C" size_t clgrpo_lmhead_fwd_workspace_bytes(int64_t T, int64_t H, int64_t V, int32_t dtype) {
  (void)H;
  (void)dtype;
  if (T <= 0 || V <= 0) return 0;
  // one record per token and vocabulary split; the split count depends on the device's CU count and never
  // exceeds kMaxFwdSplits, so this bound holds on any device
  const int64_t n_vt = (V + kFwdBM - 1) / kFwdBM;
  const int64_t splits = n_vt < kMaxFwdSplits ? n_vt : kMaxFwdSplits;
  return (size_t)splits * (size_t)T * sizeof(float4);
}

// Shared by the whole-vocabulary entry point (record == nullptr) and the shard one.
static int run_fwd(const char* who, const clgrpo_lmhead_fwd_args* a, int64_t vocab_begin, float4* record,
                   void* stream) {
  CLGRPO_REQUIRE_PTR(a, "args");
  int rc = validate_head_shape(who, a->T, a->H, a->V, a->dtype);
  if (rc) return rc;
  CLGRPO_REQUIRE_PTR(a->hidden, "hidden");
  CLGRPO_REQUIRE_PTR(a->weight, "weight");
  if (record == nullptr) {
    CLGRPO_REQUIRE_PTR(a->lse, "lse");
    if (a->labels != nullptr) CLGRPO_REQUIRE_PTR(a->logprob, "logprob");
  }
  if (vocab_begin < 0) return fail(CLGRPO_EINVAL, "%s: vocab_begin=%lld", who, (long long)vocab_begin);
  if (!(a->inv_temperature > 0.f)) return fail(CLGRPO_EINVAL, "%s: inv_temperature must be > 0", who);
  CLGRPO_REQUIRE_PTR(a->workspace, "workspace");
  const size_t need = clgrpo_lmhead_fwd_workspace_bytes(a->T, a->H, a->V, a->dtype);
  if (a->workspace_bytes < need)
    return fail(CLGRPO_EWORKSPACE, "%s: workspace %zu < %zu bytes", who, a->workspace_bytes, need);
  if (a->saved_logits != nullptr && (a->ld_saved < clgrpo_saved_logits_ld(a->V) || a->ld_saved % 64 != 0))
    return fail(CLGRPO_ESHAPE, "%s: ld_saved=%lld must be a multiple of 64 and >= %lld", who,
                (long long)a->ld_saved, (long long)clgrpo_saved_logits_ld(a->V));
  if (a->saved_logits != nullptr && (a->saved_rows <= 0 || a->saved_rows >= (1LL << 31)))
    return fail(CLGRPO_EINVAL, "%s: saved_rows=%lld", who, (long long)a->saved_rows);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (a->saved_logits != nullptr)
    return a->dtype == CLGRPO_BF16 ? launch_fwd<__bf16, true>(a, s, vocab_begin, record)
                                   : launch_fwd<float, true>(a, s, vocab_begin, record);
  return a->dtype == CLGRPO_BF16 ? launch_fwd<__bf16, false>(a, s, vocab_begin, record)
                                 : launch_fwd<float, false>(a, s, vocab_begin, record);
}

extern "C" int clgrpo_lmhead_fwd(const clgrpo_lmhead_fwd_args* a, void* stream) {
  return run_fwd("clgrpo_lmhead_fwd", a, 0, nullptr, stream);
}

extern "C" int clgrpo_lmhead_fwd_shard(const clgrpo_lmhead_fwd_args* a, int64_t vocab_begin, void* record,
                                       void* stream) {
  CLGRPO_REQUIRE_PTR(record, "record");
  return run_fwd("clgrpo_lmhead_fwd_shard", a, vocab_begin, static_cast<float4*>(record), stream);
}

extern "C" int clgrpo_lmhead_merge_shards(const void* records, int64_t n_shards, int64_t T, const int64_t* labels,
                                          int64_t V_total, float inv_temperature, float* logprob, float* entropy,
                                          float* rowmax, float* lse, void* stream) {
  CLGRPO_REQUIRE_PTR(records, "records");
  CLGRPO_REQUIRE_PTR(lse, "lse");
  if (labels != nullptr) CLGRPO_REQUIRE_PTR(logprob, "logprob");
  if (n_shards <= 0 || n_shards > 4096 || T <= 0 || T >= (1LL << 30) || V_total <= 0)
    return fail(CLGRPO_EINVAL, "clgrpo_lmhead_merge_shards: n_shards=%lld T=%lld V_total=%lld", (long long)n_shards,
                (long long)T, (long long)V_total);
  if (!(inv_temperature > 0.f)) return fail(CLGRPO_EINVAL, "clgrpo_lmhead_merge_shards: inv_temperature must be > 0");
  FinalizeParams f;
  f.part = static_cast<const float4*>(records);
  f.labels = labels;
  f.T = (int)T;
  f.V = (int)(V_total < (1LL << 31) - 1 ? V_total : (1LL << 31) - 1);
  f.n_split = (int)n_shards;
  f.c = inv_temperature * kLog2e;
  f.inv_temperature = inv_temperature;
  f.logprob = labels ? logprob : nullptr;
  f.entropy = entropy;
  f.rowmax = rowmax;
  f.lse = lse;
  f.record = nullptr;
  hipLaunchKernelGGL(lmhead_fwd_finalize_kernel, dim3((f.T + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream), f);
  return check_launch("lmhead_fwd_finalize_kernel");
}
