// NT-GEMM workgroup tile for gfx950 (CDNA4): C^[BM x BN] = A[BM x K] * B[BN x K]^T,
// both operands K-contiguous in memory, fp32 accumulation on the matrix cores.
//
// One workgroup of WAVES_M x WAVES_N wavefronts (64 lanes each) owns a BM x BN
// tile.  K is walked in slabs of 128 bytes per row (64 bf16 or 32 fp32
// elements).  A slab of A (BM rows) and of B (BN rows) travels HBM/L2 -> LDS
// directly (buffer loads with an LDS destination; no registers, no LDS store
// instructions).  Such a load fills LDS in lane order, so rows are 128 bytes
// apart with no padding; bank conflicts are avoided by an XOR swizzle of the
// 16-byte K-chunks within a row, applied on the global side of the load and
// undone by the fragment reads.  Two LDS stages: while the matrix cores work on
// stage s, the next slab lands in stage s^1; one workgroup barrier per slab,
// placed before the last K-step so that step's matrix instructions cover the
// first fragment reads of the next slab; that barrier is preceded by an
// explicit wait for the wave's outstanding loads, because a barrier alone does
// not wait for loads whose destination is LDS.
//
// Operands are either row-major (the caller's hidden states and weight) or
// K-blocked (the library's own intermediates: per tile and slab one contiguous
// 32 KB piece, see Operand).  Consecutive K loops of a workgroup that keep the
// same B rows can stream into each other: the last two slab periods of one loop
// already request the first two slabs of the next (see Stream).
//
// Accumulator layout (v_mfma_f32_32x32x*): for the 32x32 block (mi, ni) of a
// wave, lane l, register r hold
//     row (A index) = mi*32 + 8*(r/4) + 4*(l/32) + (r%4)
//     col (B index) = ni*32 + (l%32)
// so a lane owns ONE B row per ni and 16 A rows per (mi, ni).  The callers put
// the dimension they reduce over (vocabulary, for the softmax statistics) on A,
// which makes that reduction mostly lane-local.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace clgrpo {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kRowBytes = 128;    // K-slab bytes per tile row
constexpr int kChunksPerRow = 8;  // 16-byte chunks per slab row
constexpr int kBlockRows = 256;   // rows per block of a K-blocked operand

template <typename T> struct Elem;
template <> struct Elem<__bf16> { static constexpr int kSlabK = 64; };
template <> struct Elem<float> { static constexpr int kSlabK = 32; };

// Element (row, k) of a K-blocked operand with `n_kslab` slabs per row: blocks of 256 rows, each
// block holding its slabs one after another, each slab 256 rows of 128 bytes.
template <typename T>
__host__ __device__ __forceinline__ int64_t blocked_index(int64_t row, int64_t k, int64_t n_kslab) {
  constexpr int E = kRowBytes / (int)sizeof(T);
  return (((row / kBlockRows) * n_kslab + k / E) * kBlockRows + (row % kBlockRows)) * E + (k % E);
}

// Kept logits ("z-native" layout).  The forward leaves a chunk's raw logits for the backward in the
// order its accumulators hold them, so that storing them costs no shuffle: the buffer is cut into the
// same 32 KB units as a K-blocked operand (256 rows x one 128-byte K slab of vocabulary, unit (rb, ks) at
// byte (rb * n_kslab + ks) * 32768), and inside a unit into sub-blocks of 32 rows x 32 vocabulary entries,
// sub-block (rs, vs) at (rs * VSUB + vs) * PIECES KB.  A sub-block is one 32x32 accumulator block: lane
// (h, t32) = (lane / 32, lane % 32) owns row t32 and the 16 entries 8 * (r / 4) + 4 * h + r % 4, r = 0..15,
// which it stores as PIECES 16-byte pieces; piece j of all 64 lanes is one contiguous KB.  The kernel that
// turns logits into d(logits) reads a unit whole and writes the K-blocked result over it.
// 16-bit inputs keep their logits as IEEE half (10 mantissa bits against bf16's 7: the softmax the
// backward rebuilds from them is 8x closer to the fp32 one), fp32 inputs as fp32.
template <typename T> struct KeptLogit;
template <> struct KeptLogit<__bf16> { typedef _Float16 type; };
template <> struct KeptLogit<float> { typedef float type; };

template <typename T> struct ZNative {
  static constexpr int ES = (int)sizeof(T);
  static constexpr int kSlabElems = kRowBytes / ES;     // vocabulary entries per unit
  static constexpr int VSUB = kSlabElems / 32;          // sub-blocks along the vocabulary per unit
  static constexpr int PIECES = ES;                     // 16-byte pieces per lane and sub-block (16 values)
  static constexpr int kPerPiece = 16 / PIECES;         // values per piece
  static constexpr int kUnitBytes = kBlockRows * kRowBytes;
  // byte offset of piece j of lane half h for `row` and the 32-aligned vocabulary block `v32` (= vocab / 32)
  __host__ __device__ static __forceinline__ int64_t piece_offset(int64_t row, int64_t v32, int64_t n_kslab, int h, int j) {
    const int64_t rb = row / kBlockRows;
    const int R = (int)(row % kBlockRows);
    const int64_t unit = (rb * n_kslab + v32 / VSUB) * kUnitBytes;
    const int sb = (R >> 5) * VSUB + (int)(v32 % VSUB);
    return unit + (int64_t)sb * (PIECES * 1024) + j * 1024 + (h * 32 + (R & 31)) * 16;
  }
  // vocabulary offset inside its 32-block of value e of piece j for lane half h
  __host__ __device__ static __forceinline__ int col_of(int h, int j, int e) {
    const int r = j * kPerPiece + e;
    return 8 * (r >> 2) + 4 * h + (r & 3);
  }
};

// One 32-byte-of-K step for a 32x32 block: a and b each hold 16 bytes per lane.
template <typename T>
__device__ __forceinline__ void mma_block(f32x16& acc, const u32x4& a, const u32x4& b);

template <>
__device__ __forceinline__ void mma_block<__bf16>(f32x16& acc, const u32x4& a, const u32x4& b) {
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
}

template <>
__device__ __forceinline__ void mma_block<float>(f32x16& acc, const u32x4& a, const u32x4& b) {
  // Four K=2 steps; lane half h, element j stands for k = 4h + j in both operands.
  f32x4 af = __builtin_bit_cast(f32x4, a);
  f32x4 bf = __builtin_bit_cast(f32x4, b);
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[0], bf[0], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[1], bf[1], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[2], bf[2], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[3], bf[3], acc, 0, 0, 0);
}

// Row of the accumulator register r within a 32x32 block for this lane.
__device__ __forceinline__ int acc_row(int r, int lane) {
  return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
}

template <typename T, int BM_, int BN_, int WAVES_M_, int WAVES_N_>
struct GemmTile {
  static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
  static constexpr int kWaves = WAVES_M * WAVES_N;
  static constexpr int kThreads = 64 * kWaves;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int MI = WM / 32, NI = WN / 32;
  static constexpr int kRowsPerPass = kThreads / kChunksPerRow;
  static constexpr int kPassA = BM / kRowsPerPass, kPassB = BN / kRowsPerPass;
  static constexpr int kStageBytes = (BM + BN) * kRowBytes;
  static constexpr int kLdsBytes = 2 * kStageBytes;
  static constexpr int kSlabK = Elem<T>::kSlabK;
  static_assert(BM % kRowsPerPass == 0 && BN % kRowsPerPass == 0, "tile rows vs threads");
  static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be whole 32x32 blocks");

  // State a caller carries between consecutive K loops of one workgroup that share B (same
  // token rows, next block of A rows): which LDS stage holds slab 0, and whether the first two
  // slabs of the coming loop have already been requested.
  struct Stream {
    int phase = 0;
    bool loaded = false;
  };

  // Where an operand's tile lives in memory: `rows` valid rows starting at `base`, consecutive
  // rows `row_bytes` apart, consecutive 128-byte K slabs of a row `slab_bytes` apart.
  //   row-major [rows][ld]:                  row_bytes = ld * sizeof(T), slab_bytes = 128
  //   K-blocked [row block][K slab][256][128 B]: row_bytes = 128, slab_bytes = 256 * 128 (one
  //   contiguous 32 KB piece per tile and slab)
  struct Operand {
    const T* base;
    int row_bytes;
    int slab_bytes;
    int rows;
    __device__ static __forceinline__ Operand row_major(const T* base, int64_t ld, int rows) {
      return Operand{base, (int)(ld * (int64_t)sizeof(T)), kRowBytes, rows};
    }
    __device__ static __forceinline__ Operand blocked(const T* block_base, int rows) {
      return Operand{block_base, kRowBytes, kBlockRows * kRowBytes, rows};
    }
  };

  // Per-thread constants of the global -> LDS loads of one operand pair.
  struct Loader {
    const char* a_ptr;
    const char* b_ptr;
    int a_bytes, b_bytes;     // bytes the valid rows span from the tile base at slab 0
    int a_shrink, b_shrink;   // by how much that span shrinks per slab step (row-major: one slab; blocked: 0)
    int a_slab, b_slab;
    int a_voff, b_voff, a_pass, b_pass, dma_off;
  };

  typedef __attribute__((address_space(3))) char lds_char;

  // Loads go through range-checked buffer descriptors that cover exactly the valid rows, so rows
  // past them read as zero and nothing outside the operands is touched.  The hardware checks the
  // sum of the per-lane and the scalar offset against the descriptor's size, so the K-slab offset
  // travels in the descriptor's base address instead (a few scalar instructions per slab) and the
  // size is what is left of the valid rows from there.
  __device__ static __forceinline__ Loader make_loader(const Operand& a, const Operand& b) {
    const int tid = threadIdx.x;
    const int ld_row = tid >> 3;
    const int ld_chunk = tid & 7;
    Loader L;
    L.a_ptr = reinterpret_cast<const char*>(a.base);
    L.b_ptr = reinterpret_cast<const char*>(b.base);
    L.a_bytes = a.rows * a.row_bytes;
    L.b_bytes = b.rows * b.row_bytes;
    L.a_shrink = a.slab_bytes == kRowBytes ? kRowBytes : 0;
    L.b_shrink = b.slab_bytes == kRowBytes ? kRowBytes : 0;
    L.a_slab = a.slab_bytes;
    L.b_slab = b.slab_bytes;
    // A wave's load instruction fills 1 KB of LDS in lane order: 8 rows x 8 chunks of 16 bytes.
    // The lane that lands on (row, slot) fetches K-chunk slot ^ swz(row), so a fragment read of
    // K-chunk q goes to slot q ^ swz(row).
    const int ld_swz = (ld_row & 7) ^ ((ld_row >> 3) & 1);
    L.a_voff = ld_row * a.row_bytes + ((ld_chunk ^ ld_swz) * 16);
    L.b_voff = ld_row * b.row_bytes + ((ld_chunk ^ ld_swz) * 16);
    L.a_pass = kRowsPerPass * a.row_bytes;
    L.b_pass = kRowsPerPass * b.row_bytes;
    L.dma_off = __builtin_amdgcn_readfirstlane(tid >> 6) * 8 * kRowBytes;   // this wave's 8 rows within a pass
    return L;
  }

  // global -> LDS without passing registers; completion must be awaited (wait_loads) before the
  // workgroup barrier that publishes the stage.
  __device__ static __forceinline__ void dma_slab(const Loader& L, char* stage, int slab) {
    lds_char* dst = (lds_char*)(stage) + L.dma_off;
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(L.a_ptr + (int64_t)slab * L.a_slab), 0, L.a_bytes - slab * L.a_shrink, 0x00020000);
    const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(L.b_ptr + (int64_t)slab * L.b_slab), 0, L.b_bytes - slab * L.b_shrink, 0x00020000);
#pragma unroll
    for (int p = 0; p < kPassA; ++p)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, dst + p * kRowsPerPass * kRowBytes, 16,
                                               L.a_voff + p * L.a_pass, 0, 0, 0);
#pragma unroll
    for (int p = 0; p < kPassB; ++p)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, dst + (BM + p * kRowsPerPass) * kRowBytes, 16,
                                               L.b_voff + p * L.b_pass, 0, 0, 0);
  }

  // A workgroup barrier does not wait for loads whose destination is LDS: wait for this wave's
  // outstanding ones explicitly (s_waitcnt vmcnt(0), the other counters left alone).
  __device__ static __forceinline__ void wait_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }

  // acc[mi][ni] must be initialised by the caller.  `a` / `b` describe the tile's rows from K offset 0;
  // K must be a multiple of kSlabK and every row 16-byte aligned.  With next != nullptr the last
  // two slab periods request the first two slabs of the next K loop, which keeps one operand and
  // takes the other's rows from `next` (next_rows valid rows, same layout as the operand it replaces:
  // A unless next_is_b), and LDS stays in use on return; otherwise, with release_lds, all loads have
  // landed and every wave is past its last fragment read on return.
  __device__ static __forceinline__ void run(f32x16 (&acc)[MI][NI], const Operand& a, const Operand& b, int K,
                                             char* lds, Stream& st, const T* next, int next_rows,
                                             bool release_lds, bool next_is_b = false) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm = wave % WAVES_M;
    const int wn = wave / WAVES_M;
    const Loader L = make_loader(a, b);
    const int nslab = K / kSlabK;
    const bool stream_on = next != nullptr && nslab >= 2;
    Loader LN = L;
    if (stream_on) {
      if (next_is_b) {
        LN.b_ptr = reinterpret_cast<const char*>(next);
        LN.b_bytes = next_rows * b.row_bytes;
      } else {
        LN.a_ptr = reinterpret_cast<const char*>(next);
        LN.a_bytes = next_rows * a.row_bytes;
      }
    }

    const int fr_swz = (lane & 7) ^ ((lane >> 3) & 1);
    int xk[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) xk[kk] = ((kk * 2 + (lane >> 5)) ^ fr_swz) * 16;
    const int a_frag_off = (wm * WM + (lane & 31)) * kRowBytes;
    const int b_frag_off = BM * kRowBytes + (wn * WN + (lane & 31)) * kRowBytes;

    u32x4 af[2][MI], bf[2][NI];
    auto read_frags = [&](int set, const char* stage, int kk) {
#pragma unroll
      for (int mi = 0; mi < MI; ++mi)
        af[set][mi] = *reinterpret_cast<const u32x4*>(stage + a_frag_off + mi * 32 * kRowBytes + xk[kk]);
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
        bf[set][ni] = *reinterpret_cast<const u32x4*>(stage + b_frag_off + ni * 32 * kRowBytes + xk[kk]);
    };
    auto mma = [&](int set) {
#pragma unroll
      for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) mma_block<T>(acc[mi][ni], af[set][mi], bf[set][ni]);
    };
    constexpr int kFragReads = MI + NI;
    constexpr int kMma = MI * NI;
    constexpr int kLoads = kPassA + kPassB;
    // one K-step: `kFragReads` matrix ops each followed by one LDS read, then the rest
    auto pace_reads = [&]() {
#pragma unroll
      for (int i = 0; i < kFragReads; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, kMma - kFragReads, 0);
    };
    // one slab: `cur` holds slab s, the loads of slab s+1 into `nxt` are in flight; `ld` and
    // `ld_slab` name the slab requested into `cur` once everyone is done with it
    auto slab_body = [&](char* cur, char* nxt, const Loader& ld, int ld_slab) {
      read_frags(1, cur, 1);
      mma(0);
      pace_reads();
      read_frags(0, cur, 2);
      mma(1);
      pace_reads();
      read_frags(1, cur, 3);
      mma(0);
      pace_reads();
      __builtin_amdgcn_sched_barrier(0);
      // slab s+1 has landed in `nxt` for every wave; everyone holds the last fragments of `cur`
      wait_loads();
      __syncthreads();
      read_frags(0, nxt, 0);
      dma_slab(ld, cur, ld_slab);
      mma(1);
#pragma unroll
      for (int i = 0; i < kFragReads; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x020, (kLoads + kFragReads - 1) / kFragReads, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, kMma - kFragReads, 0);
      __builtin_amdgcn_sched_barrier(0);
    };

    char* const buf0 = lds + st.phase * kStageBytes;
    char* const buf1 = lds + (st.phase ^ 1) * kStageBytes;
    if (!st.loaded) {
      dma_slab(L, buf0, 0);
      wait_loads();
      __syncthreads();
      if (nslab > 1) dma_slab(L, buf1, 1);
    } else {
      wait_loads();
      __syncthreads();
    }
    read_frags(0, buf0, 0);
    int s = 0;
    for (; s + 2 < nslab; ++s)
      slab_body((s & 1) ? buf1 : buf0, (s & 1) ? buf0 : buf1, L, s + 2);
    // The last two slab periods have no slab of this loop left to request: they request the first
    // two slabs of the next loop, or the last slab again.  (Measured: leaving the loads out here
    // instead makes the whole loop slower, not faster.)
    for (; s < nslab; ++s)
      slab_body((s & 1) ? buf1 : buf0, (s & 1) ? buf0 : buf1, LN, stream_on ? s + 2 - nslab : nslab - 1);
    st.phase = (st.phase + nslab) & 1;
    st.loaded = stream_on;
    if (release_lds && !stream_on) {
      wait_loads();      // the repeated loads of the last slab still target LDS
      __syncthreads();
    }
  }

  // Single K loop: nothing carried over, LDS free on return.
  __device__ static __forceinline__ void run(f32x16 (&acc)[MI][NI], const Operand& a, const Operand& b, int K,
                                             char* lds) {
    Stream st;
    run(acc, a, b, K, lds, st, nullptr, 0, true);
  }
};

// The tile every GEMM-shaped kernel of the head path uses: 256 x 256 outputs per workgroup,
// 2 x kHeadWavesN wavefronts.
#ifndef CLGRPO_WAVES_N
#define CLGRPO_WAVES_N 4
#endif
constexpr int kHeadWavesN = CLGRPO_WAVES_N;
constexpr int kHeadThreads = 64 * 2 * kHeadWavesN;
template <typename T> using HeadTile = GemmTile<T, 256, 256, 2, kHeadWavesN>;

// Workgroup id -> logical work item so that the workgroups resident on one XCD
// (hardware deals consecutive ids round-robin over the 8 XCDs) own a contiguous
// range of logical items and therefore share operand tiles in that XCD's L2.
// grid must be padded to a multiple of 8; items >= n_items return -1.
__device__ __forceinline__ int xcd_remap(int bid, int grid) {
  const int per_xcd = grid >> 3;
  return (bid & 7) * per_xcd + (bid >> 3);
}

// The same for launches of several rounds (more items than the CUs hold at once; xcd_wgs = workgroups
// resident per XCD = CUs / 8, grid padded to a multiple of 8 * xcd_wgs): the hardware starts workgroups in
// id order, so the k-th batch of xcd_wgs workgroups of every XCD runs at about the same time.  Those 8
// batches get 8 consecutive blocks of the logical order: at any time all XCDs work inside one stretch of
// 8 * xcd_wgs consecutive items - the same few operand tiles of the slow dimension of grouped_tile, which
// the last-level cache then serves to all of them from one HBM read - instead of eight stretches a
// eighth of the launch apart.  Bit-identical results; measured on the forward: 32768 tokens at H = 7168
// (22 vocabulary splits, 11 rounds) 48.1 -> 45.2 ms, 16640 tokens at H = 4096 (35 splits, 9 rounds) 16.1 ->
// 15.4 ms, no change for launches of one or two rounds.  Used by the forward only: the kernel that recomputes
// d(logits) tile by tile got 6 % slower with it, the plain GEMM launches moved by less than 1 % either way.
__device__ __forceinline__ int xcd_round_remap(int bid, int xcd_wgs) {
  const int x = bid & 7, slot = bid >> 3;
  return ((slot / xcd_wgs) * 8 + x) * xcd_wgs + slot % xcd_wgs;
}

// Work item of this workgroup: xcd_wgs > 0 selects the mapping for launches of several rounds.
__device__ __forceinline__ int work_item(int xcd_wgs) {
  return xcd_wgs > 0 ? xcd_round_remap(blockIdx.x, xcd_wgs) : xcd_remap(blockIdx.x, gridDim.x);
}

// Host side: grid size for n_items work items on a device with `cus` CUs, and the xcd_wgs to hand to the
// kernel (0: one round or less, plain xcd_remap on a grid padded to a multiple of 8).
struct ItemGrid {
  int grid, xcd_wgs;
};
inline ItemGrid item_grid(int n_items, int cus) {
  const int xw = cus / 8;
  if (xw > 0 && n_items > 8 * xw) return ItemGrid{(n_items + 8 * xw - 1) / (8 * xw) * (8 * xw), xw};
  return ItemGrid{(n_items + 7) / 8 * 8, 0};
}

// Logical item -> (m tile, n tile), walking groups of `gm` m-tiles across all n
// tiles so neighbours in the logical order share A rows or B rows.
__device__ __forceinline__ void grouped_tile(int item, int n_m, int n_n, int gm, int& mt, int& nt) {
  const int per_group = gm * n_n;
  const int g = item / per_group;
  const int first_m = g * gm;
  const int rows = (n_m - first_m) < gm ? (n_m - first_m) : gm;
  const int in_g = item - g * per_group;
  mt = first_m + in_g % rows;
  nt = in_g / rows;
}

}  // namespace clgrpo
