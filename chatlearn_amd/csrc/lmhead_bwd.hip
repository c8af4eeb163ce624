// Backward of the fused lm_head + log-softmax statistics.
//
// Per chunk of tokens (the chunk length is set by the workspace the caller gives):
//   1. dz kernel: recompute a z^T tile [256 vocab x 256 tokens] on the matrix cores
//      exactly as the forward does, turn it into d(logits) with the stored lse,
//      and write it in both orientations, dz[token][vocab] and dzT[vocab][token].
//   2. dhidden[chunk] = dz * W        as an NT GEMM against WT = W^T (built once per call)
//   3. dW (+)= dzT * hidden[chunk]    as an NT GEMM against hidT = hidden[chunk]^T, fp32 out
// Every contraction runs through the same K-contiguous MFMA tile (gemm_core.hpp).
//
// Algorithmic work: 4*T*H*V flop (dhidden + dW); the z recomputation (2*T*H*V) is overhead.
#include "common.hpp"
#include "gemm_core.hpp"

namespace clgrpo {

int validate_head_shape(const char* who, int64_t T, int64_t H, int64_t V, int32_t dtype);

constexpr float kLog2e = 1.4426950408889634f;

template <typename T> struct Pack4;
template <> struct Pack4<float> {
  typedef float4 type;
  __device__ static __forceinline__ type make(float a, float b, float c, float d) { return make_float4(a, b, c, d); }
};
template <> struct Pack4<__bf16> {
  typedef uint2 type;
  __device__ static __forceinline__ type make(float a, float b, float c, float d) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    bf16x2 lo = {(__bf16)a, (__bf16)b};
    bf16x2 hi = {(__bf16)c, (__bf16)d};
    return make_uint2(__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi));
  }
};

struct DzParams {
  const void* hidden;   // chunk base: [Tc, H]
  const void* weight;   // [V, H]
  const int64_t* labels;  // chunk base
  int64_t label_offset;   // first vocabulary id of `weight` (0 unless this is a vocabulary shard)
  const float* lse;
  const float* entropy;   // or nullptr
  const float* g_lp;
  const float* g_ent;     // or nullptr
  int Tc;       // valid tokens in the chunk
  int ldt;      // K extent of dzT = Tc rounded up to 64
  int H, V;
  int ldv;      // K extent of dz = V rounded up to 64
  int n_tb, n_vt;
  float c, inv_temperature;
  void* dz;     // Tc x ldv, K-blocked (see blocked_index)
  void* dzT;    // V x ldt, K-blocked
};

template <typename T>
__global__ __launch_bounds__(kHeadThreads) void lmhead_dz_kernel(DzParams p) {
  using Tile = HeadTile<T>;
  constexpr int MI = Tile::MI, NI = Tile::NI, WM = Tile::WM, WN = Tile::WN;
  extern __shared__ __align__(16) char lds[];

  const int item = xcd_remap(blockIdx.x, gridDim.x);
  if (item >= p.n_tb * p.n_vt) return;
  int vt, tb;
  grouped_tile(item, p.n_vt, p.n_tb, 4, vt, tb);

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave % 2, wn = wave / 2;
  const int t0 = tb * 256, v0 = vt * 256;
  const int b_rows = (p.Tc - t0) < 256 ? (p.Tc - t0) : 256;
  const int a_rows = (p.V - v0) < 256 ? (p.V - v0) : 256;
  const T* hidden = static_cast<const T*>(p.hidden) + (int64_t)t0 * p.H;
  const T* weight = static_cast<const T*>(p.weight) + (int64_t)v0 * p.H;

  // Per-token coefficients.  Tokens past the chunk get zero gradient and a huge lse, so p = 0.
  int lab[NI], tl[NI];
  float lse2[NI], lse[NI], glp[NI], gent[NI], ent[NI];
  bool any_grad = false;
#pragma unroll
  for (int ni = 0; ni < NI; ++ni) {
    tl[ni] = t0 + wn * WN + ni * 32 + (lane & 31);
    const bool ok = tl[ni] < p.Tc;
    lab[ni] = -1;
    if (ok) {
      const int64_t rel = p.labels[tl[ni]] - p.label_offset;   // a label outside these rows matches nothing
      if (rel >= 0 && rel < p.V) lab[ni] = (int)rel;
    }
    lse[ni] = ok ? p.lse[tl[ni]] : 1e30f;
    lse2[ni] = lse[ni] * kLog2e;
    glp[ni] = ok ? p.g_lp[tl[ni]] : 0.f;
    gent[ni] = (ok && p.g_ent) ? p.g_ent[tl[ni]] : 0.f;
    ent[ni] = (ok && p.g_ent) ? p.entropy[tl[ni]] : 0.f;
    any_grad |= (glp[ni] != 0.f) | (gent[ni] != 0.f);
  }
  // A token block whose upstream gradients are all zero (e.g. prompt-only rows) needs no GEMM.
  const bool block_live = __syncthreads_or(any_grad);

  f32x16 acc[MI][NI];
#pragma unroll
  for (int mi = 0; mi < MI; ++mi)
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.f;
  if (block_live)
    Tile::run(acc, Tile::Operand::row_major(weight, p.H, a_rows), Tile::Operand::row_major(hidden, p.H, b_rows), p.H, lds);

  T* dz = static_cast<T*>(p.dz);
  T* dzT = static_cast<T*>(p.dzT);
  const float it = p.inv_temperature;
#pragma unroll
  for (int ni = 0; ni < NI; ++ni) {
    const int rel = lab[ni] - (v0 + wm * WM);
    const float hot = it * glp[ni];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float d[4];
        const int row0 = wm * WM + mi * 32 + 8 * q + 4 * (lane >> 5);  // tile row of r = 4q
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float zraw = acc[mi][ni][4 * q + j];
          const float pr = __builtin_amdgcn_exp2f(fmaf(zraw, p.c, -lse2[ni]));
          const float logp = fmaf(zraw, it, -lse[ni]);
          // dz = it * ( glp*(1[v==y] - p) - gent * p * (logp + ent) )
          float v = -it * pr * fmaf(gent[ni], logp + ent[ni], glp[ni]);
          if (rel == (row0 - wm * WM) + j) v += hot;
          if (row0 + j >= a_rows || !block_live) v = 0.f;   // vocabulary padding columns / dead block
          d[j] = v;
        }
        const int v_idx = v0 + row0;
        if (tl[ni] < p.Tc && v_idx < p.ldv) {
          typedef typename Pack4<T>::type P4;
          *reinterpret_cast<P4*>(dz + blocked_index<T>(tl[ni], v_idx, p.ldv / Tile::kSlabK)) =
              Pack4<T>::make(d[0], d[1], d[2], d[3]);
        }
        if (tl[ni] < p.ldt) {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (v_idx + j < p.V) dzT[blocked_index<T>(v_idx + j, tl[ni], p.ldt / Tile::kSlabK)] = (T)d[j];
        }
      }
    }
  }
}

// d(logits) from kept logits, in place, plus its transpose.  One workgroup per 32 KB unit of the kept
// logits (256 token rows x one 128-byte slab of vocabulary, z-native layout, see ZNative): every thread
// reads its 128 bytes of the unit, forms dz with its rows' coefficients and drops the values into two LDS
// tiles, [token][vocab] and [vocab][token]; after a barrier the first goes back over the unit as the
// K-blocked dz operand (the unit's 32 KB are exactly that operand's piece for these rows and this slab)
// and the second to the K-blocked dzT operand (per 64-token slab one contiguous piece of 64 vocabulary
// rows).  All global accesses are 16 bytes per lane and contiguous per wavefront.  HBM-bound: reads 1x,
// writes 2x the chunk.
struct DzFromZParams {
  void* z;            // Tc x ldv: in kept logits (z-native, KeptLogit<T>), out dz (K-blocked, T)
  void* dzT;          // V x ldt, K-blocked
  const int64_t* labels;
  int64_t label_offset;
  const float* lse;
  const float* entropy;
  const float* g_lp;
  const float* g_ent;
  int Tc, ldt, V, ldv;
  float c, inv_temperature;
};

template <typename T>
__global__ __launch_bounds__(256) void dz_from_z_kernel(DzFromZParams p) {
  typedef typename KeptLogit<T>::type ZT;
  typedef ZNative<ZT> ZL;
  static_assert(sizeof(ZT) == sizeof(T), "d(logits) overwrites the kept logits in place");
  constexpr int E = ZL::kSlabElems;                 // vocabulary entries of this unit (64 or 32)
  constexpr int VEC = 16 / (int)sizeof(T);          // elements per 16-byte piece
  constexpr int kSub = 8 * ZL::VSUB;                // 32x32 sub-blocks per unit
  constexpr int kSubPerWave = kSub / 4;
  constexpr int kTPitch = kBlockRows * (int)sizeof(T) + 16;   // bytes per vocabulary row of the transposed tile
  // one LDS region, used twice: [token R][vocab c] with the 16-byte chunks XOR-swizzled by R % 8 (32 KB),
  // then [vocab c][token R] with padded rows
  __shared__ __align__(16) char tile[E * kTPitch > kBlockRows * kRowBytes ? E * kTPitch : kBlockRows * kRowBytes];
  const int rb = blockIdx.x, ks = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int h = lane >> 5, t32 = lane & 31;
  const int64_t n_kslab = p.ldv / E;
  char* unit = static_cast<char*>(p.z) + ((int64_t)rb * n_kslab + ks) * ZL::kUnitBytes;
  const float it = p.inv_temperature;

  u32x4 raw[kSubPerWave][ZL::PIECES];
#pragma unroll
  for (int s = 0; s < kSubPerWave; ++s)
#pragma unroll
    for (int j = 0; j < ZL::PIECES; ++j)
      raw[s][j] = *reinterpret_cast<const u32x4*>(unit + (wave + 4 * s) * (ZL::PIECES * 1024) + j * 1024 + lane * 16);

  // this lane's 16 values of each of its sub-blocks, as d(logits) in the operand dtype
  T dz[kSubPerWave][16];
#pragma unroll
  for (int s = 0; s < kSubPerWave; ++s) {
    const int sb = wave + 4 * s;
    const int R = (sb / ZL::VSUB) * 32 + t32;       // token row inside the unit
    const int c0 = (sb % ZL::VSUB) * 32;            // first vocabulary entry of the sub-block inside the unit
    const int t = rb * kBlockRows + R;
    float glp = 0.f, gen = 0.f, lse = 0.f, ent = 0.f;
    int lab = -1;
    if (t < p.Tc) {
      glp = p.g_lp[t];
      gen = p.g_ent ? p.g_ent[t] : 0.f;
      lse = p.lse[t];
      ent = p.g_ent ? p.entropy[t] : 0.f;
      const int64_t rel = p.labels[t] - p.label_offset - ((int64_t)ks * E + c0);   // relative to the sub-block
      lab = (rel >= 0 && rel < 32) ? (int)rel : -1;
    }
    const bool live = glp != 0.f || gen != 0.f;     // rows past the chunk and rows without a gradient give zeros
    const float lse2 = lse * kLog2e;
#pragma unroll
    for (int j = 0; j < ZL::PIECES; ++j) {
      const ZT* in = reinterpret_cast<const ZT*>(&raw[s][j]);
#pragma unroll
      for (int e = 0; e < ZL::kPerPiece; ++e) {
        const int c32 = ZL::col_of(h, j, e);
        float d = 0.f;
        if (live) {
          const float zraw = (float)in[e];
          const float pr = __builtin_amdgcn_exp2f(fmaf(zraw, p.c, -lse2));
          const float logp = fmaf(zraw, it, -lse);
          d = -it * pr * fmaf(gen, logp + ent, glp);
          if (c32 == lab) d += it * glp;
          if (ks * E + c0 + c32 >= p.V) d = 0.f;    // vocabulary padding columns
        }
        dz[s][j * ZL::kPerPiece + e] = (T)d;
      }
    }
  }

  // pass 1: [token][vocab] through LDS, back over the unit as the K-blocked dz operand
#pragma unroll
  for (int s = 0; s < kSubPerWave; ++s) {
    const int sb = wave + 4 * s;
    const int R = (sb / ZL::VSUB) * 32 + t32;
    const int c0 = (sb % ZL::VSUB) * 32;
    // registers 4m .. 4m+3 are consecutive vocabulary entries: 4 * sizeof(T) bytes of the token's row
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int byte = (c0 + 8 * m + 4 * h) * (int)sizeof(T);
      char* dst = tile + R * kRowBytes + (((byte >> 4) ^ (R & 7)) << 4) + (byte & 15);
      if (sizeof(T) == 2) *reinterpret_cast<uint2*>(dst) = *reinterpret_cast<const uint2*>(&dz[s][4 * m]);
      else *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(&dz[s][4 * m]);
    }
  }
  __syncthreads();     // also: every thread has its part of the unit in registers before anyone overwrites it
  for (int pc = threadIdx.x; pc < kBlockRows * kChunksPerRow; pc += 256) {
    const int R = pc >> 3, q = pc & 7;              // row R, 16-byte chunk q of the operand is piece R * 8 + q
    *reinterpret_cast<u32x4*>(unit + pc * 16) = *reinterpret_cast<const u32x4*>(tile + R * kRowBytes + ((q ^ (R & 7)) << 4));
  }
  __syncthreads();

  // pass 2: [vocab][token] through LDS, out to the K-blocked dzT operand (vocabulary row v, token slabs of E)
#pragma unroll
  for (int s = 0; s < kSubPerWave; ++s) {
    const int sb = wave + 4 * s;
    const int R = (sb / ZL::VSUB) * 32 + t32;
    const int c0 = (sb % ZL::VSUB) * 32;
#pragma unroll
    for (int r = 0; r < 16; ++r)
      *reinterpret_cast<T*>(tile + (c0 + 8 * (r >> 2) + 4 * h + (r & 3)) * kTPitch + R * (int)sizeof(T)) = dz[s][r];
  }
  __syncthreads();
  T* dzT = static_cast<T*>(p.dzT);
  const int64_t n_tslab = p.ldt / E;
  for (int pc = threadIdx.x; pc < E * (kBlockRows / VEC); pc += 256) {
    const int sl = pc / (E * kChunksPerRow);        // token slab inside the unit
    const int c = (pc / kChunksPerRow) % E;         // vocabulary row inside the unit
    const int q = pc % kChunksPerRow;
    const int v = ks * E + c;
    const int tok = rb * kBlockRows + sl * E + q * VEC;
    if (v < p.V && tok < p.ldt)
      *reinterpret_cast<u32x4*>(dzT + blocked_index<T>(v, tok, n_tslab)) =
          *reinterpret_cast<const u32x4*>(tile + c * kTPitch + (sl * E + q * VEC) * (int)sizeof(T));
  }
}

// C (+)= A B^T with A [M x K] and B [N x K] K-blocked, C row-major in one of two orientations:
//   kMContig = false: C[m][n], ld = ldc.  The N index runs along the lanes of an accumulator block
//     (see gemm_core.hpp), so one store instruction writes whole 128-byte lines (32 lanes x 4 bytes,
//     two rows): the orientation for fp32 outputs (dW: A = dz^T, B = hidden^T).
//   kMContig = true:  C[n][m], ld = ldc.  The M index runs along a lane's registers, so a lane owns 4
//     consecutive elements of a row per register quad: one 8-byte access instead of four 2-byte ones
//     for 16-bit outputs (dhidden: A = W^T, B = dz).
// Measured on the Qwen3-8B head: fp32 out, C[n][m] with 16-byte accesses (32 rows x 32 bytes per
// instruction) is 4 % slower than C[m][n] with 4-byte ones (2 rows x 128 bytes): whole lines matter
// more than the number of memory instructions; bf16 out gains 2 % from the 8-byte accesses.
struct GemmParams {
  const void* A;      // M x K, K-blocked with a_kslabs slabs per row block
  const void* B;      // N x K, K-blocked with b_kslabs slabs per row block
  void* C;
  int64_t a_kslabs, b_kslabs, ldc;
  int M, N, K;
  int n_mt, n_nt;
  int accumulate;
  int k_split;        // > 1: work item = (tile, K range); fp32 partial tiles go to `partial`
  int k_per_split;    // K extent of one range, a multiple of the slab
  int n_walk;         // > 0: workgroups walk runs of tiles (see gemm_nt_kernel); needs k_split == 1
  float* partial;     // [k_split] copies of C's shape in fp32, densely packed (row stride N or M)
};

// Addresses of a 256 x 256 output tile for the accumulator layout: a range-checked buffer descriptor over
// the tile's valid rows, one per-lane byte offset per 32-wide block of the lane dimension, and an offset
// per accumulator register (kMContig: per register quad, a compile-time constant; otherwise a uniform
// multiple of the row pitch, handed to the instruction as its scalar offset).  Along the lane dimension
// (n) elements outside the tile get a per-lane offset far outside the descriptor: loads of them give 0
// and stores are dropped.  Along the register dimension (m) nothing relies on the range check, because the
// scalar offset is not part of it: kMContig skips whole quads (its M extents are multiples of 8), and the
// other orientation tests every row against the tile's valid rows unless the tile is a full one.
template <typename T, typename OutT, bool kMContig>
struct TileAddr {
  using Tile = HeadTile<T>;
  static constexpr int ES = (int)sizeof(OutT);
  __amdgpu_buffer_rsrc_t rsrc;
  int voff[Tile::NI];
  int row_bytes, m_first, a_rows;
  int row_lim;   // valid rows from this lane's first row on: register with row offset dm is inside iff dm < row_lim
  __device__ __forceinline__ TileAddr(OutT* base, int64_t ld, int m0, int n0, int a_rows_, int b_rows) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm = wave % 2, wn = wave / 2;
    row_bytes = (int)(ld * (int64_t)ES);
    m_first = wm * Tile::WM;
    a_rows = a_rows_;
    row_lim = a_rows_ - (m_first + 4 * (lane >> 5));
    const int rows = kMContig ? b_rows : a_rows_, cols = kMContig ? a_rows_ : b_rows;
    const int bytes = rows > 0 ? (rows - 1) * row_bytes + cols * ES : 0;
    OutT* origin = kMContig ? base + (int64_t)n0 * ld + m0 : base + (int64_t)m0 * ld + n0;
    rsrc = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<char*>(origin), 0, bytes, 0x00020000);
#pragma unroll
    for (int ni = 0; ni < Tile::NI; ++ni) {
      const int n = wn * Tile::WN + ni * 32 + (lane & 31);
      const int m = m_first + 4 * (lane >> 5);
      voff[ni] = n < b_rows ? (kMContig ? n * row_bytes + m * ES : m * row_bytes + n * ES) : 0x7f000000;
    }
  }
  // offset of register r of block row mi from voff (rows 8 * (r / 4) + r % 4 of the block, plus the lane half's 4)
  __device__ __forceinline__ int reg_off(int mi, int r) const {
    const int dm = mi * 32 + 8 * (r >> 2) + (r & 3);
    return kMContig ? dm * ES : dm * row_bytes;
  }
  __device__ __forceinline__ bool quad_ok(int mi, int q) const { return m_first + mi * 32 + 8 * q < a_rows; }
  // row of register r of block row mi, relative to this lane's first row
  __device__ static __forceinline__ int row_delta(int mi, int r) { return mi * 32 + 8 * (r >> 2) + (r & 3); }
  __device__ __forceinline__ bool full_rows() const { return a_rows == Tile::BM; }
};

__device__ __forceinline__ float elem_load(const __amdgpu_buffer_rsrc_t& rsrc, int voff, int soff, float*) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, voff, soff, 0));
}
__device__ __forceinline__ float elem_load(const __amdgpu_buffer_rsrc_t& rsrc, int voff, int soff, __bf16*) {
  return (float)__builtin_bit_cast(__bf16, __builtin_amdgcn_raw_buffer_load_b16(rsrc, voff, soff, 0));
}
__device__ __forceinline__ void elem_store(float v, const __amdgpu_buffer_rsrc_t& rsrc, int voff, int soff, float*) {
  __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned int, v), rsrc, voff, soff, 0);
}
__device__ __forceinline__ void elem_store(float v, const __amdgpu_buffer_rsrc_t& rsrc, int voff, int soff, __bf16*) {
  __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, (__bf16)v), rsrc, voff, soff, 0);
}
__device__ __forceinline__ void quad_load(f32x16& a, int q, const __amdgpu_buffer_rsrc_t& rsrc, int voff, float*) {
  const f32x4 v = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, 0, 0));
  a[4 * q] = v[0]; a[4 * q + 1] = v[1]; a[4 * q + 2] = v[2]; a[4 * q + 3] = v[3];
}
__device__ __forceinline__ void quad_load(f32x16& a, int q, const __amdgpu_buffer_rsrc_t& rsrc, int voff, __bf16*) {
  typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
  const bf16x4 v = __builtin_bit_cast(bf16x4, __builtin_amdgcn_raw_buffer_load_b64(rsrc, voff, 0, 0));
  a[4 * q] = (float)v[0]; a[4 * q + 1] = (float)v[1]; a[4 * q + 2] = (float)v[2]; a[4 * q + 3] = (float)v[3];
}
__device__ __forceinline__ void quad_store(const f32x16& a, int q, const __amdgpu_buffer_rsrc_t& rsrc, int voff, float*) {
  const f32x4 v = {a[4 * q], a[4 * q + 1], a[4 * q + 2], a[4 * q + 3]};
  __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), rsrc, voff, 0, 0);
}
__device__ __forceinline__ void quad_store(const f32x16& a, int q, const __amdgpu_buffer_rsrc_t& rsrc, int voff, __bf16*) {
  typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
  typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
  const bf16x4 v = {(__bf16)a[4 * q], (__bf16)a[4 * q + 1], (__bf16)a[4 * q + 2], (__bf16)a[4 * q + 3]};
  __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2, v), rsrc, voff, 0, 0);
}

template <typename T, typename OutT, bool kMContig, typename AccT>
__device__ __forceinline__ void tile_load(const TileAddr<T, OutT, kMContig>& at, AccT& acc) {
  using Tile = HeadTile<T>;
  const bool full = at.full_rows();   // uniform over the workgroup
#pragma unroll
  for (int ni = 0; ni < Tile::NI; ++ni)
#pragma unroll
    for (int mi = 0; mi < Tile::MI; ++mi)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (!at.quad_ok(mi, q)) continue;
        if (kMContig) quad_load(acc[mi][ni], q, at.rsrc, at.voff[ni] + at.reg_off(mi, 4 * q), (OutT*)nullptr);
        else if (full) {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            acc[mi][ni][4 * q + i] = elem_load(at.rsrc, at.voff[ni], at.reg_off(mi, 4 * q + i), (OutT*)nullptr);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (at.row_delta(mi, 4 * q + i) < at.row_lim)
              acc[mi][ni][4 * q + i] = elem_load(at.rsrc, at.voff[ni], at.reg_off(mi, 4 * q + i), (OutT*)nullptr);
        }
      }
}

template <typename T, typename OutT, bool kMContig, typename AccT>
__device__ __forceinline__ void tile_store(const TileAddr<T, OutT, kMContig>& at, const AccT& acc) {
  using Tile = HeadTile<T>;
  const bool full = at.full_rows();   // uniform over the workgroup
#pragma unroll
  for (int ni = 0; ni < Tile::NI; ++ni)
#pragma unroll
    for (int mi = 0; mi < Tile::MI; ++mi)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (!at.quad_ok(mi, q)) continue;
        if (kMContig) quad_store(acc[mi][ni], q, at.rsrc, at.voff[ni] + at.reg_off(mi, 4 * q), (OutT*)nullptr);
        else if (full) {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            elem_store(acc[mi][ni][4 * q + i], at.rsrc, at.voff[ni], at.reg_off(mi, 4 * q + i), (OutT*)nullptr);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (at.row_delta(mi, 4 * q + i) < at.row_lim)
              elem_store(acc[mi][ni][4 * q + i], at.rsrc, at.voff[ni], at.reg_off(mi, 4 * q + i), (OutT*)nullptr);
        }
      }
}

// Accumulators of output tile (m0, n0) before its K loop: zeros, or - when the GEMM adds to C and one
// workgroup owns the whole K range of the tile - the tile's current contents.  Reading C here instead of
// in the epilogue puts the loads' latency in front of the K loop, where the first operand slabs are in
// flight anyway, and leaves the epilogue a pure store.
template <typename T, typename OutT, bool kMContig>
__device__ __forceinline__ void gemm_init_tile(const GemmParams& p, f32x16 (&acc)[HeadTile<T>::MI][HeadTile<T>::NI],
                                               int m0, int n0, int a_rows, int b_rows) {
  using Tile = HeadTile<T>;
#pragma unroll
  for (int mi = 0; mi < Tile::MI; ++mi)
#pragma unroll
    for (int ni = 0; ni < Tile::NI; ++ni)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.f;
  if (p.accumulate && p.k_split == 1) {
    const TileAddr<T, OutT, kMContig> at(static_cast<OutT*>(p.C), p.ldc, m0, n0, a_rows, b_rows);
    tile_load(at, acc);
  }
}

// Output tile from the accumulators: C = acc (the accumulators already hold C's previous contents
// when the GEMM adds to it, see gemm_init_tile), or the fp32 partial of K range `ks`.
template <typename T, typename OutT, bool kMContig>
__device__ __forceinline__ void gemm_store_tile(const GemmParams& p, f32x16 (&acc)[HeadTile<T>::MI][HeadTile<T>::NI],
                                                int m0, int n0, int a_rows, int b_rows, int ks) {
  if (p.k_split > 1) {
    const TileAddr<T, float, kMContig> at(p.partial + (int64_t)ks * p.M * p.N, kMContig ? p.M : p.N, m0, n0, a_rows, b_rows);
    tile_store(at, acc);
    return;
  }
  const TileAddr<T, OutT, kMContig> at(static_cast<OutT*>(p.C), p.ldc, m0, n0, a_rows, b_rows);
  tile_store(at, acc);
}

// Work item = (walk, fixed tile) when n_walk > 0: the workgroup keeps one operand's tile (A's m tile
// when C is [n][m], B's n tile when C is [m][n]) and walks a contiguous run of tiles of the other, so the
// K loops stream into each other (the next tile's first slabs are requested while the current tile
// finishes and is stored).  Otherwise work item = (K range, m tile, n tile), one K loop per workgroup.
template <typename T, typename OutT, bool kMContig>
__global__ __launch_bounds__(kHeadThreads) void gemm_nt_kernel(GemmParams p) {
  using Tile = HeadTile<T>;
  constexpr int MI = Tile::MI, NI = Tile::NI;
  constexpr int64_t kSlabElems = (int64_t)kBlockRows * Tile::kSlabK;   // elements of one block's slab
  extern __shared__ __align__(16) char lds[];

  int item = xcd_remap(blockIdx.x, gridDim.x);
  f32x16 acc[MI][NI];
  if (p.n_walk > 0) {
    const int n_fixed = kMContig ? p.n_mt : p.n_nt;       // tiles of the operand that stays
    const int n_moving = kMContig ? p.n_nt : p.n_mt;      // tiles of the operand that is walked
    if (item >= p.n_walk * n_fixed) return;
    int walk, ft;
    grouped_tile(item, p.n_walk, n_fixed, 4, walk, ft);
    const int w_begin = (int)((int64_t)walk * n_moving / p.n_walk);
    const int w_end = (int)((int64_t)(walk + 1) * n_moving / p.n_walk);
    typename Tile::Stream st;
    for (int wt = w_begin; wt < w_end; ++wt) {
      const int mt = kMContig ? ft : wt, nt = kMContig ? wt : ft;
      const int m0 = mt * 256, n0 = nt * 256;
      const int a_rows = (p.M - m0) < 256 ? (p.M - m0) : 256;
      const int b_rows = (p.N - n0) < 256 ? (p.N - n0) : 256;
      const int moving_left = (kMContig ? p.N : p.M) - (wt + 1) * 256;
      const int next_rows = moving_left < 256 ? moving_left : 256;
      const T* A = static_cast<const T*>(p.A) + (int64_t)mt * p.a_kslabs * kSlabElems;
      const T* B = static_cast<const T*>(p.B) + (int64_t)nt * p.b_kslabs * kSlabElems;
      const T* next = kMContig ? B + p.b_kslabs * kSlabElems : A + p.a_kslabs * kSlabElems;
      gemm_init_tile<T, OutT, kMContig>(p, acc, m0, n0, a_rows, b_rows);
      Tile::run(acc, Tile::Operand::blocked(A, a_rows), Tile::Operand::blocked(B, b_rows), p.K, lds, st,
                (wt + 1 < w_end) ? next : nullptr, next_rows, true, /*next_is_b=*/kMContig);
      gemm_store_tile<T, OutT, kMContig>(p, acc, m0, n0, a_rows, b_rows, 0);
    }
    return;
  }

  if (item >= p.n_mt * p.n_nt * p.k_split) return;
  const int ks = item / (p.n_mt * p.n_nt);
  item -= ks * (p.n_mt * p.n_nt);
  int mt, nt;
  grouped_tile(item, p.n_mt, p.n_nt, 8, mt, nt);
  const int m0 = mt * 256, n0 = nt * 256;
  const int a_rows = (p.M - m0) < 256 ? (p.M - m0) : 256;
  const int b_rows = (p.N - n0) < 256 ? (p.N - n0) : 256;
  const int k0 = ks * p.k_per_split;
  const int k_len = (p.K - k0) < p.k_per_split ? (p.K - k0) : p.k_per_split;
  gemm_init_tile<T, OutT, kMContig>(p, acc, m0, n0, a_rows, b_rows);

  const int64_t s0 = k0 / Tile::kSlabK;   // first slab of this K range
  Tile::run(acc, Tile::Operand::blocked(static_cast<const T*>(p.A) + ((int64_t)mt * p.a_kslabs + s0) * kSlabElems, a_rows),
            Tile::Operand::blocked(static_cast<const T*>(p.B) + ((int64_t)nt * p.b_kslabs + s0) * kSlabElems, b_rows),
            k_len, lds);
  gemm_store_tile<T, OutT, kMContig>(p, acc, m0, n0, a_rows, b_rows, ks);
}

template <typename OutT> __device__ __forceinline__ OutT cvt_out(float v);
template <> __device__ __forceinline__ float cvt_out<float>(float v) { return v; }
template <> __device__ __forceinline__ __bf16 cvt_out<__bf16>(float v) { return (__bf16)v; }

// C (+)= sum over splits of partial[s], each a dense copy of C's shape with `cols` elements per row
template <typename OutT>
__global__ void splitk_reduce_kernel(const float* __restrict__ partial, int k_split, int64_t MN, int cols, OutT* C,
                                     int64_t ldc, int accumulate) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < MN; i += (int64_t)gridDim.x * blockDim.x) {
    float v = 0.f;
    for (int s = 0; s < k_split; ++s) v += partial[(int64_t)s * MN + i];
    const int64_t row = i / cols, col = i - row * cols;
    OutT* dst = C + row * ldc + col;
    if (accumulate) v += (float)*dst;
    *dst = cvt_out<OutT>(v);
  }
}

// dst(c, r) = src[r][c] for r < R, c < C and 0 for R <= r < ld_dst, where dst is the K-blocked
// operand with C rows and ld_dst K elements (see blocked_index).  64x64 tiles, 16-byte accesses on
// both sides (C and ld_src are multiples of 32 elements here, so a 16-byte piece never straddles an edge).
template <typename T>
__global__ __launch_bounds__(256) void transpose_block_kernel(const T* __restrict__ src, int64_t ld_src,
                                                              T* __restrict__ dst, int64_t ld_dst, int R, int C) {
  constexpr int VEC = 16 / (int)sizeof(T);       // elements per 16-byte access
  constexpr int CPR = 64 / VEC;                  // accesses per 64-wide tile row
  constexpr int RPP = 256 / CPR;                 // tile rows covered per pass
  constexpr int kE = kRowBytes / (int)sizeof(T);
  __shared__ T tile[64][64 + VEC];               // [c][r], padded rows
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const int q = threadIdx.x % CPR, row = threadIdx.x / CPR;
  for (int rr = row; rr < 64; rr += RPP) {
    const int r = r0 + rr, c = c0 + q * VEC;
    alignas(16) T vals[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) vals[j] = (T)0.f;
    if (r < R && c < C) *reinterpret_cast<u32x4*>(vals) = *reinterpret_cast<const u32x4*>(src + (int64_t)r * ld_src + c);
#pragma unroll
    for (int j = 0; j < VEC; ++j) tile[q * VEC + j][rr] = vals[j];
  }
  __syncthreads();
  for (int cc = row; cc < 64; cc += RPP) {
    const int c = c0 + cc, r = r0 + q * VEC;
    if (c < C && r < ld_dst)
      *reinterpret_cast<u32x4*>(dst + blocked_index<T>(c, r, ld_dst / kE)) = *reinterpret_cast<const u32x4*>(&tile[cc][q * VEC]);
  }
}

// K ranges per tile that fill `cus` CUs best (1 = no split): work items = tiles x ranges, and a launch
// takes ceil(items / cus) rounds.  At most kMaxKSplit ranges, each at least 8 slabs long and none empty,
// and at most what `partial_bytes` can hold of fp32 partial tiles.
constexpr int kMaxKSplit = 16;
static int pick_k_split(int tiles, int M, int N, int K, int slab, size_t partial_bytes, int cus) {
  int best = 1;
  double best_eff = 0.0;
  for (int s = 1; s <= kMaxKSplit; ++s) {
    if (s > 1) {
      if ((size_t)s * M * N * sizeof(float) > partial_bytes || K / s < 8 * slab) break;
      const int64_t per = round_up64((K + s - 1) / s, slab);
      if ((int64_t)(s - 1) * per >= K) continue;     // rounding the range up to whole slabs would leave the last one empty
    }
    const long units = (long)tiles * s;
    const double eff = (double)units / (double)(((units + cus - 1) / cus) * cus);
    if (eff > best_eff + 0.04) { best_eff = eff; best = s; }   // a split must buy more than 4 % to be worth its extra pass
  }
  return best;
}

// How the dhidden GEMM (C[n][m], M = H output columns, N = token rows, K = vocabulary) is launched.  Its tile
// count rarely fills whole rounds of one workgroup per CU; cutting K into ranges (fp32 partial tiles, summed
// by a second pass) repairs that at the price of the partials' traffic.  When the tiles exceed one round the
// cheaper repair is to cut the token rows instead: a bulk launch over whole rounds of tiles without any K
// split, and a second launch over the remaining rows with the K split those few tiles want.
struct DhPlan {
  int bulk_nt;       // n tiles (256 token rows each) of the bulk launch; 0: one launch over all rows
  int k_split;       // K ranges of the single launch, or of the tail launch when bulk_nt > 0
  size_t partial_bytes;
};

static DhPlan plan_dhidden(int64_t rows, int64_t H, int64_t K, int slab, int cus, size_t partial_cap) {
  DhPlan pl{0, 1, 0};
  if (rows <= 0) return pl;
  const int n_mt = (int)((H + 255) / 256), n_nt = (int)((rows + 255) / 256);
  const int tiles = n_mt * n_nt;
  const long k_slabs = (K + slab - 1) / slab;
  auto cost = [&](long items, int s) {        // rounds x slabs per range, plus 2 % for the partials' traffic
    const long rounds = (items * s + cus - 1) / cus;
    const double c = (double)rounds * (double)((k_slabs + s - 1) / s);
    return s > 1 ? c * 1.02 : c;
  };
  const int s_one = pick_k_split(tiles, (int)H, (int)rows, (int)K, slab, partial_cap, cus);
  pl.k_split = s_one;
  double best = cost(tiles, s_one);
  const int per_round_n = cus / n_mt;
  if (per_round_n >= 1 && n_nt > per_round_n && n_nt % per_round_n != 0) {
    const int bulk_nt = n_nt / per_round_n * per_round_n;
    const int64_t tail_rows = rows - (int64_t)bulk_nt * 256;
    const int tail_tiles = (n_nt - bulk_nt) * n_mt;
    const int s_tail = pick_k_split(tail_tiles, (int)H, (int)tail_rows, (int)K, slab, partial_cap, cus);
    const double two = cost((long)bulk_nt * n_mt, 1) + cost(tail_tiles, s_tail) + 0.01 * (double)k_slabs;
    if (two < 0.98 * best) {
      pl.bulk_nt = bulk_nt;
      pl.k_split = s_tail;
      pl.partial_bytes = s_tail > 1 ? (size_t)s_tail * tail_rows * H * sizeof(float) : 0;
      return pl;
    }
  }
  pl.partial_bytes = s_one > 1 ? (size_t)s_one * rows * H * sizeof(float) : 0;
  return pl;
}

// Bytes of fp32 split-K partials the dhidden GEMM of `rows` tokens wants (planned for a 256-CU device, so
// that the workspace size does not depend on the device in use; a launch takes fewer ranges if they do not fit).
static size_t dhidden_partial_bytes(int64_t rows, int64_t H, int64_t ldv, int slab) {
  return plan_dhidden(rows, H, ldv, slab, 256, (size_t)1 << 30).partial_bytes;
}

// How the dW GEMM (C[m][n], M = vocabulary rows, N = H, K = the chunk's tokens) is launched.  With many more tiles
// than CUs its workgroups keep one tile of hidden^T and walk runs of vocabulary tiles (see gemm_nt_kernel); the walks
// are as long as the longest run, so when the vocabulary tiles do not divide by the number of walks the last
// `n_mt % n_walk` of them keep a sixteenth of the chip busy for a whole tile period (594 tiles on 16 walks: runs of
// 37 and 38).  The repair is the one of the dhidden GEMM: a bulk launch whose walks are all equally long, and a second
// launch over the remaining vocabulary tiles cut into K ranges that fill the CUs (fp32 partial tiles, summed by a small
// pass).  The partials' traffic (written and read once) is priced in, in slab periods of one tile.
struct DwPlan {
  int n_walk;        // walks of the (bulk) launch; 0: one workgroup per tile, no bulk / tail split
  int bulk_mt;       // vocabulary tiles of the bulk launch; 0: one launch over all of them
  int k_split;       // K ranges of the tail launch
  size_t partial_bytes;
};

static DwPlan plan_dweight(int64_t V, int64_t H, int64_t K, int slab, int cus, size_t partial_cap) {
  DwPlan pl{0, 0, 1, 0};
  const int n_mt = (int)((V + 255) / 256), n_nt = (int)((H + 255) / 256);
  if (!(n_nt <= cus && (long)n_mt * n_nt >= 4L * cus && K >= 2 * slab)) return pl;
  int n_walk = cus / n_nt;
  if (n_walk > n_mt) n_walk = n_mt;
  const long walk_periods = (n_mt + n_walk - 1) / n_walk;
  const long plain_rounds = ((long)n_mt * n_nt + cus - 1) / cus;
  if (walk_periods * 100 > plain_rounds * 104) return pl;     // one workgroup per tile is the better launch
  pl.n_walk = n_walk;
  const int base = n_mt / n_walk, rem = n_mt % n_walk;
  if (rem == 0 || base == 0) return pl;
  const long k_slabs = (K + slab - 1) / slab;
  const int64_t tail_rows = V - (int64_t)(n_mt - rem) * 256;
  const long tail_tiles = (long)rem * n_nt;
  // one slab period of a tile is about 1.65 us; the partials move at about 4 TB/s: 6.6 MB per slab period
  int best_s = 0;
  double best = 0.0;
  for (int s = 1; s <= kMaxKSplit; ++s) {
    const size_t bytes = s > 1 ? (size_t)s * tail_rows * H * sizeof(float) : 0;
    if (s > 1) {
      if (bytes > partial_cap || K / s < 8 * slab) break;
      const int64_t per = round_up64((K + s - 1) / s, slab);
      if ((int64_t)(s - 1) * per >= K) continue;
    }
    const long rounds = (tail_tiles * s + cus - 1) / cus;
    const double c = (double)rounds * (double)((k_slabs + s - 1) / s) + 2.0 * (double)bytes / 6.6e6 + (s > 1 ? 0.02 : 0.01) * (double)k_slabs;
    if (best_s == 0 || c < best) { best = c; best_s = s; }
  }
  const double now = (double)(base + 1) * (double)k_slabs, two = (double)base * (double)k_slabs + best;
  if (best_s == 0 || two >= 0.99 * now) return pl;
  pl.bulk_mt = n_mt - rem;
  pl.k_split = best_s;
  pl.partial_bytes = best_s > 1 ? (size_t)best_s * tail_rows * H * sizeof(float) : 0;
  return pl;
}

static size_t dweight_partial_bytes(int64_t rows, int64_t H, int64_t V, int slab) {
  return rows > 0 ? plan_dweight(V, H, round_up64(rows, 64), slab, 256, (size_t)1 << 30).partial_bytes : 0;
}

struct BwdPlan {
  int64_t ldv;        // K extent of dz / WT (V rounded up to 64)
  int64_t chunk;      // tokens per chunk (multiple of 256 unless >= T)
  int64_t ldt;        // K extent of dzT / hidT for a full chunk (tokens rounded up to 64)
  size_t off_wt, off_hidt, off_dz, off_dzt, off_part, part_bytes, total;
};

static BwdPlan bwd_plan(int64_t T, int64_t H, int64_t V, size_t es, int64_t chunk_tokens, bool saved = false,
                        bool own_wt = true) {
  BwdPlan pl;
  pl.ldv = round_up64(V, 64);
  int64_t chunk = (chunk_tokens <= 0 || chunk_tokens >= T) ? T : round_up64(chunk_tokens, 256);
  if (chunk > T) chunk = T;
  pl.chunk = chunk;
  pl.ldt = round_up64(chunk, 64);
  size_t off = 0;
  // K-blocked operands: whole blocks of 256 rows
  const size_t Hb = (size_t)round_up64(H, 256), Cb = (size_t)round_up64(chunk, 256), Vb = (size_t)round_up64(V, 256);
  pl.off_wt = off;   off += own_wt ? align_up(Hb * pl.ldv * es, 256) : 0;
  pl.off_hidt = off; off += align_up(Hb * pl.ldt * es, 256);
  pl.off_dz = off;   off += saved ? 0 : align_up(Cb * pl.ldv * es, 256);
  pl.off_dzt = off;  off += align_up(Vb * pl.ldt * es, 256);
  // split-K partials of the dhidden GEMM and of the dW GEMM's tail (used one after the other): what a full chunk and
  // the shorter last chunk want
  const int slab = (int)(kRowBytes / es);
  size_t part = 0;
  for (size_t b : {dhidden_partial_bytes(chunk, H, pl.ldv, slab), dhidden_partial_bytes(T % chunk, H, pl.ldv, slab),
                   dweight_partial_bytes(chunk, H, V, slab), dweight_partial_bytes(T % chunk, H, V, slab)})
    if (b > part) part = b;
  pl.part_bytes = align_up(part, 256);
  pl.off_part = off; off += pl.part_bytes;
  pl.total = off;
  return pl;
}

// Largest chunk (multiple of 256, or T itself) whose plan fits into `bytes`; 0 if none does.
static int64_t chunk_for_workspace(int64_t T, int64_t H, int64_t V, size_t es, size_t bytes, bool saved, bool own_wt) {
  if (bwd_plan(T, H, V, es, T, saved, own_wt).total <= bytes) return T;
  int64_t lo = 0, hi = T / 256;   // in units of 256 tokens
  while (lo < hi) {
    const int64_t mid = (lo + hi + 1) / 2;
    if (bwd_plan(T, H, V, es, mid * 256, saved, own_wt).total <= bytes) lo = mid; else hi = mid - 1;
  }
  return lo * 256;
}

template <typename T, typename OutT, bool kMContig>
static int launch_gemm_one(const void* A, int64_t a_kslabs, int M, const void* B, int64_t b_kslabs, int N, int K, void* C,
                           int64_t ldc, int accumulate, hipStream_t stream, float* partial, size_t partial_bytes,
                           int k_split_wanted) {
  using Tile = HeadTile<T>;
  int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(&gemm_nt_kernel<T, OutT, kMContig>), Tile::kLdsBytes, "gemm_nt_kernel");
  if (rc) return rc;
  GemmParams g;
  g.A = A; g.B = B; g.C = C; g.a_kslabs = a_kslabs; g.b_kslabs = b_kslabs; g.ldc = ldc;
  g.M = M; g.N = N; g.K = K;
  g.n_mt = (M + 255) / 256; g.n_nt = (N + 255) / 256;
  g.accumulate = accumulate;
  const int slab = Tile::kSlabK;
  const int cus = device_cu_count();
  g.k_split = (partial && partial_bytes) ? k_split_wanted : 1;
  auto fits = [&](int ks) {      // partials fit the buffer and no K range is empty after rounding to whole slabs
    if (ks <= 1) return true;
    if ((size_t)ks * M * N * sizeof(float) > partial_bytes) return false;
    return (int64_t)(ks - 1) * round_up64((K + ks - 1) / ks, slab) < K;
  };
  while (!fits(g.k_split)) --g.k_split;
  g.k_per_split = g.k_split > 1 ? (int)round_up64((K + g.k_split - 1) / g.k_split, slab) : K;
  g.partial = partial;
  // Many more tiles than CUs and no K split: let one workgroup per CU walk runs of tiles instead of
  // launching one workgroup per tile.
  const int n_fixed = kMContig ? g.n_mt : g.n_nt, n_moving = kMContig ? g.n_nt : g.n_mt;
  g.n_walk = 0;
  if (g.k_split == 1 && n_fixed <= cus && g.n_mt * g.n_nt >= 4 * cus && K >= 2 * slab) {
    g.n_walk = cus / n_fixed;
    if (g.n_walk > n_moving) g.n_walk = n_moving;
    // A walk is as long as its longest run; one workgroup per tile takes ceil(tiles / CUs) rounds.  Streaming the K
    // loops into each other is worth a few per cent, not a whole extra tile period (H = 7168: 28 x 64 tiles are 7
    // rounds exactly, while 9 walks over 64 tiles make runs of 7 and 8).
    const long walk_periods = (n_moving + g.n_walk - 1) / g.n_walk;
    const long plain_rounds = ((long)g.n_mt * g.n_nt + cus - 1) / cus;
    if (walk_periods * 100 > plain_rounds * 104) g.n_walk = 0;
  }
  int grid = ((g.n_walk > 0 ? g.n_walk * n_fixed : g.n_mt * g.n_nt * g.k_split) + 7) / 8 * 8;
  hipLaunchKernelGGL((gemm_nt_kernel<T, OutT, kMContig>), dim3(grid), dim3(Tile::kThreads), Tile::kLdsBytes, stream, g);
  rc = check_launch("gemm_nt_kernel");
  if (rc || g.k_split == 1) return rc;
  const int64_t MN = (int64_t)M * N;
  int blocks = (int)((MN + 255) / 256 < 4096 ? (MN + 255) / 256 : 4096);
  hipLaunchKernelGGL(splitk_reduce_kernel<OutT>, dim3(blocks), dim3(256), 0, stream, partial, g.k_split, MN, kMContig ? M : N,
                     static_cast<OutT*>(C), ldc, accumulate);
  return check_launch("splitk_reduce_kernel");
}

// C (+)= A B^T under the launch plan of its orientation: plan_dhidden (C[n][m], with `partial`) or plan_dweight (C[m][n]).
template <typename T, typename OutT, bool kMContig>
static int launch_gemm(const void* A, int64_t a_kslabs, int M, const void* B, int64_t b_kslabs, int N, int K, void* C,
                       int64_t ldc, int accumulate, hipStream_t stream, float* partial = nullptr,
                       size_t partial_bytes = 0) {
  using Tile = HeadTile<T>;
  constexpr int64_t kSlabElems = (int64_t)kBlockRows * Tile::kSlabK;
  if (!kMContig) {
    // dW: equally long walks over most vocabulary tiles, the rest cut into K ranges (plan_dweight)
    const DwPlan dw = plan_dweight(M, N, K, Tile::kSlabK, device_cu_count(), partial ? partial_bytes : 0);
    if (dw.bulk_mt == 0)
      return launch_gemm_one<T, OutT, kMContig>(A, a_kslabs, M, B, b_kslabs, N, K, C, ldc, accumulate, stream, nullptr, 0, 1);
    const int bulk_rows = dw.bulk_mt * 256;
    int rc = launch_gemm_one<T, OutT, kMContig>(A, a_kslabs, bulk_rows, B, b_kslabs, N, K, C, ldc, accumulate, stream, nullptr, 0, 1);
    if (rc) return rc;
    const T* a_tail = static_cast<const T*>(A) + (int64_t)dw.bulk_mt * a_kslabs * kSlabElems;
    OutT* c_tail = static_cast<OutT*>(C) + (int64_t)bulk_rows * ldc;
    return launch_gemm_one<T, OutT, kMContig>(a_tail, a_kslabs, M - bulk_rows, B, b_kslabs, N, K, c_tail, ldc, accumulate, stream,
                                              dw.k_split > 1 ? partial : nullptr, dw.k_split > 1 ? partial_bytes : 0, dw.k_split);
  }
  if (!(partial && partial_bytes))
    return launch_gemm_one<T, OutT, kMContig>(A, a_kslabs, M, B, b_kslabs, N, K, C, ldc, accumulate, stream, nullptr, 0, 1);
  const DhPlan pl = plan_dhidden(N, M, K, Tile::kSlabK, device_cu_count(), partial_bytes);
  if (pl.bulk_nt == 0)
    return launch_gemm_one<T, OutT, kMContig>(A, a_kslabs, M, B, b_kslabs, N, K, C, ldc, accumulate, stream, partial,
                                              partial_bytes, pl.k_split);
  const int bulk_rows = pl.bulk_nt * 256;
  int rc = launch_gemm_one<T, OutT, kMContig>(A, a_kslabs, M, B, b_kslabs, bulk_rows, K, C, ldc, accumulate, stream,
                                              nullptr, 0, 1);
  if (rc) return rc;
  const T* b_tail = static_cast<const T*>(B) + (int64_t)pl.bulk_nt * b_kslabs * kSlabElems;
  OutT* c_tail = static_cast<OutT*>(C) + (int64_t)bulk_rows * ldc;
  return launch_gemm_one<T, OutT, kMContig>(A, a_kslabs, M, b_tail, b_kslabs, N - bulk_rows, K, c_tail, ldc, accumulate,
                                            stream, partial, partial_bytes, pl.k_split);
}

template <typename T>
static int launch_transpose(const T* src, int64_t ld_src, T* dst, int64_t ld_dst, int R, int C, hipStream_t stream) {
  dim3 grid((C + 63) / 64, (int)((ld_dst + 63) / 64));
  hipLaunchKernelGGL(transpose_block_kernel<T>, grid, dim3(256), 0, stream, src, ld_src, dst, ld_dst, R, C);
  return check_launch("transpose_block_kernel");
}

template <typename T>
static int run_bwd(const clgrpo_lmhead_bwd_args* a, hipStream_t stream, int64_t label_offset) {
  using Tile = HeadTile<T>;
  const int64_t T_ = a->T, H = a->H, V = a->V;
  const bool saved = a->saved_logits != nullptr;
  const bool own_wt = a->weight_t == nullptr;
  const int64_t chunk = chunk_for_workspace(T_, H, V, sizeof(T), a->workspace_bytes, saved, own_wt);
  if (chunk <= 0)
    return fail(CLGRPO_EWORKSPACE, "clgrpo_lmhead_bwd: workspace %zu bytes cannot hold a 256-token chunk (%zu needed)",
                a->workspace_bytes, bwd_plan(T_, H, V, sizeof(T), 256, saved, own_wt).total);
  const BwdPlan pl = bwd_plan(T_, H, V, sizeof(T), chunk, saved, own_wt);
  const int64_t ldz = saved ? a->ld_saved : pl.ldv;
  char* ws = static_cast<char*>(a->workspace);
  T* wt = a->weight_t ? static_cast<T*>(a->weight_t) : reinterpret_cast<T*>(ws + pl.off_wt);
  T* hidt = reinterpret_cast<T*>(ws + pl.off_hidt);
  T* dz_ws = reinterpret_cast<T*>(ws + pl.off_dz);
  T* dzt = reinterpret_cast<T*>(ws + pl.off_dzt);
  const T* hidden = static_cast<const T*>(a->hidden);
  const T* weight = static_cast<const T*>(a->weight);

  int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(&lmhead_dz_kernel<T>), Tile::kLdsBytes, "lmhead_dz_kernel");
  if (rc) return rc;
  if (a->dhidden && !(a->weight_t && a->weight_t_ready)) {
    // WT(h, v) = W[v][h], zero for V <= v < ldv, K-blocked
    rc = launch_transpose<T>(weight, H, wt, pl.ldv, (int)V, (int)H, stream);
    if (rc) return rc;
  }
  for (int64_t c0 = 0; c0 < T_; c0 += chunk) {
    const int64_t tc = (T_ - c0) < chunk ? (T_ - c0) : chunk;
    const int64_t ldt = round_up64(tc, 64);
    T* dz = saved ? static_cast<T*>(a->saved_logits) + c0 * ldz : dz_ws;
    if (saved) {
      DzFromZParams q;
      q.z = dz;
      q.dzT = dzt;
      q.labels = a->labels + c0;
      q.label_offset = label_offset;
      q.lse = a->lse + c0;
      q.entropy = a->g_entropy ? a->entropy + c0 : nullptr;
      q.g_lp = a->g_logprob + c0;
      q.g_ent = a->g_entropy ? a->g_entropy + c0 : nullptr;
      q.Tc = (int)tc;
      q.ldt = (int)ldt;
      q.V = (int)V;
      q.ldv = (int)ldz;
      q.c = a->inv_temperature * kLog2e;
      q.inv_temperature = a->inv_temperature;
      dim3 grid((unsigned)((tc + kBlockRows - 1) / kBlockRows), (unsigned)(ldz / Elem<T>::kSlabK));
      hipLaunchKernelGGL(dz_from_z_kernel<T>, grid, dim3(256), 0, stream, q);
      rc = check_launch("dz_from_z_kernel");
      if (rc) return rc;
    } else {
      DzParams d;
      d.hidden = hidden + c0 * H;
      d.weight = weight;
      d.labels = a->labels + c0;
      d.label_offset = label_offset;
      d.lse = a->lse + c0;
      d.entropy = a->g_entropy ? a->entropy + c0 : nullptr;
      d.g_lp = a->g_logprob + c0;
      d.g_ent = a->g_entropy ? a->g_entropy + c0 : nullptr;
      d.Tc = (int)tc;
      d.ldt = (int)ldt;
      d.H = (int)H;
      d.V = (int)V;
      d.ldv = (int)pl.ldv;
      d.n_tb = (int)((ldt + 255) / 256);
      d.n_vt = (int)((V + 255) / 256);
      d.c = a->inv_temperature * kLog2e;
      d.inv_temperature = a->inv_temperature;
      d.dz = dz;
      d.dzT = dzt;
      int grid = (d.n_tb * d.n_vt + 7) / 8 * 8;
      hipLaunchKernelGGL(lmhead_dz_kernel<T>, dim3(grid), dim3(Tile::kThreads), Tile::kLdsBytes, stream, d);
      rc = check_launch("lmhead_dz_kernel");
      if (rc) return rc;
    }
    if (a->dhidden) {
      // dhidden[chunk][h] = sum_v WT[h][v] dz[t][v]   (M = H, N = tokens, C[n][m])
      rc = launch_gemm<T, T, true>(wt, pl.ldv / Tile::kSlabK, (int)H, dz, ldz / Tile::kSlabK, (int)tc, (int)pl.ldv,
                             static_cast<T*>(a->dhidden) + c0 * H, H, 0, stream,
                             reinterpret_cast<float*>(ws + pl.off_part), pl.part_bytes);
      if (rc) return rc;
    }
    if (a->dweight) {
      // hidT(h, t) = hidden[c0 + t][h], zero for tc <= t < ldt, K-blocked;  dW[v][h] (+)= sum_t dzT(v, t) hidT(h, t)   (M = V, N = H, C[m][n])
      rc = launch_transpose<T>(hidden + c0 * H, H, hidt, ldt, (int)tc, (int)H, stream);
      if (rc) return rc;
      rc = launch_gemm<T, float, false>(dzt, ldt / Tile::kSlabK, (int)V, hidt, ldt / Tile::kSlabK, (int)H, (int)ldt, a->dweight, H,
                                        (a->accumulate_dweight || c0 > 0) ? 1 : 0, stream,
                                        reinterpret_cast<float*>(ws + pl.off_part), pl.part_bytes);
      if (rc) return rc;
    }
  }
  return CLGRPO_OK;
}

}  // namespace clgrpo

using namespace clgrpo;

extern "C" size_t clgrpo_lmhead_bwd_workspace_bytes(int64_t T, int64_t H, int64_t V, int32_t dtype,
                                                    int64_t chunk_tokens, int32_t with_saved_logits) {
  if (T <= 0 || H <= 0 || V <= 0 || (dtype != CLGRPO_BF16 && dtype != CLGRPO_F32)) return 0;
  return bwd_plan(T, H, V, dtype_bytes(dtype), chunk_tokens, (with_saved_logits & 1) != 0, (with_saved_logits & 2) == 0).total;
}

extern "C" int clgrpo_lmhead_bwd_dhidden_plan(int64_t rows, int64_t H, int64_t V, int32_t dtype, int32_t cus, int32_t* out) {
  if (rows <= 0 || H <= 0 || V <= 0 || out == nullptr || (dtype != CLGRPO_BF16 && dtype != CLGRPO_F32)) return CLGRPO_EINVAL;
  const int slab = (int)(kRowBytes / dtype_bytes(dtype));
  const DhPlan pl = plan_dhidden(rows, H, round_up64(V, 64), slab, cus > 0 ? cus : 256, (size_t)1 << 30);
  out[0] = pl.bulk_nt;
  out[1] = pl.k_split;
  return CLGRPO_OK;
}

extern "C" int clgrpo_lmhead_bwd_dweight_plan(int64_t rows, int64_t H, int64_t V, int32_t dtype, int32_t cus, int32_t* out) {
  if (rows <= 0 || H <= 0 || V <= 0 || out == nullptr || (dtype != CLGRPO_BF16 && dtype != CLGRPO_F32)) return CLGRPO_EINVAL;
  const int slab = (int)(kRowBytes / dtype_bytes(dtype));
  const DwPlan pl = plan_dweight(V, H, round_up64(rows, 64), slab, cus > 0 ? cus : 256, (size_t)1 << 30);
  out[0] = pl.n_walk;
  out[1] = pl.bulk_mt;
  out[2] = pl.k_split;
  return CLGRPO_OK;
}

static int bwd_entry(const char* who, const clgrpo_lmhead_bwd_args* a, int64_t vocab_begin, void* stream) {
  CLGRPO_REQUIRE_PTR(a, "args");
  int rc = validate_head_shape(who, a->T, a->H, a->V, a->dtype);
  if (rc) return rc;
  CLGRPO_REQUIRE_PTR(a->hidden, "hidden");
  CLGRPO_REQUIRE_PTR(a->weight, "weight");
  CLGRPO_REQUIRE_PTR(a->labels, "labels");
  CLGRPO_REQUIRE_PTR(a->lse, "lse");
  CLGRPO_REQUIRE_PTR(a->g_logprob, "g_logprob");
  if (a->g_entropy != nullptr) CLGRPO_REQUIRE_PTR(a->entropy, "entropy");
  if (a->dhidden == nullptr && a->dweight == nullptr) return fail(CLGRPO_ENULL, "%s: both dhidden and dweight are NULL", who);
  if (vocab_begin < 0) return fail(CLGRPO_EINVAL, "%s: vocab_begin=%lld", who, (long long)vocab_begin);
  if (!(a->inv_temperature > 0.f)) return fail(CLGRPO_EINVAL, "%s: inv_temperature must be > 0", who);
  CLGRPO_REQUIRE_PTR(a->workspace, "workspace");
  if (a->saved_logits != nullptr && (a->ld_saved < round_up64(a->V, 64) || a->ld_saved % 64 != 0))
    return fail(CLGRPO_ESHAPE, "%s: ld_saved=%lld must be a multiple of 64 and >= %lld", who, (long long)a->ld_saved,
                (long long)round_up64(a->V, 64));
  if (a->saved_logits != nullptr && a->saved_rows < round_up64(a->T, 256))
    return fail(CLGRPO_ESHAPE, "%s: saved_rows=%lld, but the kept-logits buffer must hold %lld rows (T rounded up to 256)", who,
                (long long)a->saved_rows, (long long)round_up64(a->T, 256));
  hipStream_t s = static_cast<hipStream_t>(stream);
  return a->dtype == CLGRPO_BF16 ? run_bwd<__bf16>(a, s, vocab_begin) : run_bwd<float>(a, s, vocab_begin);
}

extern "C" int clgrpo_lmhead_bwd(const clgrpo_lmhead_bwd_args* a, void* stream) {
  return bwd_entry("clgrpo_lmhead_bwd", a, 0, stream);
}

extern "C" int clgrpo_lmhead_bwd_shard(const clgrpo_lmhead_bwd_args* a, int64_t vocab_begin, void* stream) {
  return bwd_entry("clgrpo_lmhead_bwd_shard", a, vocab_begin, stream);
}
