// bf16 / fp16 MFMA paths of scatter2scatter and groupXtY for gfx950.
//
// One workgroup owns one BM x BN output tile that never straddles two experts and walks the contraction in
// slices of 64: global -> LDS directly (double buffered, or a ring of stages for the memory-bound small-row
// classes), or global -> registers -> LDS in the one-wave-per-SIMD form of the 256 x 256 class (mainloop_rs)
// -> MFMA 32x32x16 -> LDS-staged epilogue with 16-byte global accesses.
// Operands whose contraction axis is contiguous in memory ("direct": gathered X rows, weights stored
// (N,K)) sit in LDS as [row][64] with a 16-byte XOR swizzle and are read with ds_read_b128; operands
// whose contraction axis is strided ("transposed": weights stored (K,N), both operands of X^T dY) sit
// as [64][cols] and are read with ds_read_b64_tr_b16, which hands each lane four consecutive
// contraction elements of one column.
//
// Counterparts in the reference: _scatter2scatter + _compute_expert_block
// (scattermoe/kernels/ops.py:11-42, 50-118) and _groupXtY + _xty_and_bias (ops.py:242-366).
#include "common.hpp"

// Tunables (measured on the Mixtral-shape workload unless noted):
//   ROWS*_BELOW  average rows per expert under which the 32-, 64-, 128- and 256-row ring-buffered tile classes
//                are used (weight-streaming regime, Mixtral expert shapes with 64..1536 tokens; from there on
//                the 256x256 two-stage tile)
//   GM_RING      tile rows that visit a tile column back to back in the ring classes' order (1: -15 %, 4: -4 %)
//   STRIPE_BELOW average rows per expert under which the 256x256 class uses that order too (Mixtral shape, 1536
//                tokens: 1.68 -> 1.37 ms for the two forward launches; neutral at 4096, 2 % slower at 8192)
//   GM_S2S       row super-tiles per raster band of scatter2scatter (4: +3 % on the layer-2 shaped launches)
//   GM_XTY       the same for groupXtY (4: 1-2 % over unbanded on all three training workloads)
static constexpr int ROWS32_BELOW = 24, ROWS64_BELOW = 52, ROWS128_BELOW = 112, ROWS256_BELOW = 224;
static constexpr int ROWS128W_BELOW = 136;   // wide launches: 128 x 256 ring tiles for 52..135 rows per expert, 256 x 256 from there
static constexpr int GM_RING = 8;
static constexpr int STRIPE_BELOW = 1024;
static constexpr int GM_S2S = 4;
static constexpr int GM_XTY = 4;
static constexpr int XTY_GATHER_MAX_N = 6144;   // widest dY for which groupXtY gathers the rows of X itself
static constexpr int REMAINDER_ROWS = 128;      // an expert's last tile of at most this many rows goes to a launch of 128-row tiles
#include <type_traits>
#include <algorithm>
#include <math.h>

namespace smoe {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

static constexpr int BK = 64;               // contraction slice per stage

template <typename T> struct Mfma;
template <> struct Mfma<bf16_t> {
  static __device__ __forceinline__ f32x16 run(i32x4 a, i32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float sum8(i32x4 a) {
    const bf16x8 v = __builtin_bit_cast(bf16x8, a);
    return (((float)v[0] + (float)v[1]) + ((float)v[2] + (float)v[3])) +
           (((float)v[4] + (float)v[5]) + ((float)v[6] + (float)v[7]));
  }
};
template <> struct Mfma<f16_t> {
  static __device__ __forceinline__ f32x16 run(i32x4 a, i32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float sum8(i32x4 a) {
    const f16x8 v = __builtin_bit_cast(f16x8, a);
    return (((float)v[0] + (float)v[1]) + ((float)v[2] + (float)v[3])) +
           (((float)v[4] + (float)v[5]) + ((float)v[6] + (float)v[7]));
  }
};

typedef __attribute__((address_space(3))) char lds_char;

__device__ __forceinline__ unsigned lds_address(const char* p) {
  return (unsigned)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}
__device__ __forceinline__ unsigned wave_uniform_id() {
  return __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
}
__device__ __forceinline__ i32x4 lds_read16(const char* p) { return *(const i32x4*)p; }
__device__ __forceinline__ void lds_write16(char* p, i32x4 v) { *(i32x4*)p = v; }
__device__ __forceinline__ s16x4 lds_read_tr(const char* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p);
}

typedef __attribute__((address_space(3))) void lds_void_t;
typedef __attribute__((address_space(1))) const void glb_void_t;

// 16 bytes per lane straight from global memory into LDS: lane i of the wave lands at dst + 16*i.
// Issued as inline assembly on purpose: for the builtin the compiler assumes that every later LDS read
// may alias the in-flight transfer and waits for it (vmcnt(0)) before the first ds_read, which would
// serialise the prefetch of slice k+1 with the MFMAs of slice k.  The main loop waits explicitly instead.
// `lds_addr` is the wave-uniform byte address inside the workgroup's LDS allocation; the global address is
// a wave-uniform 64-bit base (scalar registers) plus a 32-bit per-lane byte offset.  This addressing form
// matters: the same load with a full 64-bit address in each lane costs the issuing wave so much issue time
// that the matrix pipe starves (measured: +50% run time for 8 such loads per 32 MFMAs, against no
// measurable cost for the scalar-base form).
// STREAM: the non-temporal hint, for an operand the launch reads exactly once (the weights of the memory-bound
// classes), so that it does not displace the rows that are read again and again.
template <bool STREAM = false>
__device__ __forceinline__ void load_to_lds16(const char* base_uniform, unsigned off, unsigned lds_addr) {
  if constexpr (STREAM)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
                 :
                 : "s"(lds_addr), "v"(off), "s"(base_uniform)
                 : "memory", "m0");
  else
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_addr), "v"(off), "s"(base_uniform)
                 : "memory", "m0");
}
__device__ __forceinline__ const char* make_uniform(const char* p) {
  const uint64_t v = (uint64_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (const char*)(((uint64_t)hi << 32) | lo);
}

// Both operand kinds fill a 64-deep LDS tile of EXT*128 bytes in LINEAR order of 16-byte pieces: piece
// p = j*NT + t is copied by thread t in round j (a wave's 64 pieces are contiguous, which is what the
// direct-to-LDS load needs).  Which global piece lands in LDS piece p is where the two kinds differ:
// the XOR swizzles below are applied on the global side.

// ---- operand with contiguous contraction axis: LDS tile [EXT][64], 128 B per row ------------------------
// piece p = (row, phys) holds contraction chunk c = phys ^ f(row); f makes the 16 lanes of a ds_read_b128
// phase (16 consecutive rows, one chunk) hit 16 different 16-byte bank groups.
__device__ __forceinline__ int direct_swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

template <int EXT, int NT, bool STREAM = false>
struct DirectOp {
  static constexpr int PIECES = EXT * 8;
  static constexpr int R = PIECES / NT;
  static constexpr int LDS_BYTES = EXT * 128;
  static constexpr int DS_PER_FRAG = 1;
  static_assert(PIECES % NT == 0, "tile must be a whole number of rounds");
  const char* base;        // wave-uniform global address all rows are relative to
  unsigned off[R];         // byte offset of this thread's piece of load slot j at contraction 0
  // Load slot j carries round (j + rot) % R of the tile.  The workgroups of a super tile that share a panel use
  // different rotations, each starting with the rows it is the designated first toucher of: those L2 misses
  // then start earliest, and the other sharers ask for the same lines later in their own queues, when the
  // fill is under way or done, instead of piling onto a miss that has only just been issued.
  int rot = 0;
  __device__ __forceinline__ int rnd(int j) const { const int r = j + rot; return r >= R ? r - R : r; }
  // `row_off(row)` returns the byte offset (from `b`) of element (row, k = 0) of the tile's row `row`
  template <typename F>
  __device__ __forceinline__ void init(const char* b, F row_off) {
    base = make_uniform(b);
    const int t = threadIdx.x;
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int p = rnd(j) * NT + t, row = p >> 3;
      off[j] = (unsigned)row_off(row) + (((p & 7) ^ direct_swz(row)) << 4);
    }
  }
  __device__ __forceinline__ void issue_one(unsigned tile, int k0, int j) const {
    load_to_lds16<STREAM>(base + (int64_t)k0 * 2, off[j], tile + wave_uniform_id() * 1024 + rnd(j) * NT * 16);
  }
  // the same piece into registers, and where it belongs in the LDS tile
  // (whole slices only: `kend` is not looked at)
  __device__ __forceinline__ i32x4 load_piece(int k0, int, int j) const {
    const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void*)(base + (int64_t)k0 * 2), 0, -1, 0x00020000);
    return __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)off[j], 0, 0));
  }
  __device__ __forceinline__ int piece_lds(int j) const { return (rnd(j) * NT + (int)threadIdx.x) * 16; }
  __device__ __forceinline__ void issue(unsigned tile, int k0) const {
#pragma unroll
    for (int j = 0; j < R; ++j) issue_one(tile, k0, j);
  }
  // Partial last slice: pieces past `kend` are fetched from contraction 0 of the same row (always valid
  // memory) and overwritten with zeros by the same thread once its loads have landed.
  __device__ __forceinline__ void issue_tail_one(unsigned tile, int k0, int kend, int j) const {
    const int p = rnd(j) * NT + threadIdx.x;
    const int c = (p & 7) ^ direct_swz(p >> 3);
    const bool ok = k0 + c * 8 < kend;
    load_to_lds16<STREAM>(base, ok ? off[j] + (unsigned)k0 * 2 : off[j] - (c << 4),
                  tile + wave_uniform_id() * 1024 + rnd(j) * NT * 16);
  }
  __device__ __forceinline__ void issue_tail(unsigned tile, int k0, int kend) const {
#pragma unroll
    for (int j = 0; j < R; ++j) issue_tail_one(tile, k0, kend, j);
  }
  __device__ __forceinline__ void zero_tail(char* tile, int k0, int kend) const {
    const int t = threadIdx.x;
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int p = rnd(j) * NT + t;
      const int c = (p & 7) ^ direct_swz(p >> 3);
      if (k0 + c * 8 >= kend) lds_write16(tile + p * 16, i32x4{0, 0, 0, 0});
    }
  }
  // fragment of MFMA operand rows [base, base+32), contraction step ks (16 elements)
  static __device__ __forceinline__ i32x4 frag(const char* tile, int base, int ks) {
    const int l = lane_id();
    const int row = base + (l & 31);
    return lds_read16(tile + row * 128 + (((2 * ks + (l >> 5)) ^ direct_swz(row)) << 4));
  }
  // only operands that gather their contraction rows have anything to do here (see TransOp)
  __device__ __forceinline__ void fetch_rows(int, int) {}
  __device__ __forceinline__ void stage_rows(int) {}
  __device__ __forceinline__ void take_rows(int) {}
};

// ---- operand with strided contraction axis: LDS tile [64][EXT], read transposed --------------------------
// Row kr of the tile is EXT*2 bytes = G granules of 64 B (32 columns).  A ds_read_b64_tr_b16 phase touches
// one granule column in 4 consecutive rows; storing granule g of row kr at position g ^ (kr & 3) spreads
// those 4 accesses over all 64 banks.
// GATHER: the contraction rows are not consecutive in memory but picked through an index vector (row r of the
// operand is row rows[r] / fan of the source matrix).  The 64 rows of a slice are looked up once per workgroup, not
// once per thread (vector-ALU work in this loop comes straight out of the matrix pipe's time): thread t < 64 fetches
// the index of row t one slice ahead (`fetch_rows`, an ordinary load that the main loop's wait covers), turns it into
// a byte offset and puts it into LDS before the loop's barrier (`stage_rows`); after the barrier every thread picks
// the offsets of its own load slots up from there (`take_rows`).
template <int EXT, int NT, bool STREAM = false, bool GATHER = false>
struct TransOp {
  static constexpr int CPR = EXT / 8;                  // 16-byte pieces per contraction row
  static constexpr int PIECES = 64 * CPR;
  static constexpr int R = PIECES / NT;
  static constexpr int RS = EXT * 2;                   // LDS row stride, bytes
  static constexpr int DS_PER_FRAG = 2;
  static constexpr int LDS_BYTES = 64 * RS;
  static_assert(PIECES % NT == 0 && EXT % 128 == 0, "unsupported transposed tile width");
  const char* base;    // wave-uniform global address of (contraction 0, column 0 of the tile)
  unsigned off[R];     // byte offset of this thread's piece of load slot j within the first slice
                       // (GATHER: within the slice that is issued next)
  int rot = 0;         // load slot j carries round (j + rot) % R (see DirectOp)
  __device__ __forceinline__ int rnd(int j) const { const int r = j + rot; return r >= R ? r - R : r; }
  int64_t ld;          // bytes between contraction rows
  // GATHER only
  const int64_t* rows; // wave-uniform: index vector, already offset to the first contraction row
  unsigned fan;
  unsigned colb[R];    // byte offset of this thread's piece inside its contraction row
  unsigned next_row;   // thread t < 64: index of contraction row t of the slice after the one being issued
  unsigned* srow;      // LDS, [2][64]: byte offsets of the rows of the slice to be issued next, by slice parity
  // contraction row inside a slice that load slot j of this thread carries
  __device__ __forceinline__ int slot_row(int j) const { return (rnd(j) * NT + (int)threadIdx.x) / CPR; }
  // columns >= valid_cols are clamped to column 0 (they only feed outputs that are never stored)
  __device__ __forceinline__ void init(const char* b, int64_t ld_bytes, int valid_cols) {
    init_cols(b, ld_bytes, [&](int tc) { return tc < valid_cols ? tc : 0; });
  }
  // `col_of(tc)`: element column (relative to `b`, a multiple of 8, always inside the allocation) that tile
  // column tc (a multiple of 8) is fetched from
  template <typename F>
  __device__ __forceinline__ void init_cols(const char* b, int64_t ld_bytes, F col_of) {
    base = make_uniform(b);
    ld = ld_bytes;
    const int t = threadIdx.x;
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int p = rnd(j) * NT + t;
      const int kr = p / CPR, phys = p % CPR;
      const int cc = ((((phys >> 2) ^ (kr & 3)) << 2) | (phys & 3));      // logical 16-byte piece of the row
      if constexpr (GATHER) colb[j] = (unsigned)col_of(cc * 8) * 2;
      else off[j] = (unsigned)(kr * ld_bytes) + (unsigned)col_of(cc * 8) * 2;
    }
  }
  // GATHER: `b` is (row 0, column 0 of the tile) of the SOURCE matrix, `r` the index vector at the operand's first
  // contraction row, `klen` the number of contraction rows, `lds_rows` 2 x 64 words of LDS.  Ends with the first
  // slice's offsets taken (one workgroup barrier inside).
  __device__ __forceinline__ void init_gather(const char* b, int64_t ld_bytes, int valid_cols, const int64_t* r,
                                              int fan_out, int klen, unsigned* lds_rows) {
    rows = (const int64_t*)make_uniform((const char*)r);
    fan = (unsigned)fan_out;
    srow = lds_rows;
    init(b, ld_bytes, valid_cols);
    fetch_rows(0, klen);
    stage_rows(0);
    __syncthreads();
    take_rows(0);
  }
  // index of row t of the slice at contraction k0 (rows past the end repeat the last row: their data is zeroed in LDS)
  __device__ __forceinline__ void fetch_rows(int k0, int klen) {
    if constexpr (GATHER) {
      if (wave_uniform_id() == 0) {
        int r = k0 + (int)threadIdx.x;
        r = r < klen ? r : klen - 1;
        next_row = r >= 0 ? (unsigned)rows[r] : 0u;
      }
    }
  }
  // before the barrier of the iteration that issues slice number `slice`
  __device__ __forceinline__ void stage_rows(int slice) {
    if constexpr (GATHER) {
      if (wave_uniform_id() == 0) srow[(slice & 1) * 64 + threadIdx.x] = (unsigned)((int64_t)(next_row / fan) * ld);
    }
  }
  // after that barrier
  __device__ __forceinline__ void take_rows(int slice) {
    if constexpr (GATHER) {
#pragma unroll
      for (int j = 0; j < R; ++j) off[j] = srow[(slice & 1) * 64 + slot_row(j)] + colb[j];
    }
  }
  __device__ __forceinline__ void issue_one(unsigned tile, int k0, int j) const {
    if constexpr (GATHER) load_to_lds16<STREAM>(make_uniform(base), off[j], tile + wave_uniform_id() * 1024 + rnd(j) * NT * 16);
    else load_to_lds16<STREAM>(base + (int64_t)k0 * ld, off[j], tile + wave_uniform_id() * 1024 + rnd(j) * NT * 16);
  }
  // the same piece into registers (not for gathered rows), and where it belongs in the LDS tile
  // Contraction rows from `kend` on read as zeros: the buffer descriptor of the slice ends with row kend - 1
  // (a row's pieces lie inside its first `ld` bytes).
  __device__ __forceinline__ i32x4 load_piece(int k0, int kend, int j) const {
    const int64_t span = (int64_t)(kend - k0) * ld;
    const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(base + (int64_t)k0 * ld), 0, span < 0xffffffffLL ? (int)(unsigned)span : -1, 0x00020000);
    return __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)off[j], 0, 0));
  }
  __device__ __forceinline__ int piece_lds(int j) const { return (rnd(j) * NT + (int)threadIdx.x) * 16; }
  __device__ __forceinline__ void issue(unsigned tile, int k0) const {
#pragma unroll
    for (int j = 0; j < R; ++j) issue_one(tile, k0, j);
  }
  // Partial last slice: contraction rows past `kend` are fetched from row 0 of the slice (always valid
  // memory) and overwritten with zeros by the same thread once its loads have landed.
  __device__ __forceinline__ void issue_tail_one(unsigned tile, int k0, int kend, int j) const {
    if constexpr (GATHER) {
      issue_one(tile, k0, j);          // rows past the end already point at the last valid row
    } else {
      const int kr = slot_row(j);
      const bool ok = k0 + kr < kend;
      load_to_lds16<STREAM>(base + (int64_t)k0 * ld, ok ? off[j] : off[j] - (unsigned)(kr * ld),
                    tile + wave_uniform_id() * 1024 + rnd(j) * NT * 16);
    }
  }
  __device__ __forceinline__ void issue_tail(unsigned tile, int k0, int kend) const {
#pragma unroll
    for (int j = 0; j < R; ++j) issue_tail_one(tile, k0, kend, j);
  }
  __device__ __forceinline__ void zero_tail(char* tile, int k0, int kend) const {
    const int t = threadIdx.x;
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int p = rnd(j) * NT + t;
      if (k0 + p / CPR >= kend) lds_write16(tile + p * 16, i32x4{0, 0, 0, 0});
    }
  }
  // Each 16-lane block transposes a 4 (contraction) x 16 (columns) patch: lane r of the block points at
  // contraction row r/4, columns 4*(r%4)..+3 and receives column r, contraction 0..3.  Blocks 0/1 cover
  // columns 0-15 / 16-31 of the 32-wide fragment, blocks 2/3 the contraction elements 8..15; a second
  // read 4 rows further down completes the 8 elements per lane the MFMA expects (k = 8*(lane/32) + 0..7).
  static __device__ __forceinline__ i32x4 frag(const char* tile, int base, int ks) {
    const int l = lane_id();
    const int b = l >> 4, r = l & 15;
    const int kr = ks * 16 + 8 * (b >> 1) + (r >> 2);
    const int gran = (base >> 5) ^ (r >> 2);                       // (kr & 3) == r >> 2
    const char* p = tile + kr * RS + (gran << 6) + (16 * (b & 1) + 4 * (r & 3)) * 2;
    const s16x4 lo = lds_read_tr(p);
    const s16x4 hi = lds_read_tr(p + 4 * RS);
    const s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(i32x4, v);
  }
};

// One slice of both operands, load slots interleaved (A0 B0 A1 B1 ...) so that the rows each operand starts
// with (see `rot`) are requested first.
template <class AOp, class BOp>
__device__ __forceinline__ void issue_slice(const AOp& A, const BOp& B, unsigned dst, int k0) {
  constexpr int RM = AOp::R > BOp::R ? AOp::R : BOp::R;
#pragma unroll
  for (int j = 0; j < RM; ++j) {
    if (j < AOp::R) A.issue_one(dst, k0, j);
    if (j < BOp::R) B.issue_one(dst + AOp::LDS_BYTES, k0, j);
  }
}
template <class AOp, class BOp>
__device__ __forceinline__ void issue_slice_tail(const AOp& A, const BOp& B, unsigned dst, int k0, int kend) {
  constexpr int RM = AOp::R > BOp::R ? AOp::R : BOp::R;
#pragma unroll
  for (int j = 0; j < RM; ++j) {
    if (j < AOp::R) A.issue_tail_one(dst, k0, kend, j);
    if (j < BOp::R) B.issue_tail_one(dst + AOp::LDS_BYTES, k0, kend, j);
  }
}

template <int BM_, int BN_, int WM_, int WN_, int NS_ = 2, bool RS_ = false>
struct Tile {
  static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_;
  static constexpr int NS = NS_;                      // LDS stages (2: double buffer, more: ring)
  static constexpr bool RS = RS_;                     // operands travel global -> registers -> LDS (mainloop_rs)
  static constexpr int NW = WM * WN, NT = NW * 64;
  static constexpr int WTM = BM / WM, WTN = BN / WN;
  static constexpr int FM = WTM / 32, FN = WTN / 32;
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be a multiple of the 32x32 MFMA");
};

// Main loop shared by both kernels.  acc[i][j] is the 32x32 block (i, j) of this wave's tile.
// Full 64-deep slices travel global -> LDS directly (no registers, no ds_write) one slice ahead of the
// MFMAs; a trailing partial slice is zero-filled in LDS after it has landed.
// If `rowsum`, rs[i] additionally accumulates, per lane, the sum of the lane's own 8 contraction elements of
// A-fragment i; adding lanes l and l+32 afterwards gives the sum over the contraction of A row l%32.
template <typename T, class TL, class AOp, class BOp, bool CAN_ROWSUM>
__device__ __forceinline__ void mainloop(AOp& A, BOp& B, int klen, char* lds, bool rowsum,
                                         f32x16 (&acc)[TL::FM][TL::FN], float (&rs)[TL::FM]) {
  constexpr int STAGE = AOp::LDS_BYTES + BOp::LDS_BYTES;
  const int wave = threadIdx.x >> 6;
  const int wm = wave / TL::WN, wn = wave % TL::WN;
  const int nfull = klen / BK;
  const bool tail = (klen % BK) != 0;
  const int nk = nfull + (tail ? 1 : 0);
  const unsigned lds_u = lds_address(lds);
  if (nfull > 0) issue_slice(A, B, lds_u, 0);
  else if (tail) issue_slice_tail(A, B, lds_u, 0, klen);
  A.fetch_rows(BK, klen);            // gathered operands: row indices of the slice after the one just issued
  B.fetch_rows(BK, klen);
  for (int kt = 0; kt < nk; ++kt) {
    char* cur = lds + (kt & 1) * STAGE;
    const unsigned nxt = lds_u + ((kt + 1) & 1) * STAGE;
    __builtin_amdgcn_s_waitcnt(0);   // this thread's direct loads of slice kt have landed in LDS
    if (tail && kt == nfull) {
      A.zero_tail(cur, kt * BK, klen);
      B.zero_tail(cur + AOp::LDS_BYTES, kt * BK, klen);
    }
    A.stage_rows(kt + 1);
    B.stage_rows(kt + 1);
    __syncthreads();                 // ... everyone's have, and everyone is done reading `nxt`
    A.take_rows(kt + 1);
    B.take_rows(kt + 1);
    if (kt + 1 < nfull) issue_slice(A, B, nxt, (kt + 1) * BK);
    else if (tail && kt + 1 == nfull) issue_slice_tail(A, B, nxt, (kt + 1) * BK, klen);
    if (kt + 2 < nk) {
      A.fetch_rows((kt + 2) * BK, klen);
      B.fetch_rows((kt + 2) * BK, klen);
    }
    const char* ta = cur;
    const char* tb = cur + AOp::LDS_BYTES;
    i32x4 fa[2][TL::FM], fb[2][TL::FN];
#pragma unroll
    for (int i = 0; i < TL::FM; ++i) fa[0][i] = AOp::frag(ta, wm * TL::WTM + i * 32, 0);
#pragma unroll
    for (int j = 0; j < TL::FN; ++j) fb[0][j] = BOp::frag(tb, wn * TL::WTN + j * 32, 0);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      const int c = ks & 1, n = c ^ 1;
      if (ks + 1 < BK / 16) {
#pragma unroll
        for (int i = 0; i < TL::FM; ++i) fa[n][i] = AOp::frag(ta, wm * TL::WTM + i * 32, ks + 1);
#pragma unroll
        for (int j = 0; j < TL::FN; ++j) fb[n][j] = BOp::frag(tb, wn * TL::WTN + j * 32, ks + 1);
      }
#pragma unroll
      for (int i = 0; i < TL::FM; ++i)
#pragma unroll
        for (int j = 0; j < TL::FN; ++j) acc[i][j] = Mfma<T>::run(fb[c][j], fa[c][i], acc[i][j]);
      if (CAN_ROWSUM && rowsum) {
#pragma unroll
        for (int i = 0; i < TL::FM; ++i) rs[i] += Mfma<T>::sum8(fa[c][i]);
      }
      // Interleave: the LDS reads of step ks+1 are spread between the MFMAs of step ks.
      if (ks + 1 < BK / 16) {
#pragma unroll
        for (int i = 0; i < TL::FM; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x100, AOp::DS_PER_FRAG, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
#pragma unroll
        for (int j = 0; j < TL::FN; ++j) {
          __builtin_amdgcn_sched_group_barrier(0x100, BOp::DS_PER_FRAG, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, TL::FM * TL::FN - TL::FM - TL::FN, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

// Main loop of the one-wave-per-SIMD class (4 waves, 128 x 128 wave tiles): operands travel global -> registers ->
// LDS.  A burst of loads at the top of a slice holds the waves that issue it off the matrix pipe until the memory
// pipeline has taken all of them (it takes one 1 KB wave-load per ~17 cycles and CU), and loads spread over the
// slice leave the late ones too little time to land when LDS is the only place they can land in: here every
// thread's 16 pieces of a slice sit in registers for up to two slices, which LDS has no room for.
//   set S = (kt + 1) & 1 holds slice kt + 1: its pieces are written to the other LDS stage during steps 0-2 of
//   slice kt (ds_write_b128, second half of each step) and each is reloaded with slice kt + 3 one step later
//   (pieces 12-15 in step 0 of the next slice), one load per 4 MFMAs throughout;
//   one barrier per slice, after step 2: behind it the fragments of step 0 of slice kt + 1 are read while the
//   MFMAs of step 3 run.
// Whole 64-deep slices only, at least two of them (the launcher checks); loads past the end re-read the last slice.
template <typename T, class TL, class AOp, class BOp, int P, int KS>
__device__ __forceinline__ void rs_step(const AOp& A, const BOp& B, const char* __restrict__ cur, char* __restrict__ nxt,
                                        int k2, int k3, int kend, int wm, int wn,
                                        f32x16 (&acc)[TL::FM][TL::FN], i32x4 (&g)[2][16],
                                        i32x4 (&fa)[2][TL::FM], i32x4 (&fb)[2][TL::FN]) {
  constexpr int FM = TL::FM, FN = TL::FN, NM = FM * FN;
  static_assert(NM == 16 && FM + FN <= 8, "pipeline below is laid out for 16 MFMAs per step");
  constexpr int S = P ^ 1;
  constexpr int c = KS & 1, n = c ^ 1;
  // LDS traffic of the step in the order it is to be issued in (the compiler keeps reads and writes of LDS in
  // program order): one fragment of the next step behind each of the first FM + FN MFMAs - from the stage being
  // multiplied, in step 3 from the stage just filled - and one piece written behind every third MFMA of steps 0-2
  // (pieces 0-4, 5-10, 11-15).
  constexpr int W0[5] = {0, 5, 11, 16, 16};
  const char* src = KS < 3 ? cur : (const char*)nxt;
  constexpr int fstep = KS < 3 ? KS + 1 : 0;
#pragma unroll
  for (int m = 0; m < NM; ++m) {
    if (m < FM) fa[n][m] = AOp::frag(src, wm * TL::WTM + m * 32, fstep);
    else if (m < FM + FN) fb[n][m - FM] = BOp::frag(src + AOp::LDS_BYTES, wn * TL::WTN + (m - FM) * 32, fstep);
    if ((KS * NM + m) % 3 == 1 && KS < 3) {
      const int q = (KS * NM + m) / 3;
      if (q & 1) lds_write16(nxt + AOp::LDS_BYTES + B.piece_lds(q >> 1), g[S][q]);
      else lds_write16(nxt + A.piece_lds(q >> 1), g[S][q]);
    }
  }
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j) acc[i][j] = Mfma<T>::run(fb[c][j], fa[c][i], acc[i][j]);
  static_assert(W0[1] == 5 && W0[2] == 11, "pieces per step follow from one write per three MFMAs");
  // pieces loaded in this step: 12-15 of the other set (slice kt + 2), then 0-3, 4-7, 8-11 of this one (slice kt + 3)
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    constexpr int SET = KS == 0 ? P : S;
    const int q = KS == 0 ? 12 + u : (KS - 1) * 4 + u;
    const int k0 = KS == 0 ? k2 : k3;
    g[SET][q] = (q & 1) ? B.load_piece(k0, kend, q >> 1) : A.load_piece(k0, kend, q >> 1);
  }
#pragma unroll
  for (int m = 0; m < NM; ++m) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    if (m < FM) __builtin_amdgcn_sched_group_barrier(0x100, AOp::DS_PER_FRAG, 0);
    else if (m < FM + FN) __builtin_amdgcn_sched_group_barrier(0x100, BOp::DS_PER_FRAG, 0);
    if ((KS * NM + m) % 3 == 1 && KS < 3) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
    if (m % 4 == 3) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
  }
  __builtin_amdgcn_sched_barrier(0);
  if constexpr (KS == 2) {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // this thread's pieces are in LDS, its reads of `cur` done
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  }
}

template <typename T, class TL, class AOp, class BOp, int P>
__device__ __forceinline__ void rs_slice(const AOp& A, const BOp& B, const char* cur, char* nxt,
                                         int kt, int last_k0, int kend, int wm, int wn,
                                         f32x16 (&acc)[TL::FM][TL::FN], i32x4 (&g)[2][16],
                                         i32x4 (&fa)[2][TL::FM], i32x4 (&fb)[2][TL::FN]) {
  const int k2 = min((kt + 2) * BK, last_k0), k3 = min((kt + 3) * BK, last_k0);
  __builtin_amdgcn_sched_barrier(0);
  rs_step<T, TL, AOp, BOp, P, 0>(A, B, cur, nxt, k2, k3, kend, wm, wn, acc, g, fa, fb);
  rs_step<T, TL, AOp, BOp, P, 1>(A, B, cur, nxt, k2, k3, kend, wm, wn, acc, g, fa, fb);
  rs_step<T, TL, AOp, BOp, P, 2>(A, B, cur, nxt, k2, k3, kend, wm, wn, acc, g, fa, fb);
  rs_step<T, TL, AOp, BOp, P, 3>(A, B, cur, nxt, k2, k3, kend, wm, wn, acc, g, fa, fb);
}

template <typename T, class TL, class AOp, class BOp>
__device__ __forceinline__ void mainloop_rs(const AOp& A, const BOp& B, int klen, char* lds,
                                            f32x16 (&acc)[TL::FM][TL::FN]) {
  static_assert(AOp::R == 8 && BOp::R == 8 && BK == 64, "16 pieces per thread and slice");
  constexpr int STAGE = AOp::LDS_BYTES + BOp::LDS_BYTES;
  const int wave = threadIdx.x >> 6;
  const int wm = wave / TL::WN, wn = wave % TL::WN;
  // A partial last slice only with operands that zero-fill (TransOp); without any contraction rows one slice of
  // zeros is multiplied (no branch around the loop: 256 accumulator registers would have to be merged behind it).
  const int nk = max(1, (klen + BK - 1) / BK);
  const int last_k0 = (nk - 1) * BK;
  i32x4 g[2][16];
  i32x4 fa[2][TL::FM], fb[2][TL::FN];
  const int k1 = min(BK, last_k0), k2 = min(2 * BK, last_k0);
#pragma unroll
  for (int q = 0; q < 16; ++q) g[0][q] = (q & 1) ? B.load_piece(0, klen, q >> 1) : A.load_piece(0, klen, q >> 1);
#pragma unroll
  for (int q = 0; q < 16; ++q) g[1][q] = (q & 1) ? B.load_piece(k1, klen, q >> 1) : A.load_piece(k1, klen, q >> 1);
#pragma unroll
  for (int q = 0; q < 16; ++q) {
    if (q & 1) lds_write16(lds + AOp::LDS_BYTES + B.piece_lds(q >> 1), g[0][q]);
    else lds_write16(lds + A.piece_lds(q >> 1), g[0][q]);
  }
#pragma unroll
  for (int q = 0; q < 12; ++q) g[0][q] = (q & 1) ? B.load_piece(k2, klen, q >> 1) : A.load_piece(k2, klen, q >> 1);
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 0; i < TL::FM; ++i) fa[0][i] = AOp::frag(lds, wm * TL::WTM + i * 32, 0);
#pragma unroll
  for (int j = 0; j < TL::FN; ++j) fb[0][j] = BOp::frag(lds + AOp::LDS_BYTES, wn * TL::WTN + j * 32, 0);
  // The second stage starts 64 KB into LDS, beyond what the offset field of an LDS instruction can add: its
  // addresses are formed from a base of their own (kept from being folded into constants), not with one
  // vector-ALU instruction per access.
  unsigned second = STAGE;
  asm volatile("" : "+v"(second));
  char* lds1 = lds + second;
  int kt = 0;
  for (; kt + 1 < nk; kt += 2) {
    rs_slice<T, TL, AOp, BOp, 0>(A, B, lds, lds1, kt, last_k0, klen, wm, wn, acc, g, fa, fb);
    rs_slice<T, TL, AOp, BOp, 1>(A, B, lds1, lds, kt + 1, last_k0, klen, wm, wn, acc, g, fa, fb);
  }
  if (kt < nk) rs_slice<T, TL, AOp, BOp, 0>(A, B, lds, lds1, kt, last_k0, klen, wm, wn, acc, g, fa, fb);
}

// Main loop of the small-row (decode) tile class: memory bound, so what matters is bytes in flight.  The
// slices travel through a ring of NS stages; NS-1 slices are on their way while one is being multiplied.
template <typename T, class TL, class AOp, class BOp>
__device__ __forceinline__ void mainloop_ring(const AOp& A, const BOp& B, int klen, char* lds,
                                              f32x16 (&acc)[TL::FM][TL::FN]) {
  constexpr int STAGE = AOp::LDS_BYTES + BOp::LDS_BYTES;
  constexpr int NS = TL::NS;
  constexpr int LOADS = AOp::R + BOp::R;               // direct loads per thread and slice
  static_assert((NS - 2) * LOADS <= 63, "vmcnt cannot count that many loads in flight");
  const int wave = threadIdx.x >> 6;
  const int wm = wave / TL::WN, wn = wave % TL::WN;
  const int nfull = klen / BK;
  const bool tail = (klen % BK) != 0;
  const int nk = nfull + (tail ? 1 : 0);
  const unsigned lds_u = lds_address(lds);
#define SMOE_RING_ISSUE(s, slot)                                              \
  do {                                                                        \
    const unsigned dst_ = lds_u + (slot) * STAGE;                             \
    if ((s) < nfull) issue_slice(A, B, dst_, (s) * BK);                       \
    else if ((s) < nk) issue_slice_tail(A, B, dst_, (s) * BK, klen);          \
  } while (0)
#pragma unroll
  for (int s = 0; s < NS - 1; ++s) SMOE_RING_ISSUE(s, s);
  int slot = 0;                                        // stage of slice kt
  for (int kt = 0; kt < nk; ++kt) {
    // slice kt has landed; the NS-2 younger slices may stay in flight (loads complete in issue order).
    // Near the end fewer are in flight, so wait for everything there.
    if (kt + NS - 2 < nk) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NS - 2) * LOADS) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    char* cur = lds + slot * STAGE;
    if (tail && kt == nfull) {
      A.zero_tail(cur, kt * BK, klen);
      B.zero_tail(cur + AOp::LDS_BYTES, kt * BK, klen);
    }
    __syncthreads();                 // everyone's part of slice kt is there; everyone is done with slice kt-1
    const int prev = slot == 0 ? NS - 1 : slot - 1;
    SMOE_RING_ISSUE(kt + NS - 1, prev);
    i32x4 fa[BK / 16][TL::FM], fb[BK / 16][TL::FN];
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
#pragma unroll
      for (int i = 0; i < TL::FM; ++i) fa[ks][i] = AOp::frag(cur, wm * TL::WTM + i * 32, ks);
#pragma unroll
      for (int j = 0; j < TL::FN; ++j) fb[ks][j] = BOp::frag(cur + AOp::LDS_BYTES, wn * TL::WTN + j * 32, ks);
    }
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks)
#pragma unroll
      for (int i = 0; i < TL::FM; ++i)
#pragma unroll
        for (int j = 0; j < TL::FN; ++j) acc[i][j] = Mfma<T>::run(fb[ks][j], fa[ks][i], acc[i][j]);
    slot = slot + 1 == NS ? 0 : slot + 1;
  }
#undef SMOE_RING_ISSUE
}

// Store the wave's accumulators.  The MFMAs are issued with the operands swapped (column operand first), so
// acc[i][j] holds the TRANSPOSE of output block (i, j): a lane owns output row i*32 + lane%32 and, per group
// g of four registers, the four consecutive columns j*32 + 8*g + 4*(lane/32) + 0..3 - one 8-byte store per
// group instead of four 2-byte stores.  dst[m] is the element offset of output row m of the tile (or -1),
// columns n0 + [0, BN) clipped to ncols (contiguous); optional bias (already offset to the expert), stride sb.
template <typename T, class TL>
__device__ __forceinline__ void epilogue(const f32x16 (&acc)[TL::FM][TL::FN], T* __restrict__ out,
                                         const int64_t* dst, int n0, int ncols,
                                         const T* __restrict__ bias, int64_t sb) {
  typedef T T4 __attribute__((ext_vector_type(4)));
  const int wave = threadIdx.x >> 6, l = lane_id();
  const int wm = wave / TL::WN, wn = wave % TL::WN;
  const bool base_ok = ((uintptr_t)out & 7) == 0;
#pragma unroll
  for (int i = 0; i < TL::FM; ++i) {
    const int64_t d = dst[wm * TL::WTM + i * 32 + (l & 31)];
#pragma unroll
    for (int j = 0; j < TL::FN; ++j) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n0 + wn * TL::WTN + j * 32 + g * 8 + (l >> 5) * 4;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] = acc[i][j][g * 4 + e];
          if (bias != nullptr && n + e < ncols) v[e] += to_f32(bias[(int64_t)(n + e) * sb]);
        }
        if (d < 0) continue;
        if (base_ok && n + 3 < ncols && ((d + n) & 3) == 0) {
          T4 p;
#pragma unroll
          for (int e = 0; e < 4; ++e) p[e] = from_f32<T>(v[e]);
          *(T4*)(out + d + n) = p;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < ncols) out[d + n + e] = from_f32<T>(v[e]);
        }
      }
    }
  }
}

// ---- epilogues that go through LDS ------------------------------------------------------------------
// Two floats rounded to the storage type by one instruction (element-wise casts cost a conversion and a merge per
// element); same rounding as the scalar cast.  `set_pair` puts the pair into elements 2k, 2k + 1 of a vector.
template <typename T, typename V>
__device__ __forceinline__ void set_pair(V& v, int k, float a, float b) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef T T2 __attribute__((ext_vector_type(2)));
  const T2 r = __builtin_convertvector((f32x2_t){a, b}, T2);
  v[2 * k] = r[0];
  v[2 * k + 1] = r[1];
}

// After the main loop the operand buffers are free.  The accumulators (transposed blocks, see `epilogue`) are
// rounded to the storage type and written to LDS as a row-major BM x BN tile, so that the global traffic of the
// epilogue can be 16 bytes per lane with a wave covering whole 128-byte lines: 16-byte piece c of row r sits at
// chunk c ^ (r & (CPR-1)) of the row, which keeps both the 8-byte column-strided writes and the 16-byte
// row-major reads free of bank conflicts.
template <class TL>
__device__ __forceinline__ int staged_addr(int row, int col) {
  constexpr int CPR = TL::BN / 8;
  return row * (TL::BN * 2) + ((((col >> 3) ^ row) & (CPR - 1)) << 4) + ((col & 7) << 1);
}

// `bias_of(tile_col)` returns the value to add to that column (0 without bias).
template <typename T, class TL, typename BF>
__device__ __forceinline__ void stage_accumulators(const f32x16 (&acc)[TL::FM][TL::FN], char* lds, BF bias_of,
                                                   float* sbias) {
  typedef T T4 __attribute__((ext_vector_type(4)));
  static_assert(TL::BM * TL::BN * 2 <= TL::NS * (TL::BM + TL::BN) * 128, "staged tile must fit the operand buffers");
  const int wave = threadIdx.x >> 6, l = lane_id();
  const int wm = wave / TL::WN, wn = wave % TL::WN;
  // One wave per SIMD: the additions per column come from LDS (written here, one column per thread), so that the
  // walk over the 256 accumulator registers below is one straight piece of code without loads or branches.
  if constexpr (TL::RS) {
    for (int t = threadIdx.x; t < TL::BN; t += TL::NT) sbias[t] = bias_of(t);
  }
  __syncthreads();                                   // every wave is done reading operands
#pragma unroll
  for (int j = 0; j < TL::FN; ++j) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int col = wn * TL::WTN + j * 32 + g * 8 + (l >> 5) * 4;
      float bv[4];
      if constexpr (TL::RS) {
        typedef float f32x4_t __attribute__((ext_vector_type(4)));
        const f32x4_t b4 = *(const f32x4_t*)(sbias + col);
#pragma unroll
        for (int e = 0; e < 4; ++e) bv[e] = b4[e];
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) bv[e] = bias_of(col + e);
      }
#pragma unroll
      for (int i = 0; i < TL::FM; ++i) {
        const int row = wm * TL::WTM + i * 32 + (l & 31);
        T4 v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = from_f32<T>(acc[i][j][g * 4 + e] + bv[e]);
        *(T4*)(lds + staged_addr<TL>(row, col)) = v;
      }
    }
  }
  __syncthreads();
}

// Fused gated-linear-unit epilogues (rows in grouped order: output row = row0 + m).
// Forward: the column operand of the tile is laid out so that each wave owns WTN/2 "first half" columns
// (accumulator blocks j < FN/2) and the matching WTN/2 "second half" columns (blocks j + FN/2).  Both are
// rounded to the storage type first and the hidden value is computed from the rounded values, i.e. the same
// arithmetic as storing the pre-activation and running the stand-alone pass over it.
template <typename T, class TL>
__device__ __forceinline__ void epilogue_glu_fwd(const f32x16 (&acc)[TL::FM][TL::FN], const S2SArgs& a, int row0,
                                                 int rows, int nh0, const T* __restrict__ bias) {
  if constexpr (TL::FN % 2 == 0) {
    typedef T T4 __attribute__((ext_vector_type(4)));
    constexpr int FH = TL::FN / 2;
    const int wave = threadIdx.x >> 6, l = lane_id();
    const int wm = wave / TL::WN, wn = wave % TL::WN;
    const int F = a.N;
    const bool gf = (a.act & 1) != 0;
    T* pre = (T*)a.Y;
    T* hid = (T*)a.H;
    const bool vec_ok = (((uintptr_t)pre | (uintptr_t)hid) & 7) == 0 && ((a.sym | a.shm | F) & 3) == 0;
#pragma unroll
    for (int i = 0; i < TL::FM; ++i) {
      const int m = wm * TL::WTM + i * 32 + (l & 31);
      const int64_t row = row0 + m;
#pragma unroll
      for (int j = 0; j < FH; ++j) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int n = nh0 + wn * (TL::WTN / 2) + j * 32 + g * 8 + (l >> 5) * 4;
          T first[4], second[4], h[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float v1 = acc[i][j][g * 4 + e], v2 = acc[i][j + FH][g * 4 + e];
            if (bias != nullptr && n + e < F) {
              v1 += to_f32(bias[(int64_t)(n + e) * a.sbn]);
              v2 += to_f32(bias[(int64_t)(F + n + e) * a.sbn]);
            }
            first[e] = from_f32<T>(v1);
            second[e] = from_f32<T>(v2);
            const float lin = to_f32(gf ? second[e] : first[e]), gat = to_f32(gf ? first[e] : second[e]);
            h[e] = from_f32<T>(glu_h(a.act, gat, lin));
          }
          if (m >= rows) continue;
          if (vec_ok && n + 3 < F) {
            if (pre != nullptr) {
              *(T4*)(pre + row * a.sym + n) = T4{first[0], first[1], first[2], first[3]};
              *(T4*)(pre + row * a.sym + F + n) = T4{second[0], second[1], second[2], second[3]};
            }
            *(T4*)(hid + row * a.shm + n) = T4{h[0], h[1], h[2], h[3]};
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              if (n + e >= F) continue;
              if (pre != nullptr) {
                pre[row * a.sym + n + e] = first[e];
                pre[row * a.sym + F + n + e] = second[e];
              }
              hid[row * a.shm + n + e] = h[e];
            }
          }
        }
      }
    }
  }
}

// Backward: the product is d(hidden); it is rounded to the storage type and turned into d(pre-activation)
// with the saved pre-activation, exactly as the stand-alone pass would do from a stored d(hidden).
template <typename T, class TL>
__device__ __forceinline__ void epilogue_glu_bwd(const f32x16 (&acc)[TL::FM][TL::FN], const S2SArgs& a, int row0,
                                                 int rows, int n0) {
  typedef T T4 __attribute__((ext_vector_type(4)));
  const int wave = threadIdx.x >> 6, l = lane_id();
  const int wm = wave / TL::WN, wn = wave % TL::WN;
  const int F = a.N;
  const bool gf = (a.act & 1) != 0;
  const T* pre = (const T*)a.aux;
  T* dpre = (T*)a.Y;
  const bool vec_ok = (((uintptr_t)pre | (uintptr_t)dpre) & 7) == 0 && ((a.sym | a.saux | F) & 3) == 0;
#pragma unroll
  for (int i = 0; i < TL::FM; ++i) {
    const int m = wm * TL::WTM + i * 32 + (l & 31);
    if (m >= rows) continue;
    const int64_t row = row0 + m;
#pragma unroll
    for (int j = 0; j < TL::FN; ++j) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n0 + wn * TL::WTN + j * 32 + g * 8 + (l >> 5) * 4;
        if (n >= F) continue;
        const bool vec = vec_ok && n + 3 < F;
        T p1[4], p2[4], o1[4], o2[4];
        if (vec) {
          const T4 v1 = *(const T4*)(pre + row * a.saux + n), v2 = *(const T4*)(pre + row * a.saux + F + n);
#pragma unroll
          for (int e = 0; e < 4; ++e) { p1[e] = v1[e]; p2[e] = v2[e]; }
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const bool ok = n + e < F;
            p1[e] = ok ? pre[row * a.saux + n + e] : from_f32<T>(0.0f);
            p2[e] = ok ? pre[row * a.saux + F + n + e] : from_f32<T>(0.0f);
          }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float dv = to_f32(from_f32<T>(acc[i][j][g * 4 + e]));
          const float lin = to_f32(gf ? p2[e] : p1[e]), gat = to_f32(gf ? p1[e] : p2[e]);
          float f_lin, f_gat;
          glu_grad(a.act, dv, gat, lin, f_lin, f_gat);
          const T d_lin = from_f32<T>(f_lin), d_gat = from_f32<T>(f_gat);
          o1[e] = gf ? d_gat : d_lin;
          o2[e] = gf ? d_lin : d_gat;
        }
        if (vec) {
          *(T4*)(dpre + row * a.sym + n) = T4{o1[0], o1[1], o1[2], o1[3]};
          *(T4*)(dpre + row * a.sym + F + n) = T4{o2[0], o2[1], o2[2], o2[3]};
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (n + e >= F) continue;
            dpre[row * a.sym + n + e] = o1[e];
            dpre[row * a.sym + F + n + e] = o2[e];
          }
        }
      }
    }
  }
}

// Plain store through LDS: dst[m] is the element offset of output row m of the tile (or -1).
// Output tiles are written once and not read again by the launch: stored with the non-temporal hint so that they
// do not displace operand panels in the L2 (c4: -1 % step time, c2: -0.2 %).
template <typename V>
__device__ __forceinline__ void stream_store(const V& v, V* p) { __builtin_nontemporal_store(v, p); }

// 16-byte store through a buffer descriptor: the hardware drops it when `offset` (bytes) lies beyond the descriptor's
// range, so a piece outside the tile's valid part needs no branch around its store.  That matters where loads are in
// flight across the stores: stores and loads share one counter, and behind a store that a branch may have skipped
// the compiler can only wait for everything, the prefetched loads of the next group included.
template <typename V>
__device__ __forceinline__ void range_checked_store(const V& v, __amdgpu_buffer_rsrc_t r, unsigned offset) {
  static_assert(sizeof(V) == 16, "16-byte pieces");
  typedef unsigned u32x4_st __attribute__((ext_vector_type(4)));
  __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_st, v), r, (int)offset, 0, 2 /* non-temporal */);
}
// Descriptor over the valid rows of a tile's output: `row_bytes` per row from `base` on.
// (Base and range are the same for every lane; saying so keeps the compiler from wrapping each store into a loop
// over the distinct descriptors of the wave.)
__device__ __forceinline__ __amdgpu_buffer_rsrc_t tile_rows_rsrc(void* base, int rows, int64_t row_bytes) {
  const int64_t span = (int64_t)rows * row_bytes;
  const int range = __builtin_amdgcn_readfirstlane(span < 0xffffffffLL ? (int)(unsigned)span : -1);
  return __builtin_amdgcn_make_buffer_rsrc((void*)make_uniform((const char*)base), 0, range, 0x00020000);
}

template <typename T, class TL>
__device__ __forceinline__ void epilogue_staged(const f32x16 (&acc)[TL::FM][TL::FN], T* __restrict__ out,
                                                const int64_t* dst, int n0, int ncols, const T* __restrict__ bias,
                                                int64_t sb, char* lds, float* sbias = nullptr) {
  typedef T T8 __attribute__((ext_vector_type(8)));
  constexpr int CPR = TL::BN / 8, PIECES = TL::BM * CPR, PP = PIECES / TL::NT;
  static_assert(PIECES % TL::NT == 0, "pieces must divide evenly");
  stage_accumulators<T, TL>(acc, lds, [&](int tc) {
    return bias != nullptr && n0 + tc < ncols ? to_f32(bias[(int64_t)(n0 + tc) * sb]) : 0.0f;
  }, sbias);
  // In groups: the row offsets of a group, then its pieces, are read from LDS back to back before the first of its
  // stores (written as one conditional store per piece, every piece would wait for two LDS round trips of its own)
  constexpr int GRP = PP >= 16 ? 16 : PP;
  static_assert(PP % GRP == 0, "groups must divide the pieces");
#pragma unroll
  for (int q0 = 0; q0 < PP; q0 += GRP) {
    int64_t d[GRP];
    T8 v[GRP];
#pragma unroll
    for (int g = 0; g < GRP; ++g) d[g] = dst[((q0 + g) * TL::NT + threadIdx.x) / CPR];
#pragma unroll
    for (int g = 0; g < GRP; ++g) {
      const int p = (q0 + g) * TL::NT + threadIdx.x;
      v[g] = *(const T8*)(lds + staged_addr<TL>(p / CPR, (p % CPR) * 8));
    }
#pragma unroll
    for (int g = 0; g < GRP; ++g) asm volatile("" : "+v"(v[g]), "+v"(d[g]));      // keeps the reads above the branches
#pragma unroll
    for (int g = 0; g < GRP; ++g) {
      const int n = n0 + (((q0 + g) * TL::NT + threadIdx.x) % CPR) * 8;
      if (d[g] >= 0 && n < ncols) stream_store(v[g], (T8*)(out + d[g] + n));
    }
  }
}

// Forward GLU through LDS: both halves staged (tile column order: per wave block WTN/2 first-half columns, then
// the matching second-half columns); per 16-byte piece of hidden columns two LDS reads, three coalesced stores.
template <typename T, class TL>
__device__ __forceinline__ void epilogue_glu_fwd_staged(const f32x16 (&acc)[TL::FM][TL::FN], const S2SArgs& a,
                                                        int row0, int rows, int nh0, const T* __restrict__ bias,
                                                        char* lds, float* sbias = nullptr) {
  {
    typedef T T8 __attribute__((ext_vector_type(8)));
    constexpr int HALF = TL::WTN / 2;
    constexpr int CPR = TL::BN / 16, PIECES = TL::BM * CPR, PP = PIECES / TL::NT;
    static_assert(PIECES % TL::NT == 0 && HALF % 8 == 0, "pieces must divide evenly");
    const int F = a.N;
    stage_accumulators<T, TL>(acc, lds, [&](int tc) {
      const int j = tc % TL::WTN;
      const int hc = nh0 + (tc / TL::WTN) * HALF + j % HALF;
      return bias != nullptr && hc < F ? to_f32(bias[(int64_t)(hc + (j >= HALF ? F : 0)) * a.sbn]) : 0.0f;
    }, sbias);
    T* pre = (T*)a.Y;
    T* hid = (T*)a.H;
    // a group's LDS reads are issued back to back ahead of its arithmetic and stores (see epilogue_staged)
    constexpr int GRP = PP >= 8 ? 8 : PP;
    static_assert(PP % GRP == 0, "groups must divide the pieces");
    // which half holds the gate is the same for the whole launch: one copy of the loop for each case instead of a
    // select per element (the accumulators are in LDS by now, so the branch has nothing to carry)
    auto pieces = [&](auto gate_first) {
    const bool gf = gate_first;       // a constant in the two copies of the one-wave-per-SIMD class
#pragma unroll
    for (int q0 = 0; q0 < PP; q0 += GRP) {
      T8 v1[GRP], v2[GRP];
#pragma unroll
      for (int g = 0; g < GRP; ++g) {
        const int p = (q0 + g) * TL::NT + threadIdx.x;
        const int row = p / CPR, hc = (p % CPR) * 8;          // hidden column inside the tile
        const int tc = (hc / HALF) * TL::WTN + hc % HALF;     // tile column of the first-half value
        v1[g] = *(const T8*)(lds + staged_addr<TL>(row, tc));
        v2[g] = *(const T8*)(lds + staged_addr<TL>(row, tc + HALF));
      }
#pragma unroll
      for (int g = 0; g < GRP; ++g) asm volatile("" : "+v"(v1[g]), "+v"(v2[g]));
#pragma unroll
      for (int g = 0; g < GRP; ++g) {
        const int p = (q0 + g) * TL::NT + threadIdx.x;
        const int row = p / CPR, n = nh0 + (p % CPR) * 8;
        if (row >= rows || n >= F) continue;
        const T8 first = v1[g], second = v2[g];
        T8 h;
#pragma unroll
        for (int e = 0; e < 8; e += 2)
          set_pair<T>(h, e / 2, glu_h(a.act, to_f32(gf ? first[e] : second[e]), to_f32(gf ? second[e] : first[e])),
                      glu_h(a.act, to_f32(gf ? first[e + 1] : second[e + 1]), to_f32(gf ? second[e + 1] : first[e + 1])));
        const int64_t r = row0 + row;
        if (pre != nullptr) {
          stream_store(first, (T8*)(pre + r * a.sym + n));
          stream_store(second, (T8*)(pre + r * a.sym + F + n));
        }
        stream_store(h, (T8*)(hid + r * a.shm + n));
      }
    }
    };
    // (the 8-wave classes, with half the registers per wave, keep one copy and select per element: two copies
    // there cost 130 spilled registers)
    if constexpr (!TL::RS) pieces((a.act & 1) != 0);
    else if ((a.act & 1) != 0) pieces(std::true_type());
    else pieces(std::false_type());
  }
}

// Backward through LDS: d(hidden) tile staged, then every thread handles 16-byte pieces (8 columns of one row):
// two coalesced 16-byte loads of the saved pre-activation, two coalesced 16-byte stores of its gradient.
template <typename T, class TL>
__device__ __forceinline__ void epilogue_glu_bwd_staged(const f32x16 (&acc)[TL::FM][TL::FN], const S2SArgs& a,
                                                        int row0, int rows, int n0, char* lds, float* sbias = nullptr) {
  typedef T T8 __attribute__((ext_vector_type(8)));
  constexpr int CPR = TL::BN / 8, PIECES = TL::BM * CPR, PP = PIECES / TL::NT;
  constexpr int GRP = PP >= 8 ? 4 : (PP >= 2 ? PP / 2 : 1);       // pieces per group, two groups in flight
  static_assert(PIECES % TL::NT == 0 && (PP == 1 || PP % (2 * GRP) == 0), "pieces must divide evenly");
  stage_accumulators<T, TL>(acc, lds, [](int) { return 0.0f; }, sbias);
  const int F = a.N;
  const T* pre = (const T*)a.aux;
  T* dpre = (T*)a.Y;
  const __amdgpu_buffer_rsrc_t out_rows = tile_rows_rsrc(dpre + (int64_t)row0 * a.sym, rows, a.sym * 2);
  // The saved pre-activation of the next group of pieces is on its way while the current group is worked on (loads of
  // rows and columns outside the tile's valid part are redirected to its first row / column and their results dropped).
  // One copy of the loop for each position of the gate half (see epilogue_glu_fwd_staged).
  auto pieces = [&](auto gate_first) {
  const bool gf = gate_first;       // a constant in the two copies of the one-wave-per-SIMD class
  T8 p1[2][GRP], p2[2][GRP];
  auto fetch = [&](auto buf, int q0) {
#pragma unroll
    for (int u = 0; u < GRP; ++u) {
      const int p = (q0 + u) * TL::NT + threadIdx.x;
      const int row = p / CPR, n = n0 + (p % CPR) * 8;
      const T* src = pre + (int64_t)(row0 + (row < rows ? row : 0)) * a.saux + (n < F ? n : 0);
      // read exactly once per step: the non-temporal hint keeps it from displacing operand panels in the L2 (-0.3 %)
      p1[decltype(buf)::value][u] = __builtin_nontemporal_load((const T8*)src);
      p2[decltype(buf)::value][u] = __builtin_nontemporal_load((const T8*)(src + F));
    }
  };
  auto work = [&](auto buf, int q0) {
    T8 dh[GRP];
#pragma unroll
    for (int u = 0; u < GRP; ++u) {
      const int p = (q0 + u) * TL::NT + threadIdx.x;
      dh[u] = *(const T8*)(lds + staged_addr<TL>(p / CPR, (p % CPR) * 8));
    }
#pragma unroll
    for (int u = 0; u < GRP; ++u) {
      const int p = (q0 + u) * TL::NT + threadIdx.x;
      const int row = p / CPR, n = n0 + (p % CPR) * 8;
      T8 o1, o2;
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        float f_lin[2], f_gat[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const T v1 = p1[decltype(buf)::value][u][e + h], v2 = p2[decltype(buf)::value][u][e + h];
          glu_grad(a.act, to_f32(dh[u][e + h]), to_f32(gf ? v1 : v2), to_f32(gf ? v2 : v1), f_lin[h], f_gat[h]);
        }
        set_pair<T>(o1, e / 2, gf ? f_gat[0] : f_lin[0], gf ? f_gat[1] : f_lin[1]);
        set_pair<T>(o2, e / 2, gf ? f_lin[0] : f_gat[0], gf ? f_lin[1] : f_gat[1]);
      }
      const unsigned at = row < rows && n < F ? (unsigned)(((int64_t)row * a.sym + n) * 2) : 0xffffffffu;
      range_checked_store(o1, out_rows, at);
      range_checked_store(o2, out_rows, at == 0xffffffffu ? at : at + (unsigned)F * 2);
    }
  };
  fetch(std::integral_constant<int, 0>(), 0);
  // two trips per pass: at the head of a loop the compiler waits for every outstanding load and store
#pragma unroll 2
  for (int q0 = 0; q0 < PP; q0 += 2 * GRP) {
    if constexpr (PP > 1) fetch(std::integral_constant<int, 1>(), q0 + GRP);
    work(std::integral_constant<int, 0>(), q0);
    if constexpr (PP > 1) {
      if (q0 + 2 * GRP < PP) fetch(std::integral_constant<int, 0>(), q0 + 2 * GRP);
      work(std::integral_constant<int, 1>(), q0 + GRP);
    }
  }
  };
  if constexpr (!TL::RS) pieces((a.act & 1) != 0);
  else if ((a.act & 1) != 0) pieces(std::true_type());
  else pieces(std::false_type());
}

// gpt-oss forward through LDS: the tile holds BN consecutive columns of the pre-activation, i.e. BN/2 (gate, up)
// pairs per row; per 16-byte piece one LDS read, one 16-byte store of the pre-activation (if wanted) and one
// 8-byte store of four hidden values.
template <typename T, class TL>
__device__ __forceinline__ void epilogue_oss_fwd_staged(const f32x16 (&acc)[TL::FM][TL::FN], const S2SArgs& a,
                                                        int row0, int rows, int n0, const T* __restrict__ bias,
                                                        char* lds, float* sbias = nullptr) {
  typedef T T8 __attribute__((ext_vector_type(8)));
  typedef T T4 __attribute__((ext_vector_type(4)));
  constexpr int CPR = TL::BN / 8, PIECES = TL::BM * CPR, PP = PIECES / TL::NT;
  static_assert(PIECES % TL::NT == 0, "pieces must divide evenly");
  stage_accumulators<T, TL>(acc, lds, [&](int tc) {
    return bias != nullptr && n0 + tc < a.N ? to_f32(bias[(int64_t)(n0 + tc) * a.sbn]) : 0.0f;
  }, sbias);
  T* pre = (T*)a.Y;
  T* hid = (T*)a.H;
  constexpr int GRP = PP >= 16 ? 16 : PP;               // LDS reads of a group back to back (see epilogue_staged)
  static_assert(PP % GRP == 0, "groups must divide the pieces");
#pragma unroll
  for (int q0 = 0; q0 < PP; q0 += GRP) {
    T8 vs[GRP];
#pragma unroll
    for (int g = 0; g < GRP; ++g) {
      const int p = (q0 + g) * TL::NT + threadIdx.x;
      vs[g] = *(const T8*)(lds + staged_addr<TL>(p / CPR, (p % CPR) * 8));
    }
#pragma unroll
    for (int g = 0; g < GRP; ++g) asm volatile("" : "+v"(vs[g]));
#pragma unroll
    for (int g = 0; g < GRP; ++g) {
      const int p = (q0 + g) * TL::NT + threadIdx.x;
      const int row = p / CPR, n = n0 + (p % CPR) * 8;
      if (row >= rows || n >= a.N) continue;
      const T8 v = vs[g];
      T4 h;
#pragma unroll
      for (int e = 0; e < 4; e += 2)
        set_pair<T>(h, e / 2, oss_h(to_f32(v[2 * e]), to_f32(v[2 * e + 1]), a.alpha, a.limit),
                    oss_h(to_f32(v[2 * e + 2]), to_f32(v[2 * e + 3]), a.alpha, a.limit));
      const int64_t r = row0 + row;
      if (pre != nullptr) stream_store(v, (T8*)(pre + r * a.sym + n));
      stream_store(h, (T4*)(hid + r * a.shm + n / 2));
    }
  }
}

// gpt-oss backward through LDS: d(hidden) tile staged; per piece of 8 hidden columns two 16-byte loads of the saved
// pre-activation pairs and two 16-byte stores of their gradient.
template <typename T, class TL>
__device__ __forceinline__ void epilogue_oss_bwd_staged(const f32x16 (&acc)[TL::FM][TL::FN], const S2SArgs& a,
                                                        int row0, int rows, int n0, char* lds, float* sbias = nullptr) {
  typedef T T8 __attribute__((ext_vector_type(8)));
  constexpr int CPR = TL::BN / 8, PIECES = TL::BM * CPR, PP = PIECES / TL::NT;
  constexpr int GRP = PP >= 8 ? 4 : (PP >= 2 ? PP / 2 : 1);       // pieces per group, two groups in flight
  static_assert(PIECES % TL::NT == 0 && (PP == 1 || PP % (2 * GRP) == 0), "pieces must divide evenly");
  stage_accumulators<T, TL>(acc, lds, [](int) { return 0.0f; }, sbias);
  const int F = a.N;
  const T* pre = (const T*)a.aux;
  T* dpre = (T*)a.Y;
  const __amdgpu_buffer_rsrc_t out_rows = tile_rows_rsrc(dpre + (int64_t)row0 * a.sym, rows, a.sym * 2);
  // next group's saved pre-activation pairs on their way while the current group is worked on (see epilogue_glu_bwd_staged)
  T8 p1[2][GRP], p2[2][GRP];
  auto fetch = [&](auto buf, int q0) {
#pragma unroll
    for (int u = 0; u < GRP; ++u) {
      const int p = (q0 + u) * TL::NT + threadIdx.x;
      const int row = p / CPR, n = n0 + (p % CPR) * 8;
      const T* src = pre + (int64_t)(row0 + (row < rows ? row : 0)) * a.saux + 2 * (n < F ? n : 0);
      p1[decltype(buf)::value][u] = *(const T8*)src;
      p2[decltype(buf)::value][u] = *(const T8*)(src + 8);
    }
  };
  auto work = [&](auto buf, int q0) {
    T8 dh[GRP];
#pragma unroll
    for (int u = 0; u < GRP; ++u) {
      const int p = (q0 + u) * TL::NT + threadIdx.x;
      dh[u] = *(const T8*)(lds + staged_addr<TL>(p / CPR, (p % CPR) * 8));
    }
#pragma unroll
    for (int u = 0; u < GRP; ++u) {
      const int p = (q0 + u) * TL::NT + threadIdx.x;
      const int row = p / CPR, n = n0 + (p % CPR) * 8;
      const T8 v1 = p1[decltype(buf)::value][u], v2 = p2[decltype(buf)::value][u];
      T8 o1, o2;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float dg, du;
        oss_grad(to_f32(v1[2 * e]), to_f32(v1[2 * e + 1]), to_f32(dh[u][e]), a.alpha, a.limit, dg, du);
        set_pair<T>(o1, e, dg, du);
        oss_grad(to_f32(v2[2 * e]), to_f32(v2[2 * e + 1]), to_f32(dh[u][4 + e]), a.alpha, a.limit, dg, du);
        set_pair<T>(o2, e, dg, du);
      }
      const unsigned at = row < rows && n < F ? (unsigned)(((int64_t)row * a.sym + 2 * n) * 2) : 0xffffffffu;
      range_checked_store(o1, out_rows, at);
      range_checked_store(o2, out_rows, at == 0xffffffffu ? at : at + 16u);
    }
  };
  fetch(std::integral_constant<int, 0>(), 0);
  // two trips per pass: at the head of a loop the compiler waits for every outstanding load and store
#pragma unroll 2
  for (int q0 = 0; q0 < PP; q0 += 2 * GRP) {
    if constexpr (PP > 1) fetch(std::integral_constant<int, 1>(), q0 + GRP);
    work(std::integral_constant<int, 0>(), q0);
    if constexpr (PP > 1) {
      if (q0 + 2 * GRP < PP) fetch(std::integral_constant<int, 0>(), q0 + 2 * GRP);
      work(std::integral_constant<int, 1>(), q0 + GRP);
    }
  }
}

// XCD-aware tile order.  Workgroup ids are dealt round-robin to the 8 XCDs (private L2 each), so the 32
// workgroups an XCD runs side by side are the ids x, x+8, ..., x+248 of one 256-block; they are mapped to
// one 8 x 4 "super tile" of output tiles.  Per 64-deep slice that group touches 8 row panels + 4 column
// panels for 32 tiles' worth of operands, i.e. 3/8 of the requests miss the XCD's L2 instead of 9/16 for
// a 16 x 2 arrangement and 33/64 for 32 x 1 (measured at the Mixtral shape: 13.3 GB fetched from the
// memory side per launch against 20.5 GB for 16 x 2).  Super tiles are numbered row-super fastest so that
// the XCDs working at the same time share column panels through the memory-side cache.
struct Raster {
  static constexpr int SM = 8, SN = 4;
  int m_tiles, n_tiles, m_supers, n_supers, supers, gm;
  int striped;                             // 1: column-striped order of the memory-bound classes (see make_striped)
  int64_t grid_size;                       // host side only: number of workgroups (may exceed what a launch takes)
  __host__ int64_t grid() const { return grid_size; }
  // (ml, nl): position of the tile inside its super tile
  __device__ __forceinline__ bool map(int pid, int& m, int& n, int& ml, int& nl) const {
    const int x = pid & 7, i = pid >> 3;
    if (striped) {
      // XCD x owns the tile columns n = x (mod 8) of every tile row; rows slowest, in groups of gm
      // (the residue class an XCD owns moves on with every group of rows, so that a column count that is not a
      // multiple of 8 does not leave the same XCDs short every time)
      const int m_lo = i % gm, j = i / gm;
      m = (j / n_supers) * gm + m_lo;
      n = (j % n_supers) * 8 + ((x + j / n_supers) & 7);
      ml = nl = 0;
      return m < m_tiles && n < n_tiles;
    }
    // The 8 supers of step j = i / 32 go to the 8 XCDs rotated by j: supers differ in how many of their tiles
    // exist (partial last column-super, empty tile rows), and a fixed assignment would give some XCDs the full
    // ones every time.
    const int j = i / (SM * SN);
    const int s = j * 8 + ((x + j) & 7), r = i % (SM * SN);
    if (s >= supers) return false;
    ml = r % SM;
    nl = r / SM;
    // bands of `gm` row-supers; inside a band column-super major, row-super fastest
    const int band = s / (gm * n_supers);
    const int rem = s - band * gm * n_supers;
    const int g = min(gm, m_supers - band * gm);
    m = (band * gm + rem % g) * SM + r % SM;
    n = (rem / g) * SN + r / SM;
    return m < m_tiles && n < n_tiles;
  }
};

// `gm`: row-supers per band.  A band's row panels (gm * 8 tiles) are reused by every column-super while the
// column panels stream past once, so the band should be small enough for its row panels to stay in the
// memory-side cache and large enough to keep all XCDs inside one band.
static Raster make_raster(int64_t m_tiles, int n_tiles, int gm) {
  Raster r;
  r.m_tiles = (int)m_tiles;
  r.n_tiles = n_tiles;
  r.m_supers = (int)((m_tiles + Raster::SM - 1) / Raster::SM);
  r.n_supers = (n_tiles + Raster::SN - 1) / Raster::SN;
  r.striped = 0;
  r.gm = gm < 1 ? 1 : (gm > r.m_supers ? r.m_supers : gm);
  const int64_t supers = (int64_t)r.m_supers * r.n_supers;
  r.grid_size = (supers + 7) / 8 * 8 * Raster::SM * Raster::SN;
  r.supers = supers > 0x7fffffffLL ? 0x7fffffff : (int)supers;   // such a grid is rejected by the launchers
  return r;
}

// Order of the memory-bound (ring) classes.  The grid covers an upper bound of the tile rows, so some rows are
// empty, and which ones is known only on the device: every XCD therefore takes the same share of every tile row
// (its own residue class of tile columns), and the empty rows, which come last, cost nothing but their launch.
// `gm` consecutive tile rows visit a tile column back to back on one XCD, so that an expert with several tile
// rows finds its weight panel in that XCD's L2.
static Raster make_striped(int64_t m_tiles, int n_tiles, int gm) {
  Raster r;
  r.striped = 1;
  r.m_tiles = (int)m_tiles;
  r.n_tiles = n_tiles;
  r.gm = gm < 1 ? 1 : (gm > m_tiles ? (int)m_tiles : gm);
  r.n_supers = (n_tiles + 7) / 8;                                        // tile columns per XCD
  r.m_supers = (int)((m_tiles + r.gm - 1) / r.gm);                       // groups of tile rows
  r.supers = 0;
  r.grid_size = (int64_t)r.m_supers * r.gm * r.n_supers * 8;
  return r;
}

// =====================================================================================================
// scatter2scatter
// =====================================================================================================
template <typename T, class TL, bool B_TR>
__global__ __launch_bounds__(TL::NT) void s2s_mfma_kernel(S2SArgs a, Raster rast) {
  typedef DirectOp<TL::BM, TL::NT> AOp;
  // Ring classes serve launches with at most a tile row or two per expert: (nearly) every weight element is read
  // once, and with the non-temporal hint it does not push the token rows, which every workgroup of a tile row reads,
  // out of the L2s (hint extended from the 32-/64-row classes to all ring classes: Mixtral layer forward at 256 /
  // 384 / 448 tokens 0.539 -> 0.505 / 0.559 -> 0.526 / 0.711 -> 0.688 ms, neutral from 768 tokens on)
  constexpr bool W_ONCE = TL::NS > 2;
  typedef typename std::conditional<B_TR, TransOp<TL::BN, TL::NT, W_ONCE>, DirectOp<TL::BN, TL::NT, W_ONCE>>::type BOp;
  constexpr int STAGE = AOp::LDS_BYTES + BOp::LDS_BYTES;
  __shared__ __attribute__((aligned(16))) char lds[TL::NS * STAGE];
  __shared__ int64_t sDst[TL::BM];
  __shared__ int sSrc[TL::BM];
  __shared__ __attribute__((aligned(16))) float sBias[TL::RS ? TL::BN : 4];

  // Contraction parts (the class of the experts' last tiles only): the grid is `ksplit` copies of the raster, copy
  // c multiplies the c-th part of the contraction (a raster is a multiple of 8 workgroups, so the XCD of a workgroup
  // is still its first index modulo 8)
  constexpr bool CAN_SPLIT = TL::BM == 128 && TL::BN == 256 && TL::NS == 3;
  // (the parts are the grid's second dimension; no division here: the compiler would do it in the vector unit and
  // everything derived from it, loop counters and LDS addresses included, would leave the scalar registers)
  const int part = CAN_SPLIT ? (int)blockIdx.y : 0;
  const int klen = CAN_SPLIT && a.ksplit > 1 ? a.k_part : a.K;
  const int k_first = part * klen;
  int m_tile, n_tile, m_loc, n_loc;
  if (!rast.map(blockIdx.x, m_tile, n_tile, m_loc, n_loc)) return;
  int e, row0, rows;
  if (a.tail_mode == 2) {
    // one tile row per expert: the rows its last 256-row tile would hold, when there are at most BM of them
    e = m_tile;
    if (!find_remainder<256>(a.off, a.E, e, TL::BM, row0, rows)) return;
  } else if (m_tile >= a.m_count ||
             !find_tile<TL::BM>(a.off, a.E, a.m_begin + m_tile, e, row0, rows, a.tail_mode == 1 ? REMAINDER_ROWS : 0)) {
    return;
  }
  // first output column of the tile; the fused forward GLU tile holds BN/2 columns of each half
  const int n0 = a.glu == 1 ? n_tile * (TL::BN / 2) : n_tile * TL::BN;

  // Row tables, one tile row per thread.  The main loop needs only the source rows; where the output rows go is
  // stored after it, so that a launch whose input is grouped and whose output is not (layer-2 forward, layer-1
  // input gradient) does not wait for the index vector before its first operand loads.
  static_assert(TL::BM <= TL::NT, "one row of the tables per thread");
  int64_t slot = 0;                                         // idx[n] where it is needed, else unused
  int64_t own_row = 0;
  {
    const int m = threadIdx.x;
    if (m < TL::BM) {
      const int mm = m < rows ? m : rows - 1;               // tail rows re-read the last valid row
      own_row = row0 + mm;
      if (!a.x_grouped || !a.y_grouped) slot = a.idx[own_row];
      sSrc[m] = a.x_grouped ? (int)own_row : (int)(slot / a.fan_out);
    }
  }
  __syncthreads();

  AOp A;
  A.rot = TL::RS ? 0 : (n_loc * AOp::R / Raster::SN) % AOp::R;      // the row panel has SN sharers
  // Lane offsets are 32-bit: grouped input rows are taken relative to the tile's first row (so that the input may
  // be of any size), gathered ones relative to the start of the token matrix.
  const int64_t sxm = a.sxm;
  const int src0 = a.x_grouped ? row0 : 0;
  const char* Xb = (const char*)a.X + ((int64_t)src0 * sxm + k_first) * 2;
  A.init(Xb, [&](int row) { return (int64_t)(sSrc[row] - src0) * sxm * 2; });
  BOp B;
  B.rot = TL::RS ? 0 : (m_loc * BOp::R / Raster::SM) % BOp::R;      // the column panel has SM sharers
  const char* Wb = (const char*)a.W + ((int64_t)e * a.swe + (int64_t)k_first * (B_TR ? a.swk : 1)) * 2;
  if (a.glu == 1) {
    // tile column tc -> weight column: wave block tc / WTN, first half of the block from [0, F), second from [F, 2F)
    const int F = a.N;
    auto wcol = [&](int tc) {
      const int j = tc % TL::WTN;
      const int hc = n0 + (tc / TL::WTN) * (TL::WTN / 2) + j % (TL::WTN / 2);
      return hc < F ? hc + (j >= TL::WTN / 2 ? F : 0) : 0;
    };
    if constexpr (B_TR) {
      B.init_cols(Wb, a.swk * 2, wcol);
    } else {
      const int64_t swn = a.swn;
      B.init(Wb, [&](int row) { return (int64_t)wcol(row) * swn * 2; });
    }
  } else if constexpr (B_TR) {
    B.init(Wb + (int64_t)n0 * 2, a.swk * 2, a.N - n0);
  } else {
    const int64_t swn = a.swn;
    const int N = a.N;
    B.init(Wb, [&](int row) { const int n = n0 + row < N ? n0 + row : N - 1; return (int64_t)n * swn * 2; });
  }

  f32x16 acc[TL::FM][TL::FN];
  float rs[TL::FM];
#pragma unroll
  for (int i = 0; i < TL::FM; ++i)
#pragma unroll
    for (int j = 0; j < TL::FN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  if constexpr (TL::RS) mainloop_rs<T, TL, AOp, BOp>(A, B, a.K, lds, acc);
  else if constexpr (TL::NS > 2) mainloop_ring<T, TL, AOp, BOp>(A, B, klen, lds, acc);
  else mainloop<T, TL, AOp, BOp, false>(A, B, a.K, lds, false, acc, rs);

  if constexpr (CAN_SPLIT) {
    if (a.ksplit > 1) {
      // This part's accumulators as they lie in the registers, 16 bytes per lane and store (whole 1 KB runs per
      // wave); splitk_reduce_kernel knows which output element each of them belongs to.
      typedef float f32x4_t __attribute__((ext_vector_type(4)));
      f32x4_t* P = (f32x4_t*)a.partial +
                   (((int64_t)e * rast.n_tiles + n_tile) * a.ksplit + part) * (TL::FM * TL::FN * 4 * TL::NT);
#pragma unroll
      for (int i = 0; i < TL::FM; ++i)
#pragma unroll
        for (int j = 0; j < TL::FN; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g)
            P[((i * TL::FN + j) * 4 + g) * TL::NT + threadIdx.x] =
                f32x4_t{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
      return;
    }
  }

  {
    asm volatile("" : "+v"(slot), "+v"(own_row));           // not looked at before this point
    const int m = threadIdx.x;
    if (m < TL::BM) sDst[m] = m < rows ? (a.y_grouped ? own_row : slot) * a.sym : -1;
  }
  __syncthreads();
  const T* bias = a.b ? (const T*)a.b + (int64_t)e * a.sbe : nullptr;
  // 16-byte pieces need every row start 16-byte aligned; otherwise the lane-wise epilogues are used (the
  // one-wave-per-SIMD class is only launched on aligned outputs)
  if constexpr (TL::RS) {
    if (a.glu == 0) epilogue_staged<T, TL>(acc, (T*)a.Y, sDst, n0, a.N, bias, a.sbn, lds, sBias);
    else if (a.glu == 1) epilogue_glu_fwd_staged<T, TL>(acc, a, row0, rows, n0, bias, lds, sBias);
    else if (a.glu == 2) epilogue_glu_bwd_staged<T, TL>(acc, a, row0, rows, n0, lds, sBias);
    else if (a.glu == 3) epilogue_oss_fwd_staged<T, TL>(acc, a, row0, rows, n0, bias, lds, sBias);
    else epilogue_oss_bwd_staged<T, TL>(acc, a, row0, rows, n0, lds, sBias);
  } else if (a.glu == 0) {
    const bool al16 = (((uintptr_t)a.Y & 15) == 0) && ((a.sym | a.N) & 7) == 0;
    if (al16) epilogue_staged<T, TL>(acc, (T*)a.Y, sDst, n0, a.N, bias, a.sbn, lds);
    else epilogue<T, TL>(acc, (T*)a.Y, sDst, n0, a.N, bias, a.sbn);
  } else if (a.glu == 1) {
    const bool al16 = ((((uintptr_t)a.Y | (uintptr_t)a.H) & 15) == 0) && ((a.sym | a.shm | a.N) & 7) == 0;
    if (al16) epilogue_glu_fwd_staged<T, TL>(acc, a, row0, rows, n0, bias, lds);
    else epilogue_glu_fwd<T, TL>(acc, a, row0, rows, n0, bias);
  } else if (a.glu == 2) {
    const bool al16 = ((((uintptr_t)a.aux | (uintptr_t)a.Y) & 15) == 0) && ((a.saux | a.sym | a.N) & 7) == 0;
    if (al16) epilogue_glu_bwd_staged<T, TL>(acc, a, row0, rows, n0, lds);
    else epilogue_glu_bwd<T, TL>(acc, a, row0, rows, n0);
  } else if (a.glu == 3) {
    epilogue_oss_fwd_staged<T, TL>(acc, a, row0, rows, n0, bias, lds);      // alignment checked by the launcher
  } else {
    epilogue_oss_bwd_staged<T, TL>(acc, a, row0, rows, n0, lds);
  }
}

// Second half of a product whose last tiles were multiplied in contraction parts: one workgroup per (expert, tile
// column) with the thread layout of the 128 x 256 class, so that thread t finds the accumulators that thread t of
// every part left behind.  The parts are added in ascending order (the same result on every run), then bias,
// rounding and the scatter of the rows as in the plain epilogue.
template <typename T>
__global__ __launch_bounds__(512) void splitk_reduce_kernel(S2SArgs a, int n_tiles) {
  typedef Tile<128, 256, 2, 4, 3> TL;
  typedef float f32x4_t __attribute__((ext_vector_type(4)));
  typedef T T4 __attribute__((ext_vector_type(4)));
  const int e = blockIdx.y, n_tile = blockIdx.x;
  int row0, rows;
  if (!find_remainder<256>(a.off, a.E, e, TL::BM, row0, rows)) return;
  const int wave = threadIdx.x >> 6, l = lane_id();
  const int wm = wave / TL::WN, wn = wave % TL::WN;
  const f32x4_t* P = (const f32x4_t*)a.partial + ((int64_t)e * n_tiles + n_tile) * a.ksplit * (TL::FM * TL::FN * 4 * TL::NT);
  const T* bias = a.b ? (const T*)a.b + (int64_t)e * a.sbe : nullptr;
  T* out = (T*)a.Y;
  const bool base_ok = ((uintptr_t)out & 7) == 0;
#pragma unroll
  for (int i = 0; i < TL::FM; ++i) {
    const int m = wm * TL::WTM + i * 32 + (l & 31);
    if (m >= rows) continue;
    const int64_t row = row0 + m;
    const int64_t d = (a.y_grouped ? row : a.idx[row]) * a.sym;
#pragma unroll
    for (int j = 0; j < TL::FN; ++j) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n_tile * TL::BN + wn * TL::WTN + j * 32 + g * 8 + (l >> 5) * 4;
        if (n >= a.N) continue;
        const int slot = ((i * TL::FN + j) * 4 + g) * TL::NT + threadIdx.x;
        f32x4_t v = P[slot];
        for (int c = 1; c < a.ksplit; ++c) v += P[(int64_t)c * (TL::FM * TL::FN * 4 * TL::NT) + slot];
        if (bias != nullptr) {
#pragma unroll
          for (int q = 0; q < 4; ++q)
            if (n + q < a.N) v[q] += to_f32(bias[(int64_t)(n + q) * a.sbn]);
        }
        if (base_ok && n + 3 < a.N && ((d + n) & 3) == 0) {
          *(T4*)(out + d + n) = T4{from_f32<T>(v[0]), from_f32<T>(v[1]), from_f32<T>(v[2]), from_f32<T>(v[3])};
        } else {
#pragma unroll
          for (int q = 0; q < 4; ++q)
            if (n + q < a.N) out[d + n + q] = from_f32<T>(v[q]);
        }
      }
    }
  }
}

template <typename T, class TL>
static int launch_s2s(const S2SArgs& a, bool b_tr, hipStream_t st) {
  const int bn = a.glu == 1 ? TL::BN / 2 : TL::BN;     // output columns per tile
  const int n_tiles = (a.N + bn - 1) / bn;
  const int64_t m_tiles = a.tail_mode == 2 ? a.E : std::min<int64_t>(max_tiles(a.L, a.E, TL::BM) - a.m_begin, a.m_count);
  // With only a few tile rows per expert no weight panel is shared by the tile rows of a super tile; the striped
  // order at least keeps the tile rows of one expert together on one XCD.
  const bool striped = TL::NS > 2 || a.L / a.E < STRIPE_BELOW;
  const Raster r = striped ? make_striped(m_tiles, n_tiles, GM_RING) : make_raster(m_tiles, n_tiles, GM_S2S);
  const int64_t grid = r.grid();
  const unsigned parts = a.ksplit > 1 ? (unsigned)a.ksplit : 1u;
  if (grid > 0x7fffffffLL || m_tiles > 0x7fffffffLL) { set_error("smoe_scatter2scatter: grid too large"); return SMOE_ERR_RANGE; }
  if constexpr (TL::BN % 128 == 0) {
    if (b_tr) {
      hipLaunchKernelGGL((s2s_mfma_kernel<T, TL, true>), dim3((unsigned)grid, parts), dim3(TL::NT), 0, st, a, r);
      return launch_status("s2s_mfma_kernel");
    }
  }
  hipLaunchKernelGGL((s2s_mfma_kernel<T, TL, false>), dim3((unsigned)grid, parts), dim3(TL::NT), 0, st, a, r);
  return launch_status("s2s_mfma_kernel");
}

// Launches of only a few rounds of 256 x 256 tiles (one tile per CU and round) lose up to a whole round to the
// partly filled last one; tiles of half the width take HALF_WIDTH_COST of the time and round off finer.  The
// number of tile rows is only known on the device; the host prices both classes with its expectation for rows
// spread evenly over the experts (binomial spread around the mean).  A wrong guess costs speed only.  Mixtral
// expert shapes, layer 1 + layer 2 forward: 896 tokens 912 -> 833 us, 1984..2112 tokens -3 %, nothing lost
// anywhere between 800 and 3136 tokens.
static constexpr int NUM_CU = 256;
static constexpr double HALF_WIDTH_COST = 0.58;
// expected number of 256-row tiles, rounded; `skip_small`: without the experts' last tiles of at most that many rows
static double expected_row_tiles(int64_t L, int E, int skip_small = 0) {
  const double avg = (double)L / E, sd = sqrt(avg * (1.0 - 1.0 / E)) + 1e-9;
  auto above = [&](double x) { return 0.5 * erfc((x - avg) / (sd * 1.41421356)); };      // P(rows > x)
  // expected ceil(rows / 256) = 1 + sum_j P(rows > 256 j); the terms more than 6 sd below the mean are 1
  const int j_lo = std::max(1, (int)((avg - 6 * sd) / 256.0));
  double per_expert = j_lo;
  for (int j = j_lo; j * 256.0 < avg + 6 * sd; ++j) per_expert += above(j * 256.0);
  if (skip_small > 0) {
    // minus P(rows mod 256 in [1, skip_small])
    for (int j = std::max(0, j_lo - 1); j * 256.0 < avg + 6 * sd; ++j)
      per_expert -= above(j * 256.0 + 0.5) - above(j * 256.0 + skip_small + 0.5);
  }
  return nearbyint(per_expert * E);
}
static bool half_width_wins(const S2SArgs& a) {
  const int cols = a.glu == 1 ? 128 : 256;               // output columns of a 256-wide tile
  const int64_t n_full = (a.N + cols - 1) / cols, n_half = (a.N + cols / 2 - 1) / (cols / 2);
  if (max_tiles(a.L, a.E, 256) * n_full > 4 * NUM_CU) return false;
  const double m = expected_row_tiles(a.L, a.E);
  if (m * n_full < 96) return false;                     // far below one round: nothing to win, keep the default
  const double full = ceil(m * n_full / NUM_CU), half = ceil(m * n_half / NUM_CU) * HALF_WIDTH_COST;
  return half < 0.95 * full;
}

// A launch of a few whole rounds plus a remainder of up to half a round pays a whole round for the remainder.
// Such a product is cut by tile rows: the whole rounds stay with the 256 x 256 class, the remaining tile rows go
// to a second launch of 256 x 128 tiles (twice the workgroups, 0.58 of the time).  Returns the number of tile
// rows of the first launch, 0 when the product is not split.  Plain products only (no fused unit behind them).
// Mixtral shape, 16384 tokens (8.25 rounds in the launches with 4096 output columns): layer-2 forward
// 3.47 -> 3.34 ms, layer-1 input gradient 7.03 -> 6.68 ms; 128 x 128 tiles for the remainder were slower
// (four times the workgroups at 0.75 of the time).
static int tail_split(const S2SArgs& a) {
  if (a.glu != 0 || a.m_begin != 0) return 0;
  const int64_t n_full = (a.N + 255) / 256;
  const int64_t upper = max_tiles(a.L, a.E, 256);
  if (upper * n_full > 26 * NUM_CU) return 0;
  const double m = expected_row_tiles(a.L, a.E, a.tail_mode == 1 ? REMAINDER_ROWS : 0);
  const int64_t whole = (int64_t)(m * n_full) / NUM_CU;           // whole rounds
  if (whole < 2) return 0;
  const int64_t m_first = whole * NUM_CU / n_full;                // tile rows that fit the whole rounds
  const int64_t rest = ((int64_t)m - m_first) * n_full;           // expected 256 x 256 tiles of the remainder
  // (no remainder expected: the second launch still stands by for a tile row more than expected, which would
  // otherwise cost the first launch a whole round; its workgroups exit at once when there is none)
  if (m_first <= 0 || rest < 0 || upper <= m_first || rest > NUM_CU / 2 + 8) return 0;
  return (int)m_first;
}

// The 256 x 256 class.  Products with a long enough contraction run on the one-wave-per-SIMD form of it
// (mainloop_rs: Mixtral shape, per 64-deep slice 2 300-2 420 cycles against 2 890-3 000; its prologue and its
// epilogue, run by half as many threads, cost about 5 000 cycles more per tile, which a 12-slice contraction does not
// earn back: K = 768 is 5 % slower, K = 1536 even, K = 2048 is 5-8 % faster).
// Both forms add up every output element in the same order: the same bits.
static constexpr int RS_MIN_K = 1792;
static constexpr int RS_XTY_MIN_ROWS = 2048;      // groupXtY: average rows per expert from which that form is used
template <typename T>
static int launch_main_class(const S2SArgs& a, bool b_tr, hipStream_t st) {
  bool al16 = true;             // the one-wave-per-SIMD form has only the LDS-staged epilogues (16-byte pieces)
  if (a.glu == 0) al16 = (((uintptr_t)a.Y & 15) == 0) && ((a.sym | a.N) & 7) == 0;
  else if (a.glu == 1) al16 = ((((uintptr_t)a.Y | (uintptr_t)a.H) & 15) == 0) && ((a.sym | a.shm | a.N) & 7) == 0;
  else if (a.glu == 2) al16 = ((((uintptr_t)a.aux | (uintptr_t)a.Y) & 15) == 0) && ((a.saux | a.sym | a.N) & 7) == 0;
  if (al16 && a.K % BK == 0 && a.K >= RS_MIN_K)
    return launch_s2s<T, Tile<256, 256, 2, 2, 2, true>>(a, b_tr, st);
  return launch_s2s<T, Tile<256, 256, 2, 4>>(a, b_tr, st);
}

// A partly filled tile costs what a full one costs, and every expert ends in one (its row count modulo 256).  Products
// with few tile rows per expert that are large enough to carry a second launch leave the last tiles of at most 128
// rows to a launch of 128 x 256 tiles, one tile row per expert (which experts have such a tile is known only on the
// device: the second launch covers all of them and the others' workgroups exit).  Same bits as one launch: every
// class adds up an output element in the same order.  Measured per training step, same box: 32 experts with skewed
// loads, 1024 rows on average (a fifth of the tile rows partly filled, several experts below 128 rows) 5.76 -> 5.51 ms;
// 128 experts of 2048 +- 45 rows 8.01 -> 7.97 ms; 8 experts of 4096 rows 29.36 -> 29.58 ms (the second launch costs
// what it saves): taken below 1536 rows per expert.
// With many rows per expert and few tile columns that second launch has too few workgroups for the chip and every one
// of them walks the whole contraction (8 experts x 16 tile columns: 64 to 128 workgroups, as long as a full tile).
// Plain products with a caller workspace then cut the contraction of those tiles into parts, one workgroup each
// (tail_ksplit), and a small launch adds the parts up: float32 partial sums in a fixed order, so the result is the
// same on every run, but no longer the same bits as the unsplit product (its additions are grouped differently).
static constexpr double REMAINDER_MIN_FLOP = 2e11;
static constexpr int REMAINDER_MAX_AVG_ROWS = 1536;
static constexpr int KSPLIT_MAX = 8;
static constexpr int KSPLIT_MIN_SLICES = 16;      // 64-deep slices a part must keep
static constexpr int64_t SPLITK_TILE_FLOATS = 128 * 256;

// Parts to cut the contraction of the last tiles into: enough for one workgroup per CU when half of the experts
// have such a tile; 1 = not split (also: no workspace, fused unit behind the product, ragged contraction).
static int tail_ksplit_for(int64_t K, int64_t N, int E, int glu) {
  if (glu != 0 || K % BK != 0) return 1;
  const int64_t n_tiles = (N + 255) / 256;
  const int64_t wgs = std::max<int64_t>(1, (int64_t)(E + 1) / 2 * n_tiles);
  int ks = 1;
  while (ks < KSPLIT_MAX && wgs * ks < NUM_CU && K % (BK * ks * 2) == 0 && K / (BK * ks * 2) >= KSPLIT_MIN_SLICES) ks *= 2;
  return ks;
}
static int64_t splitk_floats(int64_t N, int E, int ks) { return (int64_t)E * ((N + 255) / 256) * ks * SPLITK_TILE_FLOATS; }
static int tail_ksplit(const S2SArgs& a) {
  if (a.L / a.E < REMAINDER_MAX_AVG_ROWS) return 1;      // enough last tiles to fill the chip as they are
  const int ks = tail_ksplit_for(a.K, a.N, a.E, a.glu);
  if (ks <= 1 || a.partial == nullptr || a.partial_floats < splitk_floats(a.N, a.E, ks)) return 1;
  return ks;
}

int64_t s2s_workspace_floats(int64_t L, int64_t K, int64_t N, int E, int dtype) {
  if ((dtype != SMOE_BF16 && dtype != SMOE_F16) || E <= 0 || L / E < REMAINDER_MAX_AVG_ROWS) return 0;
  if (2.0 * (double)L * K * N < REMAINDER_MIN_FLOP) return 0;
  const int ks = tail_ksplit_for(K, N, E, 0);
  return ks > 1 ? splitk_floats(N, E, ks) : 0;
}

static bool cut_tails(const S2SArgs& a) {
  const bool whole = a.m_begin == 0 && a.m_count == 0x7fffffff && a.tail_mode == 0;
  if (!whole || 2.0 * (double)a.L * a.K * (a.glu == 1 ? 2.0 * a.N : (double)a.N) < REMAINDER_MIN_FLOP) return false;
  return a.L / a.E < REMAINDER_MAX_AVG_ROWS || tail_ksplit(a) > 1;
}

template <typename T>
static int launch_tails(const S2SArgs& a, bool b_tr, hipStream_t st) {
  typedef Tile<128, 256, 2, 4, 3> TailTile;
  S2SArgs rest = a;
  rest.tail_mode = 2;
  rest.ksplit = tail_ksplit(a);
  rest.k_part = a.K / rest.ksplit;
  if (const int rc = launch_s2s<T, TailTile>(rest, b_tr, st)) return rc;
  if (rest.ksplit <= 1) return 0;
  const int n_tiles = (a.N + 255) / 256;
  hipLaunchKernelGGL(splitk_reduce_kernel<T>, dim3((unsigned)n_tiles, (unsigned)a.E), dim3(512), 0, st, rest, n_tiles);
  return launch_status("splitk_reduce_kernel");
}

// A whole product in the 256-row classes: the experts' sparsely filled last tiles apart (cut_tails), the rest as
// whole rounds of 256 x 256 tiles plus a remainder of 256 x 128 tiles (tail_split) or as one launch.
template <typename T>
static int launch_main(const S2SArgs& a, bool b_tr, hipStream_t st) {
  S2SArgs m = a;
  const bool tails = cut_tails(a);
  if (tails) m.tail_mode = 1;
  int rc;
  if (const int m_first = a.L / a.E >= ROWS256_BELOW ? tail_split(m) : 0) {
    S2SArgs first = m, rest = m;
    first.m_count = m_first;
    rest.m_begin = m_first;
    // both classes have 256-row tiles, hence the same numbering of the tile rows
    rc = launch_main_class<T>(first, b_tr, st);
    if (rc == 0) rc = launch_s2s<T, Tile<256, 128, 4, 2, 3>>(rest, b_tr, st);
  } else {
    rc = launch_main_class<T>(m, b_tr, st);
  }
  if (rc != 0 || !tails) return rc;
  return launch_tails<T>(a, b_tr, st);
}

template <typename T>
static int dispatch_s2s(const S2SArgs& a, bool b_tr, hipStream_t st) {
  // the gpt-oss epilogues exist only in their LDS-staged form (16-byte pieces)
  if (a.glu == 3 && !((((uintptr_t)a.Y & 15) | ((uintptr_t)a.H & 7)) == 0 && (a.sym & 7) == 0 && (a.shm & 3) == 0 &&
                      (a.N & 7) == 0))
    return SMOE_ERR_UNSUPPORTED;
  if (a.glu == 4 && !((((uintptr_t)a.aux | (uintptr_t)a.Y) & 15) == 0 && ((a.saux | a.sym | a.N) & 7) == 0))
    return SMOE_ERR_UNSUPPORTED;
  // the backward gated epilogues address a tile's output rows with 32-bit byte offsets from its first row
  if ((a.glu == 2 || a.glu == 4) && a.sym * 2 * 256 >= 0xffffffffLL) return SMOE_ERR_UNSUPPORTED;
  const int64_t avg = a.L / a.E;
  if (avg >= ROWS256_BELOW) {
    S2SArgs m = a;
    if (cut_tails(a)) m.tail_mode = 1;
    if (tail_split(m) != 0 || !half_width_wins(a)) return launch_main<T>(a, b_tr, st);
  }
  // Wide launches (enough 256-wide tile columns to fill the chip twice even with one tile row per expert, e.g.
  // Mixtral layer 1) move half as many token rows per weight byte with 256-wide tiles as with 128-wide ones:
  // the 256 x 256 class from 136 rows per expert on (544..832 Mixtral tokens: layer 1 -9..-11 % against the
  // 256 x 128 ring), 128 x 256 ring tiles below (experts of about one 128-row tile: 448 tokens 518 -> 373 us,
  // 512 tokens 520 -> 455 us).  Launches with few tile columns (Mixtral layer 2) are faster in the classes below.
  const bool wide = (int64_t)a.E * ((a.N + (a.glu == 1 ? 127 : 255)) / (a.glu == 1 ? 128 : 256)) >= 2 * NUM_CU;
  if (wide && avg >= ROWS128W_BELOW) return launch_main<T>(a, b_tr, st);
  if (wide && avg >= ROWS64_BELOW) return launch_s2s<T, Tile<128, 256, 2, 4, 3>>(a, b_tr, st);
  // Below that the launch is a stream over the weights: ring-buffered classes, tile height by rows per expert
  if (avg >= ROWS128_BELOW) return launch_s2s<T, Tile<256, 128, 4, 2, 3>>(a, b_tr, st);
  if (avg >= ROWS32_BELOW && avg < ROWS64_BELOW) return launch_s2s<T, Tile<64, 128, 2, 2, 5>>(a, b_tr, st);
  // With one column block per wave the fused forward GLU exists only in its LDS-staged form (16-byte pieces)
  if (a.glu == 1 && !((((uintptr_t)a.Y | (uintptr_t)a.H) & 15) == 0 && ((a.sym | a.shm | a.N) & 7) == 0))
    return SMOE_ERR_UNSUPPORTED;
  if (avg >= ROWS64_BELOW) return launch_s2s<T, Tile<128, 128, 2, 4, 3>>(a, b_tr, st);
  // With few output columns the 128-wide tiles do not give every CU a workgroup, and what counts is bytes in
  // flight across the chip: narrower tiles (K-contiguous weights only) restore the count.
  const int64_t wgs128 = max_tiles(a.L, a.E, 32) * ((a.N + 127) / 128);
  if (!b_tr && wgs128 < 96) return launch_s2s<T, Tile<32, 32, 1, 1, 8>>(a, b_tr, st);
  if (!b_tr && wgs128 < 192) return launch_s2s<T, Tile<32, 64, 1, 2, 6>>(a, b_tr, st);
  return launch_s2s<T, Tile<32, 128, 1, 4, 6>>(a, b_tr, st);
}

static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }
static bool fits_u32(int64_t bytes) { return bytes >= 0 && bytes < (int64_t)0xfff00000LL; }

bool try_s2s_mfma(const S2SArgs& a, int dtype, hipStream_t st, int& rc) {
  if (dtype == SMOE_F32) return try_s2s_f32(a, st, rc);
  if (dtype != SMOE_BF16 && dtype != SMOE_F16) return false;
  if (a.K < 8 || a.K % 8 != 0) return false;
  if (a.sxk != 1 || a.sxm % 8 != 0 || !aligned16(a.X)) return false;
  if (a.syn != 1) return false;
  if (!aligned16(a.W) || a.swe % 8 != 0) return false;
  bool b_tr;
  if (a.swk == 1 && a.swn % 8 == 0) b_tr = false;
  else if (a.swn == 1 && a.swk % 8 == 0 && a.N % 8 == 0) b_tr = true;
  else return false;
  // lane offsets inside the kernel are 32-bit byte offsets from a scalar base (X, and W[e])
  const int64_t x_rows = a.x_grouped ? 256 : a.L / a.fan_out;        // grouped rows: relative to the tile's first row
  if (fits_u32((x_rows - 1) * a.sxm * 2 + (int64_t)a.K * 2) == false) return false;
  const int64_t w_cols = a.glu == 1 ? 2 * (int64_t)a.N : a.N;
  if (b_tr ? !fits_u32(BK * a.swk * 2 + w_cols * 2) : !fits_u32((w_cols - 1) * a.swn * 2 + (int64_t)a.K * 2))
    return false;
  if (!b_tr && try_s2s_rowdot(a, dtype, st, rc)) return true;
  rc = dtype == SMOE_BF16 ? dispatch_s2s<bf16_t>(a, b_tr, st) : dispatch_s2s<f16_t>(a, b_tr, st);
  return true;
}

// =====================================================================================================
// groupXtY:  OUT[e] (P x Q, Q contiguous) = sum_r  Pm[r, :]^T  Qm[r, :]   over the expert's rows
//   DW stored (E,N,K)-contiguous (the ParallelExperts layout):  P = dY (N cols), Q = X  (K cols)
//   DW stored (E,K,N)-contiguous:                              P = X  (K cols), Q = dY (N cols)
// Column sums of dY (the bias gradient) ride along: the first column of tiles adds up the dY fragments it
// already holds in registers.
// =====================================================================================================
struct XtYPlan {
  const void* P; int64_t ldp; int np;     // row-operand source: (L, np), leading dimension ldp elements
  const void* Q; int64_t ldq; int nq;     // column-operand source
  void* OUT; int64_t soe, sop;            // output: expert stride, row stride (columns contiguous)
  void* Db; int64_t sdbe, sdbn;
  const int64_t* off;
  int E;
  int db_from_p;                          // 1: dY is P (row sums of the tile), 0: dY is Q
  // X given as the token matrix it would be gathered from (row r of X = token row idx[r] / fan_out): the operand
  // that holds X (Q when db_from_p, else P) reads its rows through idx; NULL: X is already in grouped order
  const int64_t* idx;
  int fan_out;
};

template <typename T, class TL, bool GA, bool GB>
__global__ __launch_bounds__(TL::NT) void xty_mfma_kernel(XtYPlan a, Raster rast, int p_tiles) {
  typedef TransOp<TL::BM, TL::NT, false, GA> AOp;
  typedef TransOp<TL::BN, TL::NT, false, GB> BOp;
  constexpr int STAGE = AOp::LDS_BYTES + BOp::LDS_BYTES;
  __shared__ __attribute__((aligned(16))) char lds[2 * STAGE];
  __shared__ int64_t sDst[TL::BM];
  __shared__ unsigned sRows[2 * 64];       // row offsets of a gathered operand (see TransOp)
  __shared__ __attribute__((aligned(16))) float sBias[TL::RS ? TL::BN : 4];

  int m_tile, n_tile, m_loc, n_loc;
  if (!rast.map(blockIdx.x, m_tile, n_tile, m_loc, n_loc)) return;
  const int e = m_tile / p_tiles;
  const int p0 = (m_tile % p_tiles) * TL::BM;
  const int q0 = n_tile * TL::BN;
  const int r_lo = e ? (int)a.off[e - 1] : 0;
  const int r_hi = (int)a.off[e];

  for (int m = threadIdx.x; m < TL::BM; m += TL::NT)
    sDst[m] = (p0 + m < a.np) ? (int64_t)e * a.soe + (int64_t)(p0 + m) * a.sop : -1;
  __syncthreads();

  AOp A;
  if constexpr (GA) A.init_gather((const char*)a.P + (int64_t)p0 * 2, a.ldp * 2, a.np - p0, a.idx + r_lo, a.fan_out, r_hi - r_lo, sRows);
  else A.init((const char*)a.P + ((int64_t)r_lo * a.ldp + p0) * 2, a.ldp * 2, a.np - p0);
  BOp B;           // (rotated load order measured 1.5 % slower here, so both operands keep rot = 0)
  if constexpr (GB) B.init_gather((const char*)a.Q + (int64_t)q0 * 2, a.ldq * 2, a.nq - q0, a.idx + r_lo, a.fan_out, r_hi - r_lo, sRows);
  else B.init((const char*)a.Q + ((int64_t)r_lo * a.ldq + q0) * 2, a.ldq * 2, a.nq - q0);

  f32x16 acc[TL::FM][TL::FN];
  float rs[TL::FM];
#pragma unroll
  for (int i = 0; i < TL::FM; ++i) {
    rs[i] = 0.0f;
#pragma unroll
    for (int j = 0; j < TL::FN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  }
  const bool want_db = a.Db != nullptr && a.db_from_p && n_tile == 0;
  if constexpr (TL::RS) mainloop_rs<T, TL, AOp, BOp>(A, B, r_hi - r_lo, lds, acc);      // no bias gradient, no gather
  else mainloop<T, TL, AOp, BOp, true>(A, B, r_hi - r_lo, lds, want_db, acc, rs);

  if (TL::RS || ((((uintptr_t)a.OUT & 15) == 0) && ((a.soe | a.sop | a.nq) & 7) == 0))
    epilogue_staged<T, TL>(acc, (T*)a.OUT, sDst, q0, a.nq, nullptr, 0, lds, sBias);
  else
    epilogue<T, TL>(acc, (T*)a.OUT, sDst, q0, a.nq, nullptr, 0);

  if (want_db) {
    // lanes l and l+32 hold the two contraction halves of row l%32; the first wave column writes the sums
    const int wave = threadIdx.x >> 6, l = lane_id();
    const int wm = wave / TL::WN, wn = wave % TL::WN;
#pragma unroll
    for (int i = 0; i < TL::FM; ++i) {
      const float tot = rs[i] + __shfl_xor(rs[i], 32, 64);
      const int p = p0 + wm * TL::WTM + i * 32 + l;
      if (wn == 0 && l < 32 && p < a.np) ((T*)a.Db)[(int64_t)e * a.sdbe + (int64_t)p * a.sdbn] = from_f32<T>(tot);
    }
  }
}

// Bias gradient when dY is the column operand: column sums per expert segment.  A workgroup owns 256 columns of one
// expert: 32 column threads (16 bytes = 8 columns each) x 8 row lanes; every thread adds up the rows r = lane
// (mod 8) of the segment, then the 8 partial sums of a column are added in a fixed order (deterministic).
template <typename T>
__global__ __launch_bounds__(256) void colsum_kernel(const T* __restrict__ DY, int64_t ld, int N,
                                                    const int64_t* __restrict__ off, T* __restrict__ Db,
                                                    int64_t sdbe, int64_t sdbn) {
  typedef T T8 __attribute__((ext_vector_type(8)));
  __shared__ float part[8][256];
  const int e = blockIdx.y;
  const int c8 = threadIdx.x & 31, rg = threadIdx.x >> 5;
  const int n = (blockIdx.x * 32 + c8) * 8;
  const int r_lo = e ? (int)off[e - 1] : 0, r_hi = (int)off[e];
  float s[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (n < N) {
    for (int r = r_lo + rg; r < r_hi; r += 8) {
      const T8 v = *(const T8*)(DY + (int64_t)r * ld + n);
#pragma unroll
      for (int q = 0; q < 8; ++q) s[q] += to_f32(v[q]);
    }
  }
#pragma unroll
  for (int q = 0; q < 8; ++q) part[rg][c8 * 8 + q] = s[q];
  __syncthreads();
  const int col = blockIdx.x * 256 + threadIdx.x;
  if (col < N) {
    float t = 0.0f;
#pragma unroll
    for (int g = 0; g < 8; ++g) t += part[g][threadIdx.x];
    Db[(int64_t)e * sdbe + (int64_t)col * sdbn] = from_f32<T>(t);
  }
}

template <typename T, class TL>
static int launch_xty(const XtYArgs& a, hipStream_t st) {
  XtYPlan p;
  const bool k_contig = a.sdwk == 1;     // output rows = N index
  if (k_contig) {
    p.P = a.DY; p.ldp = a.sdym; p.np = a.N;
    p.Q = a.X; p.ldq = a.sxm; p.nq = a.K;
    p.sop = a.sdwn;
  } else {
    p.P = a.X; p.ldp = a.sxm; p.np = a.K;
    p.Q = a.DY; p.ldq = a.sdym; p.nq = a.N;
    p.sop = a.sdwk;
  }
  p.OUT = a.DW; p.soe = a.sdwe;
  p.Db = a.Db; p.sdbe = a.sdbe; p.sdbn = a.sdbn;
  p.off = a.off; p.E = a.E;
  p.db_from_p = k_contig ? 1 : 0;
  p.idx = a.idx; p.fan_out = a.fan_out;
  const int p_tiles = (p.np + TL::BM - 1) / TL::BM;
  const int q_tiles = (p.nq + TL::BN - 1) / TL::BN;
  const Raster r = make_raster((int64_t)a.E * p_tiles, q_tiles, GM_XTY);
  const int64_t grid = r.grid();
  if (grid > 0x7fffffffLL) { set_error("smoe_groupXtY: grid too large"); return SMOE_ERR_RANGE; }
  if constexpr (TL::RS) hipLaunchKernelGGL((xty_mfma_kernel<T, TL, false, false>), dim3((unsigned)grid), dim3(TL::NT), 0, st, p, r, p_tiles);
  else if (a.idx == nullptr) hipLaunchKernelGGL((xty_mfma_kernel<T, TL, false, false>), dim3((unsigned)grid), dim3(TL::NT), 0, st, p, r, p_tiles);
  else if (k_contig) hipLaunchKernelGGL((xty_mfma_kernel<T, TL, false, true>), dim3((unsigned)grid), dim3(TL::NT), 0, st, p, r, p_tiles);
  else hipLaunchKernelGGL((xty_mfma_kernel<T, TL, true, false>), dim3((unsigned)grid), dim3(TL::NT), 0, st, p, r, p_tiles);
  int rc = launch_status("xty_mfma_kernel");
  if (rc == 0 && a.Db != nullptr && !k_contig) {
    hipLaunchKernelGGL(colsum_kernel<T>, dim3((a.N + 255) / 256, a.E), dim3(256), 0, st, (const T*)a.DY,
                       a.sdym, a.N, a.off, (T*)a.Db, a.sdbe, a.sdbn);
    rc = launch_status("colsum_kernel");
  }
  return rc;
}

bool try_xty_mfma(const XtYArgs& a, int dtype, hipStream_t st, int& rc) {
  if (dtype == SMOE_F32) return a.idx == nullptr && try_xty_f32(a, st, rc);    // the float32 kernels do not gather
  if (dtype != SMOE_BF16 && dtype != SMOE_F16) return false;
  if (a.K % 8 != 0 || a.N % 8 != 0) return false;
  if (a.sdyn != 1 || a.sxk != 1 || a.sdym % 8 != 0 || a.sxm % 8 != 0) return false;
  if (!aligned16(a.DY) || !aligned16(a.X)) return false;
  if (a.sdwk != 1 && a.sdwn != 1) return false;
  if (!fits_u32(BK * a.sdym * 2 + (int64_t)a.N * 2) || !fits_u32(BK * a.sxm * 2 + (int64_t)a.K * 2)) return false;
  // gathered X: lane offsets are 32-bit byte offsets from the start of the token matrix
  if (a.idx != nullptr && !fits_u32(((int64_t)a.L / a.fan_out) * a.sxm * 2 + (int64_t)a.K * 2)) return false;
  // Looking the rows up costs the kernel about 4 % of its time; the gathered copy it saves costs 4 K bytes of HBM
  // traffic per row against 2 K N flops, i.e. a share of the kernel time that shrinks with N.  Measured per training
  // step: N = 1536 (Qwen-like, top-8) 9.12 -> 8.90 ms, N = 5760 (gpt-oss-like) 6.07 -> 6.03 ms, N = 28672 (Mixtral)
  // 31.3 -> 31.5 ms: wide layers keep the separate pass.
  if (a.idx != nullptr && a.N > XTY_GATHER_MAX_N) return false;
  // One-wave-per-SIMD form: needs the LDS-staged epilogue; no gathered operand, no bias gradient in the main loop.
  // Both operands are read transposed (two LDS reads per fragment), which leaves less to win than in
  // scatter2scatter: Mixtral shape (4096 rows per expert) 3.28 -> 3.12 and 6.35 -> 6.20 ms, 2048 rows per expert
  // (128 experts, 768 x 2048 and 2048 x 1536 outputs) 0.81 -> 0.77 and 1.55 -> 1.51 ms, 1024 rows per expert even.
  const bool out16 = (((uintptr_t)a.DW & 15) == 0) && ((a.sdwe | (a.sdwk == 1 ? a.sdwn : a.sdwk) | (a.sdwk == 1 ? a.K : a.N)) & 7) == 0;
  const bool db_in_loop = a.Db != nullptr && a.sdwk == 1;
  if (a.idx == nullptr && !db_in_loop && out16 && a.L / a.E >= RS_XTY_MIN_ROWS) {
    typedef Tile<256, 256, 2, 2, 2, true> RSTile;
    rc = dtype == SMOE_BF16 ? launch_xty<bf16_t, RSTile>(a, st) : launch_xty<f16_t, RSTile>(a, st);
    return true;
  }
  typedef Tile<256, 256, 2, 4> XTile;
  rc = dtype == SMOE_BF16 ? launch_xty<bf16_t, XTile>(a, st) : launch_xty<f16_t, XTile>(a, st);
  return true;
}

}  // namespace smoe

