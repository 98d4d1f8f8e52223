// Shared device-side building blocks of the gfx950 attention kernels:
// element-type traits (fp16 / bf16), MFMA 32x32x16 wrappers, the LDS transpose
// read, cross-half-wave exchange and the Philox4x32-10 dropout rule.
//
// Register layouts used throughout (wave64, v_mfma_f32_32x32x16_{f16,bf16}):
//   A operand: lane l holds row (l % 32), contraction indices 8*(l / 32) .. +7
//   B operand: lane l holds col (l % 32), contraction indices 8*(l / 32) .. +7
//   C/D      : lane l holds col (l % 32); register r (0..15) is row
//              8*(r / 4) + 4*(l / 32) + (r % 4)
// Because A and B index the contraction dimension the same way, any permutation of
// that dimension applied to both operands leaves the product unchanged; the kernels
// use this to feed an accumulator tile straight back in as the B operand of the
// next product without moving data between lanes.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fmha {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef short i16x4v __attribute__((__vector_size__(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define FMHA_LOG2E 1.4426950408889634f
#define FMHA_LN2 0.6931471805599453f
#define FMHA_DEV __device__ __forceinline__

template <typename T> struct Elem;

template <> struct Elem<_Float16> {
  using v8 = f16x8;
  using v4 = f16x4;
  static FMHA_DEV f32x16 mfma(v8 a, v8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

template <> struct Elem<__bf16> {
  using v8 = bf16x8;
  using v4 = bf16x4;
  static FMHA_DEV f32x16 mfma(v8 a, v8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};

// 16-byte and 8-byte register images used for type-agnostic moves.
union Pack16 {
  u32x4 u;
  f16x8 h;
  bf16x8 b;
};
union Pack8 {
  u32x2 u;
  f16x4 h;
  bf16x4 b;
  i16x4v s;
};

template <typename T> FMHA_DEV typename Elem<T>::v8 as_v8(u32x4 u);
template <> FMHA_DEV f16x8 as_v8<_Float16>(u32x4 u) { Pack16 p; p.u = u; return p.h; }
template <> FMHA_DEV bf16x8 as_v8<__bf16>(u32x4 u) { Pack16 p; p.u = u; return p.b; }
FMHA_DEV u32x4 as_u32x4(f16x8 v) { Pack16 p; p.h = v; return p.u; }
FMHA_DEV u32x4 as_u32x4(bf16x8 v) { Pack16 p; p.b = v; return p.u; }

template <typename T> FMHA_DEV typename Elem<T>::v4 as_v4(u32x2 u);
template <> FMHA_DEV f16x4 as_v4<_Float16>(u32x2 u) { Pack8 p; p.u = u; return p.h; }
template <> FMHA_DEV bf16x4 as_v4<__bf16>(u32x2 u) { Pack8 p; p.u = u; return p.b; }

// ds_read_b64_tr_b16: within each group of 16 lanes the instruction reads a
// 4 (rows) x 16 (cols) matrix of 16-bit elements -- lane i of the group supplies
// the address of row i/4, columns 4*(i%4)..+3 -- and returns to lane i the four
// row values of column i.  `byte_addr` is an LDS byte address.
FMHA_DEV u32x2 lds_read_tr16(const char *lds_ptr) {
  typedef __attribute__((address_space(3))) i16x4v lds_vec;
  Pack8 p;
  p.s = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_vec *)(lds_ptr));
  return p.u;
}

// A operand (32 rows x 16 contraction indices) of a product whose contraction index runs
// over the ROWS of a row-major LDS tile (pitch ROWB bytes) and whose output rows run over
// its columns -- i.e. the tile is consumed transposed.  For lane l (c32 = l%32, h = l/32)
// and step c the eight contraction indices are rows
//   row0 + 4h + 16c + {0,1,2,3, 8,9,10,11}
// which is the order in which a 32x32 accumulator tile (lane = column, registers = rows)
// presents them when it is fed back as the B operand; the column is col0 + c32.
template <typename T, int ROWB>
FMHA_DEV typename Elem<T>::v8 lds_load_a_transposed(const char *tile, int row0, int col0, int c, int l) {
  const int i16 = l & 15;
  const int h = l >> 5;
  const char *p0 = tile + (row0 + 4 * h + 16 * c + (i16 >> 2)) * ROWB + (col0 + (l & 16) + 4 * (i16 & 3)) * 2;
  const u32x2 lo = lds_read_tr16(p0);
  const u32x2 hi = lds_read_tr16(p0 + 8 * ROWB);
  const u32x4 both = {lo.x, lo.y, hi.x, hi.y};
  return as_v8<T>(both);
}

// ---------------------------------------------------------------- swizzled LDS tiles
// Operand tiles that are copied from global memory straight into LDS
// (global_load_lds_dwordx4: every lane names a 16-byte global chunk and the wave's 64
// chunks land in 1 KiB of consecutive LDS) cannot pad their rows.  They are kept as D/64
// panels of 64 columns, each panel [row][8 chunks of 16 bytes] with a 128-byte pitch, and
// chunk c of row r sits at position c ^ ((r >> 1) & 7): sixteen consecutive rows then spread
// one logical chunk over all sixteen 16-byte bank groups, which is what a conflict-free
// ds_read_b128 needs.  The copying lane simply fetches the chunk that belongs at its slot.
constexpr int kPanelRowB = 128;

// One wave-wide 16-byte-per-lane copy from global memory into LDS: lane i's chunk lands at
// LDS byte address lds_wave_base + 16*i.  Written as inline assembly with hand-placed waits
// (dma_wait_all) because the compiler, which cannot tell which LDS reads a copy may alias,
// would otherwise wait for all copies before any later LDS read.
FMHA_DEV void dma_global_to_lds_b128(const void *gptr, uint32_t lds_wave_base) {
  // the readfirstlane is free when the compiler already knows the value to be uniform
  lds_wave_base = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_wave_base);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_wave_base), "v"(gptr)
               : "memory");
}
// Wait until every copy issued with dma_global_to_lds_b128 by this wave has landed (this
// also waits for the wave's other outstanding vector loads and stores).
FMHA_DEV void dma_wait_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// LDS byte address of a __shared__ object.
FMHA_DEV uint32_t lds_address(const void *p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char *)p;
}

// The same copy with the global address given as a wave-uniform base plus a 32-bit per-lane
// byte offset, so that a lane can keep its offset for the whole kernel and the base advances
// on the scalar unit.
FMHA_DEV void dma_global_to_lds_b128(const void *uniform_base, uint32_t lane_offset, uint32_t lds_wave_base) {
  lds_wave_base = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_wave_base);
  const uint64_t b = (uint64_t)uniform_base;
  const uint64_t ub = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(b >> 32)) << 32) |
                      (uint32_t)__builtin_amdgcn_readfirstlane((int)b);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_wave_base), "v"(lane_offset),
               "s"(ub)
               : "memory");
}

// Copies rows [row0, row0 + BT) of a row-major [rows][D] matrix into a swizzled tile; NT
// threads take part.  Rows >= rend re-read row rend - 1 (callers neutralise them through
// their extra-step rows).  The lane's byte offsets inside a tile are computed once (init).
// Where the rows of head bh of a [heads..., rows, D] tensor live: head bh = (bh / heads, bh % heads)
// starts at element (bh / heads) * sb + (bh % heads) * sh and its rows are ss elements apart
// (D contiguous elements each).  The folded [B*H, rows, D] layout is heads = 1, sb = rows * D,
// ss = D; a [B, rows, H, D] tensor is heads = H, sb = rows * H * D, sh = D, ss = H * D.
// heads_rcp = floor(2^32 / heads) + 1 turns the division into a multiplication (exact while
// bh * heads < 2^32, which the host checks); offsets inside one head fit 31 bits (also checked).
struct RowMap {
  int64_t sb, sh, ss;
  int32_t heads;
  uint32_t heads_rcp;
  FMHA_DEV size_t head(int bh) const {
    const uint32_t b = heads == 1 ? (uint32_t)bh : __umulhi((uint32_t)bh, heads_rcp);
    return (size_t)b * (size_t)sb + (size_t)((uint32_t)bh - b * (uint32_t)heads) * (size_t)sh;
  }
};
// Kernels are built twice: for the folded contiguous layout, whose strides are compile-time
// constants (the row map is not read at all), and for row maps given at run time, which cost a
// few per cent in scalar address arithmetic and registers.
// Head dims between the built ones: a tensor's rows hold `dcols` < D elements (a multiple of 8: whole 16-byte
// chunks) and the kernels behave as if the rows were padded with zeros up to D -- chunks past dcols are
// never read (register loads fetch chunk 0 instead and are zeroed afterwards; direct copies to LDS take
// their 16 bytes from g_zero_chunk) and never written.  Zero columns change neither Q.K^T nor the kept
// columns of O and of the gradients.  Only the run-time-layout kernels know about it (rows dv elements
// apart are a run-time row stride anyway); in the others cols() is the constant D and all of it folds away.
static __device__ __attribute__((aligned(64))) uint32_t g_zero_chunk[16];
FMHA_DEV u32x4 chunk_or_zero(u32x4 v, bool live) {
  const u32x4 z = {0u, 0u, 0u, 0u};
  return live ? v : z;
}
template <bool STRIDED, int D> struct Rows {
  template <typename A> static FMHA_DEV int cols(const A &a) {
    if constexpr (STRIDED) return a.dcols;
    else return D;
  }
  static FMHA_DEV size_t head(const RowMap &m, int bh, int rows) {
    if constexpr (STRIDED) return m.head(bh);
    else return (size_t)bh * (size_t)rows * D;
  }
  static FMHA_DEV uint32_t ss(const RowMap &m) {
    if constexpr (STRIDED) return (uint32_t)m.ss;
    else return (uint32_t)D;
  }
};

template <typename T, int D, int BT, int NT> struct TileCopy {
  static constexpr int CHUNKS = BT * D / 8;
  static constexpr int CPT = CHUNKS / NT;
  static_assert(D % 64 == 0 && CHUNKS % NT == 0, "tile must divide evenly over the workgroup");
  uint32_t voff[CPT];
  uint32_t ss; // elements between rows of the source tensor

  // chunk slot c of a tile: panel c / (8*BT), row (c / 8) % BT, position c % 8, which holds the
  // row's chunk panel*8 + (position ^ ((row >> 1) & 7))
  static FMHA_DEV void slot(int c, int &row, int &col) {
    const int panel = c / (8 * BT), pos = c % 8;
    row = (c / 8) % BT;
    col = panel * 8 + (pos ^ ((row >> 1) & 7));
  }
  FMHA_DEV void init(int tid, int64_t row_stride) {
    ss = (uint32_t)row_stride;
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      int row, col;
      slot(tid + i * NT, row, col);
      voff[i] = (uint32_t)row * ss * 2u + (uint32_t)(col * 16);
    }
  }
  // base: row 0 of the head; lds_tile: LDS byte address of the destination tile; tid: the caller's
  // index among the NT threads
  // dv: elements a row really has (chunks past them come from g_zero_chunk)
  FMHA_DEV void issue(const T *base, int row0, int rend, uint32_t lds_tile, int tid, int dv = D) const {
    const uint32_t wave_dst = lds_tile + (uint32_t)(tid >> 6) * 1024u;
    if (dv < D) { // wave-uniform
#pragma unroll
      for (int i = 0; i < CPT; ++i) {
        int row, col;
        slot(tid + i * NT, row, col);
        int r = row0 + row;
        r = r < rend ? r : rend - 1;
        const T *src = col * 8 < dv ? base + ((uint32_t)r * ss + (uint32_t)(col * 8)) : (const T *)g_zero_chunk;
        dma_global_to_lds_b128(src, wave_dst + (uint32_t)(i * NT * 16));
      }
      return;
    }
    if (row0 + BT <= rend) { // wave-uniform: a full tile needs no per-lane address arithmetic
      const T *tb = base + (uint32_t)row0 * ss;
#pragma unroll
      for (int i = 0; i < CPT; ++i) dma_global_to_lds_b128(tb, voff[i], wave_dst + (uint32_t)(i * NT * 16));
    } else {
#pragma unroll
      for (int i = 0; i < CPT; ++i) {
        int row, col;
        slot(tid + i * NT, row, col);
        int r = row0 + row;
        r = r < rend ? r : rend - 1;
        dma_global_to_lds_b128(base + ((uint32_t)r * ss + (uint32_t)(col * 8)), wave_dst + (uint32_t)(i * NT * 16));
      }
    }
  }
};

// Per-lane offsets of the two kinds of operand read from a swizzled tile.
struct PanelLane {
  uint32_t rowofs[4]; // row (l % 32) of a 32-row block, logical chunk pair j: chunks 2j + l/32
  uint32_t trofs;     // transposed read, see panel_read_transposed
  FMHA_DEV void init(int l) {
    const int ql = l & 31, h = l >> 5;
#pragma unroll
    for (int j = 0; j < 4; ++j) rowofs[j] = (uint32_t)(ql * kPanelRowB + (((2 * j) ^ (h ^ ((ql >> 1) & 7))) << 4));
    const int i16 = l & 15;
    const int row_l = 4 * h + (i16 >> 2);
    const int lp = 2 * ((l >> 4) & 1) + ((i16 & 3) >> 1);
    trofs = (uint32_t)(row_l * kPanelRowB + ((lp ^ (row_l >> 1)) << 4) + 8 * (i16 & 1));
  }
};

// A operand whose rows are tile rows: row 32*sb + l%32, contraction indices 16*ks + 8*(l/32) .. +7.
template <typename T, int BT>
FMHA_DEV typename Elem<T>::v8 panel_read_rows(const char *tile, const PanelLane &pl, int sb, int ks) {
  return as_v8<T>(*(const u32x4 *)(tile + pl.rowofs[ks & 3] + sb * 32 * kPanelRowB + (ks >> 2) * (BT * kPanelRowB)));
}

// A operand of a product that consumes the tile transposed (contraction over tile rows), with the
// row order of lds_load_a_transposed: rows 32*sb + 4h + 16c + {0,1,2,3, 8,9,10,11}, column 32*db + l%32.
// Lane l addresses row 4h + (l%16)/4 (+ multiples of 8) and the 8 bytes at logical byte column
// 64*db + 32*((l/16)%2) + 8*(l%4); adding 8 to the row flips bit 2 of the swizzle, which exchanges
// the two 64-byte halves of the panel row.
template <typename T, int BT>
FMHA_DEV typename Elem<T>::v8 panel_read_transposed(const char *tile, const PanelLane &pl, int sb, int db, int c) {
  const char *p0 = tile + pl.trofs + (sb * 32 + 16 * c) * kPanelRowB + (db >> 1) * (BT * kPanelRowB);
  const u32x2 lo = lds_read_tr16(p0 + (db & 1) * 64);
  const u32x2 hi = lds_read_tr16(p0 + 8 * kPanelRowB + ((db & 1) ^ 1) * 64);
  const u32x4 both = {lo.x, lo.y, hi.x, hi.y};
  return as_v8<T>(both);
}

// Exchange between lane l and lane l^32 (v_permlane32_swap), reduced with max / add.
FMHA_DEV float xhalf_max(float x) {
  int v = __float_as_int(x);
  auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  return fmaxf(__int_as_float(r[0]), __int_as_float(r[1]));
}
FMHA_DEV float xhalf_sum(float x) {
  int v = __float_as_int(x);
  auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  return __int_as_float(r[0]) + __int_as_float(r[1]);
}

// Store of one 32 (rows = lanes) x 32 (columns) accumulator block, scaled and rounded to T, into a
// row-major matrix.  In the accumulator layout lane (row, h) holds the column groups
// 8g + 4h .. +3 (g = 0..3) of its row: four 8-byte pieces 16 bytes apart.  Storing them as they
// are makes every store instruction write 16-byte fragments of 32 different lines; exchanging
// pieces between the two half-waves (v_permlane32_swap) gives each lane 16 contiguous bytes --
// lane h = 0 the first half of a 32-byte group, lane h = 1 the second -- so the same data leaves
// in half as many, twice as large, writes.  dst: the lane's row; the block starts at column 0.
// ncol: columns of this block that exist in the destination row (a multiple of 8).
template <typename T> FMHA_DEV void store_acc_block_row(T *dst_row, const f32x16 &acc, float scale, int h, int ncol = 32) {
#pragma unroll
  for (int gp = 0; gp < 2; ++gp) {
    typename Elem<T>::v4 x, y; // pieces g = 2gp and g = 2gp + 1
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[i] = (T)(acc[4 * (2 * gp) + i] * scale);
      y[i] = (T)(acc[4 * (2 * gp + 1) + i] * scale);
    }
    Pack8 px, py;
    if constexpr (sizeof(T) == 2 && __is_same(T, _Float16)) {
      px.h = x;
      py.h = y;
    } else {
      px.b = x;
      py.b = y;
    }
    // after the swaps: lanes h = 0 hold (own x, partner's x), lanes h = 1 hold (partner's y, own y)
    auto r0 = __builtin_amdgcn_permlane32_swap((int)px.u.x, (int)py.u.x, false, false);
    auto r1 = __builtin_amdgcn_permlane32_swap((int)px.u.y, (int)py.u.y, false, false);
    const u32x4 both = {(uint32_t)r0[0], (uint32_t)r1[0], (uint32_t)r0[1], (uint32_t)r1[1]};
    if (16 * gp + 8 * h < ncol) *(u32x4 *)(dst_row + 16 * gp + 8 * h) = both;
  }
}

// ---------------------------------------------------------------- row <-> accumulator layout
// A wave's 32 x KEYS block of a [.., sq, sk] tensor (mask, dropout tensor, saved outputs) moves
// to and from global memory as whole row segments: 16 bytes (8 keys) per lane, KEYS/8 lanes per
// row, so instruction i of KEYS/16 covers rows RPI*i .. RPI*i + RPI-1 (RPI = 512/KEYS).  The MFMA
// accumulators hold the block the other way round: lane = row (l % 32), and for each 32-key
// sub-block sb four 8-byte pieces g at keys 32 sb + 8 g + 4 (l / 32) .. +3.  As a global access that
// layout touches 32 different cache lines per instruction; instead a wave-private LDS scratch
// (row pitch = row + 16 bytes) is written in one layout and read in the other.  The scratch belongs
// to one wave, whose LDS accesses execute in order: turn() only keeps the compiler from moving
// accesses across the change of layout.
template <int KEYS> struct RowScratch {
  static constexpr int LPR = KEYS / 8;    // lanes per row
  static constexpr int RPI = 64 / LPR;    // rows per instruction
  static constexpr int NI = 32 / RPI;     // instructions per block
  static constexpr int PITCH = KEYS * 2 + 16;
  static constexpr int BYTES = 32 * PITCH;
  char *row;  // this lane's 16 bytes of instruction 0 (+ RPI * i * PITCH for instruction i)
  char *frag; // this lane's piece (0, 0) (+ 64 sb + 16 g)
  int rsub, chunk; // the lane's row within an instruction's rows, and its 8-key chunk of the row
  FMHA_DEV void init(char *base, int l) {
    rsub = l / LPR;
    chunk = l % LPR;
    row = base + rsub * PITCH + chunk * 16;
    frag = base + (l & 31) * PITCH + (l >> 5) * 8;
  }
  static FMHA_DEV void turn() {
    __builtin_amdgcn_wave_barrier();
    asm volatile("" ::: "memory");
  }
  FMHA_DEV void rows_in(const u32x4 (&r)[NI]) const {
#pragma unroll
    for (int i = 0; i < NI; ++i) *(u32x4 *)(row + RPI * i * PITCH) = r[i];
  }
  FMHA_DEV u32x4 row_out(int i) const { return *(const u32x4 *)(row + RPI * i * PITCH); }
  FMHA_DEV u32x2 piece(int sb, int g) const { return *(const u32x2 *)(frag + sb * 64 + g * 16); }
  template <typename T> FMHA_DEV void put_piece(int sb, int g, const typename Elem<T>::v4 &v) const {
    Pack8 pk;
    if constexpr (__is_same(T, _Float16)) pk.h = v;
    else pk.b = v;
    *(u32x2 *)(frag + sb * 64 + g * 16) = pk.u;
  }
};

FMHA_DEV float max3(float a, float b, float c) { return __builtin_fmaxf(__builtin_fmaxf(a, b), c); }
FMHA_DEV float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
FMHA_DEV float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// ---------------------------------------------------------------- Philox4x32-10
// Salmon et al., SC'11; constants and round function as in Random123.
struct Philox {
  static constexpr uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u;
  static constexpr uint32_t W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
  static __host__ __device__ inline void run(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                             uint32_t k0, uint32_t k1, uint32_t out[4]) {
#pragma unroll
    for (int r = 0; r < 10; ++r) {
      uint64_t p0 = (uint64_t)M0 * c0;
      uint64_t p1 = (uint64_t)M1 * c2;
#if defined(__HIP_DEVICE_COMPILE__)
      // three-input xor in one instruction (v_bitop3_b32, truth table 0x96): 41 instead of 55 VALU per call
      uint32_t n0 = __builtin_amdgcn_bitop3_b32((uint32_t)(p1 >> 32), c1, k0, 0x96);
      uint32_t n2 = __builtin_amdgcn_bitop3_b32((uint32_t)(p0 >> 32), c3, k1, 0x96);
#else
      uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
      uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
#endif
      c1 = (uint32_t)p1;
      c3 = (uint32_t)p0;
      c0 = n0;
      c2 = n2;
      k0 += W0;
      k1 += W1;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
  }
};

// Dropout keep rule.  Elements are grouped into 4 (queries) x 4 (keys) blocks and one
// Philox call serves a block:
//   key = (seed_lo, seed_hi); ctr = (offset_lo, offset_hi, blk_lo, blk_hi)
//   blk = (bh * ceil(sq/4) + q/4) * ceil(sk/4) + k/4
//   random byte of element (q,k) = (out[q%4] >> 8*(k%4)) & 0xff; keep iff byte >= thr
struct DropCtx {
  uint32_t seed_lo, seed_hi, off_lo, off_hi;
  uint32_t thr;
  uint32_t qb4, kb4; // ceil(sq/4), ceil(sk/4)
};

// The 32-bit word holding the four key-consecutive random bytes of query row q,
// keys 4*k4 .. 4*k4+3.
FMHA_DEV uint32_t drop_word(const DropCtx &c, uint32_t bh, uint32_t q, uint32_t k4) {
  uint64_t blk = ((uint64_t)bh * c.qb4 + (q >> 2)) * c.kb4 + k4;
  uint32_t o[4];
  Philox::run(c.off_lo, c.off_hi, (uint32_t)blk, (uint32_t)(blk >> 32), c.seed_lo, c.seed_hi, o);
  uint32_t s = q & 3u;
  return s == 0 ? o[0] : s == 1 ? o[1] : s == 2 ? o[2] : o[3];
}

// All four words of the block holding query rows 4*q4..4*q4+3 and keys 4*k4..4*k4+3.
FMHA_DEV void drop_block(const DropCtx &c, uint32_t bh, uint32_t q4, uint32_t k4, uint32_t o[4]) {
  uint64_t blk = ((uint64_t)bh * c.qb4 + q4) * c.kb4 + k4;
  Philox::run(c.off_lo, c.off_hi, (uint32_t)blk, (uint32_t)(blk >> 32), c.seed_lo, c.seed_hi, o);
}

// ---- sharing one Philox call per 4x4 block among the four lanes that need it
// (v_mov_b32 with a DPP quad permutation; lanes 4n..4n+3 form a quad)
template <int CTRL> FMHA_DEV uint32_t quad_perm(uint32_t x) {
  // every lane of a quad is a valid source, so the previous value of the destination never shows:
  // leave it undefined instead of clearing it first
  return (uint32_t)__builtin_amdgcn_mov_dpp((int)x, CTRL, 0xf, 0xf, true);
}

// 4x4 transpose inside a quad: on entry lane i holds a[0..3]; on exit a[g] is what lane g held
// in a[i].  Two butterfly stages (partner lane ^1, then ^2), written as selects so that they
// compile to v_cndmask rather than to moves under a narrowed exec mask.
FMHA_DEV void quad_transpose4(uint32_t a[4], int lane) {
  const bool odd = lane & 1;
  // stage 1: exchange a[1]<->a[0] and a[3]<->a[2] with the lane ^ 1
  const uint32_t s0 = quad_perm<0xB1>(odd ? a[0] : a[1]);
  const uint32_t s1 = quad_perm<0xB1>(odd ? a[2] : a[3]);
  const uint32_t b0 = odd ? s0 : a[0], b1 = odd ? a[1] : s0, b2 = odd ? s1 : a[2], b3 = odd ? a[3] : s1;
  // stage 2: exchange the (2,3) pair of lanes 0,1 with the (0,1) pair of lanes 2,3
  const bool hi = lane & 2;
  const uint32_t u0 = quad_perm<0x4E>(hi ? b0 : b2);
  const uint32_t u1 = quad_perm<0x4E>(hi ? b1 : b3);
  a[0] = hi ? u0 : b0;
  a[1] = hi ? u1 : b1;
  a[2] = hi ? b2 : u0;
  a[3] = hi ? b3 : u1;
}

// Lane = query layout.  The lane owns query q and, in one 32-key block starting at key kb32, the
// keys 4h + 8g + t (g, t = 0..3).  Returns in w[g] the word holding the four random bytes of
// (q, keys 4h+8g .. +3).  The four lanes of a quad share q/4: each evaluates the block of ONE g
// and the words are exchanged, instead of every lane evaluating all four.
FMHA_DEV void drop_words_q(const DropCtx &c, uint32_t bh, uint32_t q, uint32_t kb32, int h, int lane,
                           uint32_t w[4]) {
  const uint32_t g = (uint32_t)lane & 3u;
  drop_block(c, bh, q >> 2, (kb32 >> 2) + (uint32_t)h + 2u * g, w); // w[j] = word of query row 4*(q/4)+j
  quad_transpose4(w, lane);                                        // w[g] = word of row q in block g
}

// Lane = key layout.  The lane owns key k and, in one 32-query block starting at qb32, the queries 4h + 8g + t
// (g, t = 0..3).  Lanes of a quad share k / 4: lane i evaluates the block of g = i.  Of every word (row t of block
// g) a lane uses one byte only, byte k % 4 = lane % 4, so for each t the quad transposes a 4 x 4 matrix of BYTES
// (row = the lane that evaluated block g, column = the byte) instead of broadcasting whole words.  Returns r[t]
// whose byte g is the random byte of (query qb32 + 4h + 8g + t, key k): a compare with a static byte selector per
// element, no extraction.  Two butterfly stages per word, each a quad-permuted move and a v_perm_b32 with a
// selector that depends on the lane's position in the quad only (16 instructions per block; broadcasting the
// sixteen words and extracting the lane's byte of each took 32).
FMHA_DEV void drop_bytes_k(const DropCtx &c, uint32_t bh, uint32_t qb32, uint32_t k, int h, int lane, uint32_t r[4]) {
  const uint32_t g = (uint32_t)lane & 3u;
  uint32_t o[4];
  drop_block(c, bh, (qb32 >> 2) + (uint32_t)h + 2u * g, k >> 2, o);
  // v_perm_b32(hi, lo, sel): selector values 0-3 take bytes of lo (own), 4-7 bytes of hi (partner)
  const uint32_t sel1 = (lane & 1) ? 0x03070105u : 0x06020400u; // with lane ^ 1: (own0, partner0, own2, partner2) / (partner1, own1, partner3, own3)
  const uint32_t sel2 = (lane & 2) ? 0x03020706u : 0x05040100u; // with lane ^ 2: (own0, own1, partner0, partner1) / (partner2, partner3, own2, own3)
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const uint32_t a1 = __builtin_amdgcn_perm(quad_perm<0xB1>(o[t]), o[t], sel1);
    r[t] = __builtin_amdgcn_perm(quad_perm<0x4E>(a1), a1, sel2);
  }
}

// Zeroes the dropped elements of four packed 16-bit values (two registers: elements t = 0,1 and
// t = 2,3) whose random bytes are the four bytes of `word`.  Packed 16-bit arithmetic instead of a
// compare and a select per element: the bytes are spread to 16-bit lanes (v_perm_b32), (thr-1) - byte
// is negative exactly for kept elements, and its sign, smeared over the lane, is the keep mask.
// thr_m1_x2 = (thr - 1) in both halves.
FMHA_DEV void drop_apply_pk4(uint32_t word, uint32_t thr_m1_x2, uint32_t &pair01, uint32_t &pair23) {
  typedef short s16x2 __attribute__((ext_vector_type(2)));
  union {
    uint32_t u;
    s16x2 s;
  } b01, b23, t, m01, m23;
  b01.u = __builtin_amdgcn_perm(0u, word, 0x0c010c00u); // (byte0, byte1) zero-extended
  b23.u = __builtin_amdgcn_perm(0u, word, 0x0c030c02u); // (byte2, byte3)
  t.u = thr_m1_x2;
  m01.s = (t.s - b01.s) >> 15;
  m23.s = (t.s - b23.s) >> 15;
  pair01 &= m01.u;
  pair23 &= m23.u;
}

FMHA_DEV bool drop_keep_byte(uint32_t word, int t, uint32_t thr) {
  return ((word >> (8 * t)) & 0xffu) >= thr;
}

} // namespace fmha
