// Tile GEMM for gfx950 (MI355X): C = alpha * op(A) * op(B) + beta * C, column-major, fp64 and fp32.
//
// This is the compute of one PARALiA "subkernel": the reference hands each T x T x T tile product to
// cublasDgemm / cublasSgemm through backend_run_operation (Library_scheduler/src/Subkernel.cpp:168,228;
// direct call form Database_builder/CuCuBLAS/src/dgemm_microbench.cu:141-142).  Here it is a hand-written
// MFMA kernel:
//   * one workgroup = 256 threads = 4 wavefronts (2 x 2), macro tile 128 x 128 (each wave owns 64 x 64, two
//     workgroups per CU); fp32 also has 256 x 128 (two workgroups per CU) and 256 x 256 (each wave owns 128 x 128
//     with 256 accumulator registers, one workgroup per CU) for problems with enough such tiles to fill the CUs;
//   * fp64 uses v_mfma_f64_16x16x4_f64 (4 x 4 blocks per wave), fp32 uses v_mfma_f32_32x32x2_f32 (2 x 2 or 4 x 4);
//   * A and B k-panels (16 elements deep; 32 for the fp32 tiles with direct panels) sit in LDS, double-buffered, one
//     barrier per k-panel.  They get there straight from global memory (global_load_lds_dwordx4, one panel ahead, each
//     request addressed by a scalar base and a 32-bit lane offset): MN-major panel rows of 1 KiB one per request
//     (fp64 128 x 128, fp32 256 x 256), of 512 bytes two per request (fp32 128 x 128), K-major panels in a swizzled
//     unpadded layout, eight or sixteen rows per request.  Direct: fp64 128 x 128 and fp32 128 x 128 and 256 x 256, every
//     transpose.  Through registers (global loads two panels ahead, LDS stores one ahead, both spread between the
//     MFMAs): the fp32 256 x 128 tile, and any operand whose leading dimension the lane offsets cannot span;
//   * LDS rows are padded (or, where a request fills them, swizzled or read in half-wave passes) so that the MFMA
//     operand reads do not collide in the banks;
//   * the MFMA "row" index is mapped to n and the "column" index (the lane-contiguous one) to m, so that the
//     16 / 32 lanes of a group write 128 contiguous bytes of a column of the column-major C;
//   * workgroup ids are re-mapped so the eight XCDs each own a compact block of C tiles (private L2 per XCD),
//     and inside an XCD neighbouring ids share A row-panels; the tiles of a ragged last block row, whose workgroups are
//     slow, go to all eight XCDs first.
// Arbitrary M, N, K and leading dimensions are handled; 16-byte vector loads are used when pointer and
// leading dimension allow it and the workgroup's tile is interior, element loads with zero fill otherwise.  What K
// leaves beyond its last whole panel is one guarded step behind the pipelined loop.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include "paralia_hip.h"

// Build-time switches (timing experiments; the defaults are what ships).
#ifndef PLK_F64_BK
#define PLK_F64_BK 16
#endif
#ifndef PLK_F32_BK
#define PLK_F32_BK 16
#endif
// panel depth of the fp32 128 x 128 tile where k allows it (see launch_gemm)
#ifndef PLK_F32_DEEP_BK
#define PLK_F32_DEEP_BK 32
#endif
#ifndef PLK_F64_PAIR
#define PLK_F64_PAIR 0
#endif
// Bit 0: fp64, bit 1: fp32 -- operand panels go global -> LDS without passing registers where every panel of the tile
// can (see dma_row, dma_krows).
#ifndef PLK_DIRECT
#define PLK_DIRECT 3
#endif
// Bit 0: fp64, bit 1: fp32 -- K-major panels in the swizzled, unpadded LDS layout that an LDS-DMA load can write.
#ifndef PLK_SWZ
#define PLK_SWZ 3
#endif
// 1: the permuted k order of gemm_kernel's V2 (fp32 256 x 256 tiles with a K-major operand)
// fp64 workgroups whose k extent is shorter than this keep the panels staged through registers (0: none does.  With
// 64-bit lane addresses in the row requests, short k chunks ran 7 - 12 % slower direct than staged and the limit was
// 1536; with scalar bases direct panels win or tie from K = 128 on, split-K chunks included)
#ifndef PLK_F64_STAGE_BELOW
#define PLK_F64_STAGE_BELOW 0
#endif
// which MFMA of its stretch a row request of the fp32 256 x 256 tile goes behind (see the V2 loop)
#ifndef PLK_DMA_BEHIND
#define PLK_DMA_BEHIND 2
#endif
// 1: the fp32 128 x 128 tile requests its panels straight into LDS too
#ifndef PLK_F32_SMALL_DIRECT
#define PLK_F32_SMALL_DIRECT 1
#endif
#ifndef PLK_V2
#define PLK_V2 1
#endif
// scheduling class the compiler's instruction-group pass files the LDS-DMA loads under (all DS instructions)
#ifndef PLK_DMA_MASK
#define PLK_DMA_MASK 0x080
#endif
// Row index (MFMA i) of accumulator element r for lane group g = lane / 16 in the 16x16 fp64 result block.
#ifndef PLK_F64_DROW
#define PLK_F64_DROW(r, g) (4 * (r) + (g))
#endif

namespace plk {

typedef double double4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef double dvec2 __attribute__((ext_vector_type(2)));
typedef float fvec4 __attribute__((ext_vector_type(4)));

constexpr int NTHREADS = 256;
#ifndef PLK_F32_BIG_BK
#define PLK_F32_BIG_BK 32
#endif

template <typename T> struct Traits;

template <> struct Traits<double> {
  using vec_t = dvec2;
  using acc_t = double4_t;
  static constexpr int VEC = 2;      // elements per 16-byte vector
  static constexpr int BLK = 16;     // MFMA block edge
  static constexpr int KSTEP = 4;    // k consumed per MFMA
  static constexpr int KV = 1;       // MFMA k-steps served by one refresh of the operand registers
  static constexpr int NACC = 4;     // accumulator elements per lane per block
  static constexpr int PAD_MN = 16;  // [k][mn] rows are extent + PAD_MN elements apart (128 B past a multiple of 256 B)
  static __device__ __forceinline__ acc_t mfma(double a, double b, acc_t c) {
    return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
  }
  // Row (MFMA i index) held by accumulator element r of a lane in lane-group g = lane / 16.
  static __device__ __forceinline__ int drow(int r, int g) { return PLK_F64_DROW(r, g); }
};

template <> struct Traits<float> {
  using vec_t = fvec4;
  using acc_t = float16_t;
  static constexpr int VEC = 4;
  static constexpr int BLK = 32;
  static constexpr int KSTEP = 2;
  static constexpr int KV = 2;       // two k-steps per refresh: their operands come with one LDS instruction
  static constexpr int NACC = 16;
  static constexpr int PAD_MN = 32;
  static __device__ __forceinline__ acc_t mfma(float a, float b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ int drow(int r, int g) { return 8 * (r >> 2) + 4 * g + (r & 3); }
};

// One staged operand panel: EXT rows or columns of op(X) by BK values of k.
// [mn][k] layout (K-major operands): rows BK + 2 elements apart.  fp32: lane (idx, kk) of an operand read sits in bank
// ((BK + 2) * idx + kk) mod 64, all distinct; rows are then only 8-byte aligned, so a 16-byte vector goes to LDS as two
// 8-byte stores (lds_put).  A 16-byte aligned stride costs two-way conflicts on every operand read.
template <typename T, bool KMAJOR, int EXT, int BK, bool SWZ = false, bool ROW2 = false> struct Lds {
  using Tr = Traits<T>;
  // SWZ (K-major only): rows exactly BK elements apart, no padding, and the 16-byte chunks of row mn stored at chunk
  // position c ^ swz(mn).  That is the layout an LDS-DMA load can write (a wave instruction fills 1 KiB of consecutive
  // LDS, lane by lane, while every lane picks its own global address), and the XOR keeps the 16-byte operand reads of
  // eight consecutive rows in eight different bank groups.
  static constexpr int NC = BK / Tr::VEC;                         // 16-byte chunks per K-major row
  static constexpr int RPB = 256 / (BK * (int)sizeof(T)) > 0 ? 256 / (BK * (int)sizeof(T)) : 1;  // rows per 256 B (all 64 banks)
  static constexpr __host__ __device__ __forceinline__ int swz(int mn) { return (mn / RPB) % NC; }
  // ROW2 (MN-major only): rows of 512 bytes kept two by two without padding -- rows 2q and 2q + 1 are the 1 KiB that one
  // LDS-DMA request fills (dma_row2), pairs 2 * EXT apart.  An operand read of the fp32 MFMA takes k = 2q from lanes
  // 0 - 31 and k = 2q + 1 from lanes 32 - 63, 8 bytes per lane: each half-wave pass covers 256 contiguous bytes.
  static constexpr int S_K = (KMAJOR && SWZ) ? BK : BK + 2, S_MN = ROW2 ? EXT : EXT + Tr::PAD_MN;
  static constexpr int SIZE = KMAJOR ? EXT * S_K : BK * S_MN;  // elements, padding included
  static constexpr int NV = EXT * BK / Tr::VEC / NTHREADS;     // 16-byte vectors per thread per panel
  static constexpr bool SPLIT_PUT = KMAJOR && !SWZ && sizeof(T) == 4;  // rows only 8-byte aligned: a vector goes as two halves
  static constexpr __host__ __device__ __forceinline__ int at(int k, int mn) {
    if (KMAJOR && SWZ) return mn * S_K + (((k / Tr::VEC) ^ swz(mn)) * Tr::VEC) + k % Tr::VEC;
    return KMAJOR ? mn * S_K + k : k * S_MN + mn;
  }
  // Vector i of thread tid: "c" runs along the memory-contiguous dimension (mn for MN-major operands, k for K-major
  // ones), "s" along the leading-dimension stride.
  static constexpr int CVECS = (KMAJOR ? BK : EXT) / Tr::VEC;  // vectors per contiguous run
  static __device__ __forceinline__ void coords(int tid, int i, int& c, int& s) {
    int v = tid + NTHREADS * i;
    c = (v % CVECS) * Tr::VEC;
    s = v / CVECS;
  }
  static __device__ __forceinline__ int slot_offset(int tid, int i) {
    int c, s;
    coords(tid, i, c, s);
    return KMAJOR ? at(c, s) : at(s, c);  // a 16-byte vector stays together in LDS in every layout
  }
};

template <typename L, typename T, bool GUARD>
__device__ __forceinline__ void gload(const T* __restrict__ base, long ld, int crem, int srem, bool vec_ok,
                                      typename Traits<T>::vec_t (&regs)[L::NV], int tid) {
  using Tr = Traits<T>;
  using vec_t = typename Tr::vec_t;
#pragma unroll
  for (int i = 0; i < L::NV; ++i) {
    int c, s;
    L::coords(tid, i, c, s);
    const T* p = base + c + (long)s * ld;
    if (!GUARD) {
      regs[i] = *reinterpret_cast<const vec_t*>(p);
    } else {
      vec_t v;
#pragma unroll
      for (int e = 0; e < Tr::VEC; ++e) v[e] = T(0);
      if (s < srem) {
        if (vec_ok && c + Tr::VEC <= crem) {
          v = *reinterpret_cast<const vec_t*>(p);
        } else {
#pragma unroll
          for (int e = 0; e < Tr::VEC; ++e)
            if (c + e < crem) v[e] = p[e];
        }
      }
      regs[i] = v;
    }
  }
}

// Slot i only, unguarded: the pieces the pipelined loop spreads between MFMAs.
template <typename L, typename T>
__device__ __forceinline__ void gload_one(const T* __restrict__ base, long ld, typename Traits<T>::vec_t& reg, int tid, int i) {
  int c, s;
  L::coords(tid, i, c, s);
  reg = *reinterpret_cast<const typename Traits<T>::vec_t*>(base + c + (long)s * ld);
}
typedef float fvec2 __attribute__((ext_vector_type(2)));

// One 16-byte vector into LDS; PUTS<L> is the number of store instructions that takes.
template <typename L> constexpr int PUTS = L::SPLIT_PUT ? 2 : 1;
template <typename L, typename T>
__device__ __forceinline__ void lds_put(T* __restrict__ p, const typename Traits<T>::vec_t& v) {
  if constexpr (L::SPLIT_PUT) {
    fvec2 lo, hi;
    lo.x = v[0]; lo.y = v[1]; hi.x = v[2]; hi.y = v[3];
    *reinterpret_cast<fvec2*>(p) = lo;
    *reinterpret_cast<fvec2*>(p + 2) = hi;
  } else {
    *reinterpret_cast<typename Traits<T>::vec_t*>(p) = v;
  }
}

template <typename L, typename T>
__device__ __forceinline__ void lds_store_one(T* __restrict__ xs, const typename Traits<T>::vec_t& reg, int tid, int i) {
  lds_put<L, T>(xs + L::slot_offset(tid, i), reg);
}

template <typename L, typename T>
__device__ __forceinline__ void lds_store(T* __restrict__ xs, const typename Traits<T>::vec_t (&regs)[L::NV], int tid) {
#pragma unroll
  for (int i = 0; i < L::NV; ++i) lds_put<L, T>(xs + L::slot_offset(tid, i), regs[i]);
}

// A wave-uniform pointer pinned to scalar registers.  The address arithmetic in front of it stays on the scalar unit and
// the compiler cannot merge it with the per-lane offset added behind it, so an LDS-DMA request is issued as
// "scalar base + 32-bit lane offset": between two MFMAs the wave spends two scalar adds and the request, no vector
// instruction and one address register instead of two.  With 64-bit per-lane addresses (a v_lshl_add_u64 per request)
// the requests cost 2 - 3.5 % of the fp32 256 x 256 tile's rate at 8192^3, with this form 0.2 %.
template <typename T>
__device__ __forceinline__ const char* scalar_base(const T* p) {
  const unsigned long long b = reinterpret_cast<unsigned long long>(p);
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)b), hi = __builtin_amdgcn_readfirstlane((unsigned)(b >> 32));
  return reinterpret_cast<const char*>(((unsigned long long)hi << 32) | lo);
}

// Row `row` of an MN-major panel straight from global memory into LDS (global_load_lds_dwordx4): the 64 lanes of a wave
// fetch 16 bytes each and the hardware puts lane l's at the wave's LDS base + 16 l, so one instruction moves one 1 KiB
// row (256 floats or 128 doubles) and neither staging registers nor LDS store instructions are spent on it.  The LDS
// base is wave-uniform, which is why the row stride of the padded layout can stay.  voff: dma_lane_offset<.., false>.
template <typename T, int EXT>
__device__ __forceinline__ void dma_row(const T* __restrict__ g, long ld, T* xs, int inst, int s_mn, unsigned voff) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int PER = 1024 / (int)sizeof(T), PARTS = EXT / PER > 0 ? EXT / PER : 1;  // elements per instruction, instructions per row
  const int row = inst / PARTS, part = inst % PARTS;
  const char* base = scalar_base(g + part * PER + (long)row * ld);
  __builtin_amdgcn_global_load_lds(reinterpret_cast<const T*>(base + voff), xs + row * s_mn + part * PER, 16, 0, 0);
#endif
}

// Rows of a K-major panel (each BK elements = NC 16-byte chunks) straight into the swizzled layout of Lds<.., SWZ>: wave
// instruction number `inst` of the panel fills 64 / NC consecutive rows; lane l fills chunk position l % NC of row
// l / NC with the global chunk (l % NC) ^ swz(row).  voff: dma_lane_offset<.., true>.
template <typename L, typename T>
__device__ __forceinline__ void dma_krows(const T* __restrict__ g, long ld, T* xs, int inst, unsigned voff) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int RPI = 64 / L::NC;
  const char* base = scalar_base(g + (long)(inst * RPI) * ld);
  __builtin_amdgcn_global_load_lds(reinterpret_cast<const T*>(base + voff), xs + inst * RPI * L::S_K, 16, 0, 0);
#endif
}

// Two rows of 512 bytes (128 floats) of an MN-major panel with one request: lanes 0 - 31 fetch row 2 * inst, lanes 32 - 63
// row 2 * inst + 1, and the 1 KiB lands as those two rows of the unpadded layout (Lds<.., ROW2>).
template <typename T, int EXT>
__device__ __forceinline__ void dma_row2(const T* __restrict__ g, long ld, T* xs, int inst, unsigned voff) {
#if defined(__HIP_DEVICE_COMPILE__)
  static_assert(EXT * sizeof(T) == 512, "dma_row2 moves rows of 512 bytes");
  const char* base = scalar_base(g + (long)(2 * inst) * ld);
  __builtin_amdgcn_global_load_lds(reinterpret_cast<const T*>(base + voff), xs + 2 * inst * EXT, 16, 0, 0);
#endif
}

// Where a lane's 16 bytes of a dma_row / dma_row2 / dma_krows request sit relative to the request's wave-uniform base, in bytes.
// The same for every request a wave makes for an operand: its requests are 4 apart and 4 * RPI rows are a whole swizzle
// period.  K-major: up to 64 / NC - 1 rows of ld elements, which is why the launcher keeps operands whose leading
// dimension does not fit 32 bits that way on the staged path (PLK_DMA_MAX_LD_BYTES).
template <typename L, typename T, bool KMAJOR, bool ROW2 = false>
__device__ __forceinline__ unsigned dma_lane_offset(long ld, int wave, int lane) {
  if constexpr (!KMAJOR && ROW2) {
    return (unsigned)(lane / 32) * (unsigned)ld * (unsigned)sizeof(T) + (unsigned)(16 * (lane % 32));
  } else if constexpr (KMAJOR) {
    constexpr int NC = L::NC, RPI = 64 / NC;
    static_assert((4 * RPI / L::RPB) % NC == 0, "the requests of a wave must share their swizzle");
    const int row = wave * RPI + lane / NC;
    const int gc = (lane % NC) ^ L::swz(row);
    return (unsigned)(lane / NC) * (unsigned)ld * (unsigned)sizeof(T) + (unsigned)(gc * 16);
  } else {
    return (unsigned)(16 * lane);
  }
}
// largest row stride in bytes of a K-major operand loaded by dma_krows (8 rows of it must stay under 2^32)
#define PLK_DMA_MAX_LD_BYTES (1L << 29)

// Workgroup id -> (block row, block column).  Hardware deals workgroup ids round-robin over the 8 XCDs;
// give each XCD a contiguous range of logical ids, then walk that range in groups of 8 block rows.
// A ragged last block row or column (M or N not a multiple of the tile) is dealt out first and evenly: its workgroups
// take the guarded loop, about twice the time of an interior one.  In the walk above the last row's would all fall into
// the last XCD's range, one in eight of its workgroups, so that XCD finished a sixth later than the other seven (8100 x
// 8192 x 8192 fp64: 62.7 TFLOP/s against 73.1 for 8192 x 8100 x 8192), and the last column's close every band of eight
// rows, so whichever XCD's range ends with a band starts its slowest workgroups last (7808 x 3126 x 16384, three rounds:
// 63.7 TFLOP/s, 68.1 now).  The slow tiles are numbered along the last row, then up the last column; tile j goes to
// XCD j mod 8 as one of its first workgroups, and the rectangle that is left is walked as before.
__device__ __forceinline__ void block_coords(int bid, int gm, int gn, bool ragged_m, bool ragged_n, int& bm, int& bn) {
  const int nb = gm * gn;
  const int xcd = bid & 7, loc = bid >> 3;
  const int rm = (ragged_m && gm > 1) ? 1 : 0, rn = (ragged_n && gn > 1) ? 1 : 0;
  const int rows = gm - rm, cols = gn - rn;
  int pid;
  if (rm | rn) {
    const int in_row = rm ? gn : 0;                  // the last row, corner included
    const int slow = in_row + (rn ? rows : 0);       // and the last column above it
    const int mine = (slow - xcd + 7) >> 3;          // slow tiles with j mod 8 == xcd
    // every other one of the XCD's first workgroups where it has that many (two slow ones that share a compute unit
    // would both run at half speed), its first ones otherwise
    const bool spread = ((nb - xcd + 7) >> 3) >= 2 * mine;
    const int s = spread ? ((loc & 1) == 0 && (loc >> 1) < mine ? (loc >> 1) : -1) : (loc < mine ? loc : -1);
    if (s >= 0) {
      const int j = xcd + 8 * s;
      if (j < in_row) { bm = gm - 1; bn = j; }
      else { bm = j - in_row; bn = gn - 1; }
      return;
    }
    // the rest: XCD y keeps the (nb - y + 7) / 8 workgroups the hardware deals it, less its share of the slow ones
    int start = 0;
    for (int y = 0; y < xcd; ++y) start += ((nb - y + 7) >> 3) - ((slow - y + 7) >> 3);
    pid = start + (spread && loc < 2 * mine ? (loc >> 1) : loc - mine);
  } else {
    const int q = nb >> 3, r = nb & 7;
    pid = (xcd < r) ? xcd * (q + 1) + loc : r * (q + 1) + (xcd - r) * q + loc;
  }
  constexpr int GM = 8;
  const int width = GM * cols;
  const int group = pid / width;
  const int first_m = group * GM;
  const int gsz = min(rows - first_m, GM);
  const int in = pid - group * width;
  bm = first_m + in % gsz;
  bn = in / gsz;
}

// Macro tile BM x BN, four waves in 2 x 2, each owning BM/2 x BN/2; k-panels BK deep.  Tiles with 128 x 128 leave room
// for two workgroups per CU (two waves per SIMD that fill each other's gaps); larger ones run one workgroup per CU with
// the whole register file and fewer operand reads and global loads per MFMA.
// AK: op(A) is K-major in memory (TransA == 'T').  BKM: op(B) is K-major in memory (TransB == 'N').
// DIR = false: every panel through registers, plain layouts (what the launcher picks for fp64 operands whose K-major
// rows are too far apart for the 32-bit lane offsets of a row request).
template <typename T, bool AK, bool BKM, int BM, int BN, int BK, bool DIR = true>
__global__ __launch_bounds__(NTHREADS, (BM * BN * (int)sizeof(T) <= 128 * 128 * 8 ? 2 : 1)) void gemm_kernel(int M, int N, int K, T alpha, const T* __restrict__ A, long lda,
                                                          const T* __restrict__ B, long ldb, T beta, T* __restrict__ C,
                                                          long ldc, int gm, int gn, int vecA, int vecB, int vecC, int kchunk,
                                                          int m_read, int n_read) {
  using Tr = Traits<T>;
  using vec_t = typename Tr::vec_t;
  using acc_t = typename Tr::acc_t;
  // SWZL (the tiles whose MN-major panel rows are exactly 1 KiB: fp64 128 x 128, fp32 256 x 256): K-major panels in the
  // swizzled, unpadded layout (Lds<.., SWZ>), so every panel, K-major or MN-major, can be loaded global -> LDS directly
  // and all four transposes run without staging registers and LDS stores.
  // V2 (fp32 256 x 256 with a K-major operand) adds a k order.  Which k of a panel an MFMA step multiplies is free as
  // long as A and B agree.  Inside every 16-deep group of k, lane group kk (k index of the MFMA) takes the SPG
  // consecutive values kk * SPG .. kk * SPG + SPG - 1, one per step, instead of every KSTEP-th value.  A K-major
  // operand then has the values of KV = VEC = 4 consecutive steps side by side in LDS: ONE 16-byte read per block
  // serves four steps, where the plain order needs a read per block and two steps.  MN-major operands do not care which
  // row a step reads.  (For fp64 the same order was slower than the plain one: 71.3 against 73.0 TFLOP/s NN.)
  // fp64, 8192^3: NN 73.2 -> 74.9, NT 73.5 -> 74.6, TN 73.9 -> 74.9, TT 73.6 -> 74.9 TFLOP/s against staging every panel
  // through registers (with 64-bit lane addresses in the row requests NN had measured the same either way).
  constexpr bool SWZL = DIR && ((PLK_SWZ >> (sizeof(T) == 4 ? 1 : 0)) & 1) &&
                        ((sizeof(T) == 8 && BM == 128 && BN == 128 && BK == 16) ||
                         (sizeof(T) == 4 && BM == 256 && BN == 256 && BK % 16 == 0) ||
                         (sizeof(T) == 4 && BM == 128 && BN == 128 && BK % 16 == 0 && PLK_F32_SMALL_DIRECT));
  constexpr bool V2 = PLK_V2 && SWZL && sizeof(T) == 4 && (AK || BKM);
  // ROW2 (fp32 128 x 128): the 512-byte panel rows of an MN-major operand are requested two per instruction into the
  // unpadded layout; its K-major operands take the swizzled layout (SWZL) and the permuted k order (V2) of the large tile
  constexpr bool ROW2 = DIR && PLK_F32_SMALL_DIRECT && sizeof(T) == 4 && BM == 128 && BN == 128;
  using LA = Lds<T, AK, BM, BK, SWZL, ROW2>;
  using LB = Lds<T, BKM, BN, BK, SWZL, ROW2>;
  constexpr int BLK = Tr::BLK, WM = BM / 2, WN = BN / 2, NBM = WM / BLK, NBN = WN / BLK;
  if (kchunk > 0) {
    // split K: the workgroups of grid row y multiply k in [y * kchunk, (y + 1) * kchunk) and leave their plain partial
    // product in slice y of the workspace passed as C (M x N, dense); splitk_reduce_kernel combines the slices
    const int k0 = blockIdx.y * kchunk;
    A += AK ? (long)k0 : (long)k0 * lda;
    B += BKM ? (long)k0 : (long)k0 * ldb;
    K = min(K - k0, kchunk);
    C += (long)blockIdx.y * M * N;
  }
  constexpr int ASZ = LA::SIZE, BSZ = LB::SIZE;

  __shared__ __attribute__((aligned(32))) T smem[2 * (ASZ + BSZ)];
  constexpr int STAGE = ASZ + BSZ;  // buffer b holds A at smem + b*STAGE and B right behind it

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int idx = lane % BLK, kk = lane / BLK;
  const int wm = (wave & 1) * WM, wn = (wave >> 1) * WN;

  int bm, bn;
  block_coords(blockIdx.x, gm, gn, M % BM != 0, N % BN != 0, bm, bn);
  // the divisions above run on the vector unit; back in scalar registers the tile origins and every address derived
  // from them are scalar arithmetic
  bm = __builtin_amdgcn_readfirstlane(bm);
  bn = __builtin_amdgcn_readfirstlane(bn);
  const int m0 = bm * BM, n0 = bn * BN;
  const int mrem = min(M - m0, BM), nrem = min(N - n0, BN);
  // Unguarded loads for every workgroup whose whole tile of op(A) rows and op(B) columns may be READ: the interior
  // ones, and on the edge of C those for which the caller vouches that the memory behind the operands' last rows is
  // there (m_read, n_read >= M, N: tiles that live in larger blocks).  What is read from beyond M or N only reaches
  // elements of C that the guarded epilogue does not store.
  const bool fast = (m0 + BM <= m_read) && (n0 + BN <= n_read) && vecA && vecB;

  // tile origins; element (mn, k) of op(X) lives at base[mn + k*ld] (MN-major) or base[k + mn*ld] (K-major)
  const T* Ab = AK ? A + (long)m0 * lda : A + m0;
  const T* Bb = BKM ? B + (long)n0 * ldb : B + (long)n0;
  const long a_kstep = AK ? (long)BK : (long)BK * lda;
  const long b_kstep = BKM ? (long)BK : (long)BK * ldb;

  acc_t acc[NBN][NBM];
#pragma unroll
  for (int i = 0; i < NBN; ++i)
#pragma unroll
    for (int j = 0; j < NBM; ++j)
#pragma unroll
      for (int r = 0; r < Tr::NACC; ++r) acc[i][j][r] = T(0);

  const int nkt = (K + BK - 1) / BK;
  const int nfull = K / BK;
  constexpr int NVA = LA::NV, NVB = LB::NV;
  vec_t ra[NVA], rb[NVB];

  auto fetch = [&](int kt) {
    const T* ap = Ab + kt * a_kstep;
    const T* bp = Bb + kt * b_kstep;
    if (fast && kt < nfull) {
      gload<LA, T, false>(ap, lda, 0, 0, true, ra, tid);
      gload<LB, T, false>(bp, ldb, 0, 0, true, rb, tid);
    } else {
      const int krem = min(K - kt * BK, BK);
      gload<LA, T, true>(ap, lda, AK ? krem : mrem, AK ? mrem : krem, vecA, ra, tid);
      gload<LB, T, true>(bp, ldb, BKM ? krem : nrem, BKM ? nrem : krem, vecB, rb, tid);
    }
  };

  // fp32 operands in the [k][mn] layout: lane idx of block j takes row NB * idx + j instead of j * BLK + idx, so the
  // rows a lane needs for its NB blocks are adjacent in LDS and come with one 8- or 16-byte read instead of NB 4-byte
  // ones (every operand read issued between MFMAs costs MFMA issue slots: 1 read per MFMA loses 8 % of the pipe rate,
  // 1 per 2 about half of that).  The epilogue maps the accumulators back with the same rule.
  constexpr bool PAIRED = sizeof(T) == 4 || PLK_F64_PAIR;
  constexpr bool A_PAIR = PAIRED && !AK, B_PAIR = PAIRED && !BKM;
  // rows of an MN-major operand a lane holds side by side: all its blocks' (8 or 16 bytes).  Block j of a lane is row
  // (j / PF) * BLK * PF + PF * idx + j % PF of the wave's part -- with PF = 1 the plain rule.
  constexpr int PFA = A_PAIR ? NBM : 1, PFB = B_PAIR ? NBN : 1;
  auto row_a = [&](int j) { return wm + (j / PFA) * (BLK * PFA) + PFA * idx + j % PFA; };
  auto row_b = [&](int i, int r) { return wn + (i / PFB) * (BLK * PFB) + PFB * r + i % PFB; };
  constexpr int G = 16, SPG = G / Tr::KSTEP;   // V2: k group depth, MFMA steps per group
  // this lane's A / B operand of k-step 0, block 0 (V2: of the first step of a group)
  const T* const lane_a = smem + LA::at(V2 ? kk * SPG : kk, wm + PFA * idx);
  const T* const lane_b = smem + ASZ + LB::at(V2 ? kk * SPG : kk, wn + PFB * idx);
  constexpr int A_KS = LA::at(Tr::KSTEP, 0), B_KS = LB::at(Tr::KSTEP, 0);    // strides per k-step
  // where block j sits relative to block 0 of the lane
  auto a_blk = [](int j) { return AK ? LA::at(0, j * BLK) : (j / PFA) * (BLK * PFA) + j % PFA; };
  auto b_blk = [](int i) { return BKM ? LB::at(0, i * BLK) : (i / PFB) * (BLK * PFB) + i % PFB; };
  constexpr int KV = V2 ? SPG / 2 : Tr::KV;    // V2: == VEC, the steps one 16-byte read of a K-major operand serves
  static_assert(!V2 || KV == Tr::VEC, "a 16-byte chunk of a K-major row must hold exactly KV steps");
  constexpr int KS = BK / (Tr::KSTEP * KV);  // operand refreshes ("steps") per panel
  // LDS read instructions per refresh
  constexpr int RD_A = V2 ? (AK ? NBM : KV * (NBM / PFA)) : (A_PAIR ? 1 : NBM);
  constexpr int RD_B = V2 ? (BKM ? NBN : KV * (NBN / PFB)) : (B_PAIR ? 1 : NBN);
  constexpr int NREADS = RD_A + RD_B;
  // K-major operand in the swizzled layout: where this lane finds its values in its row of block 0 (the same place in
  // every block: a block is a multiple of the swizzle period).  V2: the chunk of refresh (g, h) -- group g of the panel,
  // half h of the lane's SPG steps -- is chunk g * (16 / VEC) + 2 kk + h, moved by the row's swizzle.  Plain order: the
  // value of k-step t is element t * KSTEP + kk of the row, its chunk moved likewise.
  constexpr int NKP = !SWZL ? 1 : V2 ? (BK / G) * 2 : BK / Tr::KSTEP;
  const T* a_kp[NKP];
  const T* b_kp[NKP];
#pragma unroll
  for (int q = 0; q < NKP; ++q) {
    const int k_q = V2 ? ((q / 2) * (G / Tr::VEC) + 2 * kk + q % 2) * Tr::VEC : q * Tr::KSTEP + kk;
    a_kp[q] = smem + LA::at(k_q, wm + idx);
    b_kp[q] = smem + ASZ + LB::at(k_q, wn + idx);
  }

  auto read_ops = [&](int buf, int ks, T (&am)[KV][NBM], T (&bnv)[KV][NBN]) {
    if constexpr (V2) {
      const int g = (ks * KV) / SPG, h = ((ks * KV) % SPG) / KV;
      if constexpr (AK) {
#pragma unroll
        for (int j = 0; j < NBM; ++j) {
          const vec_t x = *reinterpret_cast<const vec_t*>(a_kp[2 * g + h] + buf * STAGE + j * BLK * LA::S_K);
#pragma unroll
          for (int v = 0; v < KV; ++v) am[v][j] = x[v];
        }
      } else {
        typedef T opv_t __attribute__((ext_vector_type(PFA)));
#pragma unroll
        for (int v = 0; v < KV; ++v)
#pragma unroll
          for (int q = 0; q < NBM / PFA; ++q) {
            const opv_t x = *reinterpret_cast<const opv_t*>(lane_a + buf * STAGE + (g * G + h * KV + v) * LA::S_MN + q * BLK * PFA);
#pragma unroll
            for (int e = 0; e < PFA; ++e) am[v][q * PFA + e] = x[e];
          }
      }
      if constexpr (BKM) {
#pragma unroll
        for (int i = 0; i < NBN; ++i) {
          const vec_t x = *reinterpret_cast<const vec_t*>(b_kp[2 * g + h] + buf * STAGE + i * BLK * LB::S_K);
#pragma unroll
          for (int v = 0; v < KV; ++v) bnv[v][i] = x[v];
        }
      } else {
        typedef T opv_t __attribute__((ext_vector_type(PFB)));
#pragma unroll
        for (int v = 0; v < KV; ++v)
#pragma unroll
          for (int q = 0; q < NBN / PFB; ++q) {
            const opv_t x = *reinterpret_cast<const opv_t*>(lane_b + buf * STAGE + (g * G + h * KV + v) * LB::S_MN + q * BLK * PFB);
#pragma unroll
            for (int e = 0; e < PFB; ++e) bnv[v][q * PFB + e] = x[e];
          }
      }
      return;
    }
#pragma unroll
    for (int v = 0; v < KV; ++v) {
#pragma unroll
      for (int j = 0; j < NBM; ++j)
        am[v][j] = (SWZL && AK) ? a_kp[ks * KV + v][buf * STAGE + j * BLK * LA::S_K] : lane_a[buf * STAGE + (ks * KV + v) * A_KS + a_blk(j)];
#pragma unroll
      for (int i = 0; i < NBN; ++i)
        bnv[v][i] = (SWZL && BKM) ? b_kp[ks * KV + v][buf * STAGE + i * BLK * LB::S_K] : lane_b[buf * STAGE + (ks * KV + v) * B_KS + b_blk(i)];
    }
  };
  // one LDS read instruction of read_ops, by its number (A's first); V2 only
  auto read_one = [&](int buf, int ks, T (&am)[KV][NBM], T (&bnv)[KV][NBN], int e) {
    if constexpr (V2) {
      const int g = (ks * KV) / SPG, h = ((ks * KV) % SPG) / KV;
      if (e < RD_A) {
        if constexpr (AK) {
          const vec_t x = *reinterpret_cast<const vec_t*>(a_kp[2 * g + h] + buf * STAGE + e * BLK * LA::S_K);
#pragma unroll
          for (int v = 0; v < KV; ++v) am[v][e] = x[v];
        } else {
          typedef T opv_t __attribute__((ext_vector_type(PFA)));
          const int v = e / (NBM / PFA), q = e % (NBM / PFA);
          const opv_t x = *reinterpret_cast<const opv_t*>(lane_a + buf * STAGE + (g * G + h * KV + v) * LA::S_MN + q * BLK * PFA);
#pragma unroll
          for (int f = 0; f < PFA; ++f) am[v][q * PFA + f] = x[f];
        }
      } else {
        const int eb = e - RD_A;
        if constexpr (BKM) {
          const vec_t x = *reinterpret_cast<const vec_t*>(b_kp[2 * g + h] + buf * STAGE + eb * BLK * LB::S_K);
#pragma unroll
          for (int v = 0; v < KV; ++v) bnv[v][eb] = x[v];
        } else {
          typedef T opv_t __attribute__((ext_vector_type(PFB)));
          const int v = eb / (NBN / PFB), q = eb % (NBN / PFB);
          const opv_t x = *reinterpret_cast<const opv_t*>(lane_b + buf * STAGE + (g * G + h * KV + v) * LB::S_MN + q * BLK * PFB);
#pragma unroll
          for (int f = 0; f < PFB; ++f) bnv[v][q * PFB + f] = x[f];
        }
      }
    }
  };
  auto mfma_step = [&](const T (&am)[KV][NBM], const T (&bnv)[KV][NBN]) {
#pragma unroll
    for (int v = 0; v < KV; ++v)
#pragma unroll
      for (int i = 0; i < NBN; ++i)
#pragma unroll
        for (int j = 0; j < NBM; ++j) acc[i][j] = Tr::mfma(bnv[v][i], am[v][j], acc[i][j]);
  };

  if (fast && nfull > 0) {
    // Software-pipelined main loop over the whole panels of K (interior workgroup; a ragged rest of K follows it in a
    // guarded step of its own).  Per k-panel:
    //   k-step 0     : store the prefetched panel kt+1 (registers -> LDS buffer cur^1), issue the global loads of
    //                  panel kt+2, read the operands of k-step 1, multiply with the operands of k-step 0;
    //   k-steps 1..  : read the operands of the next k-step while multiplying the current one;
    //   last k-step  : barrier first (everyone is done reading buffer cur and writing buffer cur^1), read the
    //                  operands of panel kt+1's first k-step, multiply the last operands of panel kt.
    // So every LDS read, LDS write and global load is issued under the shadow of MFMAs, and one barrier per panel sits
    // where the MFMA queue still has a k-step of work behind it.  The loop body has no branches: past the end, the
    // loads re-read the last panel and the stores fill a buffer nobody reads.
    T am[2][KV][NBM], bnv[2][KV][NBN];
    // MN-major operands whose panel rows are 1 KiB skip the registers (dma_row): panel kt+1 is requested while panel kt
    // is multiplied and must have landed (vmcnt) before the panel's barrier; operands staged through registers are
    // loaded two panels ahead as before.
    constexpr bool DIR_T = DIR && ((PLK_DIRECT >> (sizeof(T) == 4 ? 1 : 0)) & 1) != 0;
    // only when both operands qualify: with one operand direct and one staged the wait in front of the barrier also
    // covers the staged operand's newer loads (fp32 256 x 128 NN: 143.8 -> 137.4 TFLOP/s).  SWZL: every operand does.
    constexpr bool A_DIR = DIR_T && (SWZL || ROW2 || (!AK && !BKM && BM * sizeof(T) == 1024 && BN * sizeof(T) == 1024));
    constexpr bool B_DIR = A_DIR;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const unsigned voff_a0 = dma_lane_offset<LA, T, AK, ROW2>(lda, wave_u, lane), voff_b0 = dma_lane_offset<LB, T, BKM, ROW2>(ldb, wave_u, lane);
    if constexpr (A_DIR) {
#pragma unroll
      for (int i = 0; i < NVA; ++i) {
        if constexpr (AK) dma_krows<LA, T>(Ab, lda, smem, wave_u + 4 * i, voff_a0);
        else if constexpr (ROW2) dma_row2<T, BM>(Ab, lda, smem, wave_u + 4 * i, voff_a0);
        else dma_row<T, BM>(Ab, lda, smem, wave_u + 4 * i, LA::S_MN, voff_a0);
      }
    } else {
      gload<LA, T, false>(Ab, lda, 0, 0, true, ra, tid);
      lds_store<LA, T>(smem, ra, tid);
      gload<LA, T, false>(Ab + min(1, nfull - 1) * a_kstep, lda, 0, 0, true, ra, tid);
    }
    if constexpr (B_DIR) {
#pragma unroll
      for (int i = 0; i < NVB; ++i) {
        if constexpr (BKM) dma_krows<LB, T>(Bb, ldb, smem + ASZ, wave_u + 4 * i, voff_b0);
        else if constexpr (ROW2) dma_row2<T, BN>(Bb, ldb, smem + ASZ, wave_u + 4 * i, voff_b0);
        else dma_row<T, BN>(Bb, ldb, smem + ASZ, wave_u + 4 * i, LB::S_MN, voff_b0);
      }
    } else {
      gload<LB, T, false>(Bb, ldb, 0, 0, true, rb, tid);
      lds_store<LB, T>(smem + ASZ, rb, tid);
      gload<LB, T, false>(Bb + min(1, nfull - 1) * b_kstep, ldb, 0, 0, true, rb, tid);
    }
    if constexpr (A_DIR || B_DIR) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the requested rows are in LDS
    __syncthreads();
    read_ops(0, 0, am[0], bnv[0]);
    // side instructions of a panel, in issue order: the row requests of the direct operands, then for the staged ones
    // NREG LDS stores and NREG global loads
    constexpr int NDIR = (A_DIR ? NVA : 0) + (B_DIR ? NVB : 0), NREG = NVA + NVB - NDIR;
    constexpr int SIDE = NDIR + 2 * NREG;
    constexpr int PER_STEP = (SIDE + KS - 2) / (KS - 1);     // side instructions placed in each pre-barrier k-step
    constexpr int MFMAS = KV * NBM * NBN;
    constexpr bool ALT = sizeof(T) == 8;
    // staged vector number r -> index into (A vectors, then B vectors)
    constexpr int REG0 = A_DIR ? NVA : 0;
    // one side instruction of the panel (row request, LDS store or global load), by its number in issue order
    auto side_item = [&](int slot, T* nxt_a, T* nxt_b, const T* ga, const T* gb, unsigned voff_a, unsigned voff_b) {
      if (slot < NDIR) {
        const int vec = (A_DIR ? 0 : NVA) + slot;  // direct rows: A's first when both are direct
        if (vec < NVA) {
          if constexpr (AK) dma_krows<LA, T>(ga, lda, nxt_a, wave_u + 4 * vec, voff_a);
          else if constexpr (ROW2) dma_row2<T, BM>(ga, lda, nxt_a, wave_u + 4 * vec, voff_a);
          else dma_row<T, BM>(ga, lda, nxt_a, wave_u + 4 * vec, LA::S_MN, voff_a);
        } else {
          if constexpr (BKM) dma_krows<LB, T>(gb, ldb, nxt_b, wave_u + 4 * (vec - NVA), voff_b);
          else if constexpr (ROW2) dma_row2<T, BN>(gb, ldb, nxt_b, wave_u + 4 * (vec - NVA), voff_b);
          else dma_row<T, BN>(gb, ldb, nxt_b, wave_u + 4 * (vec - NVA), LB::S_MN, voff_b);
        }
        return;
      }
      // staged side instruction number r of the panel: fp64 alternates store / load vector by vector (the load
      // refills the registers the store has just read), fp32 issues all stores first, then all loads;
      // measured at 8192^3: fp64 73.5 against 72.0 TFLOP/s, fp32 141.3 against 139.9 the other way round
      const int r = slot - NDIR;
      const bool is_store = ALT ? (r % 2 == 0) : (r < NREG);
      const int vec = REG0 + (ALT ? r / 2 : (r < NREG ? r : r - NREG));  // 0 .. NVA-1: A, NVA .. : B
      if (is_store) {
        if (vec < NVA) lds_store_one<LA, T>(nxt_a, ra[vec], tid, vec);
        else lds_store_one<LB, T>(nxt_b, rb[vec - NVA], tid, vec - NVA);
      } else {
        if (vec < NVA) gload_one<LA, T>(ga, lda, ra[vec], tid, vec);
        else gload_one<LB, T>(gb, ldb, rb[vec - NVA], tid, vec - NVA);
      }
    };
    for (int kt = 0; kt < nfull; ++kt) {
      const int cur = kt & 1;
      T* const nxt_a = smem + (cur ^ 1) * STAGE;
      T* const nxt_b = nxt_a + ASZ;
      const int kt2 = min(kt + 2, nfull - 1), kt1 = min(kt + 1, nfull - 1);
      const T* const ga = Ab + (A_DIR ? kt1 : kt2) * a_kstep;
      const T* const gb = Bb + (B_DIR ? kt1 : kt2) * b_kstep;
      // the lane offsets of the row requests, opaque per panel: hoisted out of the loop the compiler widens them to 64
      // bits once and adds the scalar bases on the vector unit again
      unsigned voff_a = voff_a0, voff_b = voff_b0;
      if constexpr (NDIR > 0) asm volatile("" : "+v"(voff_a), "+v"(voff_b));
      if constexpr (V2 && NREG == 0) {
        // fp32 256 x 256 with a K-major operand, all panels direct.  The source is written in issue order -- an MFMA, then
        // the operand read or row request that goes behind it -- because the compiler keeps a row request (an LDS write
        // as far as it knows) in program order with every LDS read: with all reads of a step in front of its requests
        // the requests end up three in a row behind the step's last read, and the four waves of the compute unit send
        // twelve to the one address unit at once.  Spread one at a time, 10 or 11 MFMAs apart: NN 152.3 -> 152.8, TN and
        // TT 151.8 -> 152.7 TFLOP/s at 8192^3 (NT, which is not V2, loses 0.5 that way and keeps the order below).
        constexpr int PER_STEP_D = (SIDE + KS - 2) / (KS - 1), DMA_BEHIND = PLK_DMA_BEHIND;
#pragma unroll
        for (int ks = 0; ks < KS - 1; ++ks) {
#pragma unroll
          for (int m = 0; m < MFMAS; ++m) {
            const int v = m / (NBN * NBM), i = (m / NBM) % NBN, j = m % NBM;
            acc[i][j] = Tr::mfma(bnv[ks & 1][v][i], am[ks & 1][v][j], acc[i][j]);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
#pragma unroll
            for (int e = 0; e < NREADS; ++e)
              if (e * MFMAS / NREADS == m) {
                read_one(cur, ks + 1, am[(ks + 1) & 1], bnv[(ks + 1) & 1], e);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
              }
#pragma unroll
            for (int c = 0; c < PER_STEP_D; ++c)
              if (c * MFMAS / PER_STEP_D + DMA_BEHIND == m && ks * PER_STEP_D + c < SIDE) {
                side_item(ks * PER_STEP_D + c, nxt_a, nxt_b, ga, gb, voff_a, voff_b);
                __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
              }
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
#pragma unroll
      for (int ks = 0; ks < KS - 1; ++ks) {
        read_ops(cur, ks + 1, am[(ks + 1) & 1], bnv[(ks + 1) & 1]);
#pragma unroll
        for (int q = 0; q < PER_STEP; ++q) {
          const int slot = ks * PER_STEP + q;
          if (slot < SIDE) side_item(slot, nxt_a, nxt_b, ga, gb, voff_a, voff_b);
        }
        mfma_step(am[ks & 1], bnv[ks & 1]);
        // Issue order: the NREADS operand reads of the next step and the PER_STEP side instructions alternate and are
        // spread evenly over this step's MFMAs, each behind an MFMA, so that a wave issues them while its own MFMA
        // occupies the pipe.  With everything in front of the MFMAs the two waves of a SIMD reach their non-MFMA
        // stretch together and the pipe idles (fp32: 130 -> 138 TFLOP/s; fp64: 72.0 -> 73.5 together with the
        // alternating side order).
        constexpr int EXTRA = NREADS + PER_STEP, BOTH = 2 * (NREADS < PER_STEP ? NREADS : PER_STEP);
#pragma unroll
        for (int m = 0; m < MFMAS; ++m) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
#pragma unroll
          for (int e = 0; e < EXTRA; ++e) {
            if (e * MFMAS / EXTRA != m) continue;
            const bool is_read = e < BOTH ? (e % 2 == 0) : (NREADS > PER_STEP);
            if (is_read) {
              __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            } else {
              const int slot = ks * PER_STEP + (e < BOTH ? e / 2 : e - NREADS);
              if (slot >= SIDE) continue;
              if (slot < NDIR) { __builtin_amdgcn_sched_group_barrier(PLK_DMA_MASK, 1, 0); continue; }
              const int r = slot - NDIR;
              const bool is_store = ALT ? (r % 2 == 0) : (r < NREG);
              const int vec = REG0 + (ALT ? r / 2 : (r < NREG ? r : r - NREG));
              if (!is_store) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
              else if (vec < NVA) __builtin_amdgcn_sched_group_barrier(0x200, PUTS<LA>, 0);
              else __builtin_amdgcn_sched_group_barrier(0x200, PUTS<LB>, 0);
            }
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      }
      if constexpr (A_DIR || B_DIR) __builtin_amdgcn_s_waitcnt(0x0F70);  // the rows requested during this panel are in LDS
      __syncthreads();
      read_ops(cur ^ 1, 0, am[KS & 1], bnv[KS & 1]);
      mfma_step(am[(KS - 1) & 1], bnv[(KS - 1) & 1]);
#pragma unroll
      for (int m = 0; m < MFMAS; ++m) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
#pragma unroll
        for (int e = 0; e < NREADS; ++e)
          if (e * MFMAS / NREADS == m) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (nkt > nfull) {
      // The rest of K, less than a panel: guarded loads with zero fill (fetch), through registers into buffer 0, once
      // every wave has left the loop above (its last step reads the buffer it would have filled next).  Without this
      // step a K that is not a multiple of the panel depth sent every workgroup to the general loop below: 8192 x 8192
      // x 8100 fp64 66.3 TFLOP/s against 75.2 at K = 8192, fp32 132 against 152.
      fetch(nfull);
      __syncthreads();
      lds_store<LA, T>(smem, ra, tid);
      lds_store<LB, T>(smem + ASZ, rb, tid);
      __syncthreads();
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        T am_r[KV][NBM], bnv_r[KV][NBN];
        read_ops(0, ks, am_r, bnv_r);
        mfma_step(am_r, bnv_r);
      }
    }
  } else {
    // General loop: edge workgroups, ragged K, unaligned operands.  Same double buffering, loads guarded.
    if (nkt > 0) {
      fetch(0);
      lds_store<LA, T>(smem, ra, tid);
      lds_store<LB, T>(smem + ASZ, rb, tid);
    }
    __syncthreads();
    for (int kt = 0; kt < nkt; ++kt) {
      const int cur = kt & 1;
      if (kt + 1 < nkt) fetch(kt + 1);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        T am[KV][NBM], bnv[KV][NBN];
        read_ops(cur, ks, am, bnv);
        mfma_step(am, bnv);
      }
      if (kt + 1 < nkt) {
        lds_store<LA, T>(smem + (cur ^ 1) * STAGE, ra, tid);
        lds_store<LB, T>(smem + (cur ^ 1) * STAGE + ASZ, rb, tid);
      }
      __syncthreads();
    }
  }

  // Interior tile: no guards, so the compiler can batch the reads of C.  With the paired row rule (MN-major A) a lane's
  // PFA accumulators of one column are adjacent in memory and go out as one 8- or 16-byte access when C is aligned for
  // it.  Same arithmetic per element as the guarded loop below.
  // acc[i][j][r] is C(m0 + row_a(j), n0 + row_b(i, drow(r, kk))).
  if (mrem == BM && nrem == BN) {
    if constexpr (PFA > 1) {
      typedef T cvec_t __attribute__((ext_vector_type(PFA)));
      if (vecC) {
#pragma unroll
        for (int i = 0; i < NBN; ++i) {
#pragma unroll
          for (int r = 0; r < Tr::NACC; ++r) {
            const int n = row_b(i, Tr::drow(r, kk));
#pragma unroll
            for (int q = 0; q < NBM / PFA; ++q) {
              cvec_t* const cp = reinterpret_cast<cvec_t*>(C + (long)(n0 + n) * ldc + m0 + row_a(q * PFA));
              cvec_t v;
#pragma unroll
              for (int e = 0; e < PFA; ++e) v[e] = alpha * acc[i][q * PFA + e][r];
              if (beta != T(0)) {
                const cvec_t c = *cp;
#pragma unroll
                for (int e = 0; e < PFA; ++e) v[e] += beta * c[e];
              }
              *cp = v;
            }
          }
        }
        return;
      }
    }
#pragma unroll
    for (int i = 0; i < NBN; ++i) {
#pragma unroll
      for (int r = 0; r < Tr::NACC; ++r) {
        const int n = row_b(i, Tr::drow(r, kk));
        T* const ccol = C + (long)(n0 + n) * ldc + m0;
        T v[NBM];
#pragma unroll
        for (int j = 0; j < NBM; ++j) v[j] = alpha * acc[i][j][r];
        if (beta != T(0)) {
#pragma unroll
          for (int j = 0; j < NBM; ++j) v[j] += beta * ccol[row_a(j)];
        }
#pragma unroll
        for (int j = 0; j < NBM; ++j) ccol[row_a(j)] = v[j];
      }
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < NBN; ++i) {
#pragma unroll
    for (int r = 0; r < Tr::NACC; ++r) {
      const int n = row_b(i, Tr::drow(r, kk));
      if (n < nrem) {
        T* ccol = C + (long)(n0 + n) * ldc + m0;
#pragma unroll
        for (int j = 0; j < NBM; ++j) {
          const int m = row_a(j);
          if (m < mrem) {
            T v = alpha * acc[i][j][r];
            if (beta != T(0)) v += beta * ccol[m];
            ccol[m] = v;
          }
        }
      }
    }
  }
}

template <typename T>
__global__ void scale_kernel(int M, int N, T beta, T* __restrict__ C, long ldc) {
  const long total = (long)M * N;
  for (long e = (long)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (long)gridDim.x * blockDim.x) {
    const long m = e % M, n = e / M;
    T* p = C + n * ldc + m;
    *p = (beta == T(0)) ? T(0) : beta * *p;
  }
}

// C = alpha * (slice 0 + slice 1 + ...) + beta * C, slices added in index order: the result does not depend on timing.
template <typename T>
__global__ void splitk_reduce_kernel(int M, int N, int splits, T alpha, const T* __restrict__ ws, T beta, T* __restrict__ C, long ldc) {
  const long total = (long)M * N;
  for (long e = (long)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (long)gridDim.x * blockDim.x) {
    T sum = ws[e];
    for (int z = 1; z < splits; ++z) sum += ws[(long)z * total + e];
    T* p = C + (e / M) * ldc + e % M;
    T v = alpha * sum;
    if (beta != T(0)) v += beta * *p;
    *p = v;
  }
}

// How many ways to split K so that a product with few C tiles still fills the 256 compute units.
// The estimate counts rounds of 256 workgroups, each costing its k extent plus a fixed prologue / epilogue share, and
// the pass that adds the slices (workspace written once and read once).  1 = do not split.
// The launcher's fitted constants (pl_gemm_fit in the public header): built-in values measured on an MI355X, replaced
// by what the deploy database holds once the autotuner has loaded it.
inline void fit_defaults(pl_gemm_fit* f) {
  f->lone_us_per_k[0] = 0.114; f->lone_us_per_k[1] = 0.056;
  f->lone_fixed_k = 94.0;
  f->splitk_launch_us = 3.2;
  f->pass_bytes_per_us = 6.15e6;
  f->f32_small_us_per_k = 0.1099;
  f->f32_small_fixed_us = 7.4;
  f->f32_wide_gain = 0.949;
  f->f32_wide_fixed_us[0] = 4.9; f->f32_wide_fixed_us[1] = 10.6;
  const double g[4] = {0.012, 0.011, 0.010, 0.010}, f0[4] = {11.4, 10.7, 11.1, 11.7}, f1[4] = {45.5, 44.5, 53.0, 54.4};
  for (int t = 0; t < 4; ++t) { f->f32_large_gain[t] = g[t]; f->f32_large_fixed_us[t][0] = f0[t]; f->f32_large_fixed_us[t][1] = f1[t]; }
  f->edge_rounds[0] = 0.155;
  f->edge_rounds[1] = 0.236;
}
inline pl_gemm_fit& fit_in_use() {
  static pl_gemm_fit f = [] { pl_gemm_fit d; fit_defaults(&d); return d; }();
  return f;
}

template <typename T>
int pick_splits(long M, long N, long K, int* kchunk_out) {
  constexpr int BM = 128, BN = 128;
  const long tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  *kchunk_out = 0;
  // with more than about half the compute units covered, a second product running on another stream (the way the
  // scheduler issues subkernels) fills the rest better than a split would
  if (tiles > 160 || K < 256) return 1;
  const pl_gemm_fit& fit = fit_in_use();
  const double us_per_k = fit.lone_us_per_k[sizeof(T) == 8 ? 0 : 1];  // one workgroup, one unit of k, at the measured tile rate
  auto main_us = [&](long blocks, long kc) { return (double)((blocks + 255) / 256) * ((double)kc + fit.lone_fixed_k) * us_per_k; };
  double best = main_us(tiles, K);
  int best_s = 1;
  const long max_ws = 256L << 20;  // workspace bound: the slices of very long, very thin products stay small anyway
  for (int s = 2; s <= 64; ++s) {
    // whole panels per chunk (fp32: of the 32-deep panels its 128 x 128 tile takes where it can)
    const long gran = sizeof(T) == 4 ? PLK_F32_DEEP_BK : 16;
    const long kc = (((K + s - 1) / s) + gran - 1) / gran * gran;
    if (kc < 128) break;
    const long se = (K + kc - 1) / kc;
    if (se < 2) continue;
    if (se * M * N * (long)sizeof(T) > max_ws) break;
    const double t = main_us(tiles * se, kc) + fit.splitk_launch_us + (double)(2 * se + 1) * (double)M * (double)N * sizeof(T) / fit.pass_bytes_per_us;
    if (t < best * 0.95) {
      best = t;
      best_s = (int)se;
      *kchunk_out = (int)kc;
    }
  }
  return best_s;
}

// The same choice for a product that has the device to itself (a caller's device-resident call, the end of a streamed
// one).  Nothing else fills the compute units a launch leaves idle, so what counts is whole rounds of 512 workgroups (two
// per compute unit): 576 tiles are one full round and an eighth of another that takes as long (3072 x 3072 x 16384 fp64
// alone: 52.7 TFLOP/s unsplit, 73.7 split four ways = 4.5 rounds), 256 tiles leave every unit with one workgroup (2048
// x 2048 x 16384: 65.8 unsplit, 72.6 split two to four ways).  A round of 512 takes f + kc * c2, a last round of at most
// 256 workgroups (one per unit) f + kc * c1, with c1 the lone per-k time of the fit, c2 / c1 as measured on the fp32 tile
// (f32_small_us_per_k / lone_us_per_k[1]) and f the workgroup's fixed cost (lone_fixed_k); a split adds the second launch
// and the reduction's pass over the slices and C (the slices' way out of the workgroups is part of their epilogue, as the
// write of C is).  *us_out: the predicted time of the choice.
template <typename T>
int pick_splits_alone(long M, long N, long K, long max_ws_bytes, int* kchunk_out, double* us_out) {
  constexpr int BM = 128, BN = 128;
  const long tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  const pl_gemm_fit& fit = fit_in_use();
  const double c1 = fit.lone_us_per_k[sizeof(T) == 8 ? 0 : 1];
  const double c2 = c1 * fit.f32_small_us_per_k / fit.lone_us_per_k[1];
  const double f = fit.lone_fixed_k * c1;
  auto main_us = [&](long blocks, long kc) {
    const long full = blocks / 512, rem = blocks % 512;
    double t = (double)full * (f + (double)kc * c2);
    if (rem > 0) t += f + (double)kc * (rem <= 256 ? c1 : c2);
    return t;
  };
  *kchunk_out = 0;
  double best = main_us(tiles, K);
  int best_s = 1;
  const long gran = sizeof(T) == 4 ? PLK_F32_DEEP_BK : 16;
  for (int s = 2; s <= 64 && K >= 256; ++s) {
    const long kc = (((K + s - 1) / s) + gran - 1) / gran * gran;
    if (kc < 128) break;
    const long se = (K + kc - 1) / kc;
    if (se < 2) continue;
    if (se * M * N * (long)sizeof(T) > max_ws_bytes) break;
    const double t = main_us(tiles * se, kc) + fit.splitk_launch_us + ((double)se + 1.0) * (double)M * (double)N * sizeof(T) / fit.pass_bytes_per_us;
    if (t < best * 0.98) {
      best = t;
      best_s = (int)se;
      *kchunk_out = (int)kc;
    }
  }
  if (us_out) *us_out = best;
  return best_s;
}

// A product alone on the device whose tiles do not fill whole rounds can also be cut in two along N: the first
// n_head columns of C (whole tile columns, close to whole rounds of 512 workgroups) as one unsplit launch, the rest as
// a second launch that splits K, so that only the tail's slices pass through the reduction (3072^3 fp64: 576 tiles,
// four-way split of everything 874 us, 21 tile columns unsplit and the last 3 split seven ways 820 us).  Priced with
// the terms of pick_splits_alone plus half a split's launch cost for the extra launch; taken when 3 % ahead of
// best_us, the best of the one-launch choices.  Returns the tail's split count (0: one launch stays).
template <typename T>
int pick_tail_alone(long M, long N, long K, long max_ws_bytes, double best_us, long* n_head_out, double* us_out) {
  constexpr int BM = 128, BN = 128;
  const long gm = (M + BM - 1) / BM, gn = (N + BN - 1) / BN;
  const char* const off = getenv("PARALIA_GEMM_TAIL");
  if ((off && *off == '0') || gn < 2 || K < 512 || gm * gn <= 512) return 0;
  const pl_gemm_fit& fit = fit_in_use();
  const double c1 = fit.lone_us_per_k[sizeof(T) == 8 ? 0 : 1];
  const double c2 = c1 * fit.f32_small_us_per_k / fit.lone_us_per_k[1];
  const double f = fit.lone_fixed_k * c1;
  auto main_us = [&](long blocks, long kc) {
    const long full = blocks / 512, rem = blocks % 512;
    double t = (double)full * (f + (double)kc * c2);
    if (rem > 0) t += f + (double)kc * (rem <= 256 ? c1 : c2);
    return t;
  };
  const long gran = sizeof(T) == 4 ? PLK_F32_DEEP_BK : 16;
  int best_s = 0;
  double best = best_us * 0.97;
  // tails of up to two rounds' worth of tile columns
  const long h_span = (1024 + gm - 1) / gm;
  const long h_min = gn - h_span > 1 ? gn - h_span : 1;
  for (long h = gn - 1; h >= h_min; --h) {
    const long nt = N - h * BN;
    const double head = main_us(gm * h, K) + 0.5 * fit.splitk_launch_us;
    if (head >= best) continue;
    for (int s = 2; s <= 64; ++s) {
      const long kc = (((K + s - 1) / s) + gran - 1) / gran * gran;
      if (kc < 256) break;   // shorter chunks run below the model's rate (2146 x 6400 x 512 in chunks of 176: 3 % lost)
      const long se = (K + kc - 1) / kc;
      if (se < 2) continue;
      if (se * M * nt * (long)sizeof(T) > max_ws_bytes) break;
      const double t = head + main_us(gm * (gn - h) * se, kc) + fit.splitk_launch_us +
                       ((double)se + 1.0) * (double)M * (double)nt * sizeof(T) / fit.pass_bytes_per_us;
      if (t < best) {
        best = t;
        best_s = (int)se;
        *n_head_out = h * BN;
      }
    }
  }
  if (us_out) *us_out = best;
  return best_s;
}

// Macro tile and split count of one product (alone on the device: possibly an unsplit head of n_head columns and a
// tail that splits K tail_splits ways).
struct TileChoice { int tm = 128, tn = 128, splits = 1, kchunk = 0; bool big = false, wide = false; long n_head = 0; int tail_splits = 0; double us = -1; };
template <typename T>
TileChoice choose_tile(bool an, bool bnn, long M, long N, long K, bool beta_zero, bool have_ws, long workspace_bytes, bool large_allowed = true,
                       int want_splits = 0, bool alone = false, long m_read = 0, long n_read = 0, bool small_only = false) {
  TileChoice c;
  double alone_us = -1;   // alone: the predicted time of the 128 x 128 tile with the split count chosen for it
  if (want_splits >= 1) {
    // the caller's split count (1: unsplit), in whole panels per chunk like the model's own
    const long gran = sizeof(T) == 4 ? PLK_F32_DEEP_BK : 16;
    const long kc = (((K + want_splits - 1) / want_splits) + gran - 1) / gran * gran;
    const long se = (K + kc - 1) / kc;
    if (se > 1 && have_ws && want_splits > 1) c.splits = (int)se, c.kchunk = (int)kc;
  } else if (alone) {
    c.splits = pick_splits_alone<T>(M, N, K, have_ws ? workspace_bytes : 0, &c.kchunk, &alone_us);
  } else {
    c.splits = have_ws ? pick_splits<T>(M, N, K, &c.kchunk) : 1;
  }
  if (c.splits > 1 && (long)c.splits * M * N * (long)sizeof(T) > workspace_bytes) c.splits = 1, c.kchunk = 0;
  // fp32 has two more macro tiles, chosen per call by the fitted model below when they are faster than 128 x 128.
  //  * 256 x 256 x 32 ("large", every transpose): its inner loop runs 1 % faster per k (a 16-byte operand read per
  //    block and four k-steps, half the row requests per MFMA), but a CU holds one such workgroup at a time, so
  //    nothing overlaps its prologue and its epilogue: a round of 256 large tiles takes f + 2 * c * K / (1 + g), c the
  //    per-k time of a round of 512 small tiles, with g and f (beta == 0 / beta != 0) fitted per transpose to
  //    single-stream runs at M = N = 8192, K = 512 .. 8192 (152.6 - 153.2 TFLOP/s at K = 8192, beta = 0, for all four;
  //    the small tile 150 - 151).  With beta == 0 its fixed cost per unit of work is the lower one and it wins from
  //    K of about 256 on; with beta != 0 (45 - 54 us per round) only beyond K of about 12000.
  //  * 256 x 128 x 16 ("wide", NN only, panels staged through registers): still two workgroups per CU, 5 % slower per
  //    k than the small tile since that one loads its panels directly: f_w + 2 * c * K / 0.949 per round of 512; its
  //    lower fixed cost wins for K of a few hundred.
  //  * a round of 512 small tiles: f_s + c * K.
  // The constants are pl_gemm_fit's (built-in: c = 0.1099 us, f_s = 7.4 us, f_w = 4.9 | 10.6 us, g = 0.010 - 0.012, f = 11 |
  // 45 - 54 us).  Split K keeps the small tile.  fp64 stays at 128 x 128: a 256 x 128 tile (one wave per SIMD,
  // 32-cycle MFMAs) measured 70.7 against 73.4 TFLOP/s.
  const pl_gemm_fit& fit = fit_in_use();
  const int tr = an ? (bnn ? 0 : 1) : (bnn ? 2 : 3);
  const int bi = beta_zero ? 0 : 1;
  auto tiles_of = [&](long tm, long tn) { return ((M + tm - 1) / tm) * ((N + tn - 1) / tn); };
  const double k_us = fit.f32_small_us_per_k * (double)K;
  // Alone on the device, a grid with a ragged last row or column (edge workgroups that may not read to the tile's edge
  // take the guarded loop, and nothing else fills the units that wait for them) costs a fraction of a round more,
  // whatever the number of rounds: fp32 256 x 256 tiles, 4096 x 4096 x 4096 910 us, 3712 or 4000 x 4096 x 4096 1122
  // (one round: + 0.24), 5760 x 5632 2026 against 1823 (two: + 0.23 of one), 8192 x 8064 3835 against 3628 (four: + 0.23
  // of one); 128 x 128 tiles 4000 x 4096 x 4096 998 against 926 (+ 0.16 of a round), 8000^2 x 4096 3742 against 3657 (+ 0.19).
  // Without the term the large tile was taken for every such shape that fills its rounds and ran up to 27 % behind
  // the small one (3712 x 4224 x 1024).
  const long mr = m_read > 0 ? m_read : M, nr = n_read > 0 ? n_read : N;
  auto edge = [&](long tm, long tn) { return alone_us >= 0 && ((M % tm != 0 && mr < (M + tm - 1) / tm * tm) || (N % tn != 0 && nr < (N + tn - 1) / tn * tn)); };
  const double large_round = fit.f32_large_fixed_us[tr][bi] + 2.0 * k_us / (1.0 + fit.f32_large_gain[tr]);
  const double wide_round = fit.f32_wide_fixed_us[bi] + 2.0 * k_us / fit.f32_wide_gain;
  // (a round of small tiles as pick_splits_alone prices it)
  const double lone_c1 = fit.lone_us_per_k[sizeof(T) == 8 ? 0 : 1];
  const double small_round = fit.lone_fixed_k * lone_c1 + (double)(c.kchunk > 0 ? c.kchunk : K) * lone_c1 * fit.f32_small_us_per_k / fit.lone_us_per_k[1];
  const double small_edge_us = edge(128, 128) ? fit.edge_rounds[0] * small_round : 0.0;
  // the small tile's best, alone: one launch (split or not) or the head / tail cut
  long cut_head = 0;
  int cut_splits = 0;
  if (alone_us >= 0 && have_ws) {
    double cut_us = -1;
    cut_splits = pick_tail_alone<T>(M, N, K, workspace_bytes, alone_us, &cut_head, &cut_us);
    if (cut_splits > 1) alone_us = cut_us;
  }
  if (alone_us >= 0) alone_us += small_edge_us;
  const double small_us = alone_us >= 0 ? alone_us : (double)((tiles_of(128, 128) + 511) / 512) * (fit.f32_small_fixed_us + k_us);
  const double large_us = (double)((tiles_of(256, 256) + 255) / 256) * large_round + (edge(256, 256) ? fit.edge_rounds[1] * large_round : 0.0);
  const double wide_us = (double)((tiles_of(256, 128) + 511) / 512) * wide_round + (edge(256, 128) ? fit.edge_rounds[0] * wide_round : 0.0);
  // PARALIA_GEMM_LARGE_TILE: "0" small tiles only, "1" the large tile for every call, "2" the wide tile wherever it
  // exists (NN), unset: the model
  const char* const pin = getenv("PARALIA_GEMM_LARGE_TILE");
  const int pinv = (pin && *pin) ? atoi(pin) : -1;
  // (alone, the bigger tiles are weighed against the split small tile too; a caller's own split count keeps the small one)
  const bool other = sizeof(T) == 4 && (c.splits == 1 || alone_us >= 0) && pinv != 0 && !small_only;
  // partly filled rounds cost the bigger tiles more than the model's rounding says (measured: -1 % at 3072 and 5120)
  auto fills = [](long tiles, long places) { return 10 * tiles >= 9 * ((tiles + places - 1) / places) * places; };
  const bool wide_ok = other && an && bnn && (pinv == 2 || (pinv < 0 && fills(tiles_of(256, 128), 512)));
  const bool big_ok = other && large_allowed && (pinv == 1 || (pinv < 0 && fills(tiles_of(256, 256), 256)));
  c.big = big_ok && (pinv == 1 || (large_us < small_us && (!wide_ok || large_us <= wide_us)));
  c.wide = !c.big && wide_ok && (pinv == 2 || wide_us < small_us);
  if (c.big || c.wide) c.splits = 1, c.kchunk = 0;
  c.tm = c.big || c.wide ? 256 : 128;
  c.tn = c.big ? 256 : 128;
  // the model's time for the choice (a product alone on the device only: the two-stream terms price shared rounds)
  if (alone_us >= 0) c.us = c.big ? large_us : c.wide ? wide_us : alone_us;
  if (cut_splits > 1 && !c.big && !c.wide) c.tail_splits = cut_splits, c.n_head = cut_head, c.splits = 1, c.kchunk = 0;
  return c;
}

template <typename T>
int launch_gemm(char ta, char tb, long M, long N, long K, T alpha, const T* A, long lda, const T* B, long ldb, T beta,
                T* C, long ldc, hipStream_t stream, T* workspace = nullptr, long workspace_bytes = 0, int want_splits = 0,
                bool alone = false, long m_read = 0, long n_read = 0, bool small_only = false) {
  using Tr = Traits<T>;
  const bool at = (ta == 'T' || ta == 't'), an = (ta == 'N' || ta == 'n');
  const bool bt = (tb == 'T' || tb == 't'), bnn = (tb == 'N' || tb == 'n');
  if (!(at || an) || !(bt || bnn)) return 1;
  if (M < 0 || N < 0 || K < 0) return 2;
  if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return 2;
  const long rowsA = an ? M : K, rowsB = bnn ? K : N;
  if (lda < (rowsA > 1 ? rowsA : 1) || ldb < (rowsB > 1 ? rowsB : 1) || ldc < (M > 1 ? M : 1)) return 3;
  // rows of op(A) / columns of op(B) that may be read (0: as many as there are)
  if (m_read == 0) m_read = M;
  if (n_read == 0) n_read = N;
  if (m_read < M || n_read < N || m_read > INT32_MAX || n_read > INT32_MAX) return 2;
  if (M == 0 || N == 0) return 0;
  if (K == 0 || alpha == T(0)) {
    if (beta == T(1)) return 0;
    const long total = M * N;
    int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
    hipLaunchKernelGGL(scale_kernel<T>, dim3(blocks), dim3(256), 0, stream, (int)M, (int)N, beta, C, ldc);
    return hipGetLastError() == hipSuccess ? 0 : 4;
  }
  if (!A || !B || !C) return 5;
  // a K-major operand loaded straight into LDS takes eight rows per request with 32-bit lane offsets: leading dimensions
  // beyond that keep the tiles that stage through registers
  const bool dma_fits = (!at || lda * (long)sizeof(T) <= PLK_DMA_MAX_LD_BYTES) && (!bnn || ldb * (long)sizeof(T) <= PLK_DMA_MAX_LD_BYTES);
  const TileChoice choice = choose_tile<T>(an, bnn, M, N, K, beta == T(0), workspace != nullptr, workspace_bytes, dma_fits, want_splits, alone, m_read, n_read, small_only);
  if (choice.tail_splits > 1) {
    // head: whole tile columns, unsplit, in the 128 x 128 tiles the cut was priced with; tail: the remaining columns of
    // op(B) and C with K split
    const long nh = choice.n_head;
    const int rc = launch_gemm<T>(ta, tb, M, nh, K, alpha, A, lda, B, ldb, beta, C, ldc, stream, nullptr, 0, 1, false, m_read, n_read, true);
    if (rc != 0) return rc;
    return launch_gemm<T>(ta, tb, M, N - nh, K, alpha, A, lda, bnn ? B + nh * ldb : B + nh, ldb, beta, C + nh * ldc, ldc, stream, workspace,
                          workspace_bytes, choice.tail_splits, false, m_read, n_read - nh);
  }
  const int kchunk = choice.kchunk, splits = choice.splits;
  const bool big = choice.big, wide = choice.wide;
  const int TM_RT = choice.tm, TN_RT = choice.tn;
  const int gm = (int)((M + TM_RT - 1) / TM_RT), gn = (int)((N + TN_RT - 1) / TN_RT);
  if ((long)gm * gn > INT32_MAX) return 2;
  const int vecA = ((reinterpret_cast<uintptr_t>(A) & 15) == 0 && lda % Tr::VEC == 0) ? 1 : 0;
  const int vecB = ((reinterpret_cast<uintptr_t>(B) & 15) == 0 && ldb % Tr::VEC == 0) ? 1 : 0;
  // C (or the split-K slices) aligned for 16-byte accesses
  const int vecC = ((reinterpret_cast<uintptr_t>(splits > 1 ? workspace : C) & 15) == 0 && (splits > 1 ? M : ldc) % 4 == 0) ? 1 : 0;
  dim3 grid(gm * gn, splits), block(NTHREADS);
  // split: plain partial products into the dense workspace slices, alpha and beta applied by the reduction
  const T k_alpha = splits > 1 ? T(1) : alpha, k_beta = splits > 1 ? T(0) : beta;
  T* const k_C = splits > 1 ? workspace : C;
  const long k_ldc = splits > 1 ? M : ldc;
  constexpr int BK_SMALL = sizeof(T) == 4 ? PLK_F32_BK : PLK_F64_BK;
  // fp64: panels staged through registers only where the row requests cannot address the operand
  // (the fp32 128 x 128 tile: a request covers sixteen rows of a K-major operand, or two of an MN-major one)
  const bool small_fits = (at ? lda * (long)sizeof(T) <= PLK_DMA_MAX_LD_BYTES / 2 : lda * (long)sizeof(T) < (1L << 32) - 1024) &&
                          (bnn ? ldb * (long)sizeof(T) <= PLK_DMA_MAX_LD_BYTES / 2 : ldb * (long)sizeof(T) < (1L << 32) - 1024);
  const bool stage = sizeof(T) == 8 ? ((splits > 1 ? kchunk : K) < PLK_F64_STAGE_BELOW || !dma_fits) : !small_fits;
  // fp32 128 x 128 with direct panels: 32-deep panels where every workgroup's k extent is a whole number of them (a
  // K-major row is then a full 128-byte line per request: TN 141.8 -> 148.9, TT 146.8 -> 149.4 TFLOP/s at 8192^3, NN and
  // NT + 0.5 %; same bits), 16-deep ones otherwise
  const bool deep = sizeof(T) == 4 && (splits > 1 ? kchunk : K) % PLK_F32_DEEP_BK == 0 && dma_fits;
#define PLK_LAUNCH_T(AKF, BKF, TM, TN, TK, DIRF)                                                                            \
  hipLaunchKernelGGL((gemm_kernel<T, AKF, BKF, TM, TN, TK, DIRF>), grid, block, 0, stream, (int)M, (int)N, (int)K, k_alpha, \
                     A, lda, B, ldb, k_beta, k_C, k_ldc, gm, gn, vecA, vecB, vecC, kchunk, (int)m_read, (int)n_read)
#define PLK_LAUNCH(AKF, BKF)                                                        \
  do {                                                                              \
    if constexpr (sizeof(T) == 4) {                                                 \
      if (big) { PLK_LAUNCH_T(AKF, BKF, 256, 256, PLK_F32_BIG_BK, true); break; }   \
      if (wide) { PLK_LAUNCH_T(AKF, BKF, 256, 128, PLK_F32_BK, true); break; }      \
    }                                                                               \
    if (stage) { PLK_LAUNCH_T(AKF, BKF, 128, 128, BK_SMALL, false); break; }        \
    if constexpr (sizeof(T) == 4) {                                                 \
      if (deep) { PLK_LAUNCH_T(AKF, BKF, 128, 128, PLK_F32_DEEP_BK, true); break; } \
    }                                                                               \
    PLK_LAUNCH_T(AKF, BKF, 128, 128, BK_SMALL, true);                               \
  } while (0)
  // op(A) K-major <=> TransA == 'T'; op(B) K-major <=> TransB == 'N'
  if (an && bnn) PLK_LAUNCH(false, true);
  else if (an && bt) PLK_LAUNCH(false, false);
  else if (at && bnn) PLK_LAUNCH(true, true);
  else PLK_LAUNCH(true, false);
#undef PLK_LAUNCH_T
#undef PLK_LAUNCH
  if (splits > 1) {
    const long total = M * N;
    const int blocks = (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192);
    hipLaunchKernelGGL(splitk_reduce_kernel<T>, dim3(blocks), dim3(256), 0, stream, (int)M, (int)N, splits, alpha, workspace, beta, C, ldc);
  }
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

template <typename T>
long workspace_bytes_for(long M, long N, long K) {
  if (M <= 0 || N <= 0 || K <= 0 || M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return 0;
  int kchunk = 0;
  const int s = pick_splits<T>(M, N, K, &kchunk);
  return s > 1 ? (long)s * M * N * (long)sizeof(T) : 0;
}

}  // namespace plk

extern "C" int pl_dgemm_tile(char transA, char transB, long M, long N, long K, double alpha, const double* A, long lda,
                             const double* B, long ldb, double beta, double* C, long ldc, void* stream) {
  return plk::launch_gemm<double>(transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, (hipStream_t)stream);
}

extern "C" int pl_sgemm_tile(char transA, char transB, long M, long N, long K, float alpha, const float* A, long lda,
                             const float* B, long ldb, float beta, float* C, long ldc, void* stream) {
  return plk::launch_gemm<float>(transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, (hipStream_t)stream);
}

extern "C" void pl_gemm_fit_defaults(pl_gemm_fit* fit) {
  if (fit) plk::fit_defaults(fit);
}
extern "C" int pl_gemm_set_fit(const pl_gemm_fit* fit) {
  if (!fit) { plk::fit_defaults(&plk::fit_in_use()); return 0; }
  // a fit that would divide by zero or run backwards is refused as a whole
  const bool sane = fit->lone_us_per_k[0] > 0 && fit->lone_us_per_k[1] > 0 && fit->lone_fixed_k >= 0 && fit->splitk_launch_us >= 0 &&
                    fit->pass_bytes_per_us > 0 && fit->f32_small_us_per_k > 0 && fit->f32_small_fixed_us >= 0 && fit->f32_wide_gain > 0.5;
  bool large_sane = true;
  for (int t = 0; t < 4; ++t) large_sane = large_sane && fit->f32_large_gain[t] > -0.5 && fit->f32_large_fixed_us[t][0] >= 0 && fit->f32_large_fixed_us[t][1] >= 0;
  if (!sane || !large_sane || fit->f32_wide_fixed_us[0] < 0 || fit->f32_wide_fixed_us[1] < 0) return PL_ERR_ARG;
  if (!(fit->edge_rounds[0] >= 0 && fit->edge_rounds[0] <= 2 && fit->edge_rounds[1] >= 0 && fit->edge_rounds[1] <= 2)) return PL_ERR_ARG;
  plk::fit_in_use() = *fit;
  return 0;
}
extern "C" int pl_gemm_get_fit(pl_gemm_fit* fit) {
  if (!fit) return PL_ERR_NULL;
  *fit = plk::fit_in_use();
  return 0;
}
extern "C" int pl_gemm_tile_choice(int elem_size, char transA, char transB, long M, long N, long K, int beta_is_zero, long workspace_bytes,
                                   int* tile_m, int* tile_n, int* splits) {
  const bool at = (transA == 'T' || transA == 't'), an = (transA == 'N' || transA == 'n');
  const bool bt = (transB == 'T' || transB == 't'), bnn = (transB == 'N' || transB == 'n');
  if (!(at || an) || !(bt || bnn)) return PL_ERR_TRANS;
  if (M <= 0 || N <= 0 || K <= 0 || (elem_size != 8 && elem_size != 4)) return PL_ERR_DIM;
  const plk::TileChoice c = elem_size == 8 ? plk::choose_tile<double>(an, bnn, M, N, K, beta_is_zero != 0, workspace_bytes > 0, workspace_bytes)
                                           : plk::choose_tile<float>(an, bnn, M, N, K, beta_is_zero != 0, workspace_bytes > 0, workspace_bytes);
  if (tile_m) *tile_m = c.tm;
  if (tile_n) *tile_n = c.tn;
  if (splits) *splits = c.splits;
  return 0;
}

extern "C" long pl_gemm_tile_workspace_bytes(long M, long N, long K, int elem_size) {
  return elem_size == 8 ? plk::workspace_bytes_for<double>(M, N, K) : elem_size == 4 ? plk::workspace_bytes_for<float>(M, N, K) : 0;
}

extern "C" int pl_dgemm_tile_split(char transA, char transB, long M, long N, long K, double alpha, const double* A, long lda,
                                   const double* B, long ldb, double beta, double* C, long ldc, void* workspace,
                                   long workspace_bytes, int splits, void* stream) {
  if (splits < 1) return PL_ERR_ARG;
  return plk::launch_gemm<double>(transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, (hipStream_t)stream,
                                  (double*)workspace, workspace_bytes, splits);
}

extern "C" int pl_sgemm_tile_split(char transA, char transB, long M, long N, long K, float alpha, const float* A, long lda,
                                   const float* B, long ldb, float beta, float* C, long ldc, void* workspace,
                                   long workspace_bytes, int splits, void* stream) {
  if (splits < 1) return PL_ERR_ARG;
  return plk::launch_gemm<float>(transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, (hipStream_t)stream,
                                 (float*)workspace, workspace_bytes, splits);
}

extern "C" int pl_dgemm_tile_padded(char transA, char transB, long M, long N, long K, double alpha, const double* A, long lda,
                                    const double* B, long ldb, double beta, double* C, long ldc, void* workspace,
                                    long workspace_bytes, int splits, long m_readable, long n_readable, void* stream) {
  if (splits < -1) return PL_ERR_ARG;
  return plk::launch_gemm<double>(transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, (hipStream_t)stream,
                                  (double*)workspace, workspace_bytes, splits < 0 ? 0 : splits, splits < 0, m_readable, n_readable);
}

extern "C" int pl_sgemm_tile_padded(char transA, char transB, long M, long N, long K, float alpha, const float* A, long lda,
                                    const float* B, long ldb, float beta, float* C, long ldc, void* workspace,
                                    long workspace_bytes, int splits, long m_readable, long n_readable, void* stream) {
  if (splits < -1) return PL_ERR_ARG;
  return plk::launch_gemm<float>(transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, (hipStream_t)stream,
                                 (float*)workspace, workspace_bytes, splits < 0 ? 0 : splits, splits < 0, m_readable, n_readable);
}

// workspace a product alone on the device is given at most (the slices of its split)
#define PLK_ALONE_MAX_WS_BYTES (1L << 30)

extern "C" int pl_dgemm_tile_alone(char transA, char transB, long M, long N, long K, double alpha, const double* A, long lda,
                                   const double* B, long ldb, double beta, double* C, long ldc, void* workspace,
                                   long workspace_bytes, void* stream) {
  return plk::launch_gemm<double>(transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, (hipStream_t)stream,
                                  (double*)workspace, workspace_bytes, 0, true);
}

extern "C" int pl_sgemm_tile_alone(char transA, char transB, long M, long N, long K, float alpha, const float* A, long lda,
                                   const float* B, long ldb, float beta, float* C, long ldc, void* workspace,
                                   long workspace_bytes, void* stream) {
  return plk::launch_gemm<float>(transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, (hipStream_t)stream,
                                 (float*)workspace, workspace_bytes, 0, true);
}

extern "C" int pl_gemm_tile_choice_alone(int elem_size, char transA, char transB, long M, long N, long K, int beta_is_zero,
                                         long workspace_bytes, int* tile_m, int* tile_n, int* splits) {
  const bool at = (transA == 'T' || transA == 't'), an = (transA == 'N' || transA == 'n');
  const bool bt = (transB == 'T' || transB == 't'), bnn = (transB == 'N' || transB == 'n');
  if (!(at || an) || !(bt || bnn)) return PL_ERR_TRANS;
  if (M <= 0 || N <= 0 || K <= 0 || (elem_size != 8 && elem_size != 4)) return PL_ERR_DIM;
  const plk::TileChoice c = elem_size == 8 ? plk::choose_tile<double>(an, bnn, M, N, K, beta_is_zero != 0, workspace_bytes > 0, workspace_bytes, true, 0, true)
                                           : plk::choose_tile<float>(an, bnn, M, N, K, beta_is_zero != 0, workspace_bytes > 0, workspace_bytes, true, 0, true);
  if (tile_m) *tile_m = c.tm;
  if (tile_n) *tile_n = c.tn;
  if (splits) *splits = c.splits;
  return 0;
}

extern "C" int pl_gemm_tile_cut_alone(int elem_size, char transA, char transB, long M, long N, long K, int beta_is_zero,
                                      long workspace_bytes, long* n_head, int* tail_splits) {
  const bool at = (transA == 'T' || transA == 't'), an = (transA == 'N' || transA == 'n');
  const bool bt = (transB == 'T' || transB == 't'), bnn = (transB == 'N' || transB == 'n');
  if (!(at || an) || !(bt || bnn)) return PL_ERR_TRANS;
  if (M <= 0 || N <= 0 || K <= 0 || (elem_size != 8 && elem_size != 4)) return PL_ERR_DIM;
  const plk::TileChoice c = elem_size == 8 ? plk::choose_tile<double>(an, bnn, M, N, K, beta_is_zero != 0, workspace_bytes > 0, workspace_bytes, true, 0, true)
                                           : plk::choose_tile<float>(an, bnn, M, N, K, beta_is_zero != 0, workspace_bytes > 0, workspace_bytes, true, 0, true);
  if (n_head) *n_head = c.tail_splits > 1 ? c.n_head : N;
  if (tail_splits) *tail_splits = c.tail_splits > 1 ? c.tail_splits : 0;
  return 0;
}

extern "C" double pl_gemm_tile_alone_us(int elem_size, char transA, char transB, long M, long N, long K, int beta_is_zero, long workspace_bytes) {
  const bool at = (transA == 'T' || transA == 't'), an = (transA == 'N' || transA == 'n');
  const bool bt = (transB == 'T' || transB == 't'), bnn = (transB == 'N' || transB == 'n');
  if (!(at || an) || !(bt || bnn) || M <= 0 || N <= 0 || K <= 0 || (elem_size != 8 && elem_size != 4)) return -1.0;
  const plk::TileChoice c = elem_size == 8 ? plk::choose_tile<double>(an, bnn, M, N, K, beta_is_zero != 0, workspace_bytes > 0, workspace_bytes, true, 0, true)
                                           : plk::choose_tile<float>(an, bnn, M, N, K, beta_is_zero != 0, workspace_bytes > 0, workspace_bytes, true, 0, true);
  return c.us;
}

extern "C" long pl_gemm_tile_alone_workspace_bytes(char transA, char transB, long M, long N, long K, int beta_is_zero, int elem_size) {
  int splits = 1, tail_splits = 0;
  long n_head = N;
  if (pl_gemm_tile_choice_alone(elem_size, transA, transB, M, N, K, beta_is_zero, PLK_ALONE_MAX_WS_BYTES, nullptr, nullptr, &splits) != 0) return 0;
  if (pl_gemm_tile_cut_alone(elem_size, transA, transB, M, N, K, beta_is_zero, PLK_ALONE_MAX_WS_BYTES, &n_head, &tail_splits) != 0) return 0;
  if (tail_splits > 1) return (long)tail_splits * M * (N - n_head) * elem_size;
  return splits > 1 ? (long)splits * M * N * elem_size : 0;
}

extern "C" int pl_dgemm_tile_ws(char transA, char transB, long M, long N, long K, double alpha, const double* A, long lda,
                                const double* B, long ldb, double beta, double* C, long ldc, void* workspace,
                                long workspace_bytes, void* stream) {
  return plk::launch_gemm<double>(transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, (hipStream_t)stream,
                                  (double*)workspace, workspace_bytes);
}

extern "C" int pl_sgemm_tile_ws(char transA, char transB, long M, long N, long K, float alpha, const float* A, long lda,
                                const float* B, long ldb, float beta, float* C, long ldc, void* workspace,
                                long workspace_bytes, void* stream) {
  return plk::launch_gemm<float>(transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, (hipStream_t)stream,
                                 (float*)workspace, workspace_bytes);
}
