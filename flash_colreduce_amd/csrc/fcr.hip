// libfcr: column reduction of softmax attention for MI355X (gfx950, CDNA4).
//
// Two sweeps, both built on v_mfma_f32_16x16x32_{f16,bf16} (fp32 operands: v_mfma_f32_16x16x4_f32) with
// the product taken as S^T = K * Q^T (keys are MFMA rows, queries are MFMA columns).  In a 16x16
// accumulator a lane owns ONE query (lane & 15) and 4 keys (row 4*(lane/16) + r for register r), so
//   - everything that is per query row (softmax reference exponent, running sum, lse) is one
//     scalar per lane and needs no cross-lane traffic inside the sweep;
//   - everything that is per key column accumulates in the lane's registers over the whole
//     sweep and is reduced across the 16 query lanes once, at the end.
// The sweeps are bound by the vector instruction port (an MFMA keeps it for about 10 cycles, the fma,
// exp2 and add of the 64 scores it produces for 16 more) and, on random operands, by the package power
// limit.  The 16x16x32 shape is used because the 32x32x16 one, which would halve the MFMAs' share of the
// port, draws more power on random operands and ends up slower there.
//
//   row_lse_kernel    a workgroup keeps 256 query rows in registers (64 per wave; 128 and 32 for
//                     few or ragged M and for rows longer than 256 bytes) and streams key tiles through
//                     LDS; writes lse2[bh, i] = log2 sum_j 2^(s_ij).
//   col_reduce_kernel a workgroup keeps 256 key rows in registers and streams query tiles (and
//                     their lse2) through LDS; writes out[bh, j] = sum_i or max_i 2^(s_ij-lse2_i).
//   col_small_kernel  the same result for at most 128 query rows against many keys: queries resident
//                     in every wave, keys streamed (HBM bound).
//   col_fused_kernel  both sweeps in one for at most 128 query rows against many 16-bit keys: the scores of
//                     1024 keys stay in registers while the workgroups that share a (batch, head) pair
//                     exchange their row sums through tagged 64-bit slots, so the keys are read once.
//   topk_mask_kernel  keep-mask of the k largest columns of every row of the result (one workgroup per
//                     row; topk_spread_* kernels share a long row between workgroups).
// where s_ij = scale * log2(e) * <q_i, k_j>.  The column kernels store the result type of the caller's choice
// and divide the means as they store (store_column).  The streamed operand goes from global memory straight
// into a swizzled ring of LDS stages (buffer loads with the LDS as destination).  Nothing of size M*N
// is written anywhere and nothing in global memory is updated by read-modify-write atomics: one workgroup
// owns its output rows / columns (col_fused_kernel hands its partial row values to its team with atomic
// 64-bit stores and loads, value and round number in one word).
//
// Replaces the Triton kernel of the reference (flash_colreduce/flash.py:11-274).

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>

#include <mutex>
#include <type_traits>

#include "fcr.h"

// The file can be compiled whole, or in parts that are linked together (the build script does that to
// use several cores): part 0 holds the C ABI and the small kernels, parts 1-4 the sweeps of one element
// type each (fp16, bf16, fp32 rows up to 512 bytes, longer fp32 rows), parts 5 and 6 the sweeps over fp16 and
// bf16 rows of more than 512 bytes, parts 7 and 8 the single sweep for fp16 and bf16.
#ifndef FCR_PART
#define FCR_PART -1
#endif
#define FCR_HAS(part) (FCR_PART == -1 || FCR_PART == (part))

namespace fcr_detail {
struct Params {
  const char* q;
  const char* k;
  float* lse;        // [BH, M]
  float* part;       // [splits, BH, M] partial lse of key ranges when splits > 1
  int splits;        // key ranges per row tile in the row kernel (1 = whole sweep in one workgroup)
  void* out;         // [BH, N]: column sums or means (or the only result)
  void* out2;        // [BH, N]: column maxima when one sweep produces both
  int64_t q_sb, q_sh, q_sr;  // strides in BYTES: batch, head, row
  int64_t k_sb, k_sh, k_sr;
  int H, M, N;
  int dgran;         // D / 8: valid 16-byte granules per row
  int c;             // max(N - M, 0): the causal right-alignment offset
  float scale2;      // scale * log2(e)
  int tiles;         // resident tiles per (b,h)
  int bh_count;      // B * H
  int group;         // (b,h) pairs whose workgroups are launched together (see map_block)
  int stream_once;   // col_small_kernel: load the keys non-temporally
  int total;         // tiles * B * H workgroups
  // How the column kernels write a finished column (see store_column)
  int out_fmt;       // element type of out and out2: FCR_DTYPE_F32, FCR_DTYPE_F16 or FCR_DTYPE_BF16
  int mean_from;     // < 0: out holds the sums.  Else out holds means: columns below mean_from are
  float inv_m;       //   multiplied by inv_m = 1/M, column j from there on is divided by N - j
  // col_fused_kernel: teams of `splits` workgroups, team t takes (b,h) = t, t + teams, ..
  int teams;
  unsigned* sync;    // error word; zero at launch, like the slots at `part`
  int spin_limit;    // polls of the counter after which a wait gives up
};
// which: 0 = row statistics, 1 = column sweep, 2 = column sweep for few queries, 3 = both sweeps in one for few
// queries, mode + 4 for more than 64 of them (2 and 3: 16-bit types only)
void sweeps_f16(int which, const Params& p, int ksteps, bool causal, int mode, hipStream_t s);
void sweeps_bf16(int which, const Params& p, int ksteps, bool causal, int mode, hipStream_t s);
void sweeps_f32(int which, const Params& p, int ksteps, bool causal, int mode, hipStream_t s);
void sweeps_f32_long_rows(int which, const Params& p, int ksteps, bool causal, int mode, hipStream_t s);
void sweeps_f16_single(const Params& p, int ksteps, bool causal, int mode, hipStream_t s);    // col_fused_kernel
void sweeps_bf16_single(const Params& p, int ksteps, bool causal, int mode, hipStream_t s);
void sweeps_f16_long_rows(int which, const Params& p, int ksteps, bool causal, int mode, hipStream_t s);
void sweeps_bf16_long_rows(int which, const Params& p, int ksteps, bool causal, int mode, hipStream_t s);
extern thread_local bool fused_refused;   // set by a launcher of col_fused_kernel that did not launch
}  // namespace fcr_detail

namespace {
using fcr_detail::Params;

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
// k-steps are 64 bytes of a row: 32 16-bit elements of D, or 16 floats.  A wave keeps resident rows in groups of 16 (one MFMA operand each);
// two 32-row blocks (four groups) while their fragments fit the register file next to the
// accumulators (D <= 128: 4 k-steps), one block for larger D.  A workgroup keeps 4 * 32 * blocks rows.
__host__ __device__ constexpr int blocks_per_wave(int ksteps) { return ksteps <= 4 ? 2 : 1; }
// Compute units of the current device, asked once per device.  The tile, split and group choices below
// are stated in workgroups per CU (these kernels run two per CU).  256, an MI355X in its default
// partition mode, when no device can be asked (argument checks on a host without a GPU).
inline int chip_cus() {
  static int cached[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
    (void)hipGetLastError();
    return 256;
  }
  int n = __atomic_load_n(&cached[dev], __ATOMIC_RELAXED);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) {
      (void)hipGetLastError();
      n = 256;
    }
    __atomic_store_n(&cached[dev], n, __ATOMIC_RELAXED);
  }
  return n;
}
// The row kernel has both forms for D <= 128 and the host picks per problem.  Waves whose rows are all
// padding do no arithmetic, so a launch costs (rows in waves with at least one query) x (cost per
// row); one block per wave costs about 3 % per k-step more per row (every streamed fragment feeds
// half as many MFMAs) but rounds M up to 32 instead of 64 rows per wave: it wins for M <= 128 and
// for a few ragged M above that.
inline int64_t rows_swept(int M, int nb) {
  const int trows = kWaves * 32 * nb;
  const int rem = M % trows;
  const int waves = rem ? (rem + 31) / 32 : 0;   // blocks of the last tile that hold queries
  return (int64_t)(M / trows) * trows + (waves < kWaves ? waves : kWaves) * 32 * nb;
}
// One block also wins when two would give between one and two workgroups per CU (with fewer than
// one the keys of a tile are split over workgroups instead, see row_splits; that case does not depend
// on `causal`, so the size of the lse buffer does not either).  With the mask exactly two per CU is
// still too coarse: the chip then waits for the workgroup with the longest sweep.  Against at most
// 1024 keys one block wins below one workgroup per CU as well: twice the workgroups beat splitting
// sweeps of 16 chunks (32 heads of 1024 x 1024: 16.5 -> 14 us, 16 heads of 512 x 512: 13 -> 8.6 us).
inline int row_blocks_per_wave(int ksteps, int M, int N, int64_t bh, bool causal) {
  if (ksteps > 4) return 1;
  if (rows_swept(M, 1) * (100 + 3 * ksteps) < rows_swept(M, 2) * 100) return 1;
  const int64_t wgs2 = bh * ((M + kWaves * 64 - 1) / (kWaves * 64));
  const int cus = chip_cus();
  if (wgs2 < cus && N <= 1024) return 1;
  return (wgs2 >= cus && wgs2 < 2 * cus + (causal ? 1 : 0)) ? 1 : 2;
}
inline int row_tile_rows(int ksteps, int M, int N, int64_t bh, bool causal) {
  return kWaves * 32 * row_blocks_per_wave(ksteps, M, N, bh, causal);
}
constexpr int kMaxKSteps = 8;                 // rows of up to 512 bytes: two workgroups per CU
constexpr int kMaxKStepsF32 = 16;             // rows of up to 1 KiB (fp32: D <= 256, 16-bit elements: D <= 512), one workgroup per CU
constexpr int kChunk = 64;                    // streamed rows per LDS stage (two 32-row sub-steps)
constexpr int64_t kMaxWorkgroups = 1ll << 24; // the runtime refuses launches of 2^32 threads or more
constexpr float kNegInf = -__builtin_inff();
constexpr float kPosInf = __builtin_inff();


// D[16 keys][16 queries] += A[16 keys][32 d] * B[32 d][16 queries].  Lane l supplies, for A and for
// B alike, the 8 consecutive d-elements [8*(l/16), +8) of row / column l & 15, and receives
// D[4*(l/16) + r][l & 15] in register r.
template <int DT>
__device__ __forceinline__ f32x4 mma(u32x4 a, u32x4 b, f32x4 c) {
  if constexpr (DT == FCR_DTYPE_F16) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c,
                                                  0, 0, 0);
  } else if constexpr (DT == FCR_DTYPE_BF16) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b),
                                                   c, 0, 0, 0);
  } else {
    // fp32 operands: the same 16 bytes per lane are four floats, d = 4*(l/16) + e of a 16-float k-step.
    // v_mfma_f32_16x16x4_f32 number e contracts over the four lane groups' element e, so the four of
    // them cover the 16 floats once (the order of the terms of a dot product is free).
    const f32x4 af = __builtin_bit_cast(f32x4, a), bf = __builtin_bit_cast(f32x4, b);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(af[0], bf[0], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(af[1], bf[1], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(af[2], bf[2], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(af[3], bf[3], c, 0, 0, 0);
    return c;
  }
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// Work order.  The (b,h) pairs are taken in groups of `group`; inside a group workgroup w takes
// (b,h) = first + w % g and the tile of rank w / g, tiles ranked by the length of their sweep,
// longest first: with more workgroups than the chip holds at once, the short ones fill in behind
// the long ones and the causal triangle finishes level.  A group is sized to about what the chip
// holds at once, so all tiles of a (b,h) run at the same time and its streamed operand comes from
// HBM once.  Workgroups are dealt to the 8 XCDs round-robin by v, so with group a multiple of 8
// every (b,h) stays on XCD (b,h) % 8 and that operand is shared through the XCD's L2.
__device__ __forceinline__ void map_group(const Params& p, int per_bh, int& bh, int& r) {
  const int v = (int)blockIdx.x;
  const int per = p.group * per_bh;
  const int chunk = v / per;
  const int first = chunk * p.group;
  const int g = min(p.group, p.bh_count - first);
  const int w = v - chunk * per;
  r = w / g;
  bh = first + (w - r * g);
}

__device__ __forceinline__ void map_block(const Params& p, bool longest_is_last_tile, int& bh, int& tile) {
  int rank;
  map_group(p, p.tiles, bh, rank);
  tile = longest_is_last_tile ? p.tiles - 1 - rank : rank;
}

// Row kernel with the keys of a tile split over several workgroups (few query rows, many keys):
// inside a group the order is (b,h), then the tile, then the key range: the tiles that stream the
// same keys start next to each other on the same XCD and share them through its L2.
__device__ __forceinline__ void map_block_split(const Params& p, bool longest_is_last_tile, int& bh, int& tile,
                                                int& split) {
  int r;
  map_group(p, p.tiles * p.splits, bh, r);
  const int back = r / p.tiles;   // the last key range first: with the mask it holds the diagonal, the slow part
  const int rank = r - back * p.tiles;
  split = p.splits - 1 - back;
  tile = longest_is_last_tile ? p.tiles - 1 - rank : rank;
}

// First rows of the wave's resident 16-row groups.  With two blocks per wave a workgroup's 256
// resident rows are eight 32-row blocks and wave w keeps blocks w and 7-w: on a causal diagonal
// block b has b+1 (rows) or 8-b (columns) visible sub-tiles out of 8, so every wave gets 9 of the 36
// and the four waves reach each barrier together.  With one block per wave, wave w keeps block w
// of four.
template <int NB>
__device__ __forceinline__ void wave_groups(int tile, int wave, int (&rows)[2 * NB]) {
  const int t0 = tile * (kWaves * 32 * NB);
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    // blocks w, 7-w (, 8+w, 15-w): even positions count up, odd ones count down inside a run of eight
    const int blk = (NB == 1) ? wave : 8 * (i / 2) + ((i & 1) ? 7 - wave : wave);
    rows[2 * i] = t0 + 32 * blk;
    rows[2 * i + 1] = t0 + 32 * blk + 16;
  }
}

// Raw buffer view of rows [row0, nrows) of a row-major operand.  Loads through it return zero
// past the last row instead of faulting, so ragged tails need neither branches nor clamps.
// Offsets inside the view are 32 bit; the host checks that 64 rows fit.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t rows_view(const char* base, int64_t row_bytes, int row0,
                                                            int nrows) {
  int64_t bytes = (int64_t)(nrows - row0) * row_bytes;
  bytes = bytes < 0 ? 0 : (bytes > 0xfffffff0ll ? 0xfffffff0ll : bytes);
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(base) + (int64_t)row0 * row_bytes, 0,
                                           (int)(uint32_t)bytes, 0x00020000);
}

// AUX is the cache policy of the load: 0 = default, kLoadOnce = non-temporal, for bytes that no
// workgroup of the launch will ask for again.
constexpr int kLoadOnce = 2;
template <int AUX = 0>
__device__ __forceinline__ u32x4 view_load16(__amdgpu_buffer_rsrc_t v, uint32_t byte_off) {
  return __builtin_amdgcn_raw_buffer_load_b128(v, (int)byte_off, 0, AUX);
}

// The operand a wave keeps for the whole sweep: NG groups of 16 rows starting at rows[g], as MFMA
// fragments.  Lane l holds, for k-step ks, the 8 elements [32*ks + 8*(l/16), +8) of row l & 15.
template <int KS, int NG>
__device__ __forceinline__ void load_resident(u32x4 (&f)[NG][KS], const char* base, int64_t row_bytes,
                                              const int (&rows)[NG], int nrows, int dgran, int lane) {
  const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    const __amdgpu_buffer_rsrc_t view = rows_view(base, row_bytes, rows[g], nrows);
    const uint32_t roff = (uint32_t)(lane & 15) * (uint32_t)row_bytes;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int gi = ks * 4 + (lane >> 4);
      const u32x4 v = view_load16(view, roff + (uint32_t)min(gi, dgran - 1) * 16u);
      f[g][ks] = (gi < dgran) ? v : zero;  // zero padding of D up to the k-step
    }
  }
}

// Global -> LDS staging of the streamed operand, kChunk rows at a time, without passing through
// registers: buffer loads with the LDS as destination write 16 bytes per lane, 1 KiB per wave and
// instruction, to consecutive LDS addresses, while every lane chooses which 16 bytes of global memory it
// fetches.  A ring of stages is filled several chunks ahead of its use, so a load has one or two whole
// chunk periods to arrive and no wave ever waits for memory in the sweep.
//
// LDS layout of a stage: kChunk rows of kPitch bytes, no padding.  The 16-byte granule c of row r sits
// at granule position c ^ swz(r) of its row: a 16-byte fragment read is served in passes of lanes
// {0-7, 16-23}, {8-15, 24-31}, .. (eight consecutive rows at two neighbouring granule columns), and the
// swizzle sends those sixteen granules to sixteen different 16-byte slots modulo 256 bytes, i.e. to all
// 64 banks once.  Granule columns at or past D/8 (the zero padding up to the MFMA k-step, and up to the
// pitch) are fetched from an offset past the end of the buffer view, which yields zeros; so do rows
// past the end of the operand.  Behind the rows a stage has room for 64 floats (the column kernel's lse).
constexpr uint32_t kPastEnd = 0xfffffff0u;   // never inside a view: rows_view keeps sizes below it

// Stages of the ring in the two big sweeps: four while two workgroups of them fit a CU's 160 KiB (loads
// then have two to three chunk periods to arrive), two for the 32 KiB stages of D > 128.
__host__ __device__ constexpr int ring_stages(int ksteps) { return ksteps <= 4 ? 4 : 2; }

template <int AUX>
__device__ __forceinline__ void dma16(__amdgpu_buffer_rsrc_t view, uint32_t byte_off, char* lds_wave_base) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(view, (__attribute__((address_space(3))) void*)lds_wave_base, 16,
                                           (int)byte_off, 0, 0, AUX);
}
__device__ __forceinline__ void dma4(__amdgpu_buffer_rsrc_t view, uint32_t byte_off, char* lds_wave_base) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(view, (__attribute__((address_space(3))) void*)lds_wave_base, 4,
                                           (int)byte_off, 0, 0, 0);
}

// Waits until at most N of this wave's loads are outstanding and all its LDS reads have returned, then
// meets the other waves.  After it, what every wave loaded before its N newest loads is visible to
// all, and no wave is still reading what it read before the barrier, so those stages may be refilled.
// The empty asm statements keep the compiler from moving LDS accesses across the barrier (there is no
// fence, which would wait for every outstanding load).
// The value a float has after a round trip through the result's element type (round to nearest even,
// overflow to infinity, NaN kept), as the float16_t / bfloat16 casts of torch do it.
__device__ __forceinline__ float round_trip(int fmt, float v) {
  if (fmt == FCR_DTYPE_F16) return (float)(_Float16)v;
  if (fmt == FCR_DTYPE_BF16) {
    uint32_t b = __builtin_bit_cast(uint32_t, v);
    b = (v != v) ? 0x7fc00000u : ((b + 0x7fffu + ((b >> 16) & 1u)) & 0xffff0000u);
    return __builtin_bit_cast(float, b);
  }
  return v;
}

// Writes column `key` of row `bh` of a [BH, N] result whose elements have type p.out_fmt.  The
// reference casts its fp32 accumulation to the result type first (flash.py:308) and divides the means
// afterwards, in that type (flash.py:377-384): columns left of the causal offset by the Python scalar
// M, which torch turns into a multiplication by the fp32 reciprocal, the others by a tensor of counts
// that torch converts to the result type before the fp32 division.  The same steps, in the same order.
__device__ __forceinline__ void store_column(const Params& p, void* base, bool is_sum, int bh, int key, float v) {
  const int fmt = p.out_fmt;
  if (is_sum && p.mean_from >= 0) {
    v = round_trip(fmt, v);
    v = (key < p.mean_from) ? v * p.inv_m : v / round_trip(fmt, (float)(p.N - key));
  }
  const int64_t at = (int64_t)bh * p.N + key;
  if (fmt == FCR_DTYPE_F32) {
    static_cast<float*>(base)[at] = v;
  } else if (fmt == FCR_DTYPE_F16) {
    static_cast<_Float16*>(base)[at] = (_Float16)v;
  } else {
    static_cast<uint16_t*>(base)[at] = (uint16_t)(__builtin_bit_cast(uint32_t, round_trip(FCR_DTYPE_BF16, v)) >> 16);
  }
}

template <int N>
__device__ __forceinline__ void ring_sync() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (0 << 8));  // vmcnt(N) lgkmcnt(0)
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// clamp(x, 0, kChunk) on the scalar unit (written out because the compiler turns min(max()) into a
// three-operand median that only the vector unit has, which would make everything derived from it,
// here a buffer descriptor, a per-lane value)
__device__ __forceinline__ int rows_in_chunk(int rows_left) {
  int live;
  asm("s_max_i32 %0, %1, 0\n\ts_min_i32 %0, %0, %2" : "=s"(live) : "s"(rows_left), "n"(kChunk) : "scc");
  return live;
}

// LW: the waves that issue the loads (their index is what init() takes as wave_id)
template <int KS, int NS = ring_stages(KS), int LW = kWaves>
struct Ring {
  static constexpr int kN = NS;
  static constexpr int kPitch = KS <= 1 ? 64 : KS == 2 ? 128 : KS <= 4 ? 256 : KS <= 8 ? 512 : 1024;   // LDS row pitch
  static constexpr int kRowsPerLoad = 1024 / kPitch;                 // rows one wave-wide load covers
  static constexpr int kPer = kChunk / (LW * kRowsPerLoad);          // loads per loading wave and chunk
  static constexpr int kRows = kChunk * kPitch;                      // bytes of rows in a stage
  static constexpr int kStage = kRows + kChunk * 4;                  // rows + 64 floats
  static constexpr int kBytes = kN * kStage;
  static constexpr int kSwz = kPitch < 256 ? kPitch : 256;
  static __host__ __device__ constexpr int swz(int row) { return 2 * ((row * kSwz / 256) & (kSwz / 32 - 1)); }

  uint32_t voff[kPer];   // source byte offset inside a chunk of the granule this lane fetches, per load
  uint32_t ko[KS];       // LDS byte offset inside a 16-row group of this lane's fragment, per k-step
  int wave;              // wave-uniform

  __device__ __forceinline__ void init(int64_t row_bytes, int dgran, int lane, int wave_id) {
    wave = wave_id;
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
      const int byte = (wave * kPer + i) * 1024 + lane * 16;   // where the lane's 16 bytes land in the stage
      const int row = byte / kPitch;
      const int c = ((byte % kPitch) / 16) ^ swz(row);         // the granule that belongs there
      voff[i] = (c < dgran) ? (uint32_t)row * (uint32_t)row_bytes + (uint32_t)c * 16u : kPastEnd;
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int r = lane & 15, c = 4 * ks + (lane >> 4);
      ko[ks] = (uint32_t)(r * kPitch + ((c ^ swz(r)) * 16));
    }
  }
  // Chunks are fetched in order, so where the next one comes from is kept as a running address and a
  // count of the rows left (scalar registers, a handful of scalar instructions per chunk): rows
  // [row0, nrows) of the operand at `base` are what may be fetched, the rest arrives as zeros
  // without touching memory.
  const char* next_ptr;
  int rows_left;
  uint32_t row_bytes32;
  __device__ __forceinline__ void start(const char* base, int64_t row_bytes, int row0, int nrows) {
    next_ptr = base + (int64_t)row0 * row_bytes;
    rows_left = nrows - row0;
    row_bytes32 = (uint32_t)row_bytes;
  }
  // The next kChunk rows into `stage`.
  template <int AUX = 0>
  __device__ __forceinline__ void issue_next(char* stage) {
    const int live = rows_in_chunk(rows_left);   // the view covers this chunk's rows only
    const __amdgpu_buffer_rsrc_t view = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(next_ptr), 0, (int)((uint32_t)live * row_bytes32), 0x00020000);
#pragma unroll
    for (int i = 0; i < kPer; ++i) dma16<AUX>(view, voff[i], stage + (wave * kPer + i) * 1024);
    next_ptr += (int64_t)kChunk * row_bytes32;
    rows_left -= kChunk;
  }
  // kChunk rows from `ptr` on into `stage`, of which the first `rows` (clamped to [0, kChunk]) exist;
  // for sweeps that do not walk one operand front to back.
  template <int AUX = 0>
  __device__ __forceinline__ void issue_at(char* stage, const char* ptr, int rows) {
    const int live = rows_in_chunk(rows);
    const __amdgpu_buffer_rsrc_t view = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(ptr), 0, (int)((uint32_t)live * row_bytes32), 0x00020000);
#pragma unroll
    for (int i = 0; i < kPer; ++i) dma16<AUX>(view, voff[i], stage + (wave * kPer + i) * 1024);
  }
  // Fragment of the 16-row group sg of sub-step `sub` (32 rows) for k-step ks.
  __device__ __forceinline__ u32x4 frag(const char* stage, int sub, int sg, int ks) const {
    return *reinterpret_cast<const u32x4*>(stage + (sub * 32 + sg * 16) * kPitch + ko[ks]);
  }
};

// One sub-step of a sweep: 32 streamed rows (two groups of 16, fragments f) against the wave's NG
// resident groups: 2*NG independent 16x16 accumulator chains n[g][sg].  S^T = K * Q^T, so keys are
// the A operand.  A streamed fragment stays put for NG consecutive MFMAs.  When REFILL, each fragment
// register is reloaded for the sub-step after this one as soon as its MFMAs are issued, a whole
// sub-step ahead of its use.
template <int DT, int KS, int NG, bool RESIDENT_IS_KEYS, bool REFILL, class RingT>
__device__ __forceinline__ void mma_groups(f32x4 (&n)[NG][2], u32x4 (&f)[2][KS], const u32x4 (&res)[NG][KS],
                                           const RingT& rg, const char* next_lds, int next_sub) {
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    n[g][0] = zero;
    n[g][1] = zero;
  }
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
    for (int sg = 0; sg < 2; ++sg) {
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        if (RESIDENT_IS_KEYS) n[g][sg] = mma<DT>(res[g][ks], f[sg][ks], n[g][sg]);
        else n[g][sg] = mma<DT>(f[sg][ks], res[g][ks], n[g][sg]);
      }
      if (REFILL) f[sg][ks] = rg.frag(next_lds, next_sub, sg, ks);
      // MFMAs and LDS reads keep this order (the refill stays a sub-step ahead of its use instead of
      // sinking to just before it); vector, transcendental and scalar instructions may move across.
      __builtin_amdgcn_sched_barrier(0x2 | 0x4 | 0x400);
    }
  }
}

// Ring protocol.  advance(t) = ring_sync, then the load of the next chunk, t + kN - 1, into the stage
// chunk t - 1 lived in.  A loop calls it once per chunk, in order, before it first touches chunk t; loads are issued
// in chunk order, kPer (+1 with an lse row) per wave and chunk, so at that point "all but the newest
// kN - 2 chunks' loads have arrived" is exactly "chunk t has arrived".  Before the first advance the
// loads of the first kN - 1 chunks of the sweep have been issued.
//
// Branch-free sweep over chunks [ta, tb) of the streamed operand, none of which needs a mask.
// Steady state, per chunk t (two sub-steps s0, s1), one barrier:
//     advance(t+1)       chunk t+1 visible; nobody reads chunk t any more, its stage is being refilled
//     MFMA(s1 of t)   || VALU of s0 of t   || fragments <- s0 of t+1
//     MFMA(s0 of t+1) || VALU of s1 of t   || fragments <- s1 of t+1
// Every LDS read is issued a sub-step before its use.
// aux_of(stage, sub) reads what the consumer needs per sub-step besides the scores (the column
// kernel: lse of the lane's queries); it travels with the fragments so that it too is read before
// the barrier that lets the stage be refilled.
template <int DT, int KS, int NG, bool RESIDENT_IS_KEYS, class Aux, class RingT, class AdvF, class StageF,
          class AuxF, class ConsumeF>
__device__ __forceinline__ void pipelined_sweep(int ta, int tb, const u32x4 (&res)[NG][KS], const RingT& rg,
                                                AdvF&& advance, StageF&& stage_of, AuxF&& aux_of,
                                                ConsumeF&& consume) {
  if (ta >= tb) return;
  u32x4 f[2][KS];
  f32x4 pa[NG][2], pb[NG][2];  // scores of the sub-step being consumed / being produced, swapping roles
  Aux af, ap, an;
  advance(ta);
  {
    const char* lds = stage_of(ta);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      f[0][ks] = rg.frag(lds, 0, 0, ks);
      f[1][ks] = rg.frag(lds, 0, 1, ks);
    }
    ap = aux_of(lds, 0);
    mma_groups<DT, KS, NG, RESIDENT_IS_KEYS, true>(pa, f, res, rg, lds, 1);
    af = aux_of(lds, 1);
  }
  for (int t = ta; t + 1 < tb; ++t) {
    advance(t + 1);
    const char* nxt = stage_of(t + 1);
    an = af;
    mma_groups<DT, KS, NG, RESIDENT_IS_KEYS, true>(pb, f, res, rg, nxt, 0);
    af = aux_of(nxt, 0);
    consume(pa, ap);
    ap = af;
    mma_groups<DT, KS, NG, RESIDENT_IS_KEYS, true>(pa, f, res, rg, nxt, 1);
    af = aux_of(nxt, 1);
    consume(pb, an);
  }
  mma_groups<DT, KS, NG, RESIDENT_IS_KEYS, false>(pb, f, res, rg, nullptr, 0);
  consume(pa, ap);
  consume(pb, af);
}

// ---------------------------------------------------------------------------------------------
// Row statistics.  Per lane and resident 16-query group the state is (mref, l) with
//   sum over the keys seen so far of 2^(s) = l * 2^mref.
// mref is a reference exponent, not the running maximum: the common path (lse_fast) adds
// 2^(s - mref) without looking for a maximum.  The sum is renormalised (lse_renorm) only when it
// leaves [1, 2^64) -- the first visible keys of a row, or a jump of the scores by more than 64
// binades -- and then exactly as the classic online softmax would (new reference = old +
// max(tile max, 0)).  Invariant after the first visible key: 1 <= l < 2^64, hence
// mref <= lse < mref + 64, so terms that underflow are below 2^-126 of the total and overflow is
// caught by the range check.
// a[sg][r] is the score of the lane's query against key 16*sg + 4*(lane/16) + r of the sub-step;
// with MASK, keys whose offset 16*sg + r exceeds lim (already reduced by 4*(lane/16)) are hidden.
template <bool MASK>
__device__ __forceinline__ float lse_fast(const f32x4 (&a)[2], float scale2, float mref, float l, int lim) {
  const float nm = -mref;
  float ln = l;  // one add per score and nothing else: the groups of a wave give the adder its parallelism
#pragma unroll
  for (int sg = 0; sg < 2; ++sg)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float x = fmaf(a[sg][r], scale2, nm);
      if (MASK) x = (16 * sg + r <= lim) ? x : kNegInf;
      ln += fast_exp2(x);
    }
  return ln;
}

__device__ __forceinline__ bool lse_in_range(float l) { return (l >= 1.0f) && (l < 1.8446744e19f); }

template <bool MASK>
__device__ __forceinline__ void lse_renorm(const f32x4 (&a)[2], float scale2, float& mref, float& l, int lim) {
  const float nm = -mref;
  float t[8];
#pragma unroll
  for (int sg = 0; sg < 2; ++sg)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float x = fmaf(a[sg][r], scale2, nm);
      if (MASK) x = (16 * sg + r <= lim) ? x : kNegInf;
      t[sg * 4 + r] = x;
    }
  float tmax = t[0];
#pragma unroll
  for (int i = 1; i < 8; ++i) tmax = fmaxf(tmax, t[i]);
  // Nothing seen yet: the tile maximum becomes the reference (it may be far below zero, so the
  // empty sum must not be scaled: 0 * 2^(+big) is not a number).  Otherwise only ever move up.
  const bool empty = (l == 0.f);
  const float delta = empty ? ((tmax > kNegInf) ? tmax : 0.f) : fmaxf(tmax, 0.f);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) s += fast_exp2(t[i] - delta);
  l = empty ? s : l * fast_exp2(-delta) + s;
  mref += delta;
}

template <bool MASK>
__device__ __forceinline__ void lse_update(const f32x4 (&a)[2], float scale2, float& mref, float& l, int lim) {
  const float ln = lse_fast<MASK>(a, scale2, mref, l, lim);
  if (__builtin_amdgcn_ballot_w64(!lse_in_range(ln)) == 0) l = ln;
  else lse_renorm<MASK>(a, scale2, mref, l, lim);
}

// All groups of a fully visible sub-step; one rarely taken branch at the very end so that the
// arithmetic above it can be scheduled against the MFMAs of the next sub-step.
template <int NG>
__device__ __forceinline__ void lse_update_groups(const f32x4 (&a)[NG][2], float scale2, float (&mref)[NG],
                                                  float (&l)[NG]) {
  float ln[NG];
#pragma unroll
  for (int g = 0; g < NG; ++g) ln[g] = lse_fast<false>(a[g], scale2, mref[g], l[g], 0);
  // one range check for all groups, on the smallest and the largest sum (NaN scores stay NaN on
  // either path, so they need no test of their own)
  float lo = ln[0], hi = ln[0];
#pragma unroll
  for (int g = 1; g < NG; ++g) {
    lo = fminf(lo, ln[g]);
    hi = fmaxf(hi, ln[g]);
  }
  const bool ok = (lo >= 1.0f) && (hi < 1.8446744e19f);
  if (__builtin_amdgcn_ballot_w64(!ok) == 0) {
#pragma unroll
    for (int g = 0; g < NG; ++g) l[g] = ln[g];
  } else {
#pragma unroll
    for (int g = 0; g < NG; ++g) lse_renorm<false>(a[g], scale2, mref[g], l[g], 0);
  }
}

// log2(2^a + 2^b); a NaN in either (a row with a NaN or +inf score) stays a NaN: fmaxf / fminf alone
// would drop it.
__device__ __forceinline__ float lse_merge(float a, float b) {
  const float hi = fmaxf(a, b), lo = fminf(a, b);
  if (a != a || b != b) return a + b;
  if (hi == kNegInf) return kNegInf;
  return hi + fast_log2(1.0f + fast_exp2(lo - hi));
}

struct NoAux {};

// STREAM_ONCE: the launch has one row tile per (b,h), so every key is read by exactly one workgroup,
// and so many keys that none of them survives in a cache until the column kernel: they are loaded
// non-temporally (7.0 instead of 6.2 TB/s on 34 GB of keys).  With several row tiles, or few keys, the
// default policy is the faster one.
template <int DT, int KS, bool CAUSAL, int NB, bool STREAM_ONCE>
__global__ __launch_bounds__(kThreads, (KS > 8 ? 1 : 2)) void row_lse_kernel(const Params p) {
  using Rg = Ring<KS>;
  constexpr int NG = 2 * NB;
  constexpr int kTileRows = kWaves * 32 * NB;
  __shared__ __attribute__((aligned(1024))) char smem[Rg::kBytes];
  int bh, tile, split;
  map_block_split(p, CAUSAL, bh, tile, split);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, keeps the row views scalar
  const int b = bh / p.H, h = bh - b * p.H;
  const char* qb = p.q + (int64_t)b * p.q_sb + (int64_t)h * p.q_sh;
  const char* kb = p.k + (int64_t)b * p.k_sb + (int64_t)h * p.k_sh;

  int q0[NG];  // first query of each of this wave's groups
  wave_groups<NB>(tile, wave, q0);

  // Keys [0, kend) matter to this workgroup.  Chunks [0, t_int) are seen in full by every one of
  // its queries and lie inside [0, N): they take the branch-free pipelined sweep.  The rest (the
  // causal diagonal, the ragged tail) take the general loop.
  // With splits > 1 this workgroup only sweeps chunks [c_begin, c_end) of that range and writes a
  // partial lse; lse_combine_kernel merges the partials.
  const int kend = CAUSAL ? min(p.N, tile * kTileRows + kTileRows + p.c) : p.N;
  const int per_split = ((p.N + kChunk - 1) / kChunk + p.splits - 1) / p.splits;
  const int c_begin = split * per_split;
  const int nchunks = min((kend + kChunk - 1) / kChunk, c_begin + per_split);
  const int t_int = min(nchunks, CAUSAL ? min((tile * kTileRows + p.c + 1) / kChunk, p.N / kChunk) : p.N / kChunk);
  const int keys_end = min(p.N, nchunks * kChunk);   // nothing is fetched from here on

  float mref[NG], l[NG];
  int last[NG];  // last key a lane's query may see, minus the lane's row offset in a group
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    mref[g] = 0.f;
    l[g] = 0.f;
    const int i = q0[g] + (lane & 15);
    last[g] = (CAUSAL ? min(p.N - 1, i + p.c) : p.N - 1) - 4 * (lane >> 4);
  }

  Rg rg;
  rg.init(p.k_sr, p.dgran, lane, wave);
  auto stage_of = [&](int t) { return smem + ((uint32_t)t % Rg::kN) * Rg::kStage; };
  rg.start(kb, p.k_sr, c_begin * kChunk, keys_end);
  auto issue = [&](int t) { rg.template issue_next<(STREAM_ONCE ? kLoadOnce : 0)>(stage_of(t)); };
  auto advance = [&](int t) {
    ring_sync<(Rg::kN - 2) * Rg::kPer>();
    issue(t + Rg::kN - 1);
  };
  // The first chunks of the streamed operand are requested before the resident one, so that all of
  // them are in flight together.
#pragma unroll
  for (int i = 0; i < Rg::kN - 1; ++i) issue(c_begin + i);

  // A wave whose rows all lie past M (a ragged last tile, fewer than 128 queries) only helps staging.
  if (q0[0] >= p.M) {
    for (int t = c_begin; t < nchunks; ++t) advance(t);
    ring_sync<0>();
    return;
  }
  u32x4 qf[NG][KS];
  load_resident<KS, NG>(qf, qb, p.q_sr, q0, p.M, p.dgran, lane);

  pipelined_sweep<DT, KS, NG, false, NoAux>(
      c_begin, t_int, qf, rg, advance, stage_of, [](const char*, int) { return NoAux{}; },
      [&](const f32x4(&a)[NG][2], NoAux) { lse_update_groups<NG>(a, p.scale2, mref, l); });

  for (int t = max(t_int, c_begin); t < nchunks; ++t) {
    advance(t);
    const char* lds = stage_of(t);
#pragma unroll
    for (int sub = 0; sub < kChunk / 32; ++sub) {
      const int key0 = t * kChunk + sub * 32;
      if (key0 >= p.N) continue;
      // the sub-step's fragments once, for all groups that see it
      u32x4 kf[2][KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        kf[0][ks] = rg.frag(lds, sub, 0, ks);
        kf[1][ks] = rg.frag(lds, sub, 1, ks);
      }
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const int qg = q0[g];
        if (CAUSAL && key0 > qg + 15 + p.c) continue;  // no query of the group sees this sub-tile
        f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          acc[0] = mma<DT>(kf[0][ks], qf[g][ks], acc[0]);
          acc[1] = mma<DT>(kf[1][ks], qf[g][ks], acc[1]);
        }
        const bool need_mask = (key0 + 32 > p.N) || (CAUSAL && key0 + 31 > qg + p.c);
        if (need_mask) lse_update<true>(acc, p.scale2, mref[g], l[g], last[g] - key0);
        else lse_update<false>(acc, p.scale2, mref[g], l[g], 0);
      }
    }
  }
  ring_sync<0>();   // the loads past the last chunk write their zeros before the LDS is given back

#pragma unroll
  for (int g = 0; g < NG; ++g) {
    float v = (l[g] == 0.f) ? kNegInf : mref[g] + fast_log2(l[g]);   // l is positive, zero (no key seen) or NaN
    v = lse_merge(v, __shfl_xor(v, 16));  // the four lane groups hold different keys of the same query
    v = lse_merge(v, __shfl_xor(v, 32));
    const int i = q0[g] + lane;
    float* dst = (p.splits > 1) ? p.part + (int64_t)split * p.bh_count * p.M : p.lse;
    if (lane < 16 && i < p.M) dst[(int64_t)bh * p.M + i] = v;
  }
}

// lse[r] = log2 sum_s 2^part[s][r] over the key ranges of a split row sweep.  One thread per row; the
// partials are fetched eight at a time (independent loads: a round trip to memory per batch, not per
// value) and folded into a running (maximum, sum); a NaN partial makes the result NaN.
__global__ __launch_bounds__(256) void lse_combine_kernel(const float* __restrict__ part, float* __restrict__ lse,
                                                          int64_t rows, int splits) {
  const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (r >= rows) return;
  float m = kNegInf, acc = 0.f;
  bool nan = false;   // fmaxf drops a NaN partial
  for (int s0 = 0; s0 < splits; s0 += 8) {
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (s0 + i < splits) ? part[(int64_t)(s0 + i) * rows + r] : kNegInf;
    float bm = v[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) bm = fmaxf(bm, v[i]);
#pragma unroll
    for (int i = 0; i < 8; ++i) nan = nan || (v[i] != v[i]);
    const float nm = fmaxf(m, bm);
    if (nm > kNegInf) {
      acc *= fast_exp2(m - nm);   // m = -inf: acc is 0 and stays 0
#pragma unroll
      for (int i = 0; i < 8; ++i) acc += fast_exp2(v[i] - nm);
      m = nm;
    }
  }
  lse[r] = nan ? __builtin_nanf("") : ((m > kNegInf) ? m + fast_log2(acc) : kNegInf);
}

// ---------------------------------------------------------------------------------------------
// What a column sweep produces.
constexpr int kModeSum = 0, kModeMax = 1, kModeBoth = 2;

// a[sg][r] is the score of key 4*(lane/16) + r of a resident group against the lane's query in
// streamed group sg, whose lse is lse2[sg].  x = s*scale2 - lse is the base-2 log of the probability.
// Sums add 2^x; maxima track x itself and exponentiate once at the end of the sweep (2^x is monotone),
// so a max-only sweep has no exp.  With MASK, register r of group sg is hidden when r > lim + 16*sg.
template <bool MASK, int MODE>
__device__ __forceinline__ void col_update(const f32x4 (&a)[2], float scale2, const float (&lse2)[2], f32x4& csum,
                                           f32x4& cmax, int lim) {
#pragma unroll
  for (int sg = 0; sg < 2; ++sg)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float x = fmaf(a[sg][r], scale2, -lse2[sg]);
      if (MASK) x = (r <= lim + 16 * sg) ? x : kNegInf;
      if (MODE != kModeSum) cmax[r] = fmaxf(cmax[r], x);
      if (MODE != kModeMax) csum[r] += fast_exp2(x);
    }
}

struct LsePair {
  float v[2];
};

// MODE both keeps two sets of column registers, so a wave then holds one block of keys instead of two.
__host__ __device__ constexpr int col_blocks_per_wave(int ksteps, int mode) {
  return mode == kModeBoth ? 1 : blocks_per_wave(ksteps);
}
// Blocks per wave the host asks for.  Strictly between one and two workgroups of 256 keys per CU
// leave CUs unevenly loaded, and with the mask one or two per CU are too coarse as well (the chip
// waits for the longest sweep): those launches use 128-key tiles.
inline int col_tile_blocks(int ksteps, int mode, int N, int64_t bh, bool causal) {
  const int nb = col_blocks_per_wave(ksteps, mode);
  if (nb != 2) return nb;
  const int64_t wgs2 = bh * ((N + kWaves * 64 - 1) / (kWaves * 64));
  const int cus = chip_cus();
  // two-block tiles only when they still give two workgroups per CU; with fewer, CUs idle or run a single
  // workgroup (32 heads of 1024 x 1024: the call takes 37 us with 128 two-block tiles, 32 us with 256 one-block tiles)
  // (without the mask one workgroup on most CUs does better with two blocks: 16 heads of 4096 x 4096 76 -> 66 us)
  if (causal) return wgs2 <= 2 * cus ? 1 : 2;
  if (wgs2 <= cus) return 2 * wgs2 > cus ? 2 : 1;
  return wgs2 < 2 * cus ? 1 : 2;
}

template <int DT, int KS, bool CAUSAL, int MODE, int NB>
__global__ __launch_bounds__(kThreads, ((NB > 2 || KS > 8) ? 1 : 2)) void col_reduce_kernel(const Params p) {
  using Rg = Ring<KS>;
  constexpr int NG = 2 * NB;
  constexpr int kTileRows = kWaves * 32 * NB;
  constexpr int kRed = kWaves * NG * 4 * 64 * 4;      // end-of-sweep transpose buffer
  constexpr int kSmem = (Rg::kBytes > kRed) ? Rg::kBytes : kRed;
  __shared__ __attribute__((aligned(1024))) char smem[kSmem];
  int bh, tile;
  map_block(p, false, bh, tile);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, keeps the row views scalar
  const int b = bh / p.H, h = bh - b * p.H;
  const char* qb = p.q + (int64_t)b * p.q_sb + (int64_t)h * p.q_sh;
  const char* kb = p.k + (int64_t)b * p.k_sb + (int64_t)h * p.k_sh;
  const float* lse = p.lse + (int64_t)bh * p.M;

  int k0[NG];  // first key of each of this wave's groups
  wave_groups<NB>(tile, wave, k0);

  f32x4 csum[NG], cmax[NG];  // the set a MODE does not use is never touched and costs no registers
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    csum[g] = (f32x4){0.f, 0.f, 0.f, 0.f};
    cmax[g] = (f32x4){kNegInf, kNegInf, kNegInf, kNegInf};
  }

  // Query chunks [t0, nchunks) can see keys of this tile.  Chunks [t_int, nfull) are whole chunks whose
  // queries all see every key of the tile: they take the branch-free pipelined sweep (keys past N are
  // computed and never stored, so they need no mask).  The chunks on the causal diagonal before them
  // and a ragged last chunk (rows past M read as zeros, their lse too) take the general loop.
  const int nchunks = (p.M + kChunk - 1) / kChunk;
  const int t0 = CAUSAL ? max(0, tile * kTileRows - p.c) / kChunk : 0;
  const int nfull = max(t0, p.M / kChunk);
  const int t_int = CAUSAL ? min(nfull, max(t0, (tile * kTileRows + kTileRows - 1 - p.c + kChunk - 1) / kChunk)) : 0;
  // lim = i + c - key0(group) - 4*(lane/16), with i the lane's query in group 0 of the current sub-tile
  const int lim_lane = (lane & 15) + p.c - 4 * (lane >> 4);

  // A stage is kChunk query rows plus their lse.
  Rg rg;
  rg.init(p.q_sr, p.dgran, lane, wave);
  auto stage_of = [&](int t) { return smem + ((uint32_t)t % Rg::kN) * Rg::kStage; };
  rg.start(qb, p.q_sr, t0 * kChunk, p.M);
  const float* lse_next = lse + t0 * kChunk;   // walks along with the ring's cursor
  auto issue = [&](int t) {
    char* stage = stage_of(t);
    const int live = rows_in_chunk(rg.rows_left);
    rg.issue_next(stage);
    const __amdgpu_buffer_rsrc_t view = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(lse_next), 0, live * 4, 0x00020000);
    dma4(view, (uint32_t)lane * 4u, stage + Rg::kRows);   // every wave writes the same 64 values: no branch
    lse_next += kChunk;
  };
  auto advance = [&](int t) {
    ring_sync<(Rg::kN - 2) * (Rg::kPer + 1)>();
    issue(t + Rg::kN - 1);
  };
  auto aux_of = [&](const char* lds, int sub) {
    const float* v = reinterpret_cast<const float*>(lds + Rg::kRows) + sub * 32 + (lane & 15);
    return LsePair{{v[0], v[16]}};
  };
  // The first chunks of the streamed operand are requested before the resident one, so that all of
  // them are in flight together.
#pragma unroll
  for (int i = 0; i < Rg::kN - 1; ++i) issue(t0 + i);
  u32x4 kf[NG][KS];
  load_resident<KS, NG>(kf, kb, p.k_sr, k0, p.N, p.dgran, lane);

  auto general_chunk = [&](int t) {
    advance(t);
    const char* lds = stage_of(t);
#pragma unroll
    for (int sub = 0; sub < kChunk / 32; ++sub) {
      const int qs = t * kChunk + sub * 32;  // first query of the sub-tile
      if (qs >= p.M) continue;
      LsePair lq = aux_of(lds, sub);
      // +inf for rows past M: they contribute 2^-inf = 0
      if (qs + (lane & 15) >= p.M) lq.v[0] = kPosInf;
      if (qs + 16 + (lane & 15) >= p.M) lq.v[1] = kPosInf;
      // the sub-step's fragments once, for all groups that see it
      u32x4 qfrag[2][KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        qfrag[0][ks] = rg.frag(lds, sub, 0, ks);
        qfrag[1][ks] = rg.frag(lds, sub, 1, ks);
      }
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const int kg = k0[g];
        if (kg >= p.N) continue;
        if (CAUSAL && kg > qs + 31 + p.c) continue;  // no query of the sub-tile sees this group
        f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          acc[0] = mma<DT>(kf[g][ks], qfrag[0][ks], acc[0]);
          acc[1] = mma<DT>(kf[g][ks], qfrag[1][ks], acc[1]);
        }
        const bool need_mask = CAUSAL && (kg + 15 > qs + p.c);
        if (need_mask) col_update<true, MODE>(acc, p.scale2, lq.v, csum[g], cmax[g], lim_lane + qs - kg);
        else col_update<false, MODE>(acc, p.scale2, lq.v, csum[g], cmax[g], 0);
      }
    }
  };

  for (int t = t0; t < t_int; ++t) general_chunk(t);

  pipelined_sweep<DT, KS, NG, true, LsePair>(
      t_int, nfull, kf, rg, advance, stage_of, aux_of,
      [&](const f32x4(&a)[NG][2], const LsePair& lq) {
        // the lse values are first touched here, a sub-step after their LDS read was issued
#pragma unroll
        for (int g = 0; g < NG; ++g) col_update<false, MODE>(a[g], p.scale2, lq.v, csum[g], cmax[g], 0);
      });

  for (int t = nfull; t < nchunks; ++t) general_chunk(t);

  // Reduce over the 16 query lanes: transpose through LDS, one output key per lane and pass; a pass
  // writes out four of the wave's groups.
  float* red = reinterpret_cast<float*>(smem) + wave * (NG * 4 * 64);
  const int w = lane & 15;                 // key inside its group
  ring_sync<0>();   // every load has landed (those past the last chunk write zeros): the LDS can be reused
  if (MODE != kModeMax) {
#pragma unroll
    for (int g = 0; g < NG; ++g)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[(g * 4 + r) * 64 + lane] = csum[g][r];
    __syncthreads();
#pragma unroll
    for (int g4 = 0; g4 < NG; g4 += 4) {
      const int grp = g4 + (lane >> 4);      // which of the wave's groups this lane writes out
      if (grp < NG) {                        // lanes 32.. idle when a wave keeps two groups
        const float* src = red + (grp * 4 + (w & 3)) * 64 + (w >> 2) * 16;
        float v = 0.f;
#pragma unroll
        for (int j = 0; j < 16; ++j) v += src[(j + lane) & 15];
        const int key = k0[grp] + w;
        if (key < p.N) store_column(p, p.out, true, bh, key, v);
      }
    }
  }
  if (MODE != kModeSum) {
    if (MODE == kModeBoth) __syncthreads();
#pragma unroll
    for (int g = 0; g < NG; ++g)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[(g * 4 + r) * 64 + lane] = cmax[g][r];
    __syncthreads();
#pragma unroll
    for (int g4 = 0; g4 < NG; g4 += 4) {
      const int grp = g4 + (lane >> 4);
      if (grp < NG) {
        const float* src = red + (grp * 4 + (w & 3)) * 64 + (w >> 2) * 16;
        float v = kNegInf;
#pragma unroll
        for (int j = 0; j < 16; ++j) v = fmaxf(v, src[(j + lane) & 15]);
        const int key = k0[grp] + w;
        if (key < p.N) store_column(p, (MODE == kModeBoth) ? p.out2 : p.out, false, bh, key, fast_exp2(v));
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Column sweep for at most 128 query rows against many keys, where the sweep is bound by reading K.
// The roles are swapped: every wave keeps ALL queries resident (NG = 4 or 8 groups of 16) and the keys
// stream through LDS in chunks of 64, fully coalesced and two chunks ahead.  Wave w takes keys
// [16w, 16w+16) of each chunk with S = Q * K^T, so a lane holds one key (lane & 15) against the
// queries 16g + 4*(lane/16) + r: the column reduction is an in-register sum over g and r plus two
// cross-lane steps, and each wave stores its 16 finished columns.  Workgroup v sweeps key chunks
// [split*per, split*per + per) of one (b,h), p.splits ranges per (b,h).  Every key is read by exactly
// one workgroup; p.stream_once makes those loads non-temporal (set when K is too large to stay cached).
// The general kernel reads the same keys as MFMA fragments, 64 bytes per row and instruction, and
// reaches 4.9 TB/s where this one reaches 6 (measured on 34 GB of keys).
constexpr int kSmallRows = 128;

template <int DT, int KS, bool CAUSAL, int MODE, int NG>
__global__ __launch_bounds__(kThreads, (NG <= 4 ? 3 : 2)) void col_small_kernel(const Params p) {
  using Rg = Ring<KS, 3>;   // three workgroups share a CU: 3 x 3 stages of 16 KiB
  // Finished columns wait in obuf and go to memory kFlush chunks at a time, 1 KiB per store instruction:
  // up to 10 % faster than a 64-byte store per wave and chunk.  (What the columns cost beyond that does
  // not depend on how they are stored: 134 MB of them beside 8.6 GB of keys take 15 % of the sweep, which
  // runs at the row kernel's rate with the stores disabled.)  The ring and obuf are ONE LDS object:
  // with two, the compiler orders every read of the ring after all loads in flight.
  constexpr int kFlush = (MODE == kModeBoth) ? 8 : 16;   // 4 KiB of LDS either way
  constexpr int kObufBytes = (MODE == kModeBoth ? 2 : 1) * kFlush * kChunk * 4;
  __shared__ __attribute__((aligned(1024))) char smem[Rg::kBytes + kObufBytes];
  float* const obuf = reinterpret_cast<float*>(smem + Rg::kBytes);
  int bh, split;
  map_group(p, p.splits, bh, split);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int b = bh / p.H, h = bh - b * p.H;
  const char* qb = p.q + (int64_t)b * p.q_sb + (int64_t)h * p.q_sh;
  const char* kb = p.k + (int64_t)b * p.k_sb + (int64_t)h * p.k_sh;
  const float* lse = p.lse + (int64_t)bh * p.M;

  const int nchunks = (p.N + kChunk - 1) / kChunk;
  const int per = (nchunks + p.splits - 1) / p.splits;
  const int c0 = split * per, c1 = min(nchunks, c0 + per);
  if (c0 >= c1) return;  // the whole workgroup
  const int keys_end = min(p.N, c1 * kChunk);   // nothing is fetched from here on

  // The ring keeps two chunks of keys in flight per workgroup.
  Rg rg;
  rg.init(p.k_sr, p.dgran, lane, wave);
  const bool once = p.stream_once != 0;
  auto stage_of = [&](int t) { return smem + ((uint32_t)t % Rg::kN) * Rg::kStage; };
  rg.start(kb, p.k_sr, c0 * kChunk, keys_end);
  auto issue = [&](int t) {
    if (once) rg.template issue_next<kLoadOnce>(stage_of(t));
    else rg.template issue_next<0>(stage_of(t));
  };
#pragma unroll
  for (int i = 0; i < Rg::kN - 1; ++i) issue(c0 + i);

  // -lse of the lane's queries; -inf hides the rows past M
  const int qrow = 4 * (lane >> 4);
  float nlse[NG][4];
  int rows[NG];
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    rows[g] = 16 * g;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i = 16 * g + qrow + r;
      const float v = lse[min(i, p.M - 1)];
      nlse[g][r] = (i < p.M) ? -v : kNegInf;
    }
  }
  u32x4 qf[NG][KS];
  load_resident<KS, NG>(qf, qb, p.q_sr, rows, p.M, p.dgran, lane);

  void* const out_max = (MODE == kModeBoth) ? p.out2 : p.out;
  float* obuf_max = obuf + (MODE == kModeBoth ? kFlush * kChunk : 0);
  // Columns of chunks [ta, ta + kFlush) from obuf to memory, up to the end of this workgroup's range;
  // all waves have passed a barrier since they wrote them.
  auto flush = [&](int ta) {
    const int key0 = ta * kChunk, nkeys = keys_end - key0;
#pragma unroll
    for (int r = 0; r < kFlush * kChunk / kThreads; ++r) {
      const int i = tid + r * kThreads;
      if (i < nkeys) {
        if (MODE != kModeMax) store_column(p, p.out, true, bh, key0 + i, obuf[i]);
        if (MODE != kModeSum) store_column(p, out_max, false, bh, key0 + i, obuf_max[i]);
      }
    }
  };
  for (int t = c0; t < c1; ++t) {
    ring_sync<(Rg::kN - 2) * Rg::kPer>();   // chunk t visible, the stage of chunk t - 1 is free
    issue(t + Rg::kN - 1);
    if (t > c0 && (t - c0) % kFlush == 0) {
      flush(t - kFlush);
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();   // obuf is free again before anyone writes chunk t's columns
      asm volatile("" ::: "memory");
    }
    const char* lds = stage_of(t);
    const int key = t * kChunk + 16 * wave + (lane & 15);
    // query i sees the key iff key <= i + c; chunks that end at or before key c need no mask
    const bool need_mask = CAUSAL && (t * kChunk + kChunk - 1 > p.c);
    const int first = key - p.c - qrow;  // register (g, r) is visible iff 16g + r >= first
    float vsum = 0.f, vmax = kNegInf;
    // four query groups at a time, so that at most four accumulators are live
#pragma unroll
    for (int gb = 0; gb < NG; gb += 4) {
      f32x4 acc[4];
#pragma unroll
      for (int g = 0; g < 4; ++g) acc[g] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const u32x4 kfrag = rg.frag(lds, wave >> 1, wave & 1, ks);
#pragma unroll
        for (int g = 0; g < 4; ++g) acc[g] = mma<DT>(qf[gb + g][ks], kfrag, acc[g]);
      }
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int r2 = 0; r2 < 4; ++r2) {
          float x = fmaf(acc[g][r2], p.scale2, nlse[gb + g][r2]);
          if (need_mask) x = (16 * (gb + g) + r2 >= first) ? x : kNegInf;
          if (MODE != kModeSum) vmax = fmaxf(vmax, x);
          if (MODE != kModeMax) vsum += fast_exp2(x);
        }
    }
    // the four lane groups hold different queries of the same key
    const int slot = ((t - c0) % kFlush) * kChunk + 16 * wave + lane;
    if (MODE != kModeMax) {
      vsum += __shfl_xor(vsum, 16);
      vsum += __shfl_xor(vsum, 32);
      if (lane < 16) obuf[slot] = vsum;
    }
    if (MODE != kModeSum) {
      vmax = fmaxf(vmax, __shfl_xor(vmax, 16));
      vmax = fmaxf(vmax, __shfl_xor(vmax, 32));
      if (lane < 16) obuf_max[slot] = fast_exp2(vmax);
    }
  }
  ring_sync<0>();   // the loads past the last chunk write their zeros before the LDS is given back
  flush(c0 + (c1 - c0 - 1) / kFlush * kFlush);
}


// ---------------------------------------------------------------------------------------------
// Both sweeps in one for at most 128 query rows against many keys: the keys are read from memory ONCE.
// A team of p.splits workgroups shares a (b,h) pair; workgroup s of the team owns 16 chunks of 64 keys (8
// with more than 64 queries); a wave takes 16 keys of a chunk against 64 queries (as in col_small_kernel).
// Per pair a workgroup
//   1. streams its keys through the LDS ring and computes their scores, which STAY IN REGISTERS (16 per
//      lane and step): for column sums as 2^score, otherwise (maxima) as the scaled scores themselves;
//   2. sums 2^score per row, turns the sums into the log-sum-exp of every row over its own keys and
//      publishes the 64 or 128 values.  A sum outside [2^-60, 2^100) (scores far from zero, a row that
//      sees none of these keys, a NaN) is not trusted: the scores are then reduced the exact way, row
//      maximum first -- from the registers if they hold scores, else after a second sweep over the same
//      keys that keeps the scores;
//   3. reads the values the other workgroups of its team have published for this pair and merges them
//      into the rows' lse (every workgroup of the team does this merge for itself);
//   4. turns what it kept into probabilities (2^score * 2^-lse: one multiply-add per score), reduces them
//      down the rows and stores its columns.
// The grid is teams * splits workgroups and never more than one per CU, so every workgroup of a team is
// running when its partners wait for it; team t takes pairs t, t + teams, t + 2 teams, ..  The first keys
// of the next pair stream into the ring while a workgroup does steps 2-4, and the next pair's queries are
// staged in LDS a whole sweep ahead.  A wait is bounded: after p.spin_limit polls the workgroup gives up,
// sets the error word, stores NaN columns for that pair and goes on, so every workgroup reaches its end
// whatever happens to the others.
// Between workgroups: a partial value travels together with the number of its round as ONE 64-bit word,
// written and read with device-scope relaxed atomics (performed where every workgroup of the device
// sees them), so a word that shows the round shows the value; there is no counter, no fence and nobody
// waits for a store to complete.  The slots start at zero (a small kernel in front clears them), rounds
// count from 1, and the slots alternate between two sets by the parity of the round: a workgroup can be at
// most one round ahead of the slowest of its team.  The barriers between the steps wait for LDS only, so
// the keys in flight stay in flight.
// Registers are the limit (128 for the scores, 64 for the queries during step 1): what depends on the
// thread is derived again after step 1 from opaque copies instead of being kept across it.
// chunks of 64 keys per workgroup and pair: 16 for up to 64 queries, 8 for up to 128; 32 when a wave holds two
// groups of sixteen queries (nq) instead of four
__host__ __device__ constexpr int fused_chunks(int qh, int nq = 4) { return qh == 1 ? 16 * (4 / nq) : 8; }
constexpr int kFusedSteps = 8;
constexpr int kFusedThreads = 512;

template <int CTRL>
__device__ __forceinline__ float dpp_row(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// Sum or maximum over each row of 16 lanes; every lane of the row ends up with the result.
template <bool MAX>
__device__ __forceinline__ float row16_reduce(float v) {
  float o = dpp_row<0xB1>(v);    // quad_perm [1,0,3,2]
  v = MAX ? fmaxf(v, o) : v + o;
  o = dpp_row<0x4E>(v);          // quad_perm [2,3,0,1]
  v = MAX ? fmaxf(v, o) : v + o;
  o = dpp_row<0x141>(v);         // row_half_mirror
  v = MAX ? fmaxf(v, o) : v + o;
  o = dpp_row<0x140>(v);         // row_mirror
  v = MAX ? fmaxf(v, o) : v + o;
  return v;
}

// All LDS accesses of this wave done, then the workgroup's barrier.  Loads and stores to memory stay in flight.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt((15) | (3 << 14) | (7 << 4) | (0 << 8));   // vmcnt(63) expcnt(7) lgkmcnt(0)
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

__global__ __launch_bounds__(256) void zero_words_kernel(unsigned* __restrict__ w, int n) {
  const int i = (int)blockIdx.x * 256 + (int)threadIdx.x;
  if (i < n) w[i] = 0u;
}

// Eight waves, one workgroup per CU, eight steps per workgroup and pair.  Up to 64 queries (QH = 1, KH = 2):
// a step is two chunks of 64 keys, waves 0-3 take (and load) the first, waves 4-7 the second.  Up to 128
// queries (QH = 2, KH = 1): a step is one chunk, waves 4-7 hold queries 64-127, waves 0-3 load.
// NQ: groups of sixteen queries a wave holds (4; 2 for at most 32 queries: the registers then hold the scores of
// twice as many keys per pair, and the time between two sweeps is spread over that many.  One group and four
// times the keys was built as well and was slower than two: 1568 against 1499 us on 64 x 32 pairs of 16384 keys).
template <int DT, int KS, bool CAUSAL, int MODE, int QH, int NQ = 4>
__global__ __launch_bounds__(kFusedThreads, 2) void col_fused_kernel(const Params p) {
  static_assert(NQ == 4 || (QH == 1 && NQ == 2), "fewer query groups only with one query half");
  constexpr int KG = kFusedSteps * (4 / NQ);     // steps per pair
  constexpr int KH = 3 - QH;                     // chunks per step
  constexpr int NS = (QH == 1) ? 8 : 6;          // ring stages (chunks): 130 KiB or 98 KiB for 256-byte rows
  using Rg = Ring<KS, NS>;                       // four loads of 1 KiB per loading wave and chunk for 256-byte rows
  constexpr int kQBytes = QH * Rg::kRows;        // the queries of a pair, staged like a chunk of keys per 64 rows
  constexpr int kNumThreads = kFusedThreads;
  constexpr int kRowsWg = 16 * NQ * QH;          // query rows a workgroup holds
  constexpr int kItemKeys = KG * KH * kChunk;    // keys of a workgroup per pair
  constexpr int kBatchKeys = kFusedSteps * KH * kChunk;   // finished columns leave eight steps at a time
  constexpr int kBatches = KG / kFusedSteps;
  constexpr int kRes = (MODE == kModeBoth) ? 2 : 1;
  constexpr int kObufFloats = QH * kRes * kBatchKeys;
  constexpr int kRedFloats = 8 * 64;
  // waves per row that share the merge of the team's partial values (half of them when two results are
  // buffered for 1024 keys: the LDS is full)
  constexpr int kMergeWaves = (8 / QH) / ((kRes == 2 && QH == 1) ? 2 : 1);
  constexpr int kBatch = 4 * QH;                 // slots a lane fetches together: one round trip for teams of up to 32
  constexpr int kMrgFloats = kMergeWaves * kRowsWg * 2;
  constexpr int kAhead = NS / KH - 1;            // steps in flight in front of the one being computed
  constexpr int kInFlight = (NS / KH - 2) * Rg::kPer;   // loads a loading wave may have outstanding when a step starts
  // (one LDS object: see col_small_kernel)
  // one LDS object: ring | queries | finished columns | per-wave row partials | merge | per-row values | flags
  __shared__ __attribute__((aligned(1024))) char smem[Rg::kBytes + kQBytes + (kObufFloats + kRedFloats + kMrgFloats + kRowsWg + 4) * 4];
  char* const qlds = smem + Rg::kBytes;
  float* const obuf = reinterpret_cast<float*>(smem + Rg::kBytes + kQBytes);
  float* const red = obuf + kObufFloats;
  float* const mrg = red + kRedFloats;
  float* const rowv = mrg + kMrgFloats;
  int* const flag = reinterpret_cast<int*>(rowv + kRowsWg);

  const int tid0 = threadIdx.x, lane0 = tid0 & 63;   // (the loop over the pairs has its own copies, see there)
  const int wave = __builtin_amdgcn_readfirstlane(tid0 >> 6);
  const int qh = (QH == 2) ? (wave >> 2) : 0;    // which 64 queries
  const int kh = (KH == 2) ? (wave >> 2) : 0;    // which chunk of a step
  const int wq = wave & 3;                       // which 16 keys of the chunk
  const bool loader = (KH == 2) || (wave < 4);
  const int S = p.splits, T = p.teams;
  const int team = (int)blockIdx.x / S, split = (int)blockIdx.x - team * S;
  const int c0 = split * (KG * KH);              // first chunk of this workgroup's keys
  const int key0 = c0 * kChunk;
  const int keys_end = min(p.N, key0 + kItemKeys);
  const int rounds = (p.bh_count - team + T - 1) / T;
  const int qrow0 = 4 * (lane0 >> 4);
  int spin_limit = p.spin_limit;
  // flag[0]: a row of this workgroup has a sum that must be redone; flag[1]: the team was met.  Each is
  // written and read on different sides of a barrier.
  if (tid0 == 0) flag[0] = 0;

  Rg rg;
  rg.init(p.k_sr, p.dgran, lane0, 0);   // (for the fragment offsets; the loads are issued below)
  const bool once = p.stream_once != 0;
  auto stage_of = [&](int c) { return smem + ((uint32_t)c % NS) * Rg::kStage; };   // NS is a power of two
  // The loaders walk the workgroup's stream of chunks with a running address: KG * KH chunks of one pair,
  // then the same range of keys of the next pair of the team.  Chunk number c goes to stage c % NS.
  const int64_t chunk_bytes = (int64_t)kChunk * p.k_sr;
  const char* run_ptr = nullptr;
  int run_rows = 0, run_chunk = 0;
  auto run_to_pair = [&](int bh) {               // the cursor to the start of this workgroup's keys of pair bh
    const int bhc = min(bh, p.bh_count - 1);
    const int b = bhc / p.H, h = bhc - b * p.H;
    run_ptr = p.k + (int64_t)b * p.k_sb + (int64_t)h * p.k_sh + (int64_t)key0 * p.k_sr;
    run_rows = (bh < p.bh_count) ? keys_end - key0 : 0;   // past the last pair: zeros, nothing is fetched
  };
  // Where a lane's 16 bytes of each load come from (see Ring::init).  The swizzle repeats every eight rows,
  // so the kPer loads of a wave have at most kPat different patterns and the rest follow by adding rows.
  constexpr int kPat = (Rg::kRowsPerLoad >= 8) ? 1 : 8 / Rg::kRowsPerLoad;
  const int lw = wave & 3;                         // which of the loading waves
  uint32_t src_off[kPat];
  bool src_ok[kPat];
#pragma unroll
  for (int e = 0; e < kPat; ++e) {
    const int byte = (lw * Rg::kPer + e) * 1024 + lane0 * 16;
    const int row = byte / Rg::kPitch;
    const int c = ((byte % Rg::kPitch) / 16) ^ Rg::swz(row);
    src_ok[e] = c < p.dgran;
    src_off[e] = (uint32_t)row * (uint32_t)p.k_sr + (uint32_t)c * 16u;
  }
  const uint32_t pat_bytes = (uint32_t)(kPat * Rg::kRowsPerLoad) * (uint32_t)p.k_sr;
  auto issue_step = [&]() {   // the wave's chunk of the next step
    char* stage = stage_of(run_chunk + kh);
    const char* src = run_ptr + (KH == 2 && kh ? chunk_bytes : 0);
    const int live = rows_in_chunk(run_rows - kh * kChunk);
    run_chunk += KH;        // (every wave keeps the cursor, only the loading ones issue)
    run_ptr += KH * chunk_bytes;
    run_rows -= KH * kChunk;
    if (!loader) return;
    const __amdgpu_buffer_rsrc_t view = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(src), 0, (int)((uint32_t)live * (uint32_t)p.k_sr), 0x00020000);
    uint32_t so[kPat];   // opaque copies: the kPer offsets are made per call, not kept in registers between calls
#pragma unroll
    for (int e = 0; e < kPat; ++e) {
      so[e] = src_off[e];
      asm volatile("" : "+v"(so[e]));
    }
    if (once) {
#pragma unroll
      for (int i = 0; i < Rg::kPer; ++i) {
        const uint32_t off = src_ok[i % kPat] ? so[i % kPat] + (uint32_t)(i / kPat) * pat_bytes : kPastEnd;
        dma16<kLoadOnce>(view, off, stage + (lw * Rg::kPer + i) * 1024);
      }
    } else {
#pragma unroll
      for (int i = 0; i < Rg::kPer; ++i) {
        const uint32_t off = src_ok[i % kPat] ? so[i % kPat] + (uint32_t)(i / kPat) * pat_bytes : kPastEnd;
        dma16<0>(view, off, stage + (lw * Rg::kPer + i) * 1024);
      }
    }
  };
  int cons_chunk = 0;       // number of the next chunk to be computed (its stage: cons_chunk % NS)

  u32x4 qf[NQ][KS];
  // The queries of a pair go from memory to LDS like a chunk of keys (64 rows per stage-like tile, same
  // swizzle), long before they are needed, and from there into the registers when the pair's sweep starts:
  // no wave ever waits for them, and they take no registers between two sweeps.  Waves 0-3 load.
  auto stage_queries = [&](int bh) {
    if (wave >= 4) return;
    const int b = bh / p.H, h = bh - b * p.H;
    const char* qb = p.q + (int64_t)b * p.q_sb + (int64_t)h * p.q_sh;
#pragma unroll
    for (int t = 0; t < QH; ++t) {
      const int live = rows_in_chunk(p.M - 64 * t);
      const __amdgpu_buffer_rsrc_t view = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<char*>(qb + (int64_t)(64 * t) * p.q_sr), 0, (int)((uint32_t)live * (uint32_t)p.q_sr), 0x00020000);
#pragma unroll
      for (int i = 0; i < Rg::kPer; ++i) {
        const int byte = (lw * Rg::kPer + i) * 1024 + lane0 * 16;
        const int row = byte / Rg::kPitch;
        const int c = ((byte % Rg::kPitch) / 16) ^ Rg::swz(row);
        const uint32_t off = (c < p.dgran) ? (uint32_t)row * (uint32_t)p.q_sr + (uint32_t)c * 16u : kPastEnd;
        dma16<0>(view, off, qlds + t * Rg::kRows + (lw * Rg::kPer + i) * 1024);
      }
    }
  };
  auto read_queries = [&]() {
#pragma unroll
    for (int g = 0; g < NQ; ++g)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) qf[g][ks] = rg.frag(qlds + qh * Rg::kRows, g >> 1, g & 1, ks);
  };
  // the first pair's queries, then the first steps of its keys: the loads return in this order, so the
  // wait in front of the first step covers the queries
  stage_queries(team);
  run_to_pair(team);
#pragma unroll
  for (int i = 0; i < kAhead; ++i) issue_step();

  // Register (g, r) of a lane is query 64*qh + 16g + qrow + r against the lane's key.  It takes part iff
  // the query exists and may see the key: 16g + r in [first, mlim).
  const int mlim0 = p.M - 64 * qh - qrow0;
  const bool ragged_rows = p.M < 16 * NQ * (qh + 1);
  constexpr int kRowWaves = 8 / QH;   // row tid (tid < kRowsWg) is held by all eight waves, or by 0-3 / 4-7 for rows below / from 64

  for (int it = 0; it < rounds; ++it) {
    const int bh = team + it * T;
    // What the registers keep per score: for column sums 2^score (step 4 is then one multiply-add per score),
    // otherwise, or when a row's sum of 2^score is unusable, the score itself.  In the second case of a sum
    // the scores are gone by the time it shows, and the keys of the pair are streamed once more.
    f32x4 sc[KG][NQ];
    f32x4 rs[NQ];   // per row (register) and key (lane): sum of 2^score over the steps
    float my_lse = kNegInf;   // of row tid over this workgroup's keys, for tid < kRowsWg
    // Steps 1 and the first half of 2, in two forms (KEEP: the registers end up holding the scores).  Returns
    // whether some row's sum of 2^score is unusable.
    auto sweep = [&](auto keep_tag) -> bool {
    constexpr bool KEEP = decltype(keep_tag)::value;
    if (KEEP) {
#pragma unroll
      for (int g = 0; g < NQ; ++g) rs[g] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }
    {
    const int tid = tid0, lane = lane0, qrow = qrow0, mlim = mlim0;
    // 1. scores of this workgroup's keys, scaled, hidden ones at -inf
    // (what the mask needs is derived afresh from an opaque copy of c0 here and in step 4: kept across the
    // steps, or hoisted out of the loop over the pairs, it would cost registers that the scores need)
    int c0a = c0;
    asm volatile("" : "+s"(c0a));
#pragma unroll
    for (int j = 0; j < KG; ++j) {
      ring_sync<kInFlight>();   // the chunks of this step are visible, the stages of the step before are free
      if (j + kAhead == KG) run_to_pair(bh + T);   // the steps from here on belong to the next pair
      issue_step();
      if (j == 0) read_queries();   // (staged at least a whole sweep ago; the barrier above has published them)
      if (j == 1 && it + 1 < rounds) stage_queries(bh + T);   // every wave has read this pair's by now
      const char* lds = stage_of(cons_chunk + j * KH + kh);
#pragma unroll
      for (int g = 0; g < NQ; ++g) sc[j][g] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const u32x4 kfrag = rg.frag(lds, wq >> 1, wq & 1, ks);
#pragma unroll
        for (int g = 0; g < NQ; ++g) sc[j][g] = mma<DT>(qf[g][ks], kfrag, sc[j][g]);
      }
      const int kbase = (c0a + j * KH + kh) * kChunk;
      const int key = kbase + 16 * wq + (lane & 15);
      // Rows past M are rows of zeros: their scores are 0 and their 2^score is 1, which nothing downstream uses
      // (their factor in step 4 is 0), so the fast form of the sweep does not hide them.  Only a key with a
      // non-finite element makes them NaN; the row threads below look for that and ask for the second sweep,
      // which hides them as every sweep that keeps scores does.
      const bool need_mask = (KEEP && ragged_rows) || kbase + kChunk > p.N || (CAUSAL && kbase + kChunk - 1 > p.c + 64 * qh);
      if (need_mask) {
        int first = CAUSAL ? key - p.c - 64 * qh - qrow : -(1 << 30);
        if (key >= p.N) first = 1 << 30;
#pragma unroll
        for (int g = 0; g < NQ; ++g)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int o = 16 * g + r;
            sc[j][g][r] = (o >= first && o < mlim) ? sc[j][g][r] * p.scale2 : kNegInf;
          }
      } else {
#pragma unroll
        for (int g = 0; g < NQ; ++g) sc[j][g] *= p.scale2;
      }
      if (KEEP) {
#pragma unroll
        for (int g = 0; g < NQ; ++g)
#pragma unroll
          for (int r = 0; r < 4; ++r) rs[g][r] += fast_exp2(sc[j][g][r]);
      } else {   // (the row sums are taken after the loop: sixteen registers less while the queries are held)
#pragma unroll
        for (int g = 0; g < NQ; ++g)
#pragma unroll
          for (int r = 0; r < 4; ++r) sc[j][g][r] = fast_exp2(sc[j][g][r]);
      }
    }
    cons_chunk += KG * KH;
    }
    if (!KEEP) {
#pragma unroll
      for (int g = 0; g < NQ; ++g) {
        rs[g] = sc[0][g];
#pragma unroll
        for (int j = 1; j < KG; ++j) rs[g] += sc[j][g];
      }
    }
    // From here on, everything that depends on the thread is derived afresh from an opaque copy of its
    // number: values kept for these steps across step 1 would take registers from the scores (and come
    // back from scratch memory, a round trip each).
    int tid_again = threadIdx.x;
    asm volatile("" : "+v"(tid_again));
    const int tid = tid_again, lane = tid & 63, qrow = 4 * (lane >> 4);
    const float* const red_row = red + (QH == 2 ? (tid >> 6) * (kWaves * 64) : 0) + (tid & 63);

    // 2. log-sum-exp of every row over this workgroup's keys.  The sums of 2^x were taken as the scores
    // came; they are good unless a sum left fp32's comfortable range (or a row saw no key at all), and then
    // the scores, still in registers, are reduced again the exact way: row maximum first.
#pragma unroll
    for (int g = 0; g < NQ; ++g) {
#pragma unroll
      for (int r = 0; r < 4; ++r) rs[g][r] = row16_reduce<false>(rs[g][r]);
      if ((lane & 15) == 0) *reinterpret_cast<f32x4*>(red + wave * 64 + 16 * g + qrow) = rs[g];
    }
    lds_barrier();
    if (tid < kRowsWg) {
      float l = 0.f;
#pragma unroll
      for (int w = 0; w < kRowWaves; ++w) l += red_row[64 * w];
      my_lse = fast_log2(l);
      // 2^-60 <= l < 2^100: terms flushed to zero are far below the sum's last bit, and 2^score times 2^-lse
      // (the lse of all keys is at least this one) neither overflows nor loses anything above 2^-26
      const bool good = (l >= 8.6736174e-19f) && (l < 1.2676506e30f);
      if (!good && tid < p.M) flag[0] = 1;   // (written by whoever finds a bad row; thread 0 resets it below)
      if (!KEEP && tid >= p.M && !(l < kPosInf)) flag[0] = 1;   // a row of zeros met a non-finite key
      if (tid == 0) flag[1] = 1;
    }
    lds_barrier();
    return flag[0] != 0;   // uniform over the workgroup
    };   // sweep
    bool keep_scores = (MODE != kModeSum);
    bool bad_sum;
    if (MODE == kModeSum) {
      bad_sum = sweep(std::false_type());
      if (bad_sum) {
        // once more through the keys of this pair: the loads in flight (for the next pair) land and are
        // dropped, the loader goes back to this pair's first chunk and the ring starts afresh
        ring_sync<0>();
        if (tid0 == 0) flag[0] = 0;
        stage_queries(bh);   // (the sweep above has already replaced them by the next pair's)
        run_to_pair(bh);
        cons_chunk = run_chunk;
#pragma unroll
        for (int i = 0; i < kAhead; ++i) issue_step();
        keep_scores = true;
        bad_sum = sweep(std::true_type());
      }
    } else {
      bad_sum = sweep(std::true_type());
    }
    int tid_once_more = threadIdx.x;
    asm volatile("" : "+v"(tid_once_more));
    const int tid = tid_once_more, lane = tid & 63, qrow = 4 * (lane >> 4);
    const int mlim = p.M - 64 * qh - qrow;
    const float* const red_row = red + (QH == 2 ? (tid >> 6) * (kWaves * 64) : 0) + (tid & 63);
    if (bad_sum) {
      f32x4 rm[NQ];
#pragma unroll
      for (int g = 0; g < NQ; ++g) {
        rm[g] = sc[0][g];
#pragma unroll
        for (int j = 1; j < KG; ++j)
#pragma unroll
          for (int r = 0; r < 4; ++r) rm[g][r] = fmaxf(rm[g][r], sc[j][g][r]);
#pragma unroll
        for (int r = 0; r < 4; ++r) rm[g][r] = row16_reduce<true>(rm[g][r]);
        if ((lane & 15) == 0) *reinterpret_cast<f32x4*>(red + wave * 64 + 16 * g + qrow) = rm[g];
      }
      lds_barrier();
      float my_max = kNegInf;
      if (tid < kRowsWg) {
#pragma unroll
        for (int w = 0; w < kRowWaves; ++w) my_max = fmaxf(my_max, red_row[64 * w]);
        rowv[tid] = (my_max == kNegInf) ? 0.f : my_max;   // no visible key: any finite reference
      }
      lds_barrier();
#pragma unroll
      for (int g = 0; g < NQ; ++g) {
        const f32x4 ref = *reinterpret_cast<const f32x4*>(rowv + 64 * qh + 16 * g + qrow);
        rs[g] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < KG; ++j)
#pragma unroll
          for (int r = 0; r < 4; ++r) rs[g][r] += fast_exp2(sc[j][g][r] - ref[r]);
#pragma unroll
        for (int r = 0; r < 4; ++r) rs[g][r] = row16_reduce<false>(rs[g][r]);
        if ((lane & 15) == 0) *reinterpret_cast<f32x4*>(red + wave * 64 + 16 * g + qrow) = rs[g];
      }
      lds_barrier();
      if (tid < kRowsWg) {
        float l = 0.f;
#pragma unroll
        for (int w = 0; w < kRowWaves; ++w) l += red_row[64 * w];
        // a +inf score makes inf - inf above, a NaN score stays: both give a NaN here, as the row kernel does
        my_lse = (my_max == kNegInf) ? kNegInf : my_max + fast_log2(l);
      }
    }
    // 3. meet the team.  A partial value and the number of its round travel as ONE 64-bit word, so a word
    // that carries this round's number carries this round's value: nobody waits for a store to complete
    // and there is no counter.  The slots start at zero (round numbers start at 1).
    unsigned long long* const slots =
        reinterpret_cast<unsigned long long*>(p.part) + ((int64_t)(team * 2 + (it & 1)) * S) * kRowsWg;
    const unsigned round_no = (unsigned)it + 1u;
    if (tid < kRowsWg)
      __hip_atomic_store(slots + (int64_t)split * kRowsWg + tid,
                         ((unsigned long long)round_no << 32) | __builtin_bit_cast(unsigned, my_lse), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    // All waves share the team's slots: lane = row, the waves of a row take every kMergeWaves-th slot, poll
    // until it carries this round, and fold the values into (max, sum).  (The keys a wave has in flight
    // for the next pair return before these loads do; they were requested during the last steps above.)
    if (wave / QH < kMergeWaves) {
      const int rgroup = wave % QH, sub = wave / QH;
      const bool row_here = 64 * rgroup + lane < kRowsWg;   // (fewer than 64 rows per workgroup with NQ < 4)
      const unsigned long long* mine = slots + 64 * rgroup + lane;
      float m = kNegInf, acc = 0.f;
      bool nan = false, ok = true;
      int polls = 0;
      for (int s0 = sub; s0 < S; s0 += kMergeWaves * kBatch) {
        unsigned long long w[kBatch];
        for (;;) {
          bool all = true;
#pragma unroll
          for (int i = 0; i < kBatch; ++i) {
            const int sidx = s0 + i * kMergeWaves;
            w[i] = (sidx < S && row_here) ? __hip_atomic_load(mine + (int64_t)sidx * kRowsWg, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                              : (((unsigned long long)round_no << 32) | 0xff800000u);   // -inf: adds nothing
          }
#pragma unroll
          for (int i = 0; i < kBatch; ++i) all = all && ((unsigned)(w[i] >> 32) == round_no);
          if (all) break;
          if (++polls > spin_limit) {
            ok = false;
            break;
          }
          __builtin_amdgcn_s_sleep(8);
        }
        if (!ok) break;
        float v[kBatch];
#pragma unroll
        for (int i = 0; i < kBatch; ++i) v[i] = __builtin_bit_cast(float, (unsigned)w[i]);
        float bm = v[0];
#pragma unroll
        for (int i = 1; i < kBatch; ++i) bm = fmaxf(bm, v[i]);
#pragma unroll
        for (int i = 0; i < kBatch; ++i) nan = nan || (v[i] != v[i]);
        const float nm = fmaxf(m, bm);
        if (nm > kNegInf) {
          acc *= fast_exp2(m - nm);   // m = -inf: acc is 0 and stays 0
#pragma unroll
          for (int i = 0; i < kBatch; ++i) acc += fast_exp2(v[i] - nm);
          m = nm;
        }
      }
      if (!ok) {
        __hip_atomic_store(p.sync, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        flag[1] = 0;
      }
      // a NaN partial (fmaxf drops it) makes the row's lse NaN
      if (row_here) {
        mrg[(sub * kRowsWg + 64 * rgroup + lane) * 2] = nan ? __builtin_nanf("") : m;
        mrg[(sub * kRowsWg + 64 * rgroup + lane) * 2 + 1] = acc;
      }
    }
    lds_barrier();
    if (tid < kRowsWg) {
      float mv[kMergeWaves], av[kMergeWaves];
#pragma unroll
      for (int w = 0; w < kMergeWaves; ++w) {
        const float2 ma = *reinterpret_cast<const float2*>(mrg + (w * kRowsWg + tid) * 2);
        mv[w] = ma.x;
        av[w] = ma.y;
      }
      float m = kNegInf;
      bool nan = false;
#pragma unroll
      for (int w = 0; w < kMergeWaves; ++w) {
        nan = nan || (mv[w] != mv[w]);
        m = fmaxf(m, mv[w]);
      }
      const float ref = (m > kNegInf) ? m : 0.f;   // 2^(-inf - ref) = 0 times a finite sum: no branches
      float acc = 0.f;
#pragma unroll
      for (int w = 0; w < kMergeWaves; ++w) acc = fmaf(av[w], fast_exp2(mv[w] - ref), acc);
      const float lse = nan ? __builtin_nanf("") : ((m > kNegInf) ? m + fast_log2(acc) : kNegInf);
      // what step 4 adds to a score, or multiplies 2^score by (nothing for rows that do not exist)
      // (a NaN lse stays a NaN factor: the row's visible columns become NaN, as in the other kernels)
      rowv[tid] = keep_scores ? -lse : ((tid < p.M && lse != kNegInf) ? fast_exp2(-lse) : 0.f);
      if (split == 0 && tid < p.M) p.lse[(int64_t)bh * p.M + tid] = lse;   // (not meaningful if the team was not met)
    }
    lds_barrier();
    const bool met = flag[1] != 0;
    if (tid == 0) flag[0] = 0;
    if (!met) spin_limit = min(spin_limit, 64);   // the call has failed: later waits of this workgroup are short
    // 4. probabilities, reduced down the rows
    f32x4 nl[NQ];
#pragma unroll
    for (int g = 0; g < NQ; ++g) nl[g] = *reinterpret_cast<const f32x4*>(rowv + 64 * qh + 16 * g + qrow);
    float* const osum = obuf + qh * (kRes * kBatchKeys);
    float* const omax = osum + (MODE == kModeBoth ? kBatchKeys : 0);
    int c0b = c0;
    asm volatile("" : "+s"(c0b));
#pragma unroll
    for (int bt = 0; bt < kBatches; ++bt) {   // eight steps at a time through the column buffer
    float vs[kFusedSteps], vm[kFusedSteps];   // per step: the lane's key, reduced over the lane's queries
#pragma unroll
    for (int jj = 0; jj < kFusedSteps; ++jj) {
      const int j = bt * kFusedSteps + jj;
      const int kbase = (c0b + j * KH + kh) * kChunk;
      const int key = kbase + 16 * wq + (lane & 15);
      const bool need_mask = (keep_scores && ragged_rows) || kbase + kChunk > p.N || (CAUSAL && kbase + kChunk - 1 > p.c + 64 * qh);
      f32x4 part = {0.f, 0.f, 0.f, 0.f};   // four independent chains
      float vmax = kNegInf;
      if (MODE == kModeSum && !keep_scores) {   // the registers hold 2^score, nl holds 2^-lse
        if (need_mask) {
          int first = CAUSAL ? key - p.c - 64 * qh - qrow : -(1 << 30);
          if (key >= p.N) first = 1 << 30;
#pragma unroll
          for (int g = 0; g < NQ; ++g)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const int o = 16 * g + r;
              part[r] += (o >= first && o < mlim) ? sc[j][g][r] * nl[g][r] : 0.f;
            }
        } else {
#pragma unroll
          for (int g = 0; g < NQ; ++g)
#pragma unroll
            for (int r = 0; r < 4; ++r) part[r] = fmaf(sc[j][g][r], nl[g][r], part[r]);
        }
      } else if (need_mask) {   // hidden entries stay hidden from a row whose lse is not a number
        int first = CAUSAL ? key - p.c - 64 * qh - qrow : -(1 << 30);
        if (key >= p.N) first = 1 << 30;
#pragma unroll
        for (int g = 0; g < NQ; ++g)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int o = 16 * g + r;
            const float x = (o >= first && o < mlim) ? sc[j][g][r] + nl[g][r] : kNegInf;
            if (MODE != kModeSum) vmax = fmaxf(vmax, x);
            if (MODE != kModeMax) part[r] += fast_exp2(x);
          }
      } else {
#pragma unroll
        for (int g = 0; g < NQ; ++g)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float x = sc[j][g][r] + nl[g][r];
            if (MODE != kModeSum) vmax = fmaxf(vmax, x);
            if (MODE != kModeMax) part[r] += fast_exp2(x);
          }
      }
      vs[jj] = (part[0] + part[1]) + (part[2] + part[3]);
      vm[jj] = vmax;
    }
    // the four lane groups hold different queries of the same key: two exchanges, all steps at once
    if (MODE != kModeMax) {
      float o[kFusedSteps];
#pragma unroll
      for (int j = 0; j < kFusedSteps; ++j) o[j] = __shfl_xor(vs[j], 16);
#pragma unroll
      for (int j = 0; j < kFusedSteps; ++j) vs[j] += o[j];
#pragma unroll
      for (int j = 0; j < kFusedSteps; ++j) o[j] = __shfl_xor(vs[j], 32);
      if (lane < 16) {
#pragma unroll
        for (int j = 0; j < kFusedSteps; ++j) osum[(j * KH + kh) * kChunk + 16 * wq + lane] = vs[j] + o[j];
      }
    }
    if (MODE != kModeSum) {
      float o[kFusedSteps];
#pragma unroll
      for (int j = 0; j < kFusedSteps; ++j) o[j] = __shfl_xor(vm[j], 16);
#pragma unroll
      for (int j = 0; j < kFusedSteps; ++j) vm[j] = fmaxf(vm[j], o[j]);
#pragma unroll
      for (int j = 0; j < kFusedSteps; ++j) o[j] = __shfl_xor(vm[j], 32);
      if (lane < 16) {
#pragma unroll
        for (int j = 0; j < kFusedSteps; ++j) omax[(j * KH + kh) * kChunk + 16 * wq + lane] = fast_exp2(fmaxf(vm[j], o[j]));
      }
    }
    lds_barrier();
    void* const out_max = (MODE == kModeBoth) ? p.out2 : p.out;
    const float poison = __builtin_nanf("");
    const int bkey0 = key0 + bt * kBatchKeys;
    for (int i = tid; i < kBatchKeys; i += kNumThreads) {
      if (bkey0 + i < keys_end) {
        if (MODE != kModeMax) {
          float v = obuf[i];
          if (QH == 2) v += obuf[kRes * kBatchKeys + i];
          store_column(p, p.out, true, bh, bkey0 + i, met ? v : poison);
        }
        if (MODE != kModeSum) {
          const float* om = obuf + (MODE == kModeBoth ? kBatchKeys : 0);
          float v = om[i];
          if (QH == 2) v = fmaxf(v, om[kRes * kBatchKeys + i]);
          store_column(p, out_max, false, bh, bkey0 + i, met ? v : poison);
        }
      }
    }
    if (bt + 1 < kBatches) lds_barrier();   // the next batch writes the buffer again
    }
    // the next writers of obuf, red, rowv and flag are behind the ring barriers of the next pair
  }
  ring_sync<0>();   // the loads past the last chunk write their zeros before the LDS is given back
}

// ---------------------------------------------------------------------------------------------
// fp32 operands.  x = hi + lo with hi = fp16(x), lo = fp16(x - hi) carries 22 bits of x.  Packing
// queries as [hi | hi | lo] and keys as [hi | lo | hi] along d makes the fp16 kernels compute
// q_hi.k_hi + q_hi.k_lo + q_lo.k_hi, the product to about 2^-22 (the lo.lo term is dropped), with fp32
// accumulation.  With terms == 1 only [hi] is written (both operands rounded to fp16).
// dst rows are terms * dpad halves, each segment zero padded from D to dpad.
__global__ __launch_bounds__(256) void pack_f32_kernel(const float* __restrict__ src, _Float16* __restrict__ dst,
                                                       int64_t rows, int D, int dpad, int terms, int is_key) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= rows * dpad) return;
  const int64_t row = idx / dpad;
  const int d = (int)(idx - row * dpad);
  const float x = (d < D) ? src[row * D + d] : 0.f;
  const _Float16 hi = (_Float16)x;
  _Float16* out = dst + row * (int64_t)(terms * dpad) + d;
  out[0] = hi;
  if (terms == 3) {
    const _Float16 lo = (_Float16)(x - (float)hi);
    out[dpad] = is_key ? lo : hi;
    out[2 * dpad] = is_key ? hi : lo;
  }
}

// ---------------------------------------------------------------------------------------------
// Keep-mask of the k largest scores of every row (what a pruning caller does with the reduced
// columns).  One workgroup of 1024 threads per row.  Floats are mapped to integers of the same order and
// the key T of the k-th largest element is found from the top bits down; keys equal to T are kept from
// the lowest column up until k are kept.
//
// Rows of up to 32768 columns (topk_mask_kernel): thread t owns keys [t*VPT, t*VPT + VPT) in registers
// (VPT = 8 or 32) and T is built bit by bit: T | bit is accepted when at least k keys are >= it.  A pass
// is one compare and one add per key, one cross-lane sum, one LDS add per wave and one barrier.
// Longer rows (topk_mask_long_kernel) are re-read from memory in every pass, so T is found eight bits at
// a time from a 256-bin histogram in LDS; a wave whose keys all fall into one bin (the usual case for
// the top digits) adds its count with one atomic.
__device__ __forceinline__ uint32_t order_key(float x) {
  uint32_t b = __builtin_bit_cast(uint32_t, x);
  if (b == 0x80000000u) b = 0u;  // -0 and +0 are one value
  if ((b & 0x7fffffffu) > 0x7f800000u) return 0xffffffffu;  // a NaN of either sign: one value above +inf (torch.topk's order)
  return b ^ ((uint32_t)((int32_t)b >> 31) | 0x80000000u);  // monotone in x for all non-NaN floats
}

// Score rows come as fp32, fp16 or bf16 (what the column kernels store); keys are taken from the widened
// value, which is exact, so order and ties are those of the stored values.
template <typename ET> __device__ __forceinline__ float widen(ET x) { return (float)x; }
template <> __device__ __forceinline__ float widen<uint16_t>(uint16_t x) {   // bf16 bits
  return __builtin_bit_cast(float, (uint32_t)x << 16);
}
// keys of the 4 elements at p, which is aligned to 4 elements
template <typename ET> __device__ __forceinline__ void order_keys4(const ET* p, uint32_t* u) {
  typedef ET ETx4 __attribute__((ext_vector_type(4)));
  const ETx4 v = *reinterpret_cast<const ETx4*>(p);
#pragma unroll
  for (int e = 0; e < 4; ++e) u[e] = order_key(widen<ET>(v[e]));
}
template <typename ET> __device__ __forceinline__ bool rows_aligned_to_4(const ET* scores, int N) {
  return (N & 3) == 0 && (reinterpret_cast<uintptr_t>(scores) & (4 * sizeof(ET) - 1)) == 0;
}
__device__ __forceinline__ float key_value(uint32_t key) {
  return __builtin_bit_cast(float, (key & 0x80000000u) ? (key ^ 0x80000000u) : ~key);
}

constexpr int kTopkThreads = 1024;

// Sum of v over the 64 lanes, as a wave-uniform value: butterflies inside rows of 16 lanes, then the row
// totals are passed on to the rows behind and lane 63 holds the total.
__device__ __forceinline__ uint32_t wave_sum(uint32_t v) {
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xf, 0xf, true);    // quad_perm [1,0,3,2]
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xf, 0xf, true);    // quad_perm [2,3,0,1]
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xf, 0xf, true);   // row_half_mirror
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xf, 0xf, true);   // row_mirror: every lane has its row's sum
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1 and 3
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2 and 3
  return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}

// Exclusive rank of this thread's first tie among the ties of the row, by column, given that thread t
// owns a contiguous run of columns and has `mine` ties.
__device__ __forceinline__ uint32_t ties_before(uint32_t mine, uint32_t* wave_eq, int lane, int wave) {
  uint32_t incl = mine;   // inclusive scan over the wave
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const uint32_t o = __shfl_up(incl, d);
    if (lane >= d) incl += o;
  }
  if (lane == 63) wave_eq[wave] = incl;
  __syncthreads();
  uint32_t before = incl - mine;
  for (int w = 0; w < wave; ++w) before += wave_eq[w];
  return before;
}

template <int VPT, typename ET>
__global__ __launch_bounds__(kTopkThreads) void topk_mask_kernel(const ET* __restrict__ scores,
                                                                 uint8_t* __restrict__ mask,
                                                                 float* __restrict__ threshold, int N, int k) {
  constexpr int kW = kTopkThreads / 64;
  __shared__ uint32_t cnt[34];       // one counter per pass: nothing to reset between passes
  __shared__ uint32_t wave_eq[kW];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const ET* s = scores + (int64_t)blockIdx.x * N;
  uint8_t* m = mask + (int64_t)blockIdx.x * N;
  const uint32_t kk = (uint32_t)min(max(k, 0), N);
  const int base = tid * VPT;

  uint32_t u[VPT];
  // four elements per load when every row starts on such a boundary
  if (rows_aligned_to_4(scores, N)) {
#pragma unroll
    for (int i = 0; i < VPT; i += 4) {
      if (base + i < N) {
        order_keys4(s + base + i, u + i);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) u[i + e] = 0u;   // padding: below every candidate (candidates are >= 1)
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < VPT; ++i) u[i] = (base + i < N) ? order_key(widen<ET>(s[base + i])) : 0u;
  }
  if (tid < 34) cnt[tid] = 0;
  __syncthreads();

  // number of this wave's keys that satisfy pred(key), as a wave-uniform value: every lane counts its
  // own keys, one cross-lane sum per call
  auto wave_count = [&](auto pred) {
    uint32_t c = 0;
#pragma unroll
    for (int i = 0; i < VPT; ++i) c += pred(u[i]) ? 1u : 0u;
    return wave_sum(c);
  };

  uint32_t T = 0;
  for (int b = 31; b >= 0; --b) {
    const uint32_t cand = T | (1u << b);
    const uint32_t c = wave_count([&](uint32_t x) { return x >= cand; });
    if (lane == 0 && c != 0) atomicAdd(&cnt[31 - b], c);
    __syncthreads();
    if (cnt[31 - b] >= kk) T = cand;
  }
  // T is the key of the k-th largest element (all ones if k == 0: nothing is kept)
  {
    const uint32_t na = wave_count([&](uint32_t x) { return x > T; });
    const uint32_t ne = wave_count([&](uint32_t x) { return x == T; });
    if (lane == 0) {
      if (na) atomicAdd(&cnt[32], na);
      if (ne) atomicAdd(&cnt[33], ne);
    }
    __syncthreads();
  }
  const uint32_t above = cnt[32], ties = cnt[33];
  const uint32_t need = (kk > above) ? kk - above : 0u;   // how many of the `ties` keys equal to T are kept
  if (tid == 0 && threshold) threshold[blockIdx.x] = key_value(T);

  uint32_t before = 0;
  if (need < ties) {   // uniform over the workgroup: some ties are dropped, rank them by column
    uint32_t mine = 0;
#pragma unroll
    for (int i = 0; i < VPT; ++i) mine += (u[i] == T) ? 1u : 0u;
    before = ties_before(mine, wave_eq, lane, wave);
  }

  // the mask, VPT bytes per thread
  const bool keep_all_ties = need >= ties;
  uint8_t out[VPT];
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const bool eq = u[i] == T;
    const bool keep = (kk > 0) && ((u[i] > T) || (eq && (keep_all_ties || before < need)));
    if (eq) ++before;
    out[i] = keep ? 1 : 0;
  }
  if ((N & 7) == 0 && (reinterpret_cast<uintptr_t>(mask) & 7) == 0) {
#pragma unroll
    for (int i = 0; i < VPT; i += 8) {
      if (base + i < N) {
        uint64_t w = 0;
#pragma unroll
        for (int e = 0; e < 8; ++e) w |= (uint64_t)out[i + e] << (8 * e);
        *reinterpret_cast<uint64_t*>(m + base + i) = w;
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < VPT; ++i)
      if (base + i < N) m[base + i] = out[i];
  }
}

template <typename ET>
__global__ __launch_bounds__(kTopkThreads) void topk_mask_long_kernel(const ET* __restrict__ scores,
                                                                      uint8_t* __restrict__ mask,
                                                                      float* __restrict__ threshold, int N, int k) {
  constexpr int kW = kTopkThreads / 64;
  __shared__ uint32_t hist[256];
  __shared__ uint32_t sh_prefix, sh_need, sh_ties;
  __shared__ uint32_t wave_eq[kW];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const ET* s = scores + (int64_t)blockIdx.x * N;
  uint8_t* m = mask + (int64_t)blockIdx.x * N;
  const uint32_t kk = (uint32_t)min(max(k, 0), N);
  uint32_t prefix = 0, decided = 0, need = kk;
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
    for (int j0 = 0; j0 < N; j0 += kTopkThreads) {
      const int j = j0 + tid;
      const uint32_t x = (j < N) ? order_key(widen<ET>(s[j])) : 0u;
      const bool live = (j < N) && ((x & decided) == prefix);
      const uint32_t d = (x >> shift) & 255u;
      const uint64_t lives = __builtin_amdgcn_ballot_w64(live);
      if (lives == 0) continue;
      const uint32_t d0 = __builtin_amdgcn_readlane(d, __builtin_ctzll(lives));
      if (__builtin_amdgcn_ballot_w64(live && d == d0) == lives) {   // one bin for the whole wave
        if (lane == 0) atomicAdd(&hist[d0], (uint32_t)__builtin_popcountll(lives));
      } else if (live) {
        atomicAdd(&hist[d], 1u);
      }
    }
    __syncthreads();
    if (tid < 64) {   // one wave walks the bins from the top: 4 bins per lane, suffix sums across lanes
      uint32_t h[4], tot = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        h[e] = hist[255 - (lane * 4 + e)];   // lane 0 holds the four largest digits
        tot += h[e];
      }
      uint32_t incl = tot;
#pragma unroll
      for (int dd = 1; dd < 64; dd <<= 1) {
        const uint32_t o = __shfl_up(incl, dd);
        if (lane >= dd) incl += o;
      }
      uint32_t above = incl - tot;    // keys in larger digits than this lane's
      // the digit where the running count first reaches `need`
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (above < need && above + h[e] >= need) {
          sh_prefix = prefix | ((uint32_t)(255 - (lane * 4 + e)) << shift);
          sh_need = need - above;
          sh_ties = h[e];
        }
        above += h[e];
      }
    }
    __syncthreads();
    if (need > 0) {
      prefix = sh_prefix;
      need = sh_need;
    } else {
      prefix |= 0xffu << shift;   // k == 0: nothing is kept, any threshold above every key will do
    }
    decided |= 0xffu << shift;
    __syncthreads();
  }
  // prefix is now the key of the k-th largest element; `need` of the sh_ties keys equal to it are kept
  const uint32_t T = prefix;
  const uint32_t ties = (kk > 0) ? sh_ties : 0u;
  if (tid == 0 && threshold) threshold[blockIdx.x] = key_value(T);
  const int per = (N + kTopkThreads - 1) / kTopkThreads;   // thread t writes columns [t*per, t*per + per)
  const int base = tid * per;
  uint32_t before = 0;
  if (need < ties) {
    uint32_t mine = 0;
    for (int i = 0; i < per; ++i) mine += (base + i < N && order_key(widen<ET>(s[base + i])) == T) ? 1u : 0u;
    before = ties_before(mine, wave_eq, lane, wave);
  }
  const bool keep_all_ties = need >= ties;
  for (int i = 0; i < per; ++i) {
    const int j = base + i;
    if (j >= N) break;
    const uint32_t x = order_key(widen<ET>(s[j]));
    const bool eq = x == T;
    m[j] = ((kk > 0) && ((x > T) || (eq && (keep_all_ties || before < need)))) ? 1 : 0;
    if (eq) ++before;
  }
}

// ---------------------------------------------------------------------------------------------
// Rows of more than 32768 columns with a workspace: a row is spread over workgroups of VPT * 1024
// columns (VPT = 32 keys per thread, in registers, when that still gives a workgroup per CU, else 8).  Radix select, eight bits per launch: launch PASS
// histograms digit PASS of the keys that match the digits chosen so far, one histogram per workgroup,
// written whole (no atomics in memory, nothing to clear, bitwise reproducible).  Every workgroup of the
// next launch adds up the row's histograms and repeats the choice of the digit, so no launch is needed
// for that.  The last launch chooses the fourth digit, finds the ties in front of its columns in the
// earlier workgroups' histograms of that digit, and writes the mask.

struct TopkState {
  uint32_t prefix;   // digits chosen so far, in place
  uint32_t need;     // how many keys to keep among those that match the prefix
  uint32_t ties;     // how many keys fell into the digit chosen last
  uint32_t pad;
};

// workspace: hist[2][rows][parts][256] followed by state[rows][4]
__host__ __device__ inline size_t topk_hist_words(int64_t rows, int parts) { return (size_t)rows * parts * 256; }

// The choice of digit `pass` for one row, by the whole workgroup: the bins of the row's `parts` histograms
// are added up, then one wave walks them from the top.  prev is the state before this digit.
__device__ __forceinline__ TopkState topk_choose(const uint32_t* __restrict__ hist_row, int parts, TopkState prev,
                                                 int pass, uint32_t* bins, TopkState* chosen, int tid, int lane) {
  const int shift = 24 - 8 * pass;
  if (tid < 256) {
    uint32_t v = 0;
    for (int q = 0; q < parts; ++q) v += hist_row[q * 256 + tid];
    bins[tid] = v;
  }
  if (tid == 0) *chosen = TopkState{prev.prefix | (0xffu << shift), 0u, 0u, 0u};   // need == 0: nothing is kept
  __syncthreads();
  if (tid < 64) {   // 4 bins per lane, lane 0 holds the four largest digits; suffix sums across lanes
    uint32_t h[4], tot = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      h[e] = bins[255 - (lane * 4 + e)];
      tot += h[e];
    }
    uint32_t incl = tot;
#pragma unroll
    for (int dd = 1; dd < 64; dd <<= 1) {
      const uint32_t o = __shfl_up(incl, dd);
      if (lane >= dd) incl += o;
    }
    uint32_t above = incl - tot;   // keys in larger digits than this lane's
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (above < prev.need && above + h[e] >= prev.need)   // true for exactly one bin when need > 0
        *chosen = TopkState{prev.prefix | ((uint32_t)(255 - (lane * 4 + e)) << shift), prev.need - above, h[e], 0u};
      above += h[e];
    }
  }
  __syncthreads();
  const TopkState out = *chosen;
  __syncthreads();   // bins and chosen may be written again
  return out;
}

// The VPT keys of a thread from column col0 on; columns past N get key 0 and valid bit 0.
template <int VPT, typename ET>
__device__ __forceinline__ uint32_t topk_load(const ET* __restrict__ s, int N, int col0, bool vec, uint32_t u[VPT]) {
  if (vec && col0 + VPT <= N) {
#pragma unroll
    for (int i = 0; i < VPT; i += 4) order_keys4(s + col0 + i, u + i);
    return VPT == 32 ? 0xffffffffu : (1u << (VPT & 31)) - 1u;
  }
  uint32_t valid = 0;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const bool in = col0 + i < N;
    u[i] = in ? order_key(widen<ET>(s[in ? col0 + i : 0])) : 0u;
    valid |= in ? (1u << i) : 0u;
  }
  return valid;
}

template <int PASS, int VPT, typename ET>
__global__ __launch_bounds__(kTopkThreads) void topk_spread_hist_kernel(const ET* __restrict__ scores,
                                                                        uint32_t* __restrict__ ws, int64_t rows,
                                                                        int N, int k, int parts) {
  __shared__ uint32_t bins[256];
  __shared__ uint32_t hist[256];
  __shared__ TopkState chosen;
  const int tid = threadIdx.x, lane = tid & 63;
  const int64_t row = blockIdx.x / parts;
  const int part = (int)(blockIdx.x - row * parts);
  const size_t words = topk_hist_words(rows, parts);
  TopkState* states = reinterpret_cast<TopkState*>(ws + 2 * words) + row * 4;
  uint32_t* mine = ws + (PASS & 1) * words + ((size_t)row * parts + part) * 256;

  uint32_t u[VPT];
  const ET* s = scores + row * N;
  const bool vec = rows_aligned_to_4(scores, N);
  const uint32_t valid = topk_load<VPT>(s, N, (part * kTopkThreads + tid) * VPT, vec, u);

  TopkState st{0u, (uint32_t)min(max(k, 0), N), 0u, 0u};
  if (PASS > 0) {
    if (PASS > 1) st = states[PASS - 2];
    st = topk_choose(ws + ((PASS - 1) & 1) * words + (size_t)row * parts * 256, parts, st, PASS - 1, bins, &chosen,
                     tid, lane);
    if (part == 0 && tid == 0) states[PASS - 1] = st;
  }
  if (tid < 256) hist[tid] = 0;
  __syncthreads();
  constexpr uint32_t decided = PASS == 0 ? 0u : 0xffffffffu << (32 - 8 * PASS);
  constexpr int shift = 24 - 8 * PASS;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const bool live = ((valid >> i) & 1u) && ((u[i] & decided) == st.prefix);
    const uint32_t d = (u[i] >> shift) & 255u;
    const uint64_t lives = __builtin_amdgcn_ballot_w64(live);
    if (lives == 0) continue;
    const uint32_t d0 = __builtin_amdgcn_readlane(d, __builtin_ctzll(lives));
    if (__builtin_amdgcn_ballot_w64(live && d == d0) == lives) {   // one bin for the whole wave
      if (lane == 0) atomicAdd(&hist[d0], (uint32_t)__builtin_popcountll(lives));
    } else if (live) {
      atomicAdd(&hist[d], 1u);
    }
  }
  __syncthreads();
  if (tid < 256) mine[tid] = hist[tid];
}

template <int VPT, typename ET>
__global__ __launch_bounds__(kTopkThreads) void topk_spread_write_kernel(const ET* __restrict__ scores,
                                                                         uint8_t* __restrict__ mask,
                                                                         float* __restrict__ threshold,
                                                                         const uint32_t* __restrict__ ws, int64_t rows,
                                                                         int N, int k, int parts) {
  constexpr int kW = kTopkThreads / 64;
  __shared__ uint32_t bins[256];
  __shared__ TopkState chosen;
  __shared__ uint32_t wave_eq[kW];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t row = blockIdx.x / parts;
  const int part = (int)(blockIdx.x - row * parts);
  const size_t words = topk_hist_words(rows, parts);
  const TopkState* states = reinterpret_cast<const TopkState*>(ws + 2 * words) + row * 4;
  const uint32_t* last = ws + words + (size_t)row * parts * 256;   // the histograms of digit 3 (3 & 1 == 1)

  uint32_t u[VPT];
  const ET* s = scores + row * N;
  const bool vec = rows_aligned_to_4(scores, N);
  const int col0 = (part * kTopkThreads + tid) * VPT;
  const uint32_t valid = topk_load<VPT>(s, N, col0, vec, u);

  const uint32_t kk = (uint32_t)min(max(k, 0), N);
  const TopkState st = topk_choose(last, parts, states[2], 3, bins, &chosen, tid, lane);
  const uint32_t T = st.prefix, need = st.need, ties = (kk > 0) ? st.ties : 0u;
  if (part == 0 && tid == 0 && threshold) threshold[row] = key_value(T);

  uint32_t before = 0;
  if (need < ties) {   // uniform over the row: some ties are dropped, rank them by column
    uint32_t mine = 0;
#pragma unroll
    for (int i = 0; i < VPT; ++i) mine += (((valid >> i) & 1u) && u[i] == T) ? 1u : 0u;
    before = ties_before(mine, wave_eq, lane, wave);
    for (int q = 0; q < part; ++q) before += last[q * 256 + (T & 255u)];   // ties in the workgroups in front
  }
  const bool keep_all_ties = need >= ties;
  uint8_t* m = mask + row * N;
  const bool whole = valid == (VPT == 32 ? 0xffffffffu : (1u << (VPT & 31)) - 1u) && (N & 7) == 0 &&
                     (reinterpret_cast<uintptr_t>(mask) & 7) == 0;
#pragma unroll
  for (int i0 = 0; i0 < VPT; i0 += 8) {
    uint64_t w = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int i = i0 + e;
      const bool eq = ((valid >> i) & 1u) && u[i] == T;
      const bool keep = (kk > 0) && ((u[i] > T) || (eq && (keep_all_ties || before < need)));
      if (eq) ++before;
      w |= (uint64_t)(keep ? 1 : 0) << (8 * e);
    }
    if (whole) {
      *reinterpret_cast<uint64_t*>(m + col0 + i0) = w;
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if ((valid >> (i0 + e)) & 1u) m[col0 + i0 + e] = (uint8_t)(w >> (8 * e));
    }
  }
}

// ---------------------------------------------------------------------------------------------
thread_local char g_err[256] = "";

int fail(int code, const char* what) {
  snprintf(g_err, sizeof(g_err), "%s", what);
  return code;
}

inline int elem_bytes(int dtype) { return dtype == FCR_DTYPE_F32 ? 4 : 2; }
inline int ksteps_of(int dtype, int D) { return (D * elem_bytes(dtype) + 63) / 64; }

// dims = sizes of the batch, head and row dimensions.  The stride of a dimension of size one is never
// used to form an address, so it may be anything (torch reports arbitrary strides there, and a slice of an
// expanded tensor keeps stride 0): only the strides that matter are checked.
int check_strides(const void* ptr, const int64_t s[4], const char* name, const int dims[3], int D, int esize) {
  if (s[3] != 1) {
    snprintf(g_err, sizeof(g_err), "%s: stride of the last dimension must be 1 (got %lld)", name, (long long)s[3]);
    return FCR_E_STRIDE;
  }
  const int al = 16 / esize;   // elements per 16 bytes
  bool ok = (reinterpret_cast<uintptr_t>(ptr) & 15) == 0;
  for (int i = 0; i < 3; ++i)
    if (dims[i] > 1 && (s[i] % al != 0 || s[i] < 0)) ok = false;
  if (dims[2] > 1 && s[2] * esize >= (1 << 25)) ok = false;
  if (!ok) {
    snprintf(g_err, sizeof(g_err),
             "%s: base pointer must be 16-byte aligned, batch/head/row strides non-negative multiples of 16 bytes (%d elements), row stride < 2^25 bytes",
             name, al);
    return FCR_E_STRIDE;
  }
  // Rows that overlap (an expanded operand has row stride 0) cannot be described by the buffer views
  // the kernels read through: the view of the rows from r on is (rows - r) * stride bytes long.
  if (dims[2] > 1 && s[2] < D) {
    snprintf(g_err, sizeof(g_err), "%s: row stride (%lld) must be at least D (%d) when there is more than one row",
             name, (long long)s[2], D);
    return FCR_E_STRIDE;
  }
  return 0;
}

// (b,h) pairs per launch group, a multiple of 8.  Without a mask all sweeps of a launch are equally
// long and about one workgroup per CU (256) keeps the tiles of a (b,h) together in time.  With the
// causal mask the longest-first order needs room to level the triangle: about 1024 workgroups and
// never fewer than 32 pairs (measured: smaller groups lose up to 8 % on 32 heads of 8192 rows,
// larger ones up to 11 % on 1024 heads of 2048 rows, whose operands then come from HBM per tile).
int head_group(int64_t bh, int64_t per_bh, bool causal) {
  const int cus = chip_cus();
  int64_t g = ((causal ? 4 * cus : cus) / per_bh) & ~7ll;
  const int64_t least = causal ? 32 : 8;
  if (g < least) g = least;
  return (int)(g < bh ? g : bh);
}

int make_params(Params& p, const void* q, const void* k, int dtype, int B, int H, int M, int N, int D,
                const int64_t qs[4], const int64_t ks[4], float scale, bool by_keys, bool causal,
                int col_mode = kModeSum) {
  if (!q || !k || !qs || !ks) return fail(FCR_E_NULL, "null pointer argument");
  if (dtype != FCR_DTYPE_F16 && dtype != FCR_DTYPE_BF16 && dtype != FCR_DTYPE_F32)
    return fail(FCR_E_DTYPE, "dtype must be FCR_DTYPE_F16, FCR_DTYPE_BF16 or FCR_DTYPE_F32");
  if (B < 1 || H < 1 || M < 1 || N < 1) return fail(FCR_E_SHAPE, "B, H, M, N must be >= 1");
  const int esize = elem_bytes(dtype);
  if (D < 1 || D * esize > 64 * kMaxKStepsF32 || (D * esize) % 16 != 0)
    return fail(FCR_E_SHAPE, esize == 2 ? "D must be a multiple of 8 in [8, 512]"
                                         : "D must be a multiple of 4 in [4, 256] for FCR_DTYPE_F32");
  if (M > (1 << 30) || N > (1 << 30)) return fail(FCR_E_SHAPE, "M and N must be <= 2^30");
  const int64_t bh = (int64_t)B * H;
  // a launch may have fewer than 2^32 threads: fewer than 2^24 workgroups of 256 (the finest tiling, 128 rows)
  if (bh * (((int64_t)(by_keys ? N : M) + 127) / 128) >= kMaxWorkgroups)
    return fail(FCR_E_SHAPE, "B*H*ceil(rows/128) must be below 2^24 workgroups");
  if (!isfinite(scale)) return fail(FCR_E_SCALE, "scale must be finite");
  const int qdims[3] = {B, H, M}, kdims[3] = {B, H, N};
  int rc = check_strides(q, qs, "q", qdims, D, esize);
  if (rc) return rc;
  rc = check_strides(k, ks, "k", kdims, D, esize);
  if (rc) return rc;
  // the device is first asked (for its CU count) here, after every argument check
  const int ksteps = ksteps_of(dtype, D);
  const int trows = by_keys ? kWaves * 32 * col_tile_blocks(ksteps, col_mode, N, bh, causal) : row_tile_rows(ksteps, M, N, bh, causal);
  const int64_t tiles = ((by_keys ? N : M) + trows - 1) / trows;
  p.q = static_cast<const char*>(q);
  p.k = static_cast<const char*>(k);
  // a single row is given the stride of a dense one: the buffer views are sized rows * stride
  p.q_sb = B > 1 ? qs[0] * esize : 0; p.q_sh = H > 1 ? qs[1] * esize : 0; p.q_sr = M > 1 ? qs[2] * esize : D * esize;
  p.k_sb = B > 1 ? ks[0] * esize : 0; p.k_sh = H > 1 ? ks[1] * esize : 0; p.k_sr = N > 1 ? ks[2] * esize : D * esize;
  p.H = H; p.M = M; p.N = N;
  p.dgran = D * esize / 16;
  p.c = N > M ? N - M : 0;
  p.scale2 = (float)((double)scale * 1.4426950408889634);
  p.tiles = (int)tiles;
  p.bh_count = (int)bh;
  p.total = (int)(bh * tiles);
  p.lse = nullptr;
  p.out = nullptr;
  p.out2 = nullptr;
  p.part = nullptr;
  p.splits = 1;
  p.stream_once = 0;
  p.out_fmt = FCR_DTYPE_F32;
  p.mean_from = -1;
  p.inv_m = 0.f;
  p.teams = 0;
  p.sync = nullptr;
  p.spin_limit = 0;
  return 0;
}

// Key ranges per row tile in the row kernel.  One sweep per workgroup when there is at least one
// workgroup per CU; otherwise the keys of a tile are split so that about two per CU run, each
// keeping at least four 64-key chunks.
int row_splits(int B, int H, int M, int N, int ksteps) {
  const int trows = row_tile_rows(ksteps, M, N, (int64_t)B * H, false);  // same with the mask when wgs < 256
  const int64_t wgs = (int64_t)B * H * ((M + trows - 1) / trows);
  const int64_t chunks = (N + kChunk - 1) / kChunk;
  const int cus = chip_cus();
  if (wgs >= cus || chunks < 16) return 1;
  int64_t s = 2 * cus / wgs;
  if (s > chunks / 4) s = chunks / 4;
  if (s > 64) s = 64;
  return s < 1 ? 1 : (int)s;
}

// The single-sweep path (col_fused_kernel): 16-bit operands, rows of at most 256 bytes, at most 128 queries
// and enough keys for the sweep to matter.  A (b,h) pair is shared by `splits` workgroups of 512 keys each;
// teams * splits workgroups are launched, never more than the chip holds at once.
constexpr int kFusedMinChunks = 16;   // 1024 keys
struct FusedPlan {
  int qh;       // 1: 64 query rows per workgroup and 1024 keys per pair, 2: 128 rows and 512 keys
  int nq;       // groups of sixteen queries per wave: 4, or 2 (at most 32 queries) with 2048 keys per pair
  int splits, teams;
  int64_t part_at, sync_at;   // where the partial row values and the counters start in the workspace, in floats
  int64_t floats;             // workspace size
};
// Shape conditions only: the size of the workspace must not depend on the element type.
bool fused_shape(int64_t bh, int M, int N, FusedPlan& f) {
  const int64_t nchunks = ((int64_t)N + kChunk - 1) / kChunk;
  if (M > 2 * 64 || nchunks < kFusedMinChunks) return false;
  f.qh = M > 64 ? 2 : 1;
  const int cap = chip_cus();   // one workgroup per CU
  // With at most 32 queries a workgroup can keep the scores of 2048 keys of a pair, which spreads the time
  // between two sweeps over twice the keys, but it leaves half the workgroups per pair.  The choice is the
  // one with the least estimated time: rounds x (0.56 us per chunk + 4.5 us between sweeps).
  double best = 0.0;
  f.nq = 0;
  for (int nq = 4; nq >= 2; nq /= 2) {
    if (nq < 4 && (f.qh != 1 || M > 16 * nq)) continue;
    const int chunks = fused_chunks(f.qh, nq);
    const int64_t splits = (nchunks + chunks - 1) / chunks;
    if (splits > cap) continue;
    const int64_t teams = (cap / splits) < bh ? (cap / splits) : bh;
    const int64_t rounds = (bh + teams - 1) / teams;
    const int64_t swept = nchunks < chunks ? nchunks : chunks;
    const double cost = (double)rounds * (0.56 * (double)swept + 4.5);
    if (f.nq == 0 || cost < best) {
      best = cost;
      f.nq = nq;
      f.splits = (int)splits;
      f.teams = (int)teams;
    }
  }
  if (f.nq == 0) return false;
  f.part_at = (bh * M + 63) / 64 * 64;
  f.sync_at = f.part_at + 2 * (2ll * cap * 64 * f.qh);   // two sets of one 64-bit slot per row and workgroup
  f.floats = f.sync_at + 32;
  return true;
}

int launched(const char* what) {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return 0;
  snprintf(g_err, sizeof(g_err), "%s launch failed: %s", what, hipGetErrorString(e));
  return (int)e;
}

template <int DT, int KS, int NB, bool ONCE>
void launch_lse_blocks(const Params& p, bool causal, hipStream_t s) {
  const dim3 grid(p.total), block(kThreads);
  if (causal) hipLaunchKernelGGL((row_lse_kernel<DT, KS, true, NB, ONCE>), grid, block, 0, s, p);
  else hipLaunchKernelGGL((row_lse_kernel<DT, KS, false, NB, ONCE>), grid, block, 0, s, p);
}

template <int DT, int KS>
void launch_lse(const Params& p, bool causal, hipStream_t s) {
  if constexpr (KS <= 4) {
    if (row_blocks_per_wave(KS, p.M, p.N, p.bh_count, causal) == 2) return launch_lse_blocks<DT, KS, 2, false>(p, causal, s);
  }
  // one row tile per (b,h) and at least 1 GiB of keys: stream them past the caches
  const int64_t key_bytes = (int64_t)p.bh_count * p.N * p.dgran * 16;
  if (p.tiles == 1 && key_bytes >= (1ll << 30)) return launch_lse_blocks<DT, KS, 1, true>(p, causal, s);
  launch_lse_blocks<DT, KS, 1, false>(p, causal, s);
}

template <int DT, int KS, int MODE>
void launch_col_mode(const Params& p, bool causal, hipStream_t s) {
  const dim3 grid(p.total), block(kThreads);
  constexpr int NB = col_blocks_per_wave(KS, MODE);
  if constexpr (NB == 2) {
    if (col_tile_blocks(KS, MODE, p.N, p.bh_count, causal) == 1) {
      if (causal) hipLaunchKernelGGL((col_reduce_kernel<DT, KS, true, MODE, 1>), grid, block, 0, s, p);
      else hipLaunchKernelGGL((col_reduce_kernel<DT, KS, false, MODE, 1>), grid, block, 0, s, p);
      return;
    }
  }
  if (causal) hipLaunchKernelGGL((col_reduce_kernel<DT, KS, true, MODE, NB>), grid, block, 0, s, p);
  else hipLaunchKernelGGL((col_reduce_kernel<DT, KS, false, MODE, NB>), grid, block, 0, s, p);
}

template <int DT, int KS, int MODE, int NG>
void launch_col_small_groups(const Params& p, bool causal, hipStream_t s) {
  const dim3 grid(p.total), block(kThreads);
  if (causal) hipLaunchKernelGGL((col_small_kernel<DT, KS, true, MODE, NG>), grid, block, 0, s, p);
  else hipLaunchKernelGGL((col_small_kernel<DT, KS, false, MODE, NG>), grid, block, 0, s, p);
}

template <int DT, int KS, int MODE>
void launch_col_small_mode(const Params& p, bool causal, hipStream_t s) {
  if (p.M <= 64) launch_col_small_groups<DT, KS, MODE, 4>(p, causal, s);
  else launch_col_small_groups<DT, KS, MODE, 8>(p, causal, s);
}

template <int DT, int KS>
void launch_col_small(const Params& p, bool causal, int mode, hipStream_t s) {
  if (mode == kModeSum) launch_col_small_mode<DT, KS, kModeSum>(p, causal, s);
  else if (mode == kModeMax) launch_col_small_mode<DT, KS, kModeMax>(p, causal, s);
  else launch_col_small_mode<DT, KS, kModeBoth>(p, causal, s);
}

// Workgroups of col_fused_kernel wait for each other, so all of a launch must be on the chip together: the
// host plans with two workgroups of 256 threads, or one of 512, per CU, and the launch is refused (the caller
// then takes the two-kernel path) if the runtime says that this build of the kernel does not fit that way.
template <class K>
bool fits_per_cu(K kernel, int threads, int want) {
  int n = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, threads, 0) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return n >= want;
}

template <int DT, int KS, int MODE, int QH, int NQ = 4>
void launch_col_fused_mode(const Params& p, bool causal, hipStream_t s) {
  const dim3 grid(p.total), block(kFusedThreads);
  static int fits[2] = {-1, -1};   // asked once per kernel (the answer depends on its registers and LDS, not on the device of a kind)
  int f = __atomic_load_n(&fits[causal], __ATOMIC_RELAXED);
  if (f < 0) {
    f = causal ? fits_per_cu(col_fused_kernel<DT, KS, true, MODE, QH, NQ>, kFusedThreads, 1)
               : fits_per_cu(col_fused_kernel<DT, KS, false, MODE, QH, NQ>, kFusedThreads, 1);
    __atomic_store_n(&fits[causal], f, __ATOMIC_RELAXED);
  }
  if (!f) {
    fcr_detail::fused_refused = true;
    return;
  }
  if (causal) hipLaunchKernelGGL((col_fused_kernel<DT, KS, true, MODE, QH, NQ>), grid, block, 0, s, p);
  else hipLaunchKernelGGL((col_fused_kernel<DT, KS, false, MODE, QH, NQ>), grid, block, 0, s, p);
}

template <int DT, int KS, int QH, int NQ>
void launch_col_fused_groups(const Params& p, bool causal, int m, hipStream_t s) {
  if (m == kModeSum) launch_col_fused_mode<DT, KS, kModeSum, QH, NQ>(p, causal, s);
  else if (m == kModeMax) launch_col_fused_mode<DT, KS, kModeMax, QH, NQ>(p, causal, s);
  else launch_col_fused_mode<DT, KS, kModeBoth, QH, NQ>(p, causal, s);
}

// mode: kModeSum, kModeMax or kModeBoth, + 4 for more than 64 queries, + 8 for two groups of sixteen queries
// per wave
template <int DT, int KS>
void launch_col_fused(const Params& p, bool causal, int mode, hipStream_t s) {
  const int m = mode & 3;
  if (mode & 4) launch_col_fused_groups<DT, KS, 2, 4>(p, causal, m, s);
  else if (mode & 8) launch_col_fused_groups<DT, KS, 1, 2>(p, causal, m, s);
  else launch_col_fused_groups<DT, KS, 1, 4>(p, causal, m, s);
}

template <int DT, int KS>
void launch_col(const Params& p, bool causal, int mode, hipStream_t s) {
  if (mode == kModeSum) launch_col_mode<DT, KS, kModeSum>(p, causal, s);
  else if (mode == kModeMax) launch_col_mode<DT, KS, kModeMax>(p, causal, s);
  else launch_col_mode<DT, KS, kModeBoth>(p, causal, s);
}

#define FCR_DISPATCH_KS(DT, ksteps, CALL)                  \
  switch (ksteps) {                                        \
    case 1: CALL(DT, 1); break;                            \
    case 2: CALL(DT, 2); break;                            \
    case 3: CALL(DT, 3); break;                            \
    case 4: CALL(DT, 4); break;                            \
    case 5: CALL(DT, 5); break;                            \
    case 6: CALL(DT, 6); break;                            \
    case 7: CALL(DT, 7); break;                            \
    default: CALL(DT, 8); break;                           \
  }

// rows of more than 512 bytes: 9 to 16 k-steps
#define FCR_DISPATCH_KS_LONG(DT, ksteps, CALL)             \
  switch (ksteps) {                                        \
    case 9: CALL(DT, 9); break;                            \
    case 10: CALL(DT, 10); break;                          \
    case 11: CALL(DT, 11); break;                          \
    case 12: CALL(DT, 12); break;                          \
    case 13: CALL(DT, 13); break;                          \
    case 14: CALL(DT, 14); break;                          \
    case 15: CALL(DT, 15); break;                          \
    default: CALL(DT, 16); break;                          \
  }

#define FCR_DISPATCH_KS4(DT, ksteps, CALL)                 \
  switch (ksteps) {                                        \
    case 1: CALL(DT, 1); break;                            \
    case 2: CALL(DT, 2); break;                            \
    case 3: CALL(DT, 3); break;                            \
    default: CALL(DT, 4); break;                           \
  }

}  // namespace

// The sweeps of one element type (see the declarations at the top).
#define FCR_CALL_LSE(DT, KS) launch_lse<DT, KS>(p, causal, s)
#define FCR_CALL_COL(DT, KS) launch_col<DT, KS>(p, causal, mode, s)
#define FCR_CALL_COL_SMALL(DT, KS) launch_col_small<DT, KS>(p, causal, mode, s)
#define FCR_CALL_COL_FUSED(DT, KS) launch_col_fused<DT, KS>(p, causal, mode, s)
#define FCR_SWEEPS_16BIT(NAME, DT)                                                                       \
  void fcr_detail::NAME(int which, const Params& p, int ksteps, bool causal, int mode, hipStream_t s) { \
    if (which == 0) { FCR_DISPATCH_KS(DT, ksteps, FCR_CALL_LSE) }                                        \
    else if (which == 1) { FCR_DISPATCH_KS(DT, ksteps, FCR_CALL_COL) }                                   \
    else { FCR_DISPATCH_KS4(DT, ksteps, FCR_CALL_COL_SMALL) }                                            \
  }
#if FCR_HAS(1)
FCR_SWEEPS_16BIT(sweeps_f16, FCR_DTYPE_F16)
#endif
#if FCR_HAS(2)
FCR_SWEEPS_16BIT(sweeps_bf16, FCR_DTYPE_BF16)
#endif
#if FCR_HAS(7)
void fcr_detail::sweeps_f16_single(const Params& p, int ksteps, bool causal, int mode, hipStream_t s) {
  FCR_DISPATCH_KS4(FCR_DTYPE_F16, ksteps, FCR_CALL_COL_FUSED)
}
#endif
#if FCR_HAS(8)
void fcr_detail::sweeps_bf16_single(const Params& p, int ksteps, bool causal, int mode, hipStream_t s) {
  FCR_DISPATCH_KS4(FCR_DTYPE_BF16, ksteps, FCR_CALL_COL_FUSED)
}
#endif
#if FCR_HAS(3)
void fcr_detail::sweeps_f32(int which, const Params& p, int ksteps, bool causal, int mode, hipStream_t s) {
  if (which == 0) { FCR_DISPATCH_KS(FCR_DTYPE_F32, ksteps, FCR_CALL_LSE) }
  else { FCR_DISPATCH_KS(FCR_DTYPE_F32, ksteps, FCR_CALL_COL) }
}
#endif
#if FCR_HAS(4)
void fcr_detail::sweeps_f32_long_rows(int which, const Params& p, int ksteps, bool causal, int mode, hipStream_t s) {
  if (which == 0) { FCR_DISPATCH_KS_LONG(FCR_DTYPE_F32, ksteps, FCR_CALL_LSE) }
  else { FCR_DISPATCH_KS_LONG(FCR_DTYPE_F32, ksteps, FCR_CALL_COL) }
}
#endif
#if FCR_HAS(5)
void fcr_detail::sweeps_f16_long_rows(int which, const Params& p, int ksteps, bool causal, int mode, hipStream_t s) {
  if (which == 0) { FCR_DISPATCH_KS_LONG(FCR_DTYPE_F16, ksteps, FCR_CALL_LSE) }
  else { FCR_DISPATCH_KS_LONG(FCR_DTYPE_F16, ksteps, FCR_CALL_COL) }
}
#endif
#if FCR_HAS(6)
void fcr_detail::sweeps_bf16_long_rows(int which, const Params& p, int ksteps, bool causal, int mode, hipStream_t s) {
  if (which == 0) { FCR_DISPATCH_KS_LONG(FCR_DTYPE_BF16, ksteps, FCR_CALL_LSE) }
  else { FCR_DISPATCH_KS_LONG(FCR_DTYPE_BF16, ksteps, FCR_CALL_COL) }
}
#endif
#undef FCR_CALL_LSE
#undef FCR_CALL_COL
#undef FCR_CALL_COL_SMALL
#undef FCR_CALL_COL_FUSED

#if FCR_HAS(0)
namespace {
// sweeps of the element type `dtype`
void launch_sweeps(int dtype, int which, const Params& p, int ksteps, bool causal, int mode, hipStream_t s,
                   unsigned* zero = nullptr, int zero_words = 0) {
  if (zero_words > 0)
    hipLaunchKernelGGL(zero_words_kernel, dim3((unsigned)((zero_words + 255) / 256)), dim3(256), 0, s, zero, zero_words);
  const bool long_rows = ksteps > kMaxKSteps;
  if (which == 3) {   // the single sweep: 16-bit elements, rows of at most 256 bytes
    if (dtype == FCR_DTYPE_F16) fcr_detail::sweeps_f16_single(p, ksteps, causal, mode, s);
    else fcr_detail::sweeps_bf16_single(p, ksteps, causal, mode, s);
    return;
  }
  if (dtype == FCR_DTYPE_F16) (long_rows ? fcr_detail::sweeps_f16_long_rows : fcr_detail::sweeps_f16)(which, p, ksteps, causal, mode, s);
  else if (dtype == FCR_DTYPE_BF16) (long_rows ? fcr_detail::sweeps_bf16_long_rows : fcr_detail::sweeps_bf16)(which, p, ksteps, causal, mode, s);
  else (long_rows ? fcr_detail::sweeps_f32_long_rows : fcr_detail::sweeps_f32)(which, p, ksteps, causal, mode, s);
}

template <int VPT, typename ET>
void launch_topk_spread(const ET* scores, uint8_t* mask, float* threshold, int64_t rows, int N, int k, uint32_t* w,
                        hipStream_t s) {
  const int parts = (N + VPT * kTopkThreads - 1) / (VPT * kTopkThreads);
  const dim3 grid((unsigned)(rows * parts)), block(kTopkThreads);
  hipLaunchKernelGGL((topk_spread_hist_kernel<0, VPT, ET>), grid, block, 0, s, scores, w, rows, N, k, parts);
  hipLaunchKernelGGL((topk_spread_hist_kernel<1, VPT, ET>), grid, block, 0, s, scores, w, rows, N, k, parts);
  hipLaunchKernelGGL((topk_spread_hist_kernel<2, VPT, ET>), grid, block, 0, s, scores, w, rows, N, k, parts);
  hipLaunchKernelGGL((topk_spread_hist_kernel<3, VPT, ET>), grid, block, 0, s, scores, w, rows, N, k, parts);
  hipLaunchKernelGGL((topk_spread_write_kernel<VPT, ET>), grid, block, 0, s, scores, mask, threshold, w, rows, N, k,
                     parts);
}

// The top-k launches for one element type: spread over workgroups when the caller brought enough scratch
// for a long row, else one workgroup per row.
template <typename ET>
int topk_any(const ET* scores, uint8_t* mask, float* threshold, int64_t rows, int N, int k, void* ws, size_t ws_bytes,
             hipStream_t s) {
  const size_t want = fcr_topk_bytes(rows, N);
  if (ws && want != 0 && ws_bytes >= want) {
    uint32_t* w = static_cast<uint32_t*>(ws);
    // 32 keys per thread while that leaves a workgroup per CU, else 8
    const int64_t coarse = rows * ((N + 32 * kTopkThreads - 1) / (32 * kTopkThreads));
    if (coarse >= chip_cus()) launch_topk_spread<32>(scores, mask, threshold, rows, N, k, w, s);
    else launch_topk_spread<8>(scores, mask, threshold, rows, N, k, w, s);
    return 0;
  }
  const dim3 grid((unsigned)rows), block(kTopkThreads);
  if (N <= 8 * kTopkThreads) hipLaunchKernelGGL((topk_mask_kernel<8, ET>), grid, block, 0, s, scores, mask, threshold, N, k);
  else if (N <= 32 * kTopkThreads) hipLaunchKernelGGL((topk_mask_kernel<32, ET>), grid, block, 0, s, scores, mask, threshold, N, k);
  else hipLaunchKernelGGL(topk_mask_long_kernel<ET>, grid, block, 0, s, scores, mask, threshold, N, k);
  return 0;
}
}  // namespace

namespace {
size_t fcr_lse_bytes_two_kernels(int B, int H, int M, int N) {
  // the most any row width asks for (the tile height, hence the split count, depends a little on the
  // number of 64-byte k-steps of a row), so the size holds for every dtype and D
  int splits = 1;
  for (int ks = 1; ks <= kMaxKStepsF32; ++ks) {
    const int s = row_splits(B, H, M, N, ks);
    if (s > splits) splits = s;
  }
  const size_t rows = (size_t)B * (size_t)H * (size_t)M;
  return rows * sizeof(float) * (splits > 1 ? 1 + (size_t)splits : 1);
}

// process-wide switches (fcr_set_option)
int g_single_sweep = 1;
long long g_wait_polls = 1ll << 20;
}  // namespace
thread_local bool fcr_detail::fused_refused = false;

extern "C" {

int fcr_version(void) { return FCR_VERSION; }

const char* fcr_last_error(void) { return g_err; }

size_t fcr_lse_bytes(int B, int H, int M, int N, int D) {
  if (B < 1 || H < 1 || M < 1 || N < 1 || D < 1) return 0;
  {
    // the single-sweep path keeps partial row values and its counters behind the row statistics
    FusedPlan f;
    if (fused_shape((int64_t)B * H, M, N, f)) {
      const size_t two_kernels = fcr_lse_bytes_two_kernels(B, H, M, N);
      const size_t one = (size_t)f.floats * sizeof(float);
      return one > two_kernels ? one : two_kernels;
    }
  }
  return fcr_lse_bytes_two_kernels(B, H, M, N);
}

int fcr_row_lse(const void* q, const void* k, float* lse, int dtype, int B, int H, int M, int N, int D,
                const int64_t q_strides[4], const int64_t k_strides[4], float scale, int causal,
                void* stream) {
  Params p;
  if (!lse) return fail(FCR_E_NULL, "null pointer argument");
  int rc = make_params(p, q, k, dtype, B, H, M, N, D, q_strides, k_strides, scale, false, causal != 0);
  if (rc) return rc;
  p.lse = lse;
  p.splits = row_splits(B, H, M, N, ksteps_of(dtype, D));
  p.part = lse + (int64_t)B * H * M;  // only touched when splits > 1 (see fcr_lse_bytes)
  p.total *= p.splits;
  p.group = head_group(p.bh_count, (int64_t)p.tiles * p.splits, causal != 0);
  const int ksteps = ksteps_of(dtype, D);
  hipStream_t s = static_cast<hipStream_t>(stream);
  launch_sweeps(dtype, 0, p, ksteps, causal != 0, 0, s);
  rc = launched("row_lse_kernel");
  if (rc || p.splits == 1) return rc;
  const int64_t rows = (int64_t)B * H * M;
  hipLaunchKernelGGL(lse_combine_kernel, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, s, p.part, lse, rows,
                     p.splits);
  return launched("lse_combine_kernel");
}

namespace {
// Element type of the results and whether the sums leave the kernel as means.
struct ResultSpec {
  int fmt = FCR_DTYPE_F32;
  bool mean = false;
};

int col_reduce_any(const void* q, const void* k, const float* lse, void* out, void* out2, int mode, int dtype,
                   int B, int H, int M, int N, int D, const int64_t q_strides[4], const int64_t k_strides[4],
                   float scale, int causal, void* stream, const ResultSpec& res = ResultSpec()) {
  Params p;
  if (!lse || !out || (mode == kModeBoth && !out2)) return fail(FCR_E_NULL, "null pointer argument");
  int rc = make_params(p, q, k, dtype, B, H, M, N, D, q_strides, k_strides, scale, true, causal != 0, mode);
  if (rc) return rc;
  p.group = head_group(p.bh_count, p.tiles, causal != 0);
  p.lse = const_cast<float*>(lse);
  p.out = out;
  p.out2 = out2;
  p.out_fmt = res.fmt;
  if (res.mean) {
    p.mean_from = causal ? p.c : N;
    p.inv_m = 1.0f / (float)M;
  }
  const int ksteps = ksteps_of(dtype, D);
  hipStream_t s = static_cast<hipStream_t>(stream);
  // (fp32 operands always take the general sweep: they are bound by the fp32 matrix rate, not by reading K)
  if (M <= kSmallRows && ksteps <= 4 && dtype != FCR_DTYPE_F32) {
    // Few queries: the sweep with all of them resident in every wave and the keys streamed, if the
    // problem fills the chip that way: 512 to 1024 workgroups (at least two per CU), each sweeping at
    // least 16 chunks of keys, or 8 if that is what it takes.
    const int64_t nchunks = ((int64_t)N + kChunk - 1) / kChunk;
    int64_t splits = 0;
    const int cus = chip_cus();
    for (int64_t least = 16; least >= 8 && p.bh_count * splits < 2 * cus; least /= 2) {  // longer sweeps first
      splits = 4 * cus / p.bh_count;
      if (splits > nchunks / least) splits = nchunks / least;
      if (splits < 1) splits = 1;
      const int64_t per = (nchunks + splits - 1) / splits;
      splits = (nchunks + per - 1) / per;  // no empty ranges
    }
    if (p.bh_count * splits >= 2 * cus) {
      p.splits = (int)splits;
      p.total = (int)(p.bh_count * splits);
      p.group = head_group(p.bh_count, splits, false);
      p.stream_once = ((int64_t)p.bh_count * N * p.dgran * 16 >= (1ll << 30)) ? 1 : 0;
      launch_sweeps(dtype, 2, p, ksteps, causal != 0, mode, s);
      return launched("col_small_kernel");
    }
  }
  launch_sweeps(dtype, 1, p, ksteps, causal != 0, mode, s);
  return launched("col_reduce_kernel");
}
}  // namespace

int fcr_col_reduce(const void* q, const void* k, const float* lse, float* out, int dtype, int B, int H,
                   int M, int N, int D, const int64_t q_strides[4], const int64_t k_strides[4],
                   float scale, int reduction, int causal, void* stream) {
  if (reduction != FCR_REDUCE_SUM && reduction != FCR_REDUCE_MAX)
    return fail(FCR_E_REDUCTION, "reduction must be FCR_REDUCE_SUM or FCR_REDUCE_MAX");
  return col_reduce_any(q, k, lse, out, nullptr, reduction == FCR_REDUCE_MAX ? kModeMax : kModeSum, dtype, B, H, M,
                        N, D, q_strides, k_strides, scale, causal, stream);
}

int fcr_col_reduce_sum_max(const void* q, const void* k, const float* lse, float* out_sum, float* out_max,
                           int dtype, int B, int H, int M, int N, int D, const int64_t q_strides[4],
                           const int64_t k_strides[4], float scale, int causal, void* stream) {
  return col_reduce_any(q, k, lse, out_sum, out_max, kModeBoth, dtype, B, H, M, N, D, q_strides, k_strides, scale,
                        causal, stream);
}

size_t fcr_topk_bytes(int64_t rows, int N) {
  if (rows < 1 || N <= 32 * kTopkThreads || N > (1 << 30)) return 0;
  const int parts = (N + 8 * kTopkThreads - 1) / (8 * kTopkThreads);   // the finer of the two ways to cut a row
  if (rows * parts >= (1ll << 22)) return 0;   // more workgroups of 1024 threads than one launch may have
  return 2 * topk_hist_words(rows, parts) * sizeof(uint32_t) + (size_t)rows * 4 * sizeof(TopkState);
}

int fcr_topk_mask_typed(const void* scores, int dtype, uint8_t* mask, float* threshold, int64_t rows, int N, int k,
                        void* ws, size_t ws_bytes, void* stream) {
  if (!scores || !mask) return fail(FCR_E_NULL, "null pointer argument");
  if (dtype != FCR_DTYPE_F16 && dtype != FCR_DTYPE_BF16 && dtype != FCR_DTYPE_F32)
    return fail(FCR_E_DTYPE, "scores must be fp16, bf16 or fp32");
  // one workgroup of 1024 threads per row (or per part of a row), fewer than 2^32 threads per launch
  if (rows < 1 || rows >= (1ll << 22) || N < 1) return fail(FCR_E_SHAPE, "rows must be in [1, 2^22) and N >= 1");
  if (ws && (reinterpret_cast<uintptr_t>(ws) & 15) != 0)
    return fail(FCR_E_STRIDE, "the top-k workspace must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == FCR_DTYPE_F32) topk_any(static_cast<const float*>(scores), mask, threshold, rows, N, k, ws, ws_bytes, s);
  else if (dtype == FCR_DTYPE_F16) topk_any(static_cast<const _Float16*>(scores), mask, threshold, rows, N, k, ws, ws_bytes, s);
  else topk_any(static_cast<const uint16_t*>(scores), mask, threshold, rows, N, k, ws, ws_bytes, s);
  return launched("top-k kernels");
}

int fcr_topk_mask_ws(const float* scores, uint8_t* mask, float* threshold, int64_t rows, int N, int k, void* ws,
                     size_t ws_bytes, void* stream) {
  return fcr_topk_mask_typed(scores, FCR_DTYPE_F32, mask, threshold, rows, N, k, ws, ws_bytes, stream);
}

int fcr_topk_mask(const float* scores, uint8_t* mask, float* threshold, int64_t rows, int N, int k, void* stream) {
  return fcr_topk_mask_typed(scores, FCR_DTYPE_F32, mask, threshold, rows, N, k, nullptr, 0, stream);
}

int fcr_pack_f32(const float* src, void* dst, int64_t rows, int D, int terms, int is_key, void* stream) {
  if (!src || !dst) return fail(FCR_E_NULL, "null pointer argument");
  if (rows < 1 || D < 1) return fail(FCR_E_SHAPE, "rows and D must be >= 1");
  if (terms != 1 && terms != 3) return fail(FCR_E_SHAPE, "terms must be 1 or 3");
  const int dpad = (D + 7) / 8 * 8;
  if (terms * dpad > 32 * kMaxKSteps) return fail(FCR_E_SHAPE, "terms * D (padded to 8) must be <= 256");
  const int64_t n = rows * dpad;
  if ((n + 255) / 256 > 0x7fffffffll) return fail(FCR_E_SHAPE, "too many elements");
  hipLaunchKernelGGL(pack_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), src, static_cast<_Float16*>(dst), rows, D, dpad, terms,
                     is_key != 0);
  return launched("pack_f32_kernel");
}

namespace {
// A single sweep expects the whole chip: its workgroups wait for each other, one per CU.  Two of them issued on
// different streams could be dispatched side by side, each holding CUs the other needs, until their bounded
// waits run out.  So inside a process they are chained: a single sweep on another stream than the one before
// first waits (on the GPU; the host never blocks) for an event recorded at the end of that stream.  Calls that
// stay on one stream pay nothing (an event behind every call costs 5 us of a 18 us call).  Not under stream
// capture (a graph carries no such edge; graphs holding single sweeps must not replay side by side on one GPU),
// not for other processes on the same GPU, and not for fcr_colreduce_static, whose calls must not overlap anyway.
struct SweepOrder {
  hipEvent_t done = nullptr;
  hipStream_t last = nullptr;
  bool any = false;
};
SweepOrder g_order[64];
std::mutex g_order_mu;

// Takes the lock and returns the device's entry when the launch on stream s is to be chained, else nullptr.
SweepOrder* order_begin(hipStream_t s) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &st) != hipSuccess || st != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return nullptr;
  }
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
    (void)hipGetLastError();
    return nullptr;
  }
  g_order_mu.lock();
  SweepOrder* o = &g_order[dev];
  if (!o->done && hipEventCreateWithFlags(&o->done, hipEventDisableTiming) != hipSuccess) {
    (void)hipGetLastError();
    o->done = nullptr;
    g_order_mu.unlock();
    return nullptr;
  }
  if (o->any && o->last != s) {
    // (a stream that is being captured now, or was destroyed, is left alone: nothing of it can still run)
    hipStreamCaptureStatus lst = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(o->last, &lst) != hipSuccess || lst != hipStreamCaptureStatusNone ||
        hipEventRecord(o->done, o->last) != hipSuccess || hipStreamWaitEvent(s, o->done, 0) != hipSuccess)
      (void)hipGetLastError();
  }
  return o;
}
void order_end(SweepOrder* o, hipStream_t s, bool launched_it) {
  if (!o) return;
  if (launched_it) {
    o->last = s;
    o->any = true;
  }
  g_order_mu.unlock();
}

// Both sweeps of a call, writing `out` in its final form.  ws_bytes = bytes the caller's workspace is known
// to have (0: what fcr_lse_bytes asks for).  Few queries against many keys take the single sweep.
int whole_call(const void* q, const void* k, void* out, const ResultSpec& res, float* ws, size_t ws_bytes, int dtype,
               int B, int H, int M, int N, int D, const int64_t q_strides[4], const int64_t k_strides[4], float scale,
               int mode, int causal, void* stream, void* out2 = nullptr) {
  Params p;
  int rc = make_params(p, q, k, dtype, B, H, M, N, D, q_strides, k_strides, scale, true, causal != 0, mode);
  if (rc) return rc;
  const int ksteps = ksteps_of(dtype, D);
  FusedPlan f;
  if (__atomic_load_n(&g_single_sweep, __ATOMIC_RELAXED) && dtype != FCR_DTYPE_F32 && ksteps <= 4 &&
      fused_shape(p.bh_count, M, N, f) && (ws_bytes == 0 || (size_t)f.floats * sizeof(float) <= ws_bytes)) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    p.lse = ws;
    p.part = ws + f.part_at;
    p.sync = reinterpret_cast<unsigned*>(ws + f.sync_at);
    p.splits = f.splits;
    p.teams = f.teams;
    p.total = f.teams * f.splits;
    const long long polls = __atomic_load_n(&g_wait_polls, __ATOMIC_RELAXED);
    p.spin_limit = polls > 0x7fffffffll ? 0x7fffffff : (int)polls;
    p.out = out;
    p.out2 = out2;
    p.out_fmt = res.fmt;
    if (res.mean) {
      p.mean_from = causal ? p.c : N;
      p.inv_m = 1.0f / (float)M;
    }
    p.stream_once = ((int64_t)p.bh_count * N * p.dgran * 16 >= (1ll << 30)) ? 1 : 0;
    const int words = (int)(f.floats - f.part_at);   // the slots and the error word start at zero
    fcr_detail::fused_refused = false;
    SweepOrder* const order = (ws_bytes == 0) ? order_begin(s) : nullptr;
    launch_sweeps(dtype, 3, p, ksteps, causal != 0, mode | (f.qh == 2 ? 4 : 0) | (f.nq == 2 ? 8 : 0), s,
                  reinterpret_cast<unsigned*>(p.part), words);
    const int lrc = fcr_detail::fused_refused ? 0 : launched("col_fused_kernel");
    order_end(order, s, !fcr_detail::fused_refused && lrc == 0);
    if (!fcr_detail::fused_refused) return lrc;
  }
  rc = fcr_row_lse(q, k, ws, dtype, B, H, M, N, D, q_strides, k_strides, scale, causal, stream);
  if (rc) return rc;
  return col_reduce_any(q, k, ws, out, out2, mode, dtype, B, H, M, N, D, q_strides, k_strides, scale, causal, stream,
                        res);
}
}  // namespace

int fcr_colreduce_sum_max(const void* q, const void* k, float* out_sum, float* out_max, float* lse_ws, int dtype, int B,
                          int H, int M, int N, int D, const int64_t q_strides[4], const int64_t k_strides[4],
                          float scale, int causal, void* stream) {
  if (!out_sum || !out_max || !lse_ws) return fail(FCR_E_NULL, "null pointer argument");
  return whole_call(q, k, out_sum, ResultSpec(), lse_ws, 0, dtype, B, H, M, N, D, q_strides, k_strides, scale, kModeBoth,
                    causal, stream, out_max);
}

int fcr_colreduce(const void* q, const void* k, float* out, float* lse_ws, int dtype, int B, int H, int M,
                  int N, int D, const int64_t q_strides[4], const int64_t k_strides[4], float scale,
                  int reduction, int causal, void* stream) {
  if (!out || !lse_ws) return fail(FCR_E_NULL, "null pointer argument");
  if (reduction != FCR_REDUCE_SUM && reduction != FCR_REDUCE_MAX)
    return fail(FCR_E_REDUCTION, "reduction must be FCR_REDUCE_SUM or FCR_REDUCE_MAX");
  return whole_call(q, k, out, ResultSpec(), lse_ws, 0, dtype, B, H, M, N, D, q_strides, k_strides, scale,
                    reduction == FCR_REDUCE_MAX ? kModeMax : kModeSum, causal, stream);
}

// Scratch of fcr_colreduce_static: the row statistics and, for few query rows against many keys, the
// partial results of the split row sweep or the single sweep's partial values and counters.  One copy per
// GPU, held until the process ends.  Host code must not pass the array's name to a kernel (it is a
// host-side stand-in there): the device address is asked once per device and kept.
static __device__ __align__(256) unsigned char scratch[FCR_STATIC_SCRATCH_BYTES];

namespace {
int static_scratch(float** ptr) {
  static void* ptrs[64] = {};
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    snprintf(g_err, sizeof(g_err), "hipGetDevice failed: %s", hipGetErrorString(e));
    return (int)e;
  }
  if (dev < 0 || dev >= 64) return fail(FCR_E_SHAPE, "device ordinal must be below 64");
  void* p = __atomic_load_n(&ptrs[dev], __ATOMIC_ACQUIRE);
  if (!p) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));  // this device's copy of the array
    if (e != hipSuccess || !p) {
      snprintf(g_err, sizeof(g_err), "hipGetSymbolAddress(scratch) failed: %s", hipGetErrorString(e));
      return e != hipSuccess ? (int)e : (int)hipErrorInvalidSymbol;
    }
    __atomic_store_n(&ptrs[dev], p, __ATOMIC_RELEASE);
  }
  *ptr = static_cast<float*>(p);
  return 0;
}
}  // namespace

int fcr_colreduce_to(const void* q, const void* k, void* out, int out_dtype, float* lse_ws, int dtype, int B, int H,
                     int M, int N, int D, const int64_t q_strides[4], const int64_t k_strides[4], float scale,
                     int reduction, int causal, void* stream) {
  if (!out || !lse_ws) return fail(FCR_E_NULL, "null pointer argument");
  if (reduction != FCR_REDUCE_SUM && reduction != FCR_REDUCE_MAX && reduction != FCR_REDUCE_MEAN)
    return fail(FCR_E_REDUCTION, "reduction must be FCR_REDUCE_SUM, FCR_REDUCE_MAX or FCR_REDUCE_MEAN");
  if (out_dtype != FCR_DTYPE_F16 && out_dtype != FCR_DTYPE_BF16 && out_dtype != FCR_DTYPE_F32)
    return fail(FCR_E_DTYPE, "out_dtype must be FCR_DTYPE_F16, FCR_DTYPE_BF16 or FCR_DTYPE_F32");
  ResultSpec res;
  res.fmt = out_dtype;
  res.mean = reduction == FCR_REDUCE_MEAN;
  return whole_call(q, k, out, res, lse_ws, 0, dtype, B, H, M, N, D, q_strides, k_strides, scale,
                    reduction == FCR_REDUCE_MAX ? kModeMax : kModeSum, causal, stream);
}

int fcr_colreduce_sum_max_to(const void* q, const void* k, void* out_sum, void* out_max, int out_dtype, float* lse_ws,
                             int dtype, int B, int H, int M, int N, int D, const int64_t q_strides[4],
                             const int64_t k_strides[4], float scale, int sum_reduction, int causal, void* stream) {
  if (!out_sum || !out_max || !lse_ws) return fail(FCR_E_NULL, "null pointer argument");
  if (sum_reduction != FCR_REDUCE_SUM && sum_reduction != FCR_REDUCE_MEAN)
    return fail(FCR_E_REDUCTION, "sum_reduction must be FCR_REDUCE_SUM or FCR_REDUCE_MEAN");
  if (out_dtype != FCR_DTYPE_F16 && out_dtype != FCR_DTYPE_BF16 && out_dtype != FCR_DTYPE_F32)
    return fail(FCR_E_DTYPE, "out_dtype must be FCR_DTYPE_F16, FCR_DTYPE_BF16 or FCR_DTYPE_F32");
  ResultSpec res;
  res.fmt = out_dtype;
  res.mean = sum_reduction == FCR_REDUCE_MEAN;
  return whole_call(q, k, out_sum, res, lse_ws, 0, dtype, B, H, M, N, D, q_strides, k_strides, scale, kModeBoth, causal,
                    stream, out_max);
}

int fcr_colreduce_static(const void* q, const void* k, float* out, int dtype, int B, int H, int M, int N, int D,
                         const int64_t q_strides[4], const int64_t k_strides[4], float scale, int reduction,
                         int causal, void* stream) {
  if (!out) return fail(FCR_E_NULL, "null pointer argument");
  if (reduction != FCR_REDUCE_SUM && reduction != FCR_REDUCE_MAX)
    return fail(FCR_E_REDUCTION, "reduction must be FCR_REDUCE_SUM or FCR_REDUCE_MAX");
  // every argument check of the two kernels first (the last step of make_params asks the device for its
  // CU count; nothing else has touched it by then)
  Params p;
  int rc = make_params(p, q, k, dtype, B, H, M, N, D, q_strides, k_strides, scale, false, causal != 0);
  if (rc) return rc;
  const size_t need = fcr_lse_bytes(B, H, M, N, D);
  if (need > (size_t)FCR_STATIC_SCRATCH_BYTES) {
    snprintf(g_err, sizeof(g_err),
             "fcr_colreduce_static: this problem needs %zu bytes of scratch, the built-in buffer has %zu; "
             "use fcr_colreduce with a caller-provided buffer",
             need, (size_t)FCR_STATIC_SCRATCH_BYTES);
    return FCR_E_SCRATCH;
  }
  float* ws = nullptr;
  rc = static_scratch(&ws);
  if (rc) return rc;
  // The kernels write every value of the buffer they later read (the single sweep's counters are cleared by
  // a small kernel in front of it), so nothing has to be cleared here.
  return fcr_colreduce(q, k, out, ws, dtype, B, H, M, N, D, q_strides, k_strides, scale, reduction, causal, stream);
}

int fcr_set_option(int option, long long value) {
  if (option == FCR_OPT_SINGLE_SWEEP) {
    __atomic_store_n(&g_single_sweep, value != 0 ? 1 : 0, __ATOMIC_RELAXED);
    return 0;
  }
  if (option == FCR_OPT_WAIT_POLLS) {
    if (value < 0) return fail(FCR_E_SHAPE, "FCR_OPT_WAIT_POLLS must be >= 0");
    __atomic_store_n(&g_wait_polls, value, __ATOMIC_RELAXED);
    return 0;
  }
  return fail(FCR_E_SHAPE, "unknown option");
}

int fcr_colreduce_status(const float* lse_ws, int dtype, int B, int H, int M, int N, int D, void* stream) {
  if (!lse_ws) return fail(FCR_E_NULL, "null pointer argument");
  if (B < 1 || H < 1 || M < 1 || N < 1 || D < 1) return fail(FCR_E_SHAPE, "B, H, M, N, D must be >= 1");
  FusedPlan f;
  if (dtype == FCR_DTYPE_F32 || ksteps_of(dtype, D) > 4 || !fused_shape((int64_t)B * H, M, N, f)) return 0;
  unsigned word = 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipError_t e = hipMemcpyAsync(&word, reinterpret_cast<const unsigned*>(lse_ws + f.sync_at), sizeof(word),
                                hipMemcpyDeviceToHost, s);
  if (e == hipSuccess) e = hipStreamSynchronize(s);
  if (e != hipSuccess) {
    snprintf(g_err, sizeof(g_err), "reading the status word failed: %s", hipGetErrorString(e));
    return (int)e;
  }
  if (word != 0) return fail(FCR_E_WAIT, "a workgroup of the single sweep gave up waiting for its team; the columns of that (b,h) pair are NaN");
  return 0;
}

}  // extern "C"
#endif  // FCR_HAS(0)
