// Per-rank data path of the ring allreduce / allgather for MI355X (gfx950).
//
// Hand-written HIP kernels behind the C ABI of include/ring_abi.h. They take
// the place of the reference's device primitives
// (tensorflow/contrib/mpi_collectives/ring.cu.cc:41-69): the D2D copy, and
// elemwise_accum<<<32,256>>> followed by a host-blocking stream sync at every
// ring step.
//
// Design, in the order it matters for an HBM-bound stream:
//   * every lane moves 16 bytes per access (global_load/store_dwordx4), a
//     wave64 touches 1 KiB of contiguous memory per instruction;
//   * a workgroup is 4 waves; one tile is 4 x 256 x 16 B = 16 KiB per operand,
//     all loads of a tile are issued before the first add/store, so each wave
//     keeps 8 KiB in flight;
//   * one launch carries a whole step table (up to 64 rows by value in the
//     kernel arguments), so the n-1 accumulates (or copies) of a rank are one
//     launch, not n-1 launches and n-1 host syncs. Rows with equal tile counts
//     (the segments of an allreduce) use a 2-D grid (tiles, rows); unequal rows
//     share a 1-D grid and a workgroup finds its row by a scalar binary search;
//   * stores are aligned: a scalar head is peeled per row so that the
//     destination starts on a 128-byte line (16 bytes in the fold and fusion
//     kernels), the sources are read with element-aligned (possibly
//     16-byte-unaligned) dwordx4 loads. Ragged segment starts only cost those
//     few scalar elements;
//   * a copy runs faster when the chip reads first and writes after than with
//     the two directions interleaved: the copies of an allgather phase wait
//     for all their loads before their first store when every tile is resident
//     at once (the paced tiles), and from 31 MiB (unless those tiles fill the
//     CUs evenly) they hold the whole payload of the launch in registers, one
//     or two workgroups per CU (rows_phased_kernel). The unpack of a fused
//     buffer of 1-112 MiB runs the same way (unpack_phased_kernel).
//     Accumulates and folds, which read more than they write, gain nothing from it;
//   * what is touched once (accumulates, allgather copies, unpack) is loaded
//     and stored non-temporally; the in->out copy and the fusion pack, whose
//     output the reduce-scatter reads next, store with the ordinary policy;
//   * the average's divide rides on the accumulate that completes a segment
//     (or on the unpack), never on a pass of its own;
//   * LDS is used only by the fusion kernels, for the offset table of a tile
//     that spans several small tensors (and, in the unpack that holds its
//     payload in registers, for where each round of a workgroup goes).
// No MFMA: the path is one add per 12 bytes.

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <atomic>
#include <mutex>
#include <new>
#include <type_traits>
#include <vector>

#include "ring_abi.h"

namespace {

constexpr int kBlock = 256;   // threads per workgroup: 4 wave64
constexpr int kMaxRows = 64;  // rows one launch carries in its kernel arguments
// The scalar head of a step-table row brings its destination to a whole
// 128-byte line, so that the 1 KiB a wave stores per access covers whole lines
// (a 16-byte-aligned start would split a 32-byte sector at both ends of every
// access: 3 % more sectors written, and partial ones).
constexpr int kRowHeadAlign = 128;
constexpr int kPacedUnroll = 8;  // vectors per lane per tile of the paced copy (32 KiB tiles)

thread_local int g_last_hip_error = 0;
// Events the next kernel launches of this thread record their own begin and
// end into (ring_time_next_launch): a short queue, one pair per armed launch,
// taken in order by the launches that follow.
constexpr int kMaxArmedLaunches = 8;
struct ArmedLaunch { hipEvent_t start, stop; };
thread_local ArmedLaunch g_armed[kMaxArmedLaunches];
thread_local int g_armed_head = 0, g_armed_count = 0;

// Every kernel launch of the library goes through here. A launch armed by
// ring_time_next_launch carries its events in the dispatch itself, so they
// bracket the kernel's execution and nothing else.
template <typename... Params, typename... Args>
inline void launch(void (*kernel)(Params...), dim3 grid, dim3 block, hipStream_t stream, Args... args) {
  if (g_armed_count > 0) {
    const ArmedLaunch a = g_armed[g_armed_head];
    g_armed_head = (g_armed_head + 1) % kMaxArmedLaunches;
    --g_armed_count;
    hipExtLaunchKernelGGL(kernel, grid, block, 0, stream, a.start, a.stop, 0, args...);
  } else {
    hipLaunchKernelGGL(kernel, grid, block, 0, stream, args...);
  }
}

inline int hip_fail(hipError_t e) {
  g_last_hip_error = static_cast<int>(e);
  return RING_ERR_HIP;
}
#define RING_HIP(call)                                   \
  do {                                                   \
    hipError_t e_ = (call);                              \
    if (e_ != hipSuccess) return hip_fail(e_);           \
  } while (0)

// ---- element / vector types -------------------------------------------------
// A lane moves 16 bytes per access. Integers are ADDED as unsigned so overflow
// wraps (what the reference's hardware add does) instead of being undefined;
// they are DIVIDED as signed (floor division of the average).

template <typename T> struct VecOf;
template <> struct VecOf<float> { typedef float type __attribute__((ext_vector_type(4))); };
template <> struct VecOf<uint32_t> { typedef uint32_t type __attribute__((ext_vector_type(4))); };
template <> struct VecOf<uint64_t> { typedef uint64_t type __attribute__((ext_vector_type(2))); };
template <> struct VecOf<int32_t> { typedef int32_t type __attribute__((ext_vector_type(4))); };
template <> struct VecOf<int64_t> { typedef int64_t type __attribute__((ext_vector_type(2))); };

// The divide of allreduce(average=True): tf.div semantics (__init__.py:160-164
// of the reference): true division for float32 (a correctly rounded divide,
// NOT a multiply by 1/n), floor division for the integer types. n > 0, so
// floor differs from C's truncation only for negative x with a remainder.
// By a power of two the quotient is the same real number as the product with
// the (exact) reciprocal, so the one rounding gives the same bits, subnormal
// results included, without the divide's dozen instructions (n is uniform).
__device__ __forceinline__ float div_one(float x, int n) {
  if ((n & (n - 1)) == 0) return x * (1.0f / static_cast<float>(n));
  return x / static_cast<float>(n);
}
__device__ __forceinline__ int32_t div_one(int32_t x, int n) {
  const int32_t q = x / n;
  return q - ((x % n != 0) && (x < 0));
}
__device__ __forceinline__ int64_t div_one(int64_t x, int n) {
  const int64_t q = x / n;
  return q - ((x % n != 0) && (x < 0));
}
// never instantiated for the unsigned carrier types; present so templates compile
__device__ __forceinline__ uint32_t div_one(uint32_t x, int) { return x; }
__device__ __forceinline__ uint64_t div_one(uint64_t x, int) { return x; }

// The add of the accumulate; signed integers wrap like the unsigned carriers.
__device__ __forceinline__ float add_one(float a, float b) { return b + a; }
__device__ __forceinline__ uint32_t add_one(uint32_t a, uint32_t b) { return b + a; }
__device__ __forceinline__ uint64_t add_one(uint64_t a, uint64_t b) { return b + a; }
__device__ __forceinline__ int32_t add_one(int32_t a, int32_t b) {
  return static_cast<int32_t>(static_cast<uint32_t>(b) + static_cast<uint32_t>(a));
}
__device__ __forceinline__ int64_t add_one(int64_t a, int64_t b) {
  return static_cast<int64_t>(static_cast<uint64_t>(b) + static_cast<uint64_t>(a));
}

// kOpCopy: dst = a.  kOpAdd: dst = b + a (b may be dst itself: the in-place
// accumulate of the reference).  kOpDiv: dst = a / n (a may be dst itself).
// kOpAddDiv: dst = (b + a) / n, the last accumulate of an averaged allreduce:
// the sum is rounded exactly as kOpAdd rounds it and then divided exactly as
// kOpDiv divides it, so the result equals the two passes done separately.
enum Op { kOpCopy = 0, kOpAdd = 1, kOpDiv = 2, kOpAddDiv = 3 };

template <typename T, int OP>
__device__ __forceinline__ T apply_one(T a, T b, int n) {
  if (OP == kOpAdd) return add_one(a, b);
  if (OP == kOpDiv) return div_one(a, n);
  if (OP == kOpAddDiv) return div_one(add_one(a, b), n);
  return a;
}
template <typename T, int OP>
__device__ __forceinline__ typename VecOf<T>::type apply_vec(typename VecOf<T>::type a, typename VecOf<T>::type b, int n) {
  if (OP == kOpCopy) return a;
#pragma unroll
  for (uint32_t c = 0; c < 16 / sizeof(T); c++) a[c] = apply_one<T, OP>(a[c], b[c], n);
  return a;
}

// Launch modes of rows_kernel. kCopy: every row is a copy. kAdd: a row with a
// second operand is an add, a row without one is still a copy, so one launch
// can mix both. kAvg: as kAdd on the signed element types, and the rows whose
// bit is set in the table's div_mask also divide by the table's divisor.
enum Mode { kCopy = 0, kAdd = 1, kAvg = 2 };

// Rows of one launch, passed by value in the kernel arguments (read with
// scalar loads; uniform per workgroup).
struct Row {
  void* dst;
  const void* a;   // incoming segment
  const void* b;   // local operand of an add row, null for a copy row
  uint64_t count;  // elements
};
template <int MAXROWS>
struct RowTableT {
  int n_rows;
  int dry;  // measurement only: every workgroup returns at once
  // > 0: every row has this many tiles and the grid is (tiles, rows), so a
  // workgroup reads its row straight from blockIdx.y (the n-1 near-equal
  // segments of an allreduce). 0: rows differ; the grid is 1-D over all tiles
  // and a workgroup finds its row by binary search over tile_begin.
  uint32_t uniform_tiles;
  int divisor;                        // kAvg only
  uint64_t div_mask;                  // kAvg only: bit k set = row k divides
  uint32_t tile_begin[MAXROWS + 1];  // prefix sum of tiles per row
  Row row[MAXROWS];
};
typedef RowTableT<kMaxRows> RowTable;
// The same table with room for 8 rows (the 7 segments of an 8-rank phase): 320
// bytes of kernel arguments instead of 2.3 KB. What a launch costs the host
// grows with the size of its arguments (a stream of empty kernels: 2.4 us per
// launch at 24 bytes, 2.5 at 264, 3.0 at 648, 4.5 from 1.3 KB on), and a step on
// a small tensor costs what its launches cost the host: the three launches of a
// 1 MiB, 8-rank step driven from C++ take 8.2 us instead of 8.8 (12.0 instead
// of 13.4 on a slower host). The fold kernel gained nothing from a small table
// (its one launch per step is bound by the GPU's side of a dispatch, 3.9 us).
constexpr int kSmallRows = 8;
typedef RowTableT<kSmallRows> SmallRowTable;

// NT: bit 0 = non-temporal stores, bit 1 = non-temporal loads (3, both, is the
// default: every byte is touched once).
// Device global memory, as a type qualifier.
#define RING_GLOBAL __attribute__((address_space(1)))

// Macros, not function templates: the operand's type may carry a reduced
// alignment (element-aligned 16-byte accesses) that template deduction would drop.
#define RING_LOAD_VEC(NT, p) (((NT) & 2) ? __builtin_nontemporal_load(p) : *(p))
#define RING_STORE_VEC(NT, p, v)                            \
  do {                                                      \
    if ((NT) & 1) __builtin_nontemporal_store((v), (p));    \
    else *(p) = (v);                                        \
  } while (0)

// Blocks the wave until every vector-memory access it has issued is complete.
// (A build for another target, which has no such instruction, defines the macro
// before this point.)
#ifndef RING_WAIT_VMEM
#define RING_WAIT_VMEM() asm volatile("s_waitcnt vmcnt(0)" ::: "memory")
#endif

// Which side of a row the scalar head brings to 16-byte alignment.
enum Anchor { kOnDst = 0, kOnSrc = 1 };

// One workgroup-tile of a row: 256 * UNROLL 16-byte vectors of the row's body,
// plus the row's scalar head (tile 0) and tail (last tile). ANCHOR picks the
// side the head aligns: the destination (aligned stores, element-aligned loads
// of a and b), or the source a (aligned loads of a, element-aligned stores:
// rows whose source is known to be aligned, the tiles of an unpack, which then
// need no head at all and stay full tiles). a == dst (divide) and b == dst
// (add) are allowed: every element is read before it is written, by the same
// lane. PACE: a full tile waits until all its loads have arrived, then keeps
// one store in flight per wave. With every tile of a launch resident at the
// same time the chip then reads first and writes after, which HBM serves
// faster than the two interleaved; the launcher picks it for those launches
// only (a tile that has to wait for a free slot would pay for the short store queue).
template <typename T, int OP, int UNROLL, int NT, int ANCHOR = kOnDst, int PACE = 0, int HEAD_ALIGN = 16>
__device__ __forceinline__ void row_tile(T* dst_, const T* a_, const T* b_, uint64_t count, uint32_t tile,
                                         uint32_t tiles_in_row, int n) {
  typedef typename VecOf<T>::type V;
  typedef V VU __attribute__((aligned(sizeof(T))));  // element-aligned 16-byte access
  // Every operand is device global memory. Said explicitly: a pointer that was
  // itself read from memory (a fusion plan's tensor table) is otherwise taken
  // for a generic one and accessed with flat instructions.
  typedef T RING_GLOBAL GT;
  typedef V RING_GLOBAL GV;
  typedef VU RING_GLOBAL GVU;
  GT* dst = (GT*)dst_;
  const GT* a = (const GT*)a_;
  const GT* b = (const GT*)b_;
  constexpr uint32_t VEC = 16 / sizeof(T);
  constexpr uint32_t kTileVecs = kBlock * UNROLL;

  const uintptr_t anchor = ANCHOR == kOnSrc ? reinterpret_cast<uintptr_t>(a_) : reinterpret_cast<uintptr_t>(dst_);
  constexpr uint32_t kAlign = HEAD_ALIGN;  // 16, or a whole 128-byte line (at most 31 scalar elements, fewer than a workgroup has lanes)
  uint64_t head = ((kAlign - (static_cast<uint32_t>(anchor) & (kAlign - 1))) & (kAlign - 1)) / sizeof(T);
  if (head > count) head = count;
  const uint64_t nvec = (count - head) / VEC;
  const uint32_t tid = threadIdx.x;

  constexpr bool kTwo = OP == kOpAdd || OP == kOpAddDiv;  // reads b as well
  if (tile == 0 && tid < head) dst[tid] = apply_one<T, OP>(a[tid], kTwo ? b[tid] : T(), n);
  if (tile + 1 == tiles_in_row) {
    const uint64_t e = head + nvec * VEC + tid;
    if (e < count) dst[e] = apply_one<T, OP>(a[e], kTwo ? b[e] : T(), n);
  }

  // The tile's vectors through pointers that are uniform over the workgroup
  // plus a 32-bit lane offset (scalar base + vector offset: one address
  // register per operand). Access j of the workgroup covers 4 KiB of
  // consecutive memory, lane after lane (measured faster than giving every
  // wave 4 KiB of its own). The anchored side goes through the aligned vector
  // type, the other through the element-aligned one (spelled out: an alignment
  // attribute does not survive a template).
  const uint64_t tile_base = static_cast<uint64_t>(tile) * kTileVecs;
  if (tile_base >= nvec) return;
  const uint64_t left = nvec - tile_base;  // vectors from this tile on
  GV* dv_al = (GV*)(dst + head) + tile_base;
  GVU* dv_un = (GVU*)(dst + head) + tile_base;
  const GV* av_al = (const GV*)(a + head) + tile_base;
  const GVU* av_un = (const GVU*)(a + head) + tile_base;
  const GVU* bv = kTwo ? (const GVU*)(b + head) + tile_base : nullptr;
  const uint32_t v0 = tid;
#define ROW_LOAD_A(i) (ANCHOR == kOnSrc ? RING_LOAD_VEC(NT, &av_al[i]) : RING_LOAD_VEC(NT, &av_un[i]))
#define ROW_STORE(i, v)                                      \
  do {                                                       \
    if (ANCHOR == kOnDst) RING_STORE_VEC(NT, &dv_al[i], v);  \
    else RING_STORE_VEC(NT, &dv_un[i], v);                   \
  } while (0)

  if (left >= kTileVecs) {
    // access j through a base that is uniform over the workgroup (scalar
    // registers) and the one lane offset every access shares
    V x[UNROLL], y[UNROLL];
#pragma unroll
    for (int j = 0; j < UNROLL; j++)
      x[j] = ANCHOR == kOnSrc ? RING_LOAD_VEC(NT, &(av_al + j * kBlock)[v0]) : RING_LOAD_VEC(NT, &(av_un + j * kBlock)[v0]);
    if (kTwo) {
#pragma unroll
      for (int j = 0; j < UNROLL; j++) y[j] = RING_LOAD_VEC(NT, &(bv + j * kBlock)[v0]);
    }
#pragma unroll
    for (int j = 0; j < UNROLL; j++) x[j] = apply_vec<T, OP>(x[j], kTwo ? y[j] : x[j], n);
    if (PACE) RING_WAIT_VMEM();
#pragma unroll
    for (int j = 0; j < UNROLL; j++) {
      if (ANCHOR == kOnDst) RING_STORE_VEC(NT, &(dv_al + j * kBlock)[v0], x[j]);
      else RING_STORE_VEC(NT, &(dv_un + j * kBlock)[v0], x[j]);
      if (PACE) RING_WAIT_VMEM();
    }
  } else {
    // the one partial tile of a row. (rem is taken here, where left < kTileVecs
    // is known, rather than as min(left, kTileVecs) ahead of the branch: hipcc
    // 7.2 lowers that 64-bit uniform min to a scalar select on a stale
    // condition code, and every lane of the partial tile then runs.)
    const uint32_t rem = static_cast<uint32_t>(left);
#pragma unroll
    for (int j = 0; j < UNROLL; j++) {
      const uint32_t v = v0 + j * kBlock;
      if (v < rem) {
        V x = ROW_LOAD_A(v);
        V y = x;
        if (kTwo) y = RING_LOAD_VEC(NT, &bv[v]);
        const V r = apply_vec<T, OP>(x, y, n);
        ROW_STORE(v, r);
      }
    }
  }
#undef ROW_LOAD_A
#undef ROW_STORE
}

template <typename T, int MODE, int UNROLL, int NT, int PACE = 0>
__device__ __forceinline__ void run_row(const Row& r, uint32_t tile, uint32_t tiles, int divisor, bool divide) {
  T* dst = static_cast<T*>(r.dst);
  const T* a = static_cast<const T*>(r.a);
  const T* b = static_cast<const T*>(r.b);
  // every condition is uniform over the workgroup (kernel arguments only)
  if (MODE == kAvg && divide) {
    if (b != nullptr) row_tile<T, kOpAddDiv, UNROLL, NT, kOnDst, 0, kRowHeadAlign>(dst, a, b, r.count, tile, tiles, divisor);
    else row_tile<T, kOpDiv, UNROLL, NT, kOnDst, 0, kRowHeadAlign>(dst, a, nullptr, r.count, tile, tiles, divisor);
  } else if (MODE != kCopy && b != nullptr) {
    row_tile<T, kOpAdd, UNROLL, NT, kOnDst, 0, kRowHeadAlign>(dst, a, b, r.count, tile, tiles, 0);
  } else {
    row_tile<T, kOpCopy, UNROLL, NT, kOnDst, PACE, kRowHeadAlign>(dst, a, nullptr, r.count, tile, tiles, 0);
  }
}

// The row a tile of a 1-D grid belongs to: the number of rows that begin at or
// before it, minus one. begin[] lies in the kernel arguments and its entries
// past the last row hold 0xffffffff, so the count is a straight run of scalar
// compares on values fetched side by side, not a binary search whose every
// step waits for a load of its own (six in a row for 64 rows, at the start of
// every workgroup). Uniform over the workgroup.
template <int MAX_ROWS>
__device__ __forceinline__ int row_of_tile(const uint32_t* begin, int n_rows, uint32_t t) {
  int row = 0;
  constexpr int kShort = MAX_ROWS < 16 ? MAX_ROWS : 16;
  if (n_rows <= kShort) {
#pragma unroll
    for (int k = 1; k < kShort; k++) row += begin[k] <= t ? 1 : 0;
  } else {
#pragma unroll
    for (int k = 1; k < MAX_ROWS; k++) row += begin[k] <= t ? 1 : 0;
  }
  return row;
}

// The kernel's body, textually in each of the two kernels below (as a function
// that takes the table by reference the paced copy compiled to per-lane 64-bit
// addresses and ran 12 % slower).
#define RING_ROWS_KERNEL_BODY(MAXROWS, UNROLL, PACE)                                                              \
  if (tab.dry) return;                                                                                            \
  if (tab.uniform_tiles) {                                                                                        \
    const Row r = tab.row[blockIdx.y]; /* one scalar load, no search */                                           \
    const bool divide = MODE == kAvg && ((tab.div_mask >> blockIdx.y) & 1u);                                      \
    for (uint32_t t = blockIdx.x; t < tab.uniform_tiles; t += gridDim.x)                                          \
      run_row<T, MODE, UNROLL, NT, PACE>(r, t, tab.uniform_tiles, tab.divisor, divide);                           \
    return;                                                                                                       \
  }                                                                                                               \
  const uint32_t total = tab.tile_begin[tab.n_rows];                                                              \
  for (uint32_t t = blockIdx.x; t < total; t += gridDim.x) {                                                      \
    const int lo = row_of_tile<MAXROWS>(tab.tile_begin, tab.n_rows, t);                                           \
    const uint32_t first = tab.tile_begin[lo];                                                                    \
    run_row<T, MODE, UNROLL, NT, PACE>(tab.row[lo], t - first, tab.tile_begin[lo + 1] - first, tab.divisor,       \
                                       MODE == kAvg && ((tab.div_mask >> lo) & 1u));                              \
  }

template <typename T, int MODE, int UNROLL, int NT, int PACE = 0>
__global__ void __launch_bounds__(kBlock) rows_kernel(const RowTable tab) {
  RING_ROWS_KERNEL_BODY(kMaxRows, UNROLL, PACE)
}

// The same kernel (4 vectors per lane, plain tiles) on the 8-row table.
template <typename T, int MODE, int NT>
__global__ void __launch_bounds__(kBlock) rows_kernel_small(const SmallRowTable tab) {
  RING_ROWS_KERNEL_BODY(kSmallRows, 4, 0)
}
#undef RING_ROWS_KERNEL_BODY

// The copies of an allgather phase as ONE read phase and ONE write phase of the
// whole chip, the payload held in registers in between. One workgroup per CU,
// every one resident (512 registers per lane leave room for one wave per
// SIMD). The chip sweeps the rows one after the other, front to back: a lane
// takes vectors base, base + stride, ... of a row's body (stride = workgroups
// * 256), issues the loads of all rows, waits for the last, and stores in the
// same order. HBM serves one direction at a time faster than the two
// interleaved: measured stand-alone, a copy of 56-112 MiB runs at 76-79 % of
// the roofline this way against 72-74 % as plain tiles; in a step, behind the
// accumulate, the 7 ragged 12.2 MiB segments of the ResNet-50 set take 29.4 us
// instead of 31.2 (76 %) and 5 int64 segments of 12.7 MiB 22.8 instead of 24.2.
// What such a launch costs is its number of rounds (the most vectors any lane
// takes), not its bytes: a row whose last round is a tenth full costs a whole
// round. So the workgroup that takes the first 256 vectors of a row is not
// workgroup 0 but the one after the last workgroup of the previous row's
// last round (shift[row], set by the host): the rounds of successive rows
// chain, every lane takes the same number of vectors to within one, and the
// sweep over memory never restarts. Sweeping the rows side by side instead
// (a grid of (x, rows)) ran 10-20 % slower than plain tiles. For the same
// reason a row's scalar head and tail travel in registers like the rest: a
// load, a wait and a store ahead of the loads held workgroup 0 back by a
// memory latency per row, and the whole launch with it (32.5 us instead of 29.4).
// ROWS is a template parameter so that a register's row is known at compile
// time and the rows' pointers stay in scalar registers; a row has room for
// kPhasedMax / ROWS vectors per lane.
constexpr int kPhasedMax = 112;
constexpr int kPhasedMaxTwoWaves = 40;  // of a lane's 256 registers, with room for the rows' pointers and edges
struct PhasedShape {
  uint32_t rounds;             // most rounds any row needs (at most a row's share of the lane's vectors)
  uint32_t shift[kSmallRows];  // the workgroup that starts row k
};
#ifndef RING_WAVES_PER_SIMD
#define RING_WAVES_PER_SIMD(n) __attribute__((amdgpu_waves_per_eu(n, n)))
#endif
// WAVES: workgroups per CU (waves per SIMD). 1: 112 vectors per lane, the form
// for 56-112 MiB. 2: twice the workgroups with 56 vectors per lane each, for
// smaller launches, which want more loads in flight per CU than one wave per
// SIMD issues in the few rounds they have.
template <typename T, int ROWS, int WAVES>
__global__ void __launch_bounds__(kBlock) RING_WAVES_PER_SIMD(WAVES)
rows_phased_kernel(const SmallRowTable tab, const PhasedShape shape) {
  if (tab.dry) return;
  typedef typename VecOf<T>::type V;
  typedef V VU __attribute__((aligned(sizeof(T))));
  typedef T RING_GLOBAL GT;
  typedef V RING_GLOBAL GV;
  typedef VU RING_GLOBAL GVU;
  constexpr uint32_t VEC = 16 / sizeof(T);
  constexpr int PER = (WAVES == 1 ? kPhasedMax : kPhasedMaxTwoWaves) / ROWS;
  const uint32_t tid = threadIdx.x;
  const uint32_t stride = gridDim.x * kBlock;
  V s[ROWS * PER];
  T edge_head[ROWS], edge_tail[ROWS];
  // where a row's body starts and how many vectors it has (uniform)
  auto head_of = [](const Row& r) {
    uint64_t head = ((kRowHeadAlign - (static_cast<uint32_t>(reinterpret_cast<uintptr_t>(r.dst)) & (kRowHeadAlign - 1))) &
                     (kRowHeadAlign - 1)) / sizeof(T);
    return head > r.count ? r.count : head;
  };
  // the lane's first vector of row k: the workgroups take the row in the order shift[k], shift[k] + 1, ...
  auto first_of = [&](int k) {
    uint32_t w = blockIdx.x + gridDim.x - shape.shift[k];
    if (w >= gridDim.x) w -= gridDim.x;
    return w * kBlock + tid;
  };
#pragma unroll
  for (int k = 0; k < ROWS; k++) {
    const Row r = tab.row[k];
    const uint64_t head = head_of(r);
    const uint32_t nvec = static_cast<uint32_t>((r.count - head) / VEC);
    const GT* a = (const GT*)static_cast<const T*>(r.a);
    if (blockIdx.x == 0) {
      // the row's scalar head and tail travel in registers too: a load, a wait and a store here
      // would hold workgroup 0 back by a memory latency per row, and the launch ends with its last workgroup
      if (tid < head) edge_head[k] = a[tid];
      const uint64_t e = head + static_cast<uint64_t>(nvec) * VEC + tid;
      if (e < r.count) edge_tail[k] = a[e];
    }
    const GVU* av = (const GVU*)(a + head);
    const uint32_t base = first_of(k);
#pragma unroll
    for (int j = 0; j < PER; j++) {
      if (static_cast<uint32_t>(j) < shape.rounds) {
        if (base + j * stride < nvec) s[k * PER + j] = __builtin_nontemporal_load(&(av + j * stride)[base]);
      }
    }
  }
  RING_WAIT_VMEM();
#pragma unroll
  for (int k = 0; k < ROWS; k++) {
    const Row r = tab.row[k];
    const uint64_t head = head_of(r);
    const uint32_t nvec = static_cast<uint32_t>((r.count - head) / VEC);
    GV* dv = (GV*)((GT*)static_cast<T*>(r.dst) + head);
    const uint32_t base = first_of(k);
#pragma unroll
    for (int j = 0; j < PER; j++) {
      if (static_cast<uint32_t>(j) < shape.rounds) {
        if (base + j * stride < nvec) __builtin_nontemporal_store(s[k * PER + j], &(dv + j * stride)[base]);
      }
    }
    if (blockIdx.x == 0) {
      GT* dst = (GT*)static_cast<T*>(r.dst);
      if (tid < head) dst[tid] = edge_head[k];
      const uint64_t e = head + static_cast<uint64_t>(nvec) * VEC + tid;
      if (e < r.count) dst[e] = edge_tail[k];
    }
  }
}

// Byte copy for operands that are not 4-byte compatible (never produced by the
// three element types; kept so ring_copy_bytes is total).
__global__ void __launch_bounds__(kBlock) bytes_kernel(uint8_t* __restrict__ dst,
                                                       const uint8_t* __restrict__ src, uint64_t n) {
  for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n;
       i += static_cast<uint64_t>(gridDim.x) * kBlock)
    dst[i] = src[i];
}

// Measurement only (ring_probe_stream): ONE direction of a copy launch, in the
// tile shape of rows_kernel (256 lanes x 4 vectors of 16 bytes, one workgroup
// per tile, grid (tiles, rows)): every lane loads its four vectors and stores
// nothing, or stores four vectors and loads nothing. What the chip gives one
// direction at a given size is the floor of a copy of that size, which runs no
// faster than its two directions one after the other. count: 16-byte vectors.
template <int WRITE, int NT>
__global__ void __launch_bounds__(kBlock) stream_probe_kernel(const SmallRowTable tab) {
  typedef VecOf<uint32_t>::type V;
  typedef V RING_GLOBAL GV;
  const Row r = tab.row[blockIdx.y];
  const uint64_t base = static_cast<uint64_t>(blockIdx.x) * (kBlock * 4);
  if (base >= r.count) return;
  const uint64_t left = r.count - base;
  const uint32_t tid = threadIdx.x;
  if (WRITE) {
    GV* d = (GV*)static_cast<uint32_t*>(r.dst) + base;
    const V v = {1u, 2u, 3u, tid};
#pragma unroll
    for (uint32_t j = 0; j < 4; j++)
      if (tid + j * kBlock < left) RING_STORE_VEC(NT ? 1 : 0, &d[tid + j * kBlock], v);
  } else {
    const GV* a = (const GV*)static_cast<const uint32_t*>(r.a) + base;
    V x[4];
#pragma unroll
    for (uint32_t j = 0; j < 4; j++) {
      x[j] = V{0u, 0u, 0u, 0u};
      if (tid + j * kBlock < left) x[j] = RING_LOAD_VEC(NT ? 2 : 0, &a[tid + j * kBlock]);
    }
    const V acc = x[0] ^ x[1] ^ x[2] ^ x[3];
    // keeps the loads alive; four given words out of 2^128, and then the store goes where the loads came from
    if (acc[0] == 0x9e3779b9u && acc[1] == 0x7f4a7c15u && acc[2] == 0xf39cc060u && acc[3] == 0x5cedc834u)
      ((GV*)static_cast<const uint32_t*>(r.a))[base + tid] = acc;
  }
}

// ---- fold: a segment reduced in one pass, in ring order ---------------------------
// The ring leaves in segment s the left fold acc = x_s; acc = x_{s+1} + acc; ...
// over the ranks in ring order (ring.h:183-205 unrolled over its n-1 steps).
// Where every rank's copy of the segment is addressable at once (all ranks on
// one GPU, or peers that pushed their copies into staging slots over their own
// links) the owner computes that fold directly: m reads and one write per
// element instead of 3(m-1) accesses, the same additions in the same order.

constexpr int kMaxFoldRows = 32;
constexpr int kMaxFoldPtrs = 256;
// Tile shape, from a sweep on 8 sources of 8 MiB (the 64 MiB, N=8 segment):
// 2 vectors per lane per source with the loads of 8 sources in flight at once
// took 12.7 us; 4 sources at once 13.1; 1 vector per lane 14.2-14.9; 4 vectors
// per lane (half as many workgroups) 17.3-18.0.
constexpr int kFoldUnroll = 2;
constexpr int kFoldGroup = 8;
// A fold that stores its result to every rank (8 sources, 8 destinations of
// 64 MiB): 1 vector per lane 194 us, 2 vectors 199 us, 4 vectors 213 us.
constexpr int kFoldToAllUnroll = 1;

struct FoldRow {
  void* dst;
  uint64_t count;      // elements
  uint32_t first_ptr;  // index of the row's first source in FoldTable::src
  uint32_t m;          // sources, folded in the order they are listed; 1 = a copy row
  uint32_t first_dst;  // index in FoldTable::src of the row's further destinations
  uint32_t n_more;     // how many: the result is stored to dst and to each of them
};
struct FoldTable {
  int n_rows;
  int divisor;             // > 0: rows whose bit is set in div_mask are divided (tf.div) before they are stored
  uint32_t div_mask;
  uint32_t uniform_tiles;  // as RowTable
  uint32_t tile_begin[kMaxFoldRows + 1];
  FoldRow row[kMaxFoldRows];
  const void* src[kMaxFoldPtrs];  // the rows' sources, and their further destinations
};

// One tile of a fold row. dst may be one of the row's own sources: a lane reads
// every source of its elements before it stores them. DIV && divide: the fold
// is divided by n before it is stored (divide is uniform over the workgroup).
// more[0..n_more): further destinations of the same result (every rank's copy
// of a finished segment, written by the owner's fold instead of being copied
// from it afterwards); they may be sources of the row too, and need only be
// element-aligned. MORE_UNDIVIDED: they take the fold as it is and only dst the
// quotient (a rank's finished segment: the sum goes on the wire, the average
// into the rank's own tensors).
template <typename T, int UNROLL, int GROUP, bool DIV, int NT, bool MORE_UNDIVIDED = false>
__device__ __forceinline__ void fold_tile(T* dst, const void* const* src, int m, uint64_t count, uint32_t tile,
                                          uint32_t tiles_in_row, int n, bool divide,
                                          const void* const* more = nullptr, int n_more = 0) {
  typedef typename VecOf<T>::type V;
  typedef V VU __attribute__((aligned(sizeof(T))));
  constexpr uint32_t VEC = 16 / sizeof(T);
  constexpr uint32_t kTileVecs = kBlock * UNROLL;
  constexpr int kGroup = GROUP;  // sources whose loads are issued together

  uint64_t head = ((16u - (static_cast<uint32_t>(reinterpret_cast<uintptr_t>(dst)) & 15u)) & 15u) / sizeof(T);
  if (head > count) head = count;
  const uint64_t nvec = (count - head) / VEC;
  const uint32_t tid = threadIdx.x;

  // scalar head (tile 0) and tail (last tile)
  auto scalar = [&](uint64_t e) {
    T acc = static_cast<const T*>(src[0])[e];
    for (int k = 1; k < m; k++) acc = add_one(acc, static_cast<const T*>(src[k])[e]);
    const T r = (DIV && divide) ? div_one(acc, n) : acc;
    dst[e] = r;
    for (int d = 0; d < n_more; d++) static_cast<T*>(const_cast<void*>(more[d]))[e] = MORE_UNDIVIDED ? acc : r;
  };
  if (tile == 0 && tid < head) scalar(tid);
  if (tile + 1 == tiles_in_row) {
    const uint64_t e = head + nvec * VEC + tid;
    if (e < count) scalar(e);
  }

  V* dv = reinterpret_cast<V*>(dst + head);
  const uint64_t v0 = static_cast<uint64_t>(tile) * kTileVecs + tid;
  const bool full = static_cast<uint64_t>(tile + 1) * kTileVecs <= nvec;
  bool ok[UNROLL];
  V acc[UNROLL];
  {
    const VU* sv = reinterpret_cast<const VU*>(static_cast<const T*>(src[0]) + head);
#pragma unroll
    for (int j = 0; j < UNROLL; j++) {
      ok[j] = full || v0 + j * kBlock < nvec;
      if (ok[j]) acc[j] = RING_LOAD_VEC(NT, &sv[v0 + j * kBlock]);
    }
  }
  for (int k = 1; k < m; k += kGroup) {
    const int group = m - k < kGroup ? m - k : kGroup;  // uniform
    V x[kGroup][UNROLL];
#pragma unroll
    for (int g = 0; g < kGroup; g++) {
      if (g < group) {
        const VU* sv = reinterpret_cast<const VU*>(static_cast<const T*>(src[k + g]) + head);
#pragma unroll
        for (int j = 0; j < UNROLL; j++)
          if (ok[j]) x[g][j] = RING_LOAD_VEC(NT, &sv[v0 + j * kBlock]);
      }
    }
#pragma unroll
    for (int g = 0; g < kGroup; g++) {
      if (g < group) {
#pragma unroll
        for (int j = 0; j < UNROLL; j++)
          if (ok[j]) acc[j] = apply_vec<T, kOpAdd>(acc[j], x[g][j], 0);
      }
    }
  }
  if (MORE_UNDIVIDED) {
    // the further destinations take the sum itself (what a rank sends on), dst the quotient
    for (int d = 0; d < n_more; d++) {  // uniform
      VU* ov = reinterpret_cast<VU*>(static_cast<T*>(const_cast<void*>(more[d])) + head);
#pragma unroll
      for (int j = 0; j < UNROLL; j++)
        if (ok[j]) RING_STORE_VEC(NT, &ov[v0 + j * kBlock], acc[j]);
    }
    n_more = 0;
  }
#pragma unroll
  for (int j = 0; j < UNROLL; j++) {
    if (ok[j]) {
      if (DIV && divide) acc[j] = apply_vec<T, kOpDiv>(acc[j], acc[j], n);
      RING_STORE_VEC(NT, &dv[v0 + j * kBlock], acc[j]);
    }
  }
  for (int d = 0; d < n_more; d++) {  // uniform
    VU* ov = reinterpret_cast<VU*>(static_cast<T*>(const_cast<void*>(more[d])) + head);
#pragma unroll
    for (int j = 0; j < UNROLL; j++)
      if (ok[j]) RING_STORE_VEC(NT, &ov[v0 + j * kBlock], acc[j]);
  }
}

// A row with one source, one destination and no divide is a plain copy (the
// finished segments a rank takes in next to the fold of its own): touched once,
// so non-temporal both ways whatever the fold rows use.
template <typename T, bool DIV, int NT, int UNROLL, int GROUP>
__device__ __forceinline__ void fold_row_tile(const FoldTable& tab, int row, uint32_t tile, uint32_t tiles_in_row) {
  const FoldRow r = tab.row[row];
  const bool divide = DIV && ((tab.div_mask >> row) & 1u);
  if (r.m == 1 && r.n_more == 0 && !divide)
    fold_tile<T, UNROLL, GROUP, false, 3>(static_cast<T*>(r.dst), tab.src + r.first_ptr, 1, r.count, tile, tiles_in_row,
                                          0, false);
  else
    fold_tile<T, UNROLL, GROUP, DIV, NT>(static_cast<T*>(r.dst), tab.src + r.first_ptr, static_cast<int>(r.m), r.count,
                                         tile, tiles_in_row, tab.divisor, divide, tab.src + r.first_dst,
                                         static_cast<int>(r.n_more));
}

template <typename T, bool DIV, int NT, int UNROLL, int GROUP>
__global__ void __launch_bounds__(kBlock) fold_kernel(const FoldTable tab) {
  if (tab.uniform_tiles) {
    for (uint32_t t = blockIdx.x; t < tab.uniform_tiles; t += gridDim.x)
      fold_row_tile<T, DIV, NT, UNROLL, GROUP>(tab, static_cast<int>(blockIdx.y), t, tab.uniform_tiles);
    return;
  }
  const uint32_t total = tab.tile_begin[tab.n_rows];
  for (uint32_t t = blockIdx.x; t < total; t += gridDim.x) {
    const int lo = row_of_tile<kMaxFoldRows>(tab.tile_begin, tab.n_rows, t);
    const uint32_t first = tab.tile_begin[lo];
    fold_row_tile<T, DIV, NT, UNROLL, GROUP>(tab, lo, t - first, tab.tile_begin[lo + 1] - first);
  }
}

// ---- tensor fusion: pack / unpack -----------------------------------------------
// The fused buffer is cut into tiles of 1024 16-byte groups. A tile that lies
// inside one tensor (all of the bytes of a ResNet-sized gradient set, bar a few
// hundred KiB) is a plain aligned-store span copy. A tile that spans several
// tensors stages the offsets and base pointers of just those tensors in LDS
// and every lane finds the tensor of its 16-byte group by binary search there.
// With DIV the unpack also divides by n (the average of a fused allreduce), so
// the sum is not written and read once more just to be scaled.

constexpr uint32_t kFusionTileVecs = 1024;
constexpr uint32_t kFusionLdsCap = 512;  // tensors of one tile staged in LDS
constexpr uint32_t kUnpackPhasedTensors = 1024;  // tensors of a set whose unpack holds its payload in registers

// What a workgroup needs to know about its tile, in one 16-byte scalar load:
// the first and last tensor that overlap it and, when that is one tensor (all
// but a few hundred KiB of a ResNet-sized set), where the tile's first element
// lies in it, so that no offset or pointer table is read at all.
struct __attribute__((aligned(16))) FusionTile {
  void* addr;  // first == last: address of the tile's first element inside the tensor; else null
  uint32_t first, last;
};
// The record as one 16-byte load (field by field the compiler fetches `addr`
// only after it has branched on `first` and `last`: two loads in a row).
__device__ __forceinline__ FusionTile load_tile(const FusionTile* tiles, uint32_t tile) {
  typedef uint64_t U2 __attribute__((ext_vector_type(2)));
  const U2 raw = *reinterpret_cast<const U2*>(tiles + tile);
  FusionTile rec;
  rec.addr = reinterpret_cast<void*>(raw.x);
  rec.first = static_cast<uint32_t>(raw.y);
  rec.last = static_cast<uint32_t>(raw.y >> 32);
  return rec;
}

// A piece [b0, b1) of the fused element space that meets several tensors
// (off_tab / ptr_tab: their offsets and base pointers, tensor 0 holding b0 or
// lying before it). Every lane takes up to 4 16-byte groups, two at a time:
// it finds the tensor of each by binary search and issues the loads of both
// before the first store. GATHER: lin_out = tensor (+ lin_in when given);
// otherwise tensor = SOP(lin_in). lin_in / lin_out point at element b0 of the
// linear side. A group cut by a tensor boundary (one per boundary) or by the
// end of the piece goes element by element. Small tensors share cache lines
// with their neighbours, so the tensor side is accessed with the ordinary
// policy; NT applies to the store of the linear side only.
template <typename T, bool GATHER, int SOP, int NT>
__device__ __forceinline__ void multi_tensor_piece(const uint64_t* off_tab, T* const* ptr_tab, uint32_t ta,
                                                   uint32_t tensors, uint64_t b0, uint64_t b1, const T* lin_in,
                                                   T* lin_out, int divisor) {
  typedef typename VecOf<T>::type V;
  typedef V VU __attribute__((aligned(sizeof(T))));
  typedef T RING_GLOBAL GT;  // tensors and the linear side are device global memory
  typedef VU RING_GLOBAL GVU;
  constexpr uint32_t VEC = 16 / sizeof(T);
  constexpr int kBatch = 2;  // groups in flight per lane: more costs registers the full tiles need
  const uint32_t len = static_cast<uint32_t>(b1 - b0);  // a piece is at most one tile
  const uint32_t ngroups = (len + VEC - 1) / VEC;
#pragma unroll 1
  for (uint32_t g0 = threadIdx.x; g0 < ngroups; g0 += kBatch * kBlock) {
    T* tp[kBatch];
    uint32_t at[kBatch];
    bool whole[kBatch], cut[kBatch];
    V x[kBatch], y[kBatch];
#pragma unroll
    for (int j = 0; j < kBatch; j++) {
      const uint32_t i = (g0 + j * kBlock) * VEC;  // element of the piece
      whole[j] = cut[j] = false;
      if (i < len) {
        const uint64_t e = b0 + i;
        uint32_t l = ta, h = tensors;  // off_tab[l] <= e < off_tab[h]
        while (h - l > 1) {
          const uint32_t mid = (l + h) >> 1;
          if (off_tab[mid] <= e) l = mid; else h = mid;
        }
        at[j] = l;
        tp[j] = ptr_tab[l] + (e - off_tab[l]);
        whole[j] = e + VEC <= off_tab[l + 1] && i + VEC <= len;
        cut[j] = !whole[j];
      }
    }
#pragma unroll
    for (int j = 0; j < kBatch; j++) {
      if (whole[j]) {
        const uint32_t i = (g0 + j * kBlock) * VEC;
        if (GATHER) {
          x[j] = RING_LOAD_VEC(0, (const GVU*)tp[j]);
          if (lin_in) y[j] = RING_LOAD_VEC(0, (const GVU*)(lin_in + i));
        } else {
          x[j] = RING_LOAD_VEC(0, (const GVU*)(lin_in + i));
        }
      }
    }
#pragma unroll
    for (int j = 0; j < kBatch; j++) {
      const uint32_t i = (g0 + j * kBlock) * VEC;
      if (whole[j]) {
        if (GATHER) {
          const V r = lin_in ? apply_vec<T, kOpAdd>(y[j], x[j], 0) : x[j];
          RING_STORE_VEC(NT, (GVU*)(lin_out + i), r);
        } else {
          const V r = apply_vec<T, SOP>(x[j], x[j], divisor);
          RING_STORE_VEC(0, (GVU*)tp[j], r);
        }
      } else if (cut[j]) {
        const uint32_t end = i + VEC < len ? i + VEC : len;
        uint32_t l = at[j];
        for (uint32_t k = i; k < end; k++) {
          const uint64_t e = b0 + k;
          while (e >= off_tab[l + 1]) l++;
          GT* t = (GT*)(ptr_tab[l] + (e - off_tab[l]));
          const GT* in = (const GT*)lin_in;
          GT* out = (GT*)lin_out;
          if (GATHER) out[k] = in ? apply_one<T, kOpAdd>(in[k], *t, 0) : *t;
          else *t = apply_one<T, SOP>(in[k], T(), divisor);
        }
      }
    }
  }
}

template <typename T, bool PACK, int NT, bool DIV>
__global__ void __launch_bounds__(kBlock)
fusion_kernel(T* __restrict__ fused, const uint64_t* __restrict__ offsets, T* const* __restrict__ ptrs,
              const FusionTile* __restrict__ tiles, uint32_t ntiles, uint64_t total, int divisor) {
  constexpr uint32_t VEC = 16 / sizeof(T);
  constexpr uint64_t kTileElems = static_cast<uint64_t>(kFusionTileVecs) * VEC;
  constexpr int OP = DIV ? kOpDiv : kOpCopy;
  __shared__ uint64_t s_off[kFusionLdsCap + 1];
  __shared__ T* s_ptr[kFusionLdsCap];

  for (uint32_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
    const uint64_t e0 = static_cast<uint64_t>(tile) * kTileElems;
    const uint64_t e1 = (e0 + kTileElems < total) ? e0 + kTileElems : total;
    const FusionTile rec = load_tile(tiles, tile);
    const uint32_t t0 = rec.first;
    const uint32_t t1 = rec.last;
    if (t0 == t1) {
      T* tensor = static_cast<T*>(rec.addr);
      if (PACK) row_tile<T, kOpCopy, 4, NT>(fused + e0, tensor, nullptr, e1 - e0, 0, 1, 0);
      else row_tile<T, OP, 4, NT, kOnSrc>(tensor, fused + e0, nullptr, e1 - e0, 0, 1, divisor);
      continue;
    }
    const uint32_t span = t1 - t0 + 1;
    const uint64_t* off_tab = offsets + t0;
    T* const* ptr_tab = ptrs + t0;
    const bool staged = span <= kFusionLdsCap;  // uniform per workgroup
    if (staged) {
      for (uint32_t i = threadIdx.x; i <= span; i += kBlock) s_off[i] = offsets[t0 + i];
      for (uint32_t i = threadIdx.x; i < span; i += kBlock) s_ptr[i] = ptrs[t0 + i];
      __syncthreads();
      off_tab = s_off;
      ptr_tab = s_ptr;
    }
    if (PACK) multi_tensor_piece<T, true, kOpCopy, NT>(off_tab, ptr_tab, 0, span, e0, e1, nullptr, fused + e0, 0);
    else multi_tensor_piece<T, false, OP, NT>(off_tab, ptr_tab, 0, span, e0, e1, fused + e0, nullptr, divisor);
    if (staged) __syncthreads();  // before the next tile overwrites the table
  }
}

// ---- the unpack with the payload in registers ------------------------------------
// The unpack of a fused buffer of up to 112 MiB as rows_phased_kernel runs the
// allgather copies: one or two workgroups per CU, one read phase and one write
// phase of the whole chip. The fused side is one aligned run, so a lane's loads need
// no table at all and go out first; where the 256 vectors a workgroup takes
// in a round go (4 KiB of the fused space) is looked up while they are on
// their way: lane j reads the record of round j's tile, and when that tile
// lies inside one tensor the round's destination is an address, kept in LDS.
// A round whose tile meets several tensors (a hundred of the 6240 tiles of a
// ResNet-50 gradient set) is stored lane by lane: every lane finds the tensor
// of its vector by binary search in the offset table, which the workgroup
// staged in LDS next to the addresses. Nothing of this waits on memory a
// second time: the records and the table arrive behind the payload.
// DIV 1: the tensors receive value / divisor for a divisor that is a power of
// two: a multiplication by the exact reciprocal for float32 and an arithmetic
// shift for the integers, which are tf.div's true and floor division bit for
// bit (div_one does the same). DIV 2: float32 by any divisor, the IEEE
// division of div_one (a dozen instructions an element, which the write phase
// has the time for); the integers' general division is left to the tiles.
template <typename T, int DIV>
__device__ __forceinline__ T divide_in_registers(T x, float reciprocal, int shift, float divisor) {
  (void)reciprocal;
  (void)shift;
  (void)divisor;
  if constexpr (DIV == 0) {
    return x;
  } else if constexpr (std::is_floating_point<T>::value) {
    if constexpr (DIV == 2) return x / divisor;
    else return x * reciprocal;
  } else {
    static_assert(DIV == 1, "integers: powers of two only");
    return x >> shift;
  }
}

// The tensor that holds element e of the fused space: off[l] <= e < off[l + 1], off[0] = 0, off[m] = total.
__device__ __forceinline__ uint32_t tensor_of_element(const uint64_t* off, uint32_t m, uint64_t e) {
  uint32_t l = 0, h = m;
  while (h - l > 1) {
    const uint32_t mid = (l + h) >> 1;
    if (off[mid] <= e) l = mid; else h = mid;
  }
  return l;
}

// WAVES: workgroups per CU, as in rows_phased_kernel (2: buffers of up to 56 MiB, 40 groups a lane).
template <typename T, int DIV, int WAVES>
__global__ void __launch_bounds__(kBlock) RING_WAVES_PER_SIMD(WAVES)
unpack_phased_kernel(const T* __restrict__ fused, const uint64_t* __restrict__ offsets, T* const* __restrict__ ptrs,
                     const FusionTile* __restrict__ tiles, uint32_t m, uint64_t total, uint32_t rounds, int divisor) {
  typedef typename VecOf<T>::type V;
  typedef V VU __attribute__((aligned(sizeof(T))));
  typedef T RING_GLOBAL GT;
  typedef V RING_GLOBAL GV;
  typedef VU RING_GLOBAL GVU;
  constexpr uint32_t VEC = 16 / sizeof(T);
  constexpr int PER = WAVES == 1 ? kPhasedMax : kPhasedMaxTwoWaves;  // groups a lane holds
  __shared__ uint64_t s_off[kUnpackPhasedTensors + 1];
  __shared__ T* s_ptr[kUnpackPhasedTensors];
  __shared__ T* s_to[PER];  // where lane 0's vector of round j goes, or null: the round meets several tensors
  const uint32_t tid = threadIdx.x;
  const uint32_t stride = gridDim.x * kBlock;
  const uint32_t base = blockIdx.x * kBlock + tid;
  const uint32_t nvec = static_cast<uint32_t>(total / VEC);  // the host checked: at most PER * stride
  const uint32_t n_tail = static_cast<uint32_t>(total - static_cast<uint64_t>(nvec) * VEC);
  const GV* fv = (const GV*)fused;
  V s[PER];
  T tail = T();
#pragma unroll
  for (int j = 0; j < PER; j++) {
    if (static_cast<uint32_t>(j) < rounds) {
      if (base + j * stride < nvec) s[j] = __builtin_nontemporal_load(&(fv + j * stride)[base]);
    }
  }
  if (blockIdx.x == 0 && tid < n_tail) tail = ((const GT*)fused)[static_cast<uint64_t>(nvec) * VEC + tid];
  // behind the payload: the destinations of this workgroup's rounds and the offset table (at most
  // kUnpackPhasedTensors tensors: five offsets and four pointers a lane). Every load is issued before the
  // first is waited for, so the launch pays one memory latency for all of it, the one it pays for the payload.
  constexpr uint32_t kPtrsPerLane = kUnpackPhasedTensors / kBlock, kOffsPerLane = kPtrsPerLane + 1;
  static_assert(kUnpackPhasedTensors % kBlock == 0, "whole rounds of the workgroup over the pointer table");
  T* to = nullptr;
  const uint64_t v0 = static_cast<uint64_t>(blockIdx.x) * kBlock + static_cast<uint64_t>(tid) * stride;
  const bool has_round = tid < rounds && v0 < nvec;
  // (a lane without a round reads tile 0's record and drops it: a load under a branch would be waited for there)
  const FusionTile rec = load_tile(tiles, has_round ? static_cast<uint32_t>(v0 / kFusionTileVecs) : 0u);
  uint64_t off[kOffsPerLane];
  T* ptr[kPtrsPerLane];
#pragma unroll
  for (uint32_t i = 0; i < kOffsPerLane; i++) {
    off[i] = 0;
    if (tid + i * kBlock <= m) off[i] = offsets[tid + i * kBlock];
  }
#pragma unroll
  for (uint32_t i = 0; i < kPtrsPerLane; i++) {
    ptr[i] = nullptr;
    if (tid + i * kBlock < m) ptr[i] = ptrs[tid + i * kBlock];
  }
  if (has_round && rec.first == rec.last) to = static_cast<T*>(rec.addr) + (v0 % kFusionTileVecs) * VEC;
  if (tid < static_cast<uint32_t>(PER)) s_to[tid] = to;
#pragma unroll
  for (uint32_t i = 0; i < kOffsPerLane; i++)
    if (tid + i * kBlock <= m) s_off[tid + i * kBlock] = off[i];
#pragma unroll
  for (uint32_t i = 0; i < kPtrsPerLane; i++)
    if (tid + i * kBlock < m) s_ptr[tid + i * kBlock] = ptr[i];
  __syncthreads();
  RING_WAIT_VMEM();
  float reciprocal = 1.0f;
  int shift = 0;
  const float fdivisor = static_cast<float>(divisor);
  if (DIV == 1) {
    reciprocal = 1.0f / fdivisor;
    while ((1 << shift) < divisor) shift++;
  }
#pragma unroll
  for (int j = 0; j < PER; j++) {
    if (static_cast<uint32_t>(j) < rounds) {
      const uint32_t idx = base + j * stride;
      if (idx < nvec) {
        V r = s[j];
#pragma unroll
        for (uint32_t c = 0; c < VEC; c++) r[c] = divide_in_registers<T, DIV>(r[c], reciprocal, shift, fdivisor);
        T* to = s_to[j];
        if (to) {
          __builtin_nontemporal_store(r, &((GVU*)(GT*)to)[tid]);
        } else {
          // small tensors share cache lines with their neighbours: ordinary stores
          const uint64_t e = static_cast<uint64_t>(idx) * VEC;
          uint32_t l = tensor_of_element(s_off, m, e);
          if (e + VEC <= s_off[l + 1]) {
            *(GVU*)(GT*)(s_ptr[l] + (e - s_off[l])) = r;
          } else {
            // a vector cut by the end of a tensor (one per end that is not 16-byte aligned): element by
            // element, as a loop that stays a loop (this body is repeated for every round)
#pragma unroll 1
            for (uint32_t c = 0; c < VEC; c++) {
              while (e + c >= s_off[l + 1]) l++;
              T x = r[0];
#pragma unroll
              for (uint32_t k = 1; k < VEC; k++) x = (c == k) ? r[k] : x;
              *(GT*)(s_ptr[l] + (e + c - s_off[l])) = x;
            }
          }
        }
      }
    }
  }
  if (blockIdx.x == 0 && tid < n_tail) {
    const uint64_t e = static_cast<uint64_t>(nvec) * VEC + tid;
    const uint32_t l = tensor_of_element(s_off, m, e);
    *(GT*)(s_ptr[l] + (e - s_off[l])) = divide_in_registers<T, DIV>(tail, reciprocal, shift, fdivisor);
  }
}

// ---- tensor fusion without passes of its own -------------------------------------
// The pack before a fused allreduce and the unpack after it read and write the
// whole set once each for nothing but a change of layout. Both fold into the
// ring's own work: the first touch of a segment by the reduce-scatter can take
// its local operand straight from the tensors (gather: out = tensor + incoming,
// written to the wire buffer the next rank is sent from), and the allgather's
// finished segments can go straight to the tensors (scatter: tensor = incoming,
// optionally divided). A launch works on spans of the fused element space, one
// per ring segment; a tile of the space meets at most a few spans and, as in
// the pack / unpack kernel, either lies inside one tensor or finds its tensors
// through an offset table staged in LDS.

constexpr int kMaxFusionSpans = 64;
struct FusionSpan {
  uint64_t begin, end;  // elements of the fused space
  const void* in;       // element `begin` of what arrives (gather: may be null, then a plain pack)
  void* out;            // gather only: element `begin` of the linear destination
};
struct FusionSpanTable {
  int n;
  int divisor;  // scatter: > 0 divides
  FusionSpan span[kMaxFusionSpans];
};

template <typename T, bool GATHER, int NT, bool DIV>
__global__ void __launch_bounds__(kBlock)
fusion_span_kernel(const uint64_t* __restrict__ offsets, T* const* __restrict__ ptrs,
                   const FusionTile* __restrict__ tiles, uint32_t tile_lo, uint32_t tile_hi, uint64_t total,
                   const FusionSpanTable tab) {
  constexpr uint32_t VEC = 16 / sizeof(T);
  constexpr uint64_t kTileElems = static_cast<uint64_t>(kFusionTileVecs) * VEC;
  constexpr int SOP = DIV ? kOpDiv : kOpCopy;  // scatter
  __shared__ uint64_t s_off[kFusionLdsCap + 1];
  __shared__ T* s_ptr[kFusionLdsCap];

  for (uint32_t tile = tile_lo + blockIdx.x; tile < tile_hi; tile += gridDim.x) {
    const uint64_t e0 = static_cast<uint64_t>(tile) * kTileElems;
    const uint64_t e1 = (e0 + kTileElems < total) ? e0 + kTileElems : total;
    const FusionTile rec = load_tile(tiles, tile);
    const uint32_t t0 = rec.first;
    const uint32_t t1 = rec.last;
    const uint32_t tensors = t1 - t0 + 1;
    const uint64_t* off_tab = offsets + t0;
    T* const* ptr_tab = ptrs + t0;
    const bool staged = tensors > 1 && tensors <= kFusionLdsCap;  // uniform per workgroup
    if (staged) {
      for (uint32_t i = threadIdx.x; i <= tensors; i += kBlock) s_off[i] = offsets[t0 + i];
      for (uint32_t i = threadIdx.x; i < tensors; i += kBlock) s_ptr[i] = ptrs[t0 + i];
      __syncthreads();
      off_tab = s_off;
      ptr_tab = s_ptr;
    }
    // first span that ends after e0 (spans are sorted and disjoint)
    int lo = 0, hi = tab.n;
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (tab.span[mid].end <= e0) lo = mid + 1; else hi = mid;
    }
    for (int sp = lo; sp < tab.n && tab.span[sp].begin < e1; sp++) {
      const FusionSpan span = tab.span[sp];
      const uint64_t b0 = span.begin > e0 ? span.begin : e0;
      const uint64_t b1 = span.end < e1 ? span.end : e1;
      if (b0 >= b1) continue;
      const T* lin_in = span.in ? static_cast<const T*>(span.in) + (b0 - span.begin) : nullptr;
      T* lin_out = GATHER ? static_cast<T*>(span.out) + (b0 - span.begin) : nullptr;
      // the tensor holding b0 (uniform scalar walk over the tile's few tensors)
      uint32_t ta = 0;
      if (tensors > 1)
        while (off_tab[ta + 1] <= b0) ta++;
      if (tensors == 1 || b1 <= off_tab[ta + 1]) {
        // the piece lies inside one tensor: the aligned-store span code of the step tables
        T* tensor = tensors == 1 ? static_cast<T*>(rec.addr) + (b0 - e0) : ptr_tab[ta] + (b0 - off_tab[ta]);
        if (GATHER) {
          if (lin_in) row_tile<T, kOpAdd, 4, NT>(lin_out, lin_in, tensor, b1 - b0, 0, 1, 0);
          else row_tile<T, kOpCopy, 4, NT>(lin_out, tensor, nullptr, b1 - b0, 0, 1, 0);
        } else {
          row_tile<T, SOP, 4, NT>(tensor, lin_in, nullptr, b1 - b0, 0, 1, tab.divisor);
        }
        continue;
      }
      // several tensors: every lane finds the tensor of its 16-byte group
      multi_tensor_piece<T, GATHER, SOP, 0>(off_tab, ptr_tab, ta, tensors, b0, b1, lin_in, lin_out, tab.divisor);
    }
    if (staged) __syncthreads();  // before the next tile overwrites the table
  }
}

// ---- the direct form of a fused allreduce in one launch ---------------------------------
// One rank of a fused allreduce whose peers pushed their raw copies of the
// rank's own segment into staging slots and whose other segments arrive
// finished. Over the fused element space: inside the owned segment a piece of
// a tensor is folded from the m staged copies and the tensor itself (the
// rank's own copy, last in the ring's order for that segment), the sum goes to
// the wire buffer the other ranks are sent from and the quotient back into the
// tensor; everywhere else a finished segment is scattered into the tensors as
// by fusion_span_kernel. The owned segment is read once and written once where
// pack, fold and scatter as launches of their own read it three times.

constexpr int kMaxDirectSpans = 32;  // ranks of a ring this kernel serves
struct FusionDirectSpan {
  uint64_t begin, end;  // elements of the fused space
  const void* in;       // element `begin` of the finished segment
};
struct FusionDirectTable {
  int n;        // finished spans (sorted, disjoint, none meets the fold span)
  int divisor;  // > 0 divides what goes into the tensors
  int m;        // staged copies of the fold span
  uint64_t fold_begin, fold_end;
  void* wire;   // element fold_begin of where the fold itself is stored
  FusionDirectSpan span[kMaxDirectSpans];
  const void* staged[kMaxDirectSpans];  // element fold_begin of every staged copy, in fold order
};

template <typename T, int NT, bool DIV>
__global__ void __launch_bounds__(kBlock)
fusion_direct_kernel(const uint64_t* __restrict__ offsets, T* const* __restrict__ ptrs,
                     const FusionTile* __restrict__ tiles, uint32_t tile_lo, uint32_t tile_hi, uint64_t total,
                     const FusionDirectTable tab) {
  constexpr uint32_t VEC = 16 / sizeof(T);
  constexpr uint64_t kTileElems = static_cast<uint64_t>(kFusionTileVecs) * VEC;
  constexpr int SOP = DIV ? kOpDiv : kOpCopy;
  __shared__ uint64_t s_off[kFusionLdsCap + 1];
  __shared__ T* s_ptr[kFusionLdsCap];
  __shared__ const void* s_src[kMaxDirectSpans + 1];
  __shared__ const void* s_wire[1];

  for (uint32_t tile = tile_lo + blockIdx.x; tile < tile_hi; tile += gridDim.x) {
    const uint64_t e0 = static_cast<uint64_t>(tile) * kTileElems;
    const uint64_t e1 = (e0 + kTileElems < total) ? e0 + kTileElems : total;
    const FusionTile rec = load_tile(tiles, tile);
    const uint32_t t0 = rec.first;
    const uint32_t t1 = rec.last;
    const uint32_t tensors = t1 - t0 + 1;
    const uint64_t* off_tab = offsets + t0;
    T* const* ptr_tab = ptrs + t0;
    const bool staged = tensors > 1 && tensors <= kFusionLdsCap;  // uniform per workgroup
    if (staged) {
      for (uint32_t i = threadIdx.x; i <= tensors; i += kBlock) s_off[i] = offsets[t0 + i];
      for (uint32_t i = threadIdx.x; i < tensors; i += kBlock) s_ptr[i] = ptrs[t0 + i];
      __syncthreads();
      off_tab = s_off;
      ptr_tab = s_ptr;
    }
    // finished segments that meet the tile: scattered into the tensors
    int lo = 0, hi = tab.n;
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (tab.span[mid].end <= e0) lo = mid + 1; else hi = mid;
    }
    for (int sp = lo; sp < tab.n && tab.span[sp].begin < e1; sp++) {
      const FusionDirectSpan span = tab.span[sp];
      const uint64_t b0 = span.begin > e0 ? span.begin : e0;
      const uint64_t b1 = span.end < e1 ? span.end : e1;
      if (b0 >= b1) continue;
      const T* lin_in = static_cast<const T*>(span.in) + (b0 - span.begin);
      uint32_t ta = 0;
      if (tensors > 1)
        while (off_tab[ta + 1] <= b0) ta++;
      if (tensors == 1 || b1 <= off_tab[ta + 1]) {
        T* tensor = tensors == 1 ? static_cast<T*>(rec.addr) + (b0 - e0) : ptr_tab[ta] + (b0 - off_tab[ta]);
        row_tile<T, SOP, 4, NT>(tensor, lin_in, nullptr, b1 - b0, 0, 1, tab.divisor);
        continue;
      }
      multi_tensor_piece<T, false, SOP, 0>(off_tab, ptr_tab, ta, tensors, b0, b1, lin_in, nullptr, tab.divisor);
    }
    // the part of the owned segment in the tile, cut where a tensor ends: every
    // piece is one fold row over the staged copies and the tensor
    uint64_t b0 = tab.fold_begin > e0 ? tab.fold_begin : e0;
    const uint64_t fold_end = tab.fold_end < e1 ? tab.fold_end : e1;
    uint32_t ta = 0;
    while (b0 < fold_end) {
      if (tensors > 1)
        while (off_tab[ta + 1] <= b0) ta++;
      uint64_t b1 = fold_end;
      if (tensors > 1 && off_tab[ta + 1] < b1) b1 = off_tab[ta + 1];
      T* tensor = tensors == 1 ? static_cast<T*>(rec.addr) + (b0 - e0) : ptr_tab[ta] + (b0 - off_tab[ta]);
      const uint64_t within = b0 - tab.fold_begin;
      if (threadIdx.x < static_cast<uint32_t>(tab.m))
        s_src[threadIdx.x] = static_cast<const T*>(tab.staged[threadIdx.x]) + within;
      if (threadIdx.x == static_cast<uint32_t>(tab.m)) {
        s_src[tab.m] = tensor;
        s_wire[0] = static_cast<T*>(tab.wire) + within;
      }
      __syncthreads();
      const uint64_t count = b1 - b0;
      uint64_t head = ((16u - (static_cast<uint32_t>(reinterpret_cast<uintptr_t>(tensor)) & 15u)) & 15u) / sizeof(T);
      if (head > count) head = count;
      const uint64_t nvec = (count - head) / VEC;
      uint32_t sub_tiles = static_cast<uint32_t>((nvec + kBlock - 1) / kBlock);
      if (sub_tiles == 0) sub_tiles = 1;
      for (uint32_t sub = 0; sub < sub_tiles; sub++)
        fold_tile<T, 1, kFoldGroup, DIV, NT, true>(tensor, s_src, tab.m + 1, count, sub, sub_tiles, tab.divisor, DIV,
                                                   s_wire, 1);
      __syncthreads();  // before the next piece overwrites the pointers
      b0 = b1;
    }
    if (staged) __syncthreads();  // before the next tile overwrites the table
  }
}

// ---- a fused allreduce of ranks that share the GPU, without a fused buffer -----------
// What pack, ring and unpack compute for n resident ranks, in one pass over the
// fused element space: element e lies in ring segment s(e) of the packed
// layout, the ring leaves there the fold of the ranks' values in the order
// s, s+1, ..., s+n-1 (mod n), and every rank's tensor receives it (divided,
// for an average). A tile of the space is cut where a segment or a tensor
// ends; each piece is then one fold row with n sources and n destinations
// whose pointers the first lanes look up in the ranks' tensor tables.

constexpr int kMaxFusedRanks = 16;
// A tile of the fused space (1024 16-byte groups) is worked on by this many
// workgroups, a quarter each: the fold that stores to every rank wants short
// tiles (kFoldToAllUnroll), and what a workgroup has to look up before its
// first load is one round trip to memory, so there is nothing to share.
constexpr uint32_t kFusedAllSplit = kFusionTileVecs / (kBlock * kFoldToAllUnroll);
struct FusedRanks {
  int n;
  int divisor;
  uint64_t total;   // elements of the fused space
  uint64_t seg;     // total / n
  uint64_t rem;     // total % n: the first rem segments hold one more
  const void* const* in[kMaxFusedRanks];   // rank k's input tensor table
  void* const* out[kMaxFusedRanks];        // rank k's output tensor table
  const FusionTile* in_tiles[kMaxFusedRanks];   // rank k's tile records: where a tile inside one tensor starts
  const FusionTile* out_tiles[kMaxFusedRanks];
};

// The pointer of rank r out of a table in the kernel arguments, r different per
// lane: a run of selects on scalar registers instead of a load from the
// argument segment (one more trip to memory ahead of the loads that matter).
template <typename P>
__device__ __forceinline__ P pick_rank(const P (&table)[kMaxFusedRanks], int r) {
  P p = table[0];
#pragma unroll
  for (int j = 1; j < kMaxFusedRanks; j++) p = (r == j) ? table[j] : p;
  return p;
}

template <typename T, bool DIV, int NT>
__global__ void __launch_bounds__(kBlock)
fusion_allreduce_kernel(const uint64_t* __restrict__ offsets, const FusionTile* __restrict__ tiles, uint32_t ntiles,
                        const FusedRanks ranks) {
  constexpr uint32_t VEC = 16 / sizeof(T);
  constexpr uint64_t kTileElems = static_cast<uint64_t>(kFusionTileVecs) * VEC;
  constexpr uint64_t kPartElems = kTileElems / kFusedAllSplit;
  __shared__ const void* s_src[kMaxFusedRanks];
  __shared__ const void* s_dst[kMaxFusedRanks];
  const int n = ranks.n;
  auto seg_start = [&](uint64_t s) { return s * ranks.seg + (s < ranks.rem ? s : ranks.rem); };
  auto seg_of = [&](uint64_t e) {  // segments 0..rem-1 have seg+1 elements
    const uint64_t big = ranks.rem * (ranks.seg + 1);
    return e < big ? e / (ranks.seg + 1) : ranks.rem + (ranks.seg ? (e - big) / ranks.seg : 0);
  };
  // one piece: fold row with n sources (rank (s + k) mod n is source k, the ring's order for segment s)
  // and n destinations, whose pointers lie in s_src / s_dst
  auto fold_piece = [&](uint64_t count) {
    T* dst = static_cast<T*>(const_cast<void*>(s_dst[0]));
    uint64_t head = ((16u - (static_cast<uint32_t>(reinterpret_cast<uintptr_t>(dst)) & 15u)) & 15u) / sizeof(T);
    if (head > count) head = count;
    const uint64_t nvec = (count - head) / VEC;
    uint32_t sub_tiles = static_cast<uint32_t>((nvec + kBlock * kFoldToAllUnroll - 1) / (kBlock * kFoldToAllUnroll));
    if (sub_tiles == 0) sub_tiles = 1;
    for (uint32_t sub = 0; sub < sub_tiles; sub++)
      fold_tile<T, kFoldToAllUnroll, kFoldGroup, DIV, NT>(dst, s_src, n, count, sub, sub_tiles, ranks.divisor, DIV,
                                                          s_dst + 1, n - 1);
  };

  for (uint32_t item = blockIdx.x; item < ntiles * kFusedAllSplit; item += gridDim.x) {
    const uint32_t tile = item / kFusedAllSplit, part = item % kFusedAllSplit;
    const uint64_t e0 = static_cast<uint64_t>(tile) * kTileElems;
    const uint64_t e1 = (e0 + kTileElems < ranks.total) ? e0 + kTileElems : ranks.total;
    // Issued together, one trip to memory: the tile's record (uniform) and, by lane k < n, where the tile
    // starts in rank k's input and output tensors (meaningful when the tile lies inside one tensor).
    const FusionTile rec = load_tile(tiles, tile);
    FusionTile mine_in{nullptr, 0, 0}, mine_out{nullptr, 0, 0};
    const int k = static_cast<int>(threadIdx.x);
    if (k < n) {
      mine_in = load_tile(pick_rank(ranks.in_tiles, k), tile);
      mine_out = load_tile(pick_rank(ranks.out_tiles, k), tile);
    }
    if (rec.first == rec.last) {
      // inside one tensor: this workgroup's quarter of the tile, cut where a ring segment ends
      uint64_t b0 = e0 + part * kPartElems;
      const uint64_t end = b0 + kPartElems < e1 ? b0 + kPartElems : e1;
      uint64_t s = b0 < end ? seg_of(b0) : 0;
      while (b0 < end) {
        while (seg_start(s + 1) <= b0) s++;
        const uint64_t b1 = seg_start(s + 1) < end ? seg_start(s + 1) : end;
        if (k < n) {
          // rank k is source (k - s) mod n of this segment's fold, and destination k
          const int j = static_cast<int>((static_cast<uint64_t>(k) + static_cast<uint64_t>(n) - s % static_cast<uint64_t>(n)) %
                                         static_cast<uint64_t>(n));
          s_src[j] = static_cast<const T*>(mine_in.addr) + (b0 - e0);
          s_dst[k] = static_cast<T*>(mine_out.addr) + (b0 - e0);
        }
        __syncthreads();
        fold_piece(b1 - b0);
        __syncthreads();  // before the next piece overwrites the pointers
        b0 = b1;
      }
      continue;
    }
    // several tensors meet in the tile (a few hundred KiB of a ResNet-sized set): one workgroup takes all of
    // it, cut where a tensor or a segment ends, the pointers looked up in the ranks' tensor tables
    if (part != 0) continue;
    uint32_t t = rec.first;  // the tensor holding the current position (all uniform over the workgroup)
    uint64_t s = seg_of(e0);
    uint64_t b0 = e0;
    while (b0 < e1) {
      while (offsets[t + 1] <= b0) t++;
      while (seg_start(s + 1) <= b0) s++;
      uint64_t b1 = e1;
      if (offsets[t + 1] < b1) b1 = offsets[t + 1];
      if (seg_start(s + 1) < b1) b1 = seg_start(s + 1);
      const uint64_t within = b0 - offsets[t];
      if (k < n) {
        const int r = static_cast<int>((s + static_cast<uint64_t>(k)) % static_cast<uint64_t>(n));
        s_src[k] = static_cast<const T*>(pick_rank(ranks.in, r)[t]) + within;
        s_dst[k] = static_cast<T*>(pick_rank(ranks.out, k)[t]) + within;
      }
      __syncthreads();
      fold_piece(b1 - b0);
      __syncthreads();  // before the next piece overwrites the pointers
      b0 = b1;
    }
  }
}

// ---- launch configuration -----------------------------------------------------

constexpr uint64_t kCacheResidentBytes = 128ull << 20;

enum Role {
  kRoleCopy, kRoleAccumulate, kRoleAllgather, kRolePack, kRoleUnpack, kRoleFold, kRoleBroadcast, kRoleFoldAll, kRoles
};

// Launch options (ring_set_option), as one launch sees them: a snapshot.
struct Tuning {
  int unroll = 4;          // 16-byte vectors per lane per tile: 2, 4 or 8
  // Cache policy per role; bit 0: non-temporal stores, bit 1: non-temporal
  // loads, -1: chosen by size. Accumulates, allgather copies and the unpack
  // touch their bytes once. The in->out copy and the pack write the buffer the
  // reduce-scatter reads next, so their stores stay ordinary (measured 2-5 %
  // of a step on tensors up to 128 MiB, which the last-level cache can hold);
  // the copy's loads turn non-temporal above that size, where ordinary ones
  // only evict what the next kernel wants.
  // the fold's result is what the allgather reads next; a source that several
  // rows copy (a finished segment fetched by every other rank) is loaded with
  // the ordinary policy so that it is fetched from HBM once
  // (a fold that stores its result to every rank writes final outputs: touched once)
  int nt[kRoles] = {-1, 3, 3, 2, 3, 2, 1, 3};
  // Allgather copies whose tiles all fit on the chip at once run as one read
  // phase and one write phase (rows_kernel's PACE): -1 chosen by the size of
  // the launch, 0 never, 1 always.
  int paced_copy = -1;
  // The same idea with the whole payload of the launch in registers
  // (rows_phased_kernel): -1 chosen by the size of the launch, 0 never, 1
  // whenever the launch fits.
  int phased_copy = -1;
  int blocks_per_cu = 0;   // 0: one workgroup per tile; >0: persistent grid of CUs x this
  int dry_launch = 0;      // measurement only: the step-table kernels return at entry (what a launch of that grid costs)
  int flat_grid = 0;       // measurement only: rows of equal tile counts share the 1-D grid of unequal rows instead of (tiles, rows)
};

// Where the options live: one atomic cell each, so that ring_set_option on one
// thread and launches on others (one thread per rank drives its own stream)
// are no data race. A launch reads them once, at entry (tuning()), and works
// on that snapshot; an option set while a launch is being prepared applies to
// that launch or to the next one.
enum OptionCell { kCellUnroll, kCellPaced, kCellPhased, kCellBlocksPerCu, kCellDry, kCellFlat, kCellNt, kCells = kCellNt + kRoles };
struct OptionCells {
  std::atomic<int> v[kCells];
  OptionCells() { store(Tuning()); }
  void store(const Tuning& t) {
    v[kCellUnroll].store(t.unroll, std::memory_order_relaxed);
    v[kCellPaced].store(t.paced_copy, std::memory_order_relaxed);
    v[kCellPhased].store(t.phased_copy, std::memory_order_relaxed);
    v[kCellBlocksPerCu].store(t.blocks_per_cu, std::memory_order_relaxed);
    v[kCellDry].store(t.dry_launch, std::memory_order_relaxed);
    v[kCellFlat].store(t.flat_grid, std::memory_order_relaxed);
    for (int r = 0; r < kRoles; r++) v[kCellNt + r].store(t.nt[r], std::memory_order_relaxed);
  }
};
OptionCells g_options;

inline Tuning tuning() {
  Tuning t;
  t.unroll = g_options.v[kCellUnroll].load(std::memory_order_relaxed);
  t.paced_copy = g_options.v[kCellPaced].load(std::memory_order_relaxed);
  t.phased_copy = g_options.v[kCellPhased].load(std::memory_order_relaxed);
  t.blocks_per_cu = g_options.v[kCellBlocksPerCu].load(std::memory_order_relaxed);
  t.dry_launch = g_options.v[kCellDry].load(std::memory_order_relaxed);
  t.flat_grid = g_options.v[kCellFlat].load(std::memory_order_relaxed);
  for (int r = 0; r < kRoles; r++) t.nt[r] = g_options.v[kCellNt + r].load(std::memory_order_relaxed);
  return t;
}

struct DeviceInfo {
  bool ok = false;
  int cus = 0;
};

int device_info(DeviceInfo* out) {
  static thread_local DeviceInfo cached[64];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) { hip_fail(e); return RING_ERR_NO_DEVICE; }
  if (dev < 0 || dev >= 64) return RING_ERR_NO_DEVICE;
  if (!cached[dev].ok) {
    int cus = 0;
    RING_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    cached[dev].cus = cus > 0 ? cus : 256;
    cached[dev].ok = true;
  }
  *out = cached[dev];
  return RING_OK;
}

template <typename T, int MODE>
int launch_rows_typed(const RowTable& tab, dim3 grid, hipStream_t stream, int nt, int unroll, bool paced) {
#define RING_LAUNCH(U, N) launch(rows_kernel<T, MODE, U, N>, grid, dim3(kBlock), stream, tab)
#define RING_LAUNCH_NT(U)                       \
  switch (nt & 3) {                             \
    case 0: RING_LAUNCH(U, 0); break;           \
    case 1: RING_LAUNCH(U, 1); break;           \
    case 2: RING_LAUNCH(U, 2); break;           \
    default: RING_LAUNCH(U, 3); break;          \
  }
  if (!paced && unroll == 4 && tab.n_rows <= kSmallRows) {
    SmallRowTable small;
    small.n_rows = tab.n_rows;
    small.dry = tab.dry;
    small.uniform_tiles = tab.uniform_tiles;
    small.divisor = tab.divisor;
    small.div_mask = tab.div_mask;
    for (int k = 0; k <= kSmallRows; k++) small.tile_begin[k] = tab.tile_begin[k];
    for (int k = 0; k < tab.n_rows; k++) small.row[k] = tab.row[k];
    for (int k = tab.n_rows; k < kSmallRows; k++) small.row[k] = Row{nullptr, nullptr, nullptr, 0};
    switch (nt & 3) {
      case 0: launch(rows_kernel_small<T, MODE, 0>, grid, dim3(kBlock), stream, small); break;
      case 1: launch(rows_kernel_small<T, MODE, 1>, grid, dim3(kBlock), stream, small); break;
      case 2: launch(rows_kernel_small<T, MODE, 2>, grid, dim3(kBlock), stream, small); break;
      default: launch(rows_kernel_small<T, MODE, 3>, grid, dim3(kBlock), stream, small); break;
    }
  } else if (MODE == kCopy && paced) {
    if constexpr (MODE == kCopy) {
      switch (nt & 3) {
        case 0: launch(rows_kernel<T, kCopy, kPacedUnroll, 0, 1>, grid, dim3(kBlock), stream, tab); break;
        case 1: launch(rows_kernel<T, kCopy, kPacedUnroll, 1, 1>, grid, dim3(kBlock), stream, tab); break;
        case 2: launch(rows_kernel<T, kCopy, kPacedUnroll, 2, 1>, grid, dim3(kBlock), stream, tab); break;
        default: launch(rows_kernel<T, kCopy, kPacedUnroll, 3, 1>, grid, dim3(kBlock), stream, tab); break;
      }
    }
  } else {
    switch (unroll) {
      case 2: RING_LAUNCH_NT(2); break;
      case 8: RING_LAUNCH_NT(8); break;
      default: RING_LAUNCH_NT(4); break;
    }
  }
#undef RING_LAUNCH_NT
#undef RING_LAUNCH
  RING_HIP(hipGetLastError());
  return RING_OK;
}

// Room for n items: on the stack up to N of them (the rows of one launch), on the heap beyond.
template <typename T, size_t N>
struct RowBuffer {
  T stack[N];
  std::vector<T> heap;
  T* data;
  explicit RowBuffer(size_t n) : data(stack) {
    if (n > N) {
      heap.resize(n);
      data = heap.data();
    }
  }
};

struct HostRow {
  void* dst;
  const void* a;
  const void* b;   // null: copy row
  uint64_t count;  // elements of `esz` bytes
  bool divide;     // with a divisor: this row also divides
};

// ---- which form a launch of copy rows takes ----------------------------------------------
// The thresholds, in one place. All of them are per CU, so that they scale
// with the chip; they were measured on the 256 CUs of an MI355X, where
// 4 KiB per CU are 1 MiB.
//
// The paced tiles: every tile of the launch on the chip at the same time (at
// most 7 workgroups per CU of 32 KiB tiles, 56 MiB per side on 256 CUs) and the
// launch large enough to be bound by memory rather than by its dispatch (2 per
// CU). Measured on 7 rows: 21-56 MiB per side 1-10 % faster than the plain
// tiles (56 MiB: 19.6 against 20.8 us), slower beyond (63 MiB: 25.3 against
// 23.7 us) and no different below.
constexpr uint64_t kPacedMinTilesPerCu = 2;
constexpr uint64_t kPacedMaxTilesPerCu = 7;
// The payload in registers (rows_phased_kernel). The chip's registers hold
// 112 MiB as one workgroup per CU; up to 224 KiB per side per CU (56 MiB, where
// the 7 paced tiles per CU end) the launch runs as TWO workgroups per CU with
// fewer vectors per lane each (a few rounds of one wave per SIMD keep too
// little in flight). By itself the launcher takes the form above that size,
// and from 124 KiB per CU (31 MiB; 5 ragged rows of 6.4 MiB: 11.7 against
// 12.7 us paced; at 28 MiB the paced tiles win, 10.2 against 11.2) unless the
// paced tiles fill the chip exactly (a whole number of 32 KiB tiles per CU),
// which is their best case and beats this form by 3-4 % (7 x 8 MiB: 19.7
// against 20.4 us); with a CU or more left over they lose 3-8 % to it
// (7 x 7.5 MiB: 19.6 against 18.1 us). Not on chips of fewer than 128 CUs,
// where none of this was measured.
constexpr uint64_t kRegistersOnePerCuAbove = 224u << 10;
constexpr uint64_t kRegistersTwoPerCuFrom = 124u << 10;
constexpr int kRegistersMinCus = 128;

struct RowsChoice {
  int form;           // RING_FORM_*
  PhasedShape shape;  // the forms in registers: rounds, and the workgroup that starts each row
};

// The form of one launch of `rows` (what launch_rows was handed: rows of `esz`-byte
// elements for `role`), from the shape of the launch, the options and the
// number of CUs alone. Only the copies of an allgather phase have a choice.
RowsChoice choose_rows_form(const HostRow* rows, size_t n_rows, size_t esz, Role role, int divisor, int nt,
                            const Tuning& tun, int cus) {
  RowsChoice c;
  c.form = RING_FORM_TILES;
  c.shape.rounds = 0;
  for (int k = 0; k < kSmallRows; k++) c.shape.shift[k] = 0;
  if (role != kRoleAllgather || divisor > 0 || n_rows < 1 || cus < 1) return c;
  const uint64_t vec = 16 / esz, ucus = static_cast<uint64_t>(cus);
  bool copies = true;           // no row has a second operand (empty rows aside)
  bool copies_not_empty = true;  // and none is empty
  uint64_t bytes = 0, paced_tiles = 0;
  for (size_t k = 0; k < n_rows; k++) {
    const bool empty = rows[k].count == 0;
    copies = copies && (rows[k].b == nullptr || empty);
    copies_not_empty = copies_not_empty && rows[k].b == nullptr && !empty;
    bytes += rows[k].count * esz;
    paced_tiles += (rows[k].count / vec + kBlock * kPacedUnroll - 1) / (kBlock * kPacedUnroll);
  }
  // In registers: up to kSmallRows rows, each within its share of a lane's vectors, non-temporal both ways.
  if (n_rows <= static_cast<size_t>(kSmallRows) && (nt & 3) == 3 && tun.phased_copy != 0 && tun.blocks_per_cu == 0 &&
      copies_not_empty) {
    const uint64_t per_cu = bytes / ucus;
    const int waves = per_cu > kRegistersOnePerCuAbove ? 1 : 2;
    const uint64_t wgs = ucus * waves, stride = wgs * kBlock;
    const uint64_t room = static_cast<uint64_t>((waves == 1 ? kPhasedMax : kPhasedMaxTwoWaves) / static_cast<int>(n_rows));
    PhasedShape shape = c.shape;
    uint64_t start = 0;
    bool fits = room >= 1;
    for (size_t k = 0; k < n_rows && fits; k++) {
      const HostRow& r = rows[k];
      const uintptr_t d = reinterpret_cast<uintptr_t>(r.dst);
      uint64_t head = ((kRowHeadAlign - (d & (kRowHeadAlign - 1))) & (kRowHeadAlign - 1)) / esz;
      if (head > r.count) head = r.count;
      const uint64_t nvec = (r.count - head) / vec;
      const uint64_t rounds = (nvec + stride - 1) / stride;
      if (rounds > room) { fits = false; break; }
      if (rounds > shape.rounds) shape.rounds = static_cast<uint32_t>(rounds);
      shape.shift[k] = static_cast<uint32_t>(start);
      // the next row starts behind the last workgroup of this row's last round
      start = (start + (nvec % stride + kBlock - 1) / kBlock) % wgs;
    }
    bool by_itself = per_cu > kRegistersOnePerCuAbove;
    if (!by_itself && per_cu >= kRegistersTwoPerCuFrom) by_itself = paced_tiles % ucus != 0;
    if (fits && (tun.phased_copy > 0 || (by_itself && cus >= kRegistersMinCus))) {
      c.form = waves == 1 ? RING_FORM_REGISTERS_1 : RING_FORM_REGISTERS_2;
      c.shape = shape;
      return c;
    }
  }
  if (n_rows <= static_cast<size_t>(kMaxRows) && tun.paced_copy != 0 && copies &&
      (tun.paced_copy > 0 || (tun.blocks_per_cu == 0 && paced_tiles >= kPacedMinTilesPerCu * ucus &&
                              paced_tiles <= kPacedMaxTilesPerCu * ucus)))
    c.form = RING_FORM_PACED;
  return c;
}

// Launches rows (any number) in groups of kMaxRows. esz: 4 or 8. A table with
// no add row runs the copy-only kernel.
// divisor > 0: rows marked `divide` also divide by it (kAvg) and the element
// type is signed.
int launch_rows(const HostRow* rows, size_t n_rows, size_t esz, bool is_float, hipStream_t stream,
                Role role, int divisor = 0) {
  const Tuning tun = tuning();
  int nt = tun.nt[role];
  if (nt < 0) {
    uint64_t bytes = 0;
    for (size_t k = 0; k < n_rows; k++) bytes += rows[k].count * esz;
    nt = bytes <= kCacheResidentBytes ? 0 : 2;
  }
  int unroll = (tun.unroll == 2 || tun.unroll == 8) ? tun.unroll : 4;
  const uint64_t vec = 16 / esz;
  DeviceInfo info;
  bool paced = false;
  if (role == kRoleAllgather && divisor <= 0 && n_rows >= 1) {
    int rc = device_info(&info);
    if (rc != RING_OK) return rc;
    const RowsChoice choice = choose_rows_form(rows, n_rows, esz, role, divisor, nt, tun, info.cus);
    if (choice.form == RING_FORM_REGISTERS_1 || choice.form == RING_FORM_REGISTERS_2) {
      const int waves = choice.form == RING_FORM_REGISTERS_1 ? 1 : 2;
      const uint64_t wgs = static_cast<uint64_t>(info.cus) * waves;
      SmallRowTable tab;
      for (size_t k = 0; k < static_cast<size_t>(kSmallRows); k++)
        tab.row[k] = k < n_rows ? Row{rows[k].dst, rows[k].a, nullptr, rows[k].count} : Row{nullptr, nullptr, nullptr, 0};
      const PhasedShape shape = choice.shape;
      tab.n_rows = static_cast<int>(n_rows);
      tab.dry = tun.dry_launch;
      tab.uniform_tiles = 0;
      tab.divisor = 0;
      tab.div_mask = 0;
      for (int k = 0; k <= kSmallRows; k++) tab.tile_begin[k] = 0;
      const dim3 grid(static_cast<uint32_t>(wgs));
#define RING_PHASED(T, W)                                                                                \
  switch (n_rows) {                                                                                      \
    case 1: launch(rows_phased_kernel<T, 1, W>, grid, dim3(kBlock), stream, tab, shape); break;          \
    case 2: launch(rows_phased_kernel<T, 2, W>, grid, dim3(kBlock), stream, tab, shape); break;          \
    case 3: launch(rows_phased_kernel<T, 3, W>, grid, dim3(kBlock), stream, tab, shape); break;          \
    case 4: launch(rows_phased_kernel<T, 4, W>, grid, dim3(kBlock), stream, tab, shape); break;          \
    case 5: launch(rows_phased_kernel<T, 5, W>, grid, dim3(kBlock), stream, tab, shape); break;          \
    case 6: launch(rows_phased_kernel<T, 6, W>, grid, dim3(kBlock), stream, tab, shape); break;          \
    case 7: launch(rows_phased_kernel<T, 7, W>, grid, dim3(kBlock), stream, tab, shape); break;          \
    default: launch(rows_phased_kernel<T, 8, W>, grid, dim3(kBlock), stream, tab, shape); break;         \
  }
      if (waves == 2) {
        if (esz == 8) { RING_PHASED(uint64_t, 2) } else { RING_PHASED(uint32_t, 2) }
      } else {
        if (esz == 8) { RING_PHASED(uint64_t, 1) } else { RING_PHASED(uint32_t, 1) }
      }
#undef RING_PHASED
      RING_HIP(hipGetLastError());
      return RING_OK;
    }
    paced = choice.form == RING_FORM_PACED;
  }
  if (paced) unroll = kPacedUnroll;
  const uint64_t tile_vecs = static_cast<uint64_t>(kBlock) * unroll;
  size_t i = 0;
  while (i < n_rows) {
    RowTable tab;
    tab.n_rows = 0;
    tab.dry = tun.dry_launch;
    tab.divisor = divisor;
    tab.div_mask = 0;
    tab.tile_begin[0] = 0;
    for (int k = 1; k <= kMaxRows; k++) tab.tile_begin[k] = 0xffffffffu;  // past the last row: after every tile
    uint64_t tiles = 0;
    uint64_t first_tiles = 0;
    bool any_add = false, uniform = true;
    while (i < n_rows && tab.n_rows < kMaxRows) {
      const HostRow& r = rows[i];
      if (r.count == 0) { i++; continue; }
      const uintptr_t d = reinterpret_cast<uintptr_t>(r.dst);
      uint64_t head = ((kRowHeadAlign - (d & (kRowHeadAlign - 1))) & (kRowHeadAlign - 1)) / esz;
      if (head > r.count) head = r.count;
      const uint64_t nvec = (r.count - head) / vec;
      uint64_t t = (nvec + tile_vecs - 1) / tile_vecs;
      if (t == 0) t = 1;
      if (tiles + t > 0x7fffffffull) {
        if (tab.n_rows == 0) return RING_ERR_ARGUMENT;  // a single row beyond 2^31 tiles
        break;
      }
      const int k = tab.n_rows++;
      tab.row[k] = Row{r.dst, r.a, r.b, r.count};
      if (divisor > 0 && r.divide) tab.div_mask |= 1ull << k;
      any_add = any_add || r.b != nullptr;
      if (k == 0) first_tiles = t;
      uniform = uniform && t == first_tiles;
      tiles += t;
      tab.tile_begin[k + 1] = static_cast<uint32_t>(tiles);
      i++;
    }
    if (tab.n_rows == 0) continue;
    uint64_t cap = tiles;
    if (tun.blocks_per_cu > 0) {
      int rc = device_info(&info);
      if (rc != RING_OK) return rc;
      cap = static_cast<uint64_t>(info.cus) * tun.blocks_per_cu;
    }
    dim3 grid;
    if (uniform && !tun.flat_grid && tab.n_rows <= 65535) {
      uint64_t per_row = cap / static_cast<uint64_t>(tab.n_rows);
      if (per_row < 1) per_row = 1;
      if (per_row > first_tiles) per_row = first_tiles;
      tab.uniform_tiles = static_cast<uint32_t>(first_tiles);
      grid = dim3(static_cast<uint32_t>(per_row), static_cast<uint32_t>(tab.n_rows));
    } else {
      tab.uniform_tiles = 0;
      grid = dim3(static_cast<uint32_t>(tiles < cap ? tiles : cap));
    }
    int rc;
    if (tab.div_mask != 0) {
      rc = esz == 8 ? launch_rows_typed<int64_t, kAvg>(tab, grid, stream, nt, unroll, paced)
           : is_float ? launch_rows_typed<float, kAvg>(tab, grid, stream, nt, unroll, paced)
                      : launch_rows_typed<int32_t, kAvg>(tab, grid, stream, nt, unroll, paced);
    } else if (!any_add) {
      rc = esz == 8 ? launch_rows_typed<uint64_t, kCopy>(tab, grid, stream, nt, unroll, paced)
                    : launch_rows_typed<uint32_t, kCopy>(tab, grid, stream, nt, unroll, paced);
    } else if (esz == 8) {
      rc = launch_rows_typed<uint64_t, kAdd>(tab, grid, stream, nt, unroll, paced);
    } else if (is_float) {
      rc = launch_rows_typed<float, kAdd>(tab, grid, stream, nt, unroll, paced);
    } else {
      rc = launch_rows_typed<uint32_t, kAdd>(tab, grid, stream, nt, unroll, paced);
    }
    if (rc != RING_OK) return rc;
  }
  return RING_OK;
}

inline bool dtype_ok(int dtype) { return dtype == RING_F32 || dtype == RING_I32 || dtype == RING_I64; }
inline size_t dtype_size(int dtype) { return dtype == RING_I64 ? 8 : (dtype_ok(dtype) ? 4 : 0); }

enum StepKind { kStepCopy, kStepAddInPlace, kStepAddFrom };

// input: the local operand of kStepAddFrom rows (same element offsets as buffer).
int steps_common(const void* input, void* buffer, const ring_step* steps, int n_steps, int dtype,
                 void* stream, StepKind kind) {
  if (!dtype_ok(dtype)) return RING_ERR_DTYPE;
  if (n_steps < 0) return RING_ERR_ARGUMENT;
  if (n_steps == 0) return RING_OK;
  if (!steps) return RING_ERR_ARGUMENT;
  const size_t esz = dtype_size(dtype);
  RowBuffer<HostRow, kMaxRows> rows(static_cast<size_t>(n_steps));
  size_t n_rows = 0;
  for (int i = 0; i < n_steps; i++) {
    if (steps[i].count == 0) continue;
    if (!buffer || !steps[i].src || (kind == kStepAddFrom && !input)) return RING_ERR_ARGUMENT;
    char* d = static_cast<char*>(buffer) + steps[i].dst_offset * esz;
    const char* local = kind == kStepAddFrom ? static_cast<const char*>(input) + steps[i].dst_offset * esz : d;
    if ((reinterpret_cast<uintptr_t>(d) | reinterpret_cast<uintptr_t>(steps[i].src) |
         reinterpret_cast<uintptr_t>(local)) & (esz - 1))
      return RING_ERR_ARGUMENT;
    rows.data[n_rows++] = HostRow{d, steps[i].src, kind == kStepCopy ? nullptr : local, steps[i].count, false};
  }
  return launch_rows(rows.data, n_rows, esz, dtype == RING_F32, static_cast<hipStream_t>(stream),
                     kind == kStepCopy ? kRoleAllgather : kRoleAccumulate);
}

}  // namespace

// Host side of a fusion plan. The device table is one allocation:
// offsets[m+1] | ptrs[m] | padding to 16 bytes | tiles[ntiles].
struct ring_fusion_plan {
  int dtype = 0;
  size_t esz = 0;
  int device = 0;
  uint32_t m = 0;        // non-empty tensors
  uint32_t ntiles = 0;
  uint64_t total = 0;    // elements
  void* d_table = nullptr;
  uint64_t* d_offsets = nullptr;
  void** d_ptrs = nullptr;
  FusionTile* d_tiles = nullptr;
  std::vector<uint64_t> h_offsets;  // host copy of the offsets: what two plans must share to describe one fused space
};

namespace {

// What the pack / unpack kernel reads besides the tensors: the offset table
// of the fused buffer, wherever it lives (a plan's own allocation, or the
// static array of the allocation-free entry point).
struct FusionView {
  int dtype;
  size_t esz;
  uint32_t ntiles;
  uint64_t total;  // elements
  const uint64_t* offsets;
  void* const* ptrs;
  const FusionTile* tiles;
  uint32_t m;  // non-empty tensors: entries of ptrs, and of offsets less one
};

inline FusionView view_of(const ring_fusion_plan* p) {
  return FusionView{p->dtype, p->esz, p->ntiles, p->total, p->d_offsets, p->d_ptrs, p->d_tiles, p->m};
}

// ---- which form an unpack takes -------------------------------------------------------
// The unpack with the payload in registers (unpack_phased_kernel), by itself from 4 KiB of the fused buffer
// per CU (1 MiB on 256 CUs) up to what the registers hold. Measured behind the allgather that wrote the
// buffer, float32, sets of 79-155 tensors, against the tiles: 2-12 MiB 4.4-5.8 us against 6.7-7.8; 24 MiB
// 10.0 / 13.4; 40 MiB 16.1 / 18.3; 56 MiB 23.0 / 24.3 (two workgroups per CU); 80 MiB 31.4 / 32.9 and 97 MiB
// 34.8 / 39.4 (one per CU). Between the two, the form with two workgroups per CU holds up to 80 MiB and is
// the better one up to 72 (64 MiB: 26.4 against 27.7 as one workgroup per CU and 27.0 as tiles; 80 MiB: 33.4
// against 31.4): two per CU up to 300 KiB per CU (75 MiB).
// float32 by a divisor that is no power of two: the IEEE division in the kernel, as two workgroups per CU
// only (with 112 rounds to unroll the division makes the body too large for the compiler to keep the payload
// in registers) and up to 256 KiB per CU (64 MiB; by 6, behind the allgather: 4 MiB 5.4 against 7.2 us as
// tiles, 32 MiB 13.1 / 15.5, 64 MiB 26.1 / 27.2, 72 MiB 30.1 / 28.9); beyond, and for the integer types
// (floor division), the tiles.
constexpr uint64_t kUnpackPhasedMinPerCu = 4u << 10;
constexpr uint64_t kUnpackTwoWorkgroupsMaxPerCu = 300u << 10;
constexpr uint64_t kUnpackDivideMaxPerCu = 256u << 10;

struct UnpackChoice {
  int form;         // RING_FORM_TILES, RING_FORM_REGISTERS_1 or RING_FORM_REGISTERS_2
  uint32_t rounds;  // the forms in registers: 16-byte groups per lane
};

// total: elements of the fused buffer; m: non-empty tensors; divisor 0: no divide.
UnpackChoice choose_unpack_form(uint64_t total, uint32_t m, size_t esz, bool is_float, int divisor, const Tuning& tun,
                                int cus) {
  UnpackChoice c{RING_FORM_TILES, 0};
  const bool power_of_two = divisor <= 0 || (divisor & (divisor - 1)) == 0;
  if (tun.phased_copy == 0 || tun.blocks_per_cu != 0 || (tun.nt[kRoleUnpack] & 3) != 3 || m > kUnpackPhasedTensors ||
      cus < 1 || !(power_of_two || is_float))
    return c;
  const uint64_t per_cu = total * esz / static_cast<uint64_t>(cus);
  const int waves = per_cu > kUnpackTwoWorkgroupsMaxPerCu ? 1 : 2;
  const uint64_t stride = static_cast<uint64_t>(cus) * waves * kBlock;
  const uint64_t rounds = (total / (16 / esz) + stride - 1) / stride;
  if (rounds < 1 || rounds > static_cast<uint64_t>(waves == 1 ? kPhasedMax : kPhasedMaxTwoWaves)) return c;
  if (!(tun.phased_copy > 0 || (per_cu >= kUnpackPhasedMinPerCu && cus >= kRegistersMinCus))) return c;
  if (!power_of_two && !(waves == 2 && (tun.phased_copy > 0 || per_cu <= kUnpackDivideMaxPerCu))) return c;
  c.form = waves == 1 ? RING_FORM_REGISTERS_1 : RING_FORM_REGISTERS_2;
  c.rounds = static_cast<uint32_t>(rounds);
  return c;
}

template <typename T, bool PACK, bool DIV>
int launch_fusion(const FusionView& p, void* fused, hipStream_t stream, int divisor) {
  const Tuning tun = tuning();
  if (!PACK) {
    DeviceInfo info;
    int rc = device_info(&info);
    if (rc != RING_OK) return rc;
    const UnpackChoice choice = choose_unpack_form(p.total, p.m, sizeof(T), std::is_floating_point<T>::value,
                                                   DIV ? divisor : 0, tun, info.cus);
    if (choice.form != RING_FORM_TILES) {
      const int waves = choice.form == RING_FORM_REGISTERS_1 ? 1 : 2;
      const uint64_t wgs = static_cast<uint64_t>(info.cus) * waves;
#define RING_UNPACK_PHASED(D, W)                                                                              \
  launch(unpack_phased_kernel<T, D, W>, dim3(static_cast<uint32_t>(wgs)), dim3(kBlock), stream,               \
         static_cast<const T*>(fused), p.offsets, reinterpret_cast<T* const*>(p.ptrs), p.tiles, p.m, p.total, \
         choice.rounds, divisor)
      constexpr int kPowerOfTwo = DIV ? 1 : 0;
      if (!DIV || (divisor & (divisor - 1)) == 0) {
        if (waves == 1) RING_UNPACK_PHASED(kPowerOfTwo, 1); else RING_UNPACK_PHASED(kPowerOfTwo, 2);
      } else if constexpr (DIV && std::is_floating_point<T>::value) {
        RING_UNPACK_PHASED(2, 2);  // choose_unpack_form gives this divisor the form with two workgroups per CU only
      }
#undef RING_UNPACK_PHASED
      RING_HIP(hipGetLastError());
      return RING_OK;
    }
  }
  uint32_t grid = p.ntiles;
  if (tun.blocks_per_cu > 0) {
    DeviceInfo info;
    int rc = device_info(&info);
    if (rc != RING_OK) return rc;
    const uint64_t cap = static_cast<uint64_t>(info.cus) * tun.blocks_per_cu;
    if (grid > cap) grid = static_cast<uint32_t>(cap);
  }
#define RING_FUSION(N)                                                                                   \
  launch(fusion_kernel<T, PACK, N, DIV>, dim3(grid), dim3(kBlock), stream, static_cast<T*>(fused),       \
         p.offsets, reinterpret_cast<T* const*>(p.ptrs), p.tiles, p.ntiles, p.total, divisor)
  int nt = tun.nt[PACK ? kRolePack : kRoleUnpack];
  if (nt < 0) nt = 2;
  switch (nt & 3) {
    case 0: RING_FUSION(0); break;
    case 1: RING_FUSION(1); break;
    case 2: RING_FUSION(2); break;
    default: RING_FUSION(3); break;
  }
#undef RING_FUSION
  RING_HIP(hipGetLastError());
  return RING_OK;
}

// divisor 0: plain pack / unpack. divisor >= 1: unpack and divide.
int fusion_run(const FusionView& p, void* fused, void* stream, bool pack, int divisor) {
  if (p.total == 0) return RING_OK;
  if (!fused || (reinterpret_cast<uintptr_t>(fused) & 15u)) return RING_ERR_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (divisor > 0) {
    if (p.dtype == RING_F32) return launch_fusion<float, false, true>(p, fused, s, divisor);
    if (p.dtype == RING_I32) return launch_fusion<int32_t, false, true>(p, fused, s, divisor);
    return launch_fusion<int64_t, false, true>(p, fused, s, divisor);
  }
  if (p.esz == 8)
    return pack ? launch_fusion<uint64_t, true, false>(p, fused, s, 0) : launch_fusion<uint64_t, false, false>(p, fused, s, 0);
  return pack ? launch_fusion<uint32_t, true, false>(p, fused, s, 0) : launch_fusion<uint32_t, false, false>(p, fused, s, 0);
}

int fusion_run(const ring_fusion_plan* p, void* fused, void* stream, bool pack, int divisor) {
  if (!p) return RING_ERR_ARGUMENT;
  return fusion_run(view_of(p), fused, stream, pack, divisor);
}

// ---- the offset table in a static device array --------------------------------------
// For callers that may not allocate device memory (code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc): the table a
// plan keeps in an allocation of its own is built in a file-scope device array
// instead, by two small kernels, from values that travel in kernel arguments.
// Every call on a GPU shares that GPU's copy of the array.

constexpr uint32_t kStaticMaxTensors = 1024;  // non-empty tensors per call
constexpr uint32_t kStaticMaxTiles = 65536;   // 16 KiB tiles of the fused buffer: 1 GiB
struct StaticFusionTable {
  uint64_t offsets[kStaticMaxTensors + 1];
  void* ptrs[kStaticMaxTensors];
  FusionTile tiles[kStaticMaxTiles];
};
// 1,064,968 bytes per GPU the library runs on, held until the process ends.
static __device__ __align__(256) unsigned char scratch[sizeof(StaticFusionTable)];

// `scratch` is a host-side stand-in in host code: the array's device address is
// looked up once per device and only that pointer is ever handed to a kernel.
// With it, per device: an event recorded behind the last call's launches and
// the stream they went to, so that a call on another stream can be ordered
// behind them (every call on a GPU works in the same array).
struct ScratchState {
  StaticFusionTable* ptr = nullptr;
  hipEvent_t last_done = nullptr;   // created with the address, once per device
  hipStream_t last_stream = nullptr;
  bool recorded = false;            // last_done marks a call
};
std::mutex g_scratch_mutex;
ScratchState g_scratch_state[64];

// g_scratch_mutex held.
int scratch_of_current_device(ScratchState** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) { hip_fail(e); return RING_ERR_NO_DEVICE; }
  if (dev < 0 || dev >= 64) return RING_ERR_NO_DEVICE;
  ScratchState& st = g_scratch_state[dev];
  if (!st.ptr) {
    void* p = nullptr;
    RING_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return RING_ERR_HIP;
    hipEvent_t ev = nullptr;
    RING_HIP(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
    st.last_done = ev;
    st.ptr = static_cast<StaticFusionTable*>(p);
  }
  *out = &st;
  return RING_OK;
}

// A piece of the offset / pointer table, by value in the kernel arguments.
constexpr uint32_t kTableChunk = 128;
struct TableChunk {
  uint32_t base, n;  // entries [base, base + n) of the table
  uint64_t end;      // written to offsets[base + n]: where the next tensor starts (the total after the last chunk)
  uint64_t off[kTableChunk];
  void* ptr[kTableChunk];
};

__global__ void __launch_bounds__(kBlock) table_chunk_kernel(StaticFusionTable* tab, const TableChunk c) {
  const uint32_t i = threadIdx.x;
  if (i < c.n) {
    tab->offsets[c.base + i] = c.off[i];
    tab->ptrs[c.base + i] = c.ptr[i];
  }
  if (i == 0) tab->offsets[c.base + c.n] = c.end;
}

// The record of every tile, as ring_fusion_plan_create computes it on the
// host: the first and the last tensor that overlap the tile, and the tile's
// address inside the tensor when that is one tensor.
__global__ void __launch_bounds__(kBlock)
table_tiles_kernel(StaticFusionTable* tab, uint32_t m, uint32_t ntiles, uint64_t tile_elems, uint64_t total,
                   uint32_t esz) {
  const uint32_t tile = blockIdx.x * kBlock + threadIdx.x;
  if (tile >= ntiles) return;
  const uint64_t e0 = static_cast<uint64_t>(tile) * tile_elems;
  const uint64_t e1 = (e0 + tile_elems < total) ? e0 + tile_elems : total;
  // offsets[0..m] is strictly increasing, offsets[0] = 0, offsets[m] = total
  uint32_t lo = 0, hi = m;  // offsets[lo] <= e0 < offsets[hi]
  while (hi - lo > 1) {
    const uint32_t mid = (lo + hi) >> 1;
    if (tab->offsets[mid] <= e0) lo = mid; else hi = mid;
  }
  const uint32_t first = lo;
  hi = m;  // offsets[lo] < e1 <= offsets[hi]
  while (hi - lo > 1) {
    const uint32_t mid = (lo + hi) >> 1;
    if (tab->offsets[mid] < e1) lo = mid; else hi = mid;
  }
  FusionTile rec;
  rec.first = first;
  rec.last = lo;
  rec.addr = first == lo ? static_cast<char*>(tab->ptrs[first]) + (e0 - tab->offsets[first]) * esz : nullptr;
  tab->tiles[tile] = rec;
}

}  // namespace

// =============================================================================
// C ABI
// =============================================================================
extern "C" {

int ring_abi_version(void) { return RING_ABI_VERSION; }

const char* ring_status_string(int status) {
  switch (status) {
    case RING_OK: return "ok";
    case RING_ERR_DTYPE: return "Invalid tensor type passed.";
    case RING_ERR_ARGUMENT: return "invalid argument";
    case RING_ERR_HIP: return "HIP runtime call failed";
    case RING_ERR_NO_DEVICE: return "no usable GPU";
    case RING_ERR_LIMIT: return "beyond the capacity of the static device table (1024 tensors, 65536 tiles of 16 KiB)";
    default: return "unknown status";
  }
}

int ring_last_hip_error(void) { return g_last_hip_error; }

size_t ring_dtype_size(int dtype) { return dtype_size(dtype); }

// Tuning knobs for measurement runs; not part of the drop-in surface.
// name: "unroll" (2|4|8), "blocks_per_cu" (0 = one workgroup per tile),
// "nontemporal" (bit 0 stores, bit 1 loads; sets every role) and
// "nontemporal_copy" / "_accumulate" / "_allgather" / "_pack" / "_unpack",
// "paced_copy" and "phased_copy" (the two forms of the allgather copies that
// read first and write after: -1 by size, 0 never, 1 always), "dry_launch",
// "flat_grid".
int ring_set_option(const char* name, int value) {
  if (!name) return RING_ERR_ARGUMENT;
  auto set = [](int cell, int v) { g_options.v[cell].store(v, std::memory_order_relaxed); };
  if (!strcmp(name, "unroll")) {
    if (value != 2 && value != 4 && value != 8) return RING_ERR_ARGUMENT;
    set(kCellUnroll, value);
  } else if (!strcmp(name, "paced_copy")) {
    if (value < -1 || value > 1) return RING_ERR_ARGUMENT;
    set(kCellPaced, value);
  } else if (!strcmp(name, "phased_copy")) {
    if (value < -1 || value > 1) return RING_ERR_ARGUMENT;
    set(kCellPhased, value);
  } else if (!strncmp(name, "nontemporal", 11)) {
    static const char* const kSuffix[kRoles] = {"_copy", "_accumulate", "_allgather", "_pack", "_unpack",
                                                "_fold", "_broadcast", "_fold_all"};
    if (value < -1 || value > 3) return RING_ERR_ARGUMENT;
    const Tuning defaults;
    bool known = name[11] == 0;
    for (int r = 0; r < kRoles; r++) {
      if (name[11] == 0 || !strcmp(name + 11, kSuffix[r])) {
        set(kCellNt + r, value < 0 ? defaults.nt[r] : value);  // -1: back to the default
        known = true;
      }
    }
    if (!known) return RING_ERR_ARGUMENT;
  } else if (!strcmp(name, "blocks_per_cu")) {
    if (value < 0 || value > 64) return RING_ERR_ARGUMENT;
    set(kCellBlocksPerCu, value);
  } else if (!strcmp(name, "dry_launch")) {
    set(kCellDry, value != 0);
  } else if (!strcmp(name, "flat_grid")) {
    set(kCellFlat, value != 0);
  } else {
    return RING_ERR_ARGUMENT;
  }
  return RING_OK;
}

// ---- which form a launch takes, as a query --------------------------------------------

int ring_describe_rows_launch(const ring_row* rows, int n_rows, int dtype, int role, int cus, int* form) {
  if (!dtype_ok(dtype)) return RING_ERR_DTYPE;
  if (!form || n_rows < 0 || (n_rows > 0 && !rows) || cus < 1) return RING_ERR_ARGUMENT;
  if (role != RING_ROLE_COPY && role != RING_ROLE_ACCUMULATE && role != RING_ROLE_ALLGATHER) return RING_ERR_ARGUMENT;
  const size_t esz = dtype_size(dtype);
  // the rows as the entry points hand them to the launcher: empty ones dropped
  RowBuffer<HostRow, kMaxRows> host(static_cast<size_t>(n_rows));
  size_t n_host = 0;
  uint64_t bytes = 0;
  for (int i = 0; i < n_rows; i++) {
    if (rows[i].count == 0) continue;
    host.data[n_host++] = HostRow{rows[i].dst, rows[i].a, rows[i].b, rows[i].count, false};
    bytes += rows[i].count * esz;
  }
  const Tuning tun = tuning();
  const Role r = role == RING_ROLE_COPY ? kRoleCopy : role == RING_ROLE_ACCUMULATE ? kRoleAccumulate : kRoleAllgather;
  int nt = tun.nt[r];
  if (nt < 0) nt = bytes <= kCacheResidentBytes ? 0 : 2;
  *form = choose_rows_form(host.data, n_host, esz, r, 0, nt, tun, cus).form;
  return RING_OK;
}

int ring_describe_unpack_launch(uint64_t total_elements, int n_tensors, int dtype, int divisor, int cus, int* form) {
  if (!dtype_ok(dtype)) return RING_ERR_DTYPE;
  if (!form || n_tensors < 0 || divisor < 0 || cus < 1) return RING_ERR_ARGUMENT;
  *form = choose_unpack_form(total_elements, static_cast<uint32_t>(n_tensors), dtype_size(dtype), dtype == RING_F32,
                             divisor, tuning(), cus).form;
  return RING_OK;
}

// ---- measurement hooks --------------------------------------------------------------

int ring_event_create(void** event) {
  if (!event) return RING_ERR_ARGUMENT;
  hipEvent_t e = nullptr;
  RING_HIP(hipEventCreate(&e));
  *event = e;
  return RING_OK;
}

int ring_event_destroy(void* event) {
  if (!event) return RING_OK;
  RING_HIP(hipEventDestroy(static_cast<hipEvent_t>(event)));
  return RING_OK;
}

int ring_event_elapsed_us(void* start, void* stop, double* us) {
  if (!start || !stop || !us) return RING_ERR_ARGUMENT;
  float ms = 0.f;
  RING_HIP(hipEventElapsedTime(&ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
  *us = static_cast<double>(ms) * 1e3;
  return RING_OK;
}

int ring_event_record(void* event, void* stream) {
  if (!event) return RING_ERR_ARGUMENT;
  RING_HIP(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
  return RING_OK;
}

int ring_event_synchronize(void* event) {
  if (!event) return RING_ERR_ARGUMENT;
  RING_HIP(hipEventSynchronize(static_cast<hipEvent_t>(event)));
  return RING_OK;
}

int ring_graph_begin_capture(void* stream) {
  if (!stream) return RING_ERR_ARGUMENT;  // the null stream cannot be captured
  RING_HIP(hipStreamBeginCapture(static_cast<hipStream_t>(stream), hipStreamCaptureModeThreadLocal));
  return RING_OK;
}

int ring_graph_end_capture(void* stream, void** graph_exec) {
  if (!stream || !graph_exec) return RING_ERR_ARGUMENT;
  *graph_exec = nullptr;
  hipGraph_t graph = nullptr;
  RING_HIP(hipStreamEndCapture(static_cast<hipStream_t>(stream), &graph));
  hipGraphExec_t exec = nullptr;
  const hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  if (e != hipSuccess) return hip_fail(e);
  *graph_exec = exec;
  return RING_OK;
}

int ring_graph_launch(void* graph_exec, void* stream) {
  if (!graph_exec) return RING_ERR_ARGUMENT;
  RING_HIP(hipGraphLaunch(static_cast<hipGraphExec_t>(graph_exec), static_cast<hipStream_t>(stream)));
  return RING_OK;
}

int ring_graph_destroy(void* graph_exec) {
  if (!graph_exec) return RING_OK;
  RING_HIP(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec)));
  return RING_OK;
}

int ring_stream_wait_event(void* stream, void* event) {
  if (!event) return RING_ERR_ARGUMENT;
  RING_HIP(hipStreamWaitEvent(static_cast<hipStream_t>(stream), static_cast<hipEvent_t>(event), 0));
  return RING_OK;
}

int ring_time_next_launch(void* start_event, void* stop_event) {
  if (!start_event && !stop_event) {
    g_armed_head = g_armed_count = 0;
    return RING_OK;
  }
  if (g_armed_count == kMaxArmedLaunches) return RING_ERR_LIMIT;
  g_armed[(g_armed_head + g_armed_count) % kMaxArmedLaunches] =
      ArmedLaunch{static_cast<hipEvent_t>(start_event), static_cast<hipEvent_t>(stop_event)};
  ++g_armed_count;
  return RING_OK;
}

int ring_probe_stream(const ring_row* rows, int n_rows, int dtype, int mode, void* stream) {
  if (!dtype_ok(dtype)) return RING_ERR_DTYPE;
  if (!rows || n_rows < 1 || n_rows > kSmallRows || mode < 0 || mode > 3) return RING_ERR_ARGUMENT;
  const size_t esz = dtype_size(dtype);
  const bool write = (mode & 1) != 0;
  SmallRowTable tab;
  tab.n_rows = n_rows;
  tab.dry = 0;
  tab.uniform_tiles = 0;
  tab.divisor = 0;
  tab.div_mask = 0;
  for (int k = 0; k <= kSmallRows; k++) tab.tile_begin[k] = 0;
  uint64_t tiles = 1;
  for (int k = 0; k < kSmallRows; k++) {
    tab.row[k] = Row{nullptr, nullptr, nullptr, 0};
    if (k >= n_rows) continue;
    const void* p = write ? rows[k].dst : rows[k].a;
    if (!p || (reinterpret_cast<uintptr_t>(p) & 15u)) return RING_ERR_ARGUMENT;
    const uint64_t nvec = rows[k].count * esz / 16;  // whole 16-byte vectors; a probe has no scalar edges
    tab.row[k] = Row{rows[k].dst, rows[k].a, nullptr, nvec};
    const uint64_t t = (nvec + kBlock * 4 - 1) / (kBlock * 4);
    if (t > tiles) tiles = t;
  }
  if (tiles > 0x7fffffffull) return RING_ERR_ARGUMENT;
  const dim3 grid(static_cast<uint32_t>(tiles), static_cast<uint32_t>(n_rows));
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (mode) {
    case 0: launch(stream_probe_kernel<0, 1>, grid, dim3(kBlock), s, tab); break;
    case 1: launch(stream_probe_kernel<1, 1>, grid, dim3(kBlock), s, tab); break;
    case 2: launch(stream_probe_kernel<0, 0>, grid, dim3(kBlock), s, tab); break;
    default: launch(stream_probe_kernel<1, 0>, grid, dim3(kBlock), s, tab); break;
  }
  RING_HIP(hipGetLastError());
  return RING_OK;
}

// ---- host tables ------------------------------------------------------------

int ring_segment_table(size_t count, int n, size_t* sizes, size_t* starts) {
  if (n < 1 || !sizes || !starts) return RING_ERR_ARGUMENT;
  const size_t un = static_cast<size_t>(n);
  const size_t q = count / un, rem = count % un;
  size_t at = 0;
  for (size_t i = 0; i < un; i++) {
    sizes[i] = q + (i < rem ? 1 : 0);
    starts[i] = at;
    at += sizes[i];
  }
  return RING_OK;
}

size_t ring_temp_elements(size_t count, int n) {
  if (n < 1) return 0;
  const size_t un = static_cast<size_t>(n);
  return count / un + (count % un ? 1 : 0);
}

int ring_allgather_table(const size_t* rows, int n, size_t elems_per_row, size_t* starts) {
  if (n < 1 || !rows || !starts) return RING_ERR_ARGUMENT;
  size_t at = 0;
  for (int i = 0; i < n; i++) {
    starts[i] = at;
    // a gathered tensor that does not fit size_t is an error, not a table that wraps
    if (rows[i] != 0 && elems_per_row > SIZE_MAX / rows[i]) return RING_ERR_ARGUMENT;
    const size_t elems = elems_per_row * rows[i];
    if (elems > SIZE_MAX - at) return RING_ERR_ARGUMENT;
    at += elems;
  }
  return RING_OK;
}

int ring_schedule(int phase, int n, int r, int step, int* send_seg, int* recv_seg) {
  if (n < 1 || r < 0 || r >= n || step < 0 || step >= n - 1 || !send_seg || !recv_seg)
    return RING_ERR_ARGUMENT;
  int send, recv;
  switch (phase) {
    case RING_PHASE_REDUCE_SCATTER:
    case RING_PHASE_GATHER:
      send = r - step; recv = r - step - 1; break;
    case RING_PHASE_ALLGATHER:
      send = r - step + 1; recv = r - step; break;
    default: return RING_ERR_ARGUMENT;
  }
  *send_seg = ((send % n) + n) % n;
  *recv_seg = ((recv % n) + n) % n;
  return RING_OK;
}

// ---- stream -------------------------------------------------------------------

int ring_get_device(int* device) {
  if (!device) return RING_ERR_ARGUMENT;
  RING_HIP(hipGetDevice(device));
  return RING_OK;
}

int ring_set_device(int device) {
  RING_HIP(hipSetDevice(device));
  return RING_OK;
}

int ring_stream_create(void** stream) {
  if (!stream) return RING_ERR_ARGUMENT;
  hipStream_t s = nullptr;
  RING_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *stream = s;
  return RING_OK;
}

int ring_stream_destroy(void* stream) {
  if (!stream) return RING_OK;
  RING_HIP(hipStreamDestroy(static_cast<hipStream_t>(stream)));
  return RING_OK;
}

int ring_stream_synchronize(void* stream) {
  RING_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return RING_OK;
}

// ---- primitives -----------------------------------------------------------------

int ring_copy_bytes(void* dst, const void* src, size_t bytes, void* stream) {
  if (bytes == 0) return RING_OK;
  if (!dst || !src) return RING_ERR_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uintptr_t all = reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src) | bytes;
  if ((all & 3u) == 0) {
    HostRow row{dst, src, nullptr, bytes / 4, false};
    return launch_rows(&row, 1, 4, false, s, kRoleCopy);
  }
  uint64_t blocks = (bytes + kBlock - 1) / kBlock;
  if (blocks > 65536) blocks = 65536;
  launch(bytes_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(kBlock), s,
                     static_cast<uint8_t*>(dst), static_cast<const uint8_t*>(src),
                     static_cast<uint64_t>(bytes));
  RING_HIP(hipGetLastError());
  return RING_OK;
}

int ring_accumulate(int dtype, void* dst, const void* src, size_t count, void* stream) {
  if (!dtype_ok(dtype)) return RING_ERR_DTYPE;
  if (count == 0) return RING_OK;
  if (!dst || !src) return RING_ERR_ARGUMENT;
  const size_t esz = dtype_size(dtype);
  if ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & (esz - 1))
    return RING_ERR_ARGUMENT;
  HostRow row{dst, src, dst, count, false};
  return launch_rows(&row, 1, esz, dtype == RING_F32, static_cast<hipStream_t>(stream), kRoleAccumulate);
}

int ring_accumulate_f32(float* dst, const float* src, size_t count, void* stream) {
  return ring_accumulate(RING_F32, dst, src, count, stream);
}
int ring_accumulate_i32(int32_t* dst, const int32_t* src, size_t count, void* stream) {
  return ring_accumulate(RING_I32, dst, src, count, stream);
}
int ring_accumulate_i64(int64_t* dst, const int64_t* src, size_t count, void* stream) {
  return ring_accumulate(RING_I64, dst, src, count, stream);
}

int ring_reduce_scatter_steps(void* buffer, const ring_step* steps, int n_steps, int dtype, void* stream) {
  return steps_common(nullptr, buffer, steps, n_steps, dtype, stream, kStepAddInPlace);
}

int ring_reduce_scatter_steps_from(const void* input, void* buffer, const ring_step* steps, int n_steps,
                                   int dtype, void* stream) {
  if (input == buffer) return steps_common(nullptr, buffer, steps, n_steps, dtype, stream, kStepAddInPlace);
  return steps_common(input, buffer, steps, n_steps, dtype, stream, kStepAddFrom);
}

int ring_apply_rows(const ring_row* rows, int n_rows, int dtype, void* stream) {
  return ring_apply_rows_avg(rows, n_rows, nullptr, 0, dtype, stream);
}

int ring_apply_rows_avg(const ring_row* rows, int n_rows, const unsigned char* divide, int divisor, int dtype,
                        void* stream) {
  if (!dtype_ok(dtype)) return RING_ERR_DTYPE;
  if (n_rows < 0 || divisor < 0) return RING_ERR_ARGUMENT;
  if (n_rows == 0) return RING_OK;
  if (!rows) return RING_ERR_ARGUMENT;
  const size_t esz = dtype_size(dtype);
  RowBuffer<HostRow, kMaxRows> host(static_cast<size_t>(n_rows));
  size_t n_host = 0;
  bool copies_only = true;
  for (int i = 0; i < n_rows; i++) {
    if (rows[i].count == 0) continue;
    if (!rows[i].dst || !rows[i].a) return RING_ERR_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(rows[i].dst) | reinterpret_cast<uintptr_t>(rows[i].a) |
         reinterpret_cast<uintptr_t>(rows[i].b)) & (esz - 1))
      return RING_ERR_ARGUMENT;
    host.data[n_host++] = HostRow{rows[i].dst, rows[i].a, rows[i].b, rows[i].count,
                                  divisor > 0 && (!divide || divide[i] != 0)};
    copies_only = copies_only && rows[i].b == nullptr;
  }
  // copy rows that share a source: one buffer handed to several destinations
  Role role = kRoleAccumulate;
  if (divisor == 0 && n_host > 1 && copies_only) {
    RowBuffer<const void*, kMaxRows> sources(n_host);
    for (size_t k = 0; k < n_host; k++) sources.data[k] = host.data[k].a;
    std::sort(sources.data, sources.data + n_host);
    if (std::adjacent_find(sources.data, sources.data + n_host) != sources.data + n_host) role = kRoleBroadcast;
  }
  return launch_rows(host.data, n_host, esz, dtype == RING_F32, static_cast<hipStream_t>(stream), role, divisor);
}

int ring_allgather_steps(void* buffer, const ring_step* steps, int n_steps, int dtype, void* stream) {
  return steps_common(nullptr, buffer, steps, n_steps, dtype, stream, kStepCopy);
}

namespace {

struct HostFoldRow {
  void* dst;
  const void* const* srcs;
  int m;
  uint64_t count;
  bool divide;
  void* const* more = nullptr;  // further destinations of the result
  int n_more = 0;
};

// Launches fold rows (any number, any mix of source counts) in tables of at most
// kMaxFoldRows rows and kMaxFoldPtrs source pointers.
int launch_fold(const HostFoldRow* rows, size_t n_rows, int divisor, int dtype, hipStream_t s) {
  const size_t esz = dtype_size(dtype);
  const uint64_t vec = 16 / esz;
  bool to_all = false;
  for (size_t k = 0; k < n_rows; k++) to_all = to_all || rows[k].n_more > 0;
  const uint64_t kTileVecs = static_cast<uint64_t>(kBlock) * (to_all ? kFoldToAllUnroll : kFoldUnroll);
  int nt = tuning().nt[to_all ? kRoleFoldAll : kRoleFold];
  if (nt < 0) nt = to_all ? 3 : 2;
  size_t i = 0;
  while (i < n_rows) {
    FoldTable tab;
    tab.n_rows = 0;
    tab.divisor = divisor;
    tab.div_mask = 0;
    tab.tile_begin[0] = 0;
    for (int k = 1; k <= kMaxFoldRows; k++) tab.tile_begin[k] = 0xffffffffu;  // past the last row: after every tile
    uint64_t tiles = 0, first_tiles = 0;
    uint32_t ptrs = 0;
    bool uniform = true;
    while (i < n_rows && tab.n_rows < kMaxFoldRows) {
      const HostFoldRow& r = rows[i];
      if (r.count == 0) { i++; continue; }
      if (r.m < 1 || r.n_more < 0 || r.m + r.n_more > kMaxFoldPtrs) return RING_ERR_ARGUMENT;
      if (ptrs + static_cast<uint32_t>(r.m + r.n_more) > static_cast<uint32_t>(kMaxFoldPtrs)) break;  // next table
      if (!r.dst || !r.srcs || (reinterpret_cast<uintptr_t>(r.dst) & (esz - 1))) return RING_ERR_ARGUMENT;
      const uintptr_t d = reinterpret_cast<uintptr_t>(r.dst);
      uint64_t head = ((16u - (d & 15u)) & 15u) / esz;
      if (head > r.count) head = r.count;
      uint64_t t = ((r.count - head) / vec + kTileVecs - 1) / kTileVecs;
      if (t == 0) t = 1;
      if (tiles + t > 0x7fffffffull) {
        if (tab.n_rows == 0) return RING_ERR_ARGUMENT;
        break;
      }
      const int k = tab.n_rows++;
      tab.row[k] = FoldRow{r.dst, r.count, ptrs, static_cast<uint32_t>(r.m),
                           ptrs + static_cast<uint32_t>(r.m), static_cast<uint32_t>(r.n_more)};
      for (int j = 0; j < r.m; j++) {
        if (!r.srcs[j] || (reinterpret_cast<uintptr_t>(r.srcs[j]) & (esz - 1))) return RING_ERR_ARGUMENT;
        tab.src[ptrs++] = r.srcs[j];
      }
      for (int j = 0; j < r.n_more; j++) {
        if (!r.more[j] || (reinterpret_cast<uintptr_t>(r.more[j]) & (esz - 1))) return RING_ERR_ARGUMENT;
        tab.src[ptrs++] = r.more[j];
      }
      if (divisor > 0 && r.divide) tab.div_mask |= 1u << k;
      if (k == 0) first_tiles = t;
      uniform = uniform && t == first_tiles;
      tiles += t;
      tab.tile_begin[k + 1] = static_cast<uint32_t>(tiles);
      i++;
    }
    if (tab.n_rows == 0) continue;
    dim3 grid;
    if (uniform) {
      tab.uniform_tiles = static_cast<uint32_t>(first_tiles);
      grid = dim3(static_cast<uint32_t>(first_tiles), static_cast<uint32_t>(tab.n_rows));
    } else {
      tab.uniform_tiles = 0;
      grid = dim3(static_cast<uint32_t>(tiles));
    }
#define RING_FOLD_UG(T, D, N)                                                                      \
  if (to_all) launch(fold_kernel<T, D, N, kFoldToAllUnroll, kFoldGroup>, grid, dim3(kBlock), s, tab); \
  else launch(fold_kernel<T, D, N, kFoldUnroll, kFoldGroup>, grid, dim3(kBlock), s, tab);
#define RING_FOLD(T, D)                          \
  switch (nt & 3) {                              \
    case 0: RING_FOLD_UG(T, D, 0) break;         \
    case 1: RING_FOLD_UG(T, D, 1) break;         \
    case 2: RING_FOLD_UG(T, D, 2) break;         \
    default: RING_FOLD_UG(T, D, 3) break;        \
  }
    if (tab.div_mask != 0) {
      if (dtype == RING_F32) { RING_FOLD(float, true) }
      else if (dtype == RING_I32) { RING_FOLD(int32_t, true) }
      else { RING_FOLD(int64_t, true) }
    } else {
      if (dtype == RING_F32) { RING_FOLD(float, false) }
      else if (dtype == RING_I32) { RING_FOLD(int32_t, false) }
      else { RING_FOLD(int64_t, false) }
    }
#undef RING_FOLD_UG
#undef RING_FOLD
    RING_HIP(hipGetLastError());
  }
  return RING_OK;
}

}  // namespace

int ring_fold_rows(const ring_fold_row* rows, int n_rows, int m, int divisor, int dtype, void* stream) {
  return ring_fold_and_copy_rows(rows, n_rows, m, divisor, nullptr, 0, dtype, stream);
}

int ring_fold_and_copy_rows(const ring_fold_row* fold_rows, int n_fold, int m, int divisor, const ring_row* copy_rows,
                            int n_copy, int dtype, void* stream) {
  if (!dtype_ok(dtype)) return RING_ERR_DTYPE;
  if (n_fold < 0 || n_copy < 0 || divisor < 0) return RING_ERR_ARGUMENT;
  if (n_fold > 0 && (m < 1 || m > kMaxFoldPtrs || !fold_rows)) return RING_ERR_ARGUMENT;
  if (n_copy > 0 && !copy_rows) return RING_ERR_ARGUMENT;
  RowBuffer<HostFoldRow, kMaxRows> host(static_cast<size_t>(n_fold) + static_cast<size_t>(n_copy));
  size_t n_host = 0;
  for (int i = 0; i < n_fold; i++)
    host.data[n_host++] = HostFoldRow{fold_rows[i].dst, fold_rows[i].srcs, m, fold_rows[i].count, true};
  for (int i = 0; i < n_copy; i++) {
    if (copy_rows[i].b != nullptr) return RING_ERR_ARGUMENT;  // copy rows only
    host.data[n_host++] = HostFoldRow{copy_rows[i].dst, &copy_rows[i].a, 1, copy_rows[i].count, false};
  }
  return launch_fold(host.data, n_host, divisor, dtype, static_cast<hipStream_t>(stream));
}

int ring_fold_to_all_rows(const ring_fold_to_all_row* rows, int n_rows, int m, int n_dst, int divisor, int dtype,
                          void* stream) {
  if (!dtype_ok(dtype)) return RING_ERR_DTYPE;
  if (n_rows < 0 || divisor < 0 || (n_rows > 0 && !rows)) return RING_ERR_ARGUMENT;
  if (n_rows > 0 && (m < 1 || n_dst < 1 || m + n_dst - 1 > kMaxFoldPtrs)) return RING_ERR_ARGUMENT;
  RowBuffer<HostFoldRow, kMaxRows> host(static_cast<size_t>(n_rows));
  for (int i = 0; i < n_rows; i++) {
    if (rows[i].count > 0 && (!rows[i].dsts || !rows[i].srcs)) return RING_ERR_ARGUMENT;
    HostFoldRow r{rows[i].count > 0 ? rows[i].dsts[0] : nullptr, rows[i].srcs, m, rows[i].count, true};
    r.more = rows[i].count > 0 ? rows[i].dsts + 1 : nullptr;
    r.n_more = n_dst - 1;
    host.data[i] = r;
  }
  return launch_fold(host.data, static_cast<size_t>(n_rows), divisor, dtype, static_cast<hipStream_t>(stream));
}

int ring_scale(int dtype, void* data, size_t count, int divisor, void* stream) {
  if (!dtype_ok(dtype)) return RING_ERR_DTYPE;
  if (divisor < 1) return RING_ERR_ARGUMENT;
  if (count == 0) return RING_OK;
  if (!data || (reinterpret_cast<uintptr_t>(data) & (dtype_size(dtype) - 1))) return RING_ERR_ARGUMENT;
  HostRow row{data, data, nullptr, count, true};
  return launch_rows(&row, 1, dtype_size(dtype), dtype == RING_F32, static_cast<hipStream_t>(stream),
                     kRoleAccumulate, divisor);
}

// ---- fusion ------------------------------------------------------------------------

int ring_fusion_plan_create(const void* const* tensors, const size_t* counts, int k, int dtype,
                            ring_fusion_plan** plan) {
  if (!plan) return RING_ERR_ARGUMENT;
  *plan = nullptr;
  if (!dtype_ok(dtype)) return RING_ERR_DTYPE;
  if (k < 0 || (k > 0 && (!tensors || !counts))) return RING_ERR_ARGUMENT;
  const size_t esz = dtype_size(dtype);
  const uint64_t tile_elems = static_cast<uint64_t>(kFusionTileVecs) * (16 / esz);

  std::vector<uint64_t> offsets;
  std::vector<void*> ptrs;
  uint64_t total = 0;
  for (int j = 0; j < k; j++) {
    if (counts[j] == 0) continue;  // empty tensors occupy nothing in the fused buffer
    if (!tensors[j] || (reinterpret_cast<uintptr_t>(tensors[j]) & (esz - 1))) return RING_ERR_ARGUMENT;
    offsets.push_back(total);
    ptrs.push_back(const_cast<void*>(tensors[j]));
    // a set whose bytes do not fit 64 bits is an error, not a fused buffer that wraps
    if (counts[j] > (UINT64_MAX / esz) - total) return RING_ERR_ARGUMENT;
    total += counts[j];
  }
  offsets.push_back(total);
  const uint64_t ntiles64 = (total + tile_elems - 1) / tile_elems;
  if (ntiles64 > 0x7fffffffull || ptrs.size() > 0x7fffffffull) return RING_ERR_ARGUMENT;

  ring_fusion_plan* p = new (std::nothrow) ring_fusion_plan();
  if (!p) return RING_ERR_ARGUMENT;
  p->dtype = dtype;
  p->esz = esz;
  p->m = static_cast<uint32_t>(ptrs.size());
  p->ntiles = static_cast<uint32_t>(ntiles64);
  p->total = total;
  p->h_offsets = offsets;
  if (total == 0) { *plan = p; return RING_OK; }

  std::vector<FusionTile> tiles(p->ntiles);
  uint32_t t = 0;
  for (uint32_t tile = 0; tile < p->ntiles; tile++) {
    const uint64_t e0 = static_cast<uint64_t>(tile) * tile_elems;
    const uint64_t e1 = (e0 + tile_elems < total) ? e0 + tile_elems : total;
    while (offsets[t + 1] <= e0) t++;
    uint32_t u = t;
    while (offsets[u + 1] < e1) u++;
    tiles[tile].first = t;
    tiles[tile].last = u;
    tiles[tile].addr = t == u ? static_cast<char*>(ptrs[t]) + (e0 - offsets[t]) * esz : nullptr;
  }

  const size_t b_off = offsets.size() * sizeof(uint64_t);
  const size_t b_ptr = ptrs.size() * sizeof(void*);
  const size_t at_tiles = (b_off + b_ptr + 15) & ~static_cast<size_t>(15);
  const size_t b_tile = static_cast<size_t>(p->ntiles) * sizeof(FusionTile);
  std::vector<char> host(at_tiles + b_tile);
  memcpy(host.data(), offsets.data(), b_off);
  memcpy(host.data() + b_off, ptrs.data(), b_ptr);
  memcpy(host.data() + at_tiles, tiles.data(), b_tile);

  hipError_t e = hipGetDevice(&p->device);
  if (e == hipSuccess) e = hipMalloc(&p->d_table, host.size());
  if (e == hipSuccess) e = hipMemcpy(p->d_table, host.data(), host.size(), hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    if (p->d_table) (void)hipFree(p->d_table);
    delete p;
    return hip_fail(e);
  }
  char* base = static_cast<char*>(p->d_table);
  p->d_offsets = reinterpret_cast<uint64_t*>(base);
  p->d_ptrs = reinterpret_cast<void**>(base + b_off);
  p->d_tiles = reinterpret_cast<FusionTile*>(base + at_tiles);
  *plan = p;
  return RING_OK;
}

int ring_fusion_plan_dtype(const ring_fusion_plan* plan) { return plan ? plan->dtype : -1; }

int ring_fusion_plan_destroy(ring_fusion_plan* plan) {
  if (!plan) return RING_OK;
  hipError_t e = plan->d_table ? hipFree(plan->d_table) : hipSuccess;
  delete plan;
  if (e != hipSuccess) return hip_fail(e);
  return RING_OK;
}

size_t ring_fusion_plan_elements(const ring_fusion_plan* plan) { return plan ? plan->total : 0; }

int ring_fusion_pack(const ring_fusion_plan* plan, void* fused, void* stream) {
  return fusion_run(plan, fused, stream, true, 0);
}

int ring_fusion_unpack(const ring_fusion_plan* plan, const void* fused, void* stream) {
  return fusion_run(plan, const_cast<void*>(fused), stream, false, 0);
}

int ring_fusion_unpack_scaled(const ring_fusion_plan* plan, const void* fused, int divisor, void* stream) {
  if (divisor < 1) return RING_ERR_ARGUMENT;
  return fusion_run(plan, const_cast<void*>(fused), stream, false, divisor);
}

int ring_fusion_run_static(int unpack, const void* const* tensors, const size_t* counts, int k, int dtype, void* fused,
                           int divisor, void* stream) {
  if (!dtype_ok(dtype)) return RING_ERR_DTYPE;
  if (k < 0 || (k > 0 && (!tensors || !counts)) || divisor < 0 || (!unpack && divisor != 0)) return RING_ERR_ARGUMENT;
  const size_t esz = dtype_size(dtype);
  const uint64_t tile_elems = static_cast<uint64_t>(kFusionTileVecs) * (16 / esz);
  // first pass over the host arrays: sizes only, so that nothing is launched for a call that is refused
  uint64_t total = 0;
  uint32_t m = 0;
  for (int j = 0; j < k; j++) {
    if (counts[j] == 0) continue;
    if (!tensors[j] || (reinterpret_cast<uintptr_t>(tensors[j]) & (esz - 1))) return RING_ERR_ARGUMENT;
    if (m == kStaticMaxTensors) return RING_ERR_LIMIT;
    m++;
    if (counts[j] > static_cast<uint64_t>(kStaticMaxTiles) * tile_elems - total) return RING_ERR_LIMIT;  // (no sum that wraps)
    total += counts[j];
  }
  if (total == 0) return RING_OK;
  if (!fused || (reinterpret_cast<uintptr_t>(fused) & 15u)) return RING_ERR_ARGUMENT;
  const uint32_t ntiles = static_cast<uint32_t>((total + tile_elems - 1) / tile_elems);

  // One call at a time prepares launches on the array (the lock covers enqueueing, not execution).
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  ScratchState* st = nullptr;
  int rc = scratch_of_current_device(&st);
  if (rc != RING_OK) return rc;
  StaticFusionTable* tab = st->ptr;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // The last call's kernels may still be reading the table this call is about to rewrite. On the same
  // stream they are ordered ahead of it; on another stream this call's launches wait for the event recorded
  // behind them. A stream that is being captured is left alone (a wait would pull the other stream's work
  // into its graph, and a graph's replays run whenever its owner launches them): ordering a captured call
  // against calls on other streams stays with the caller.
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  RING_HIP(hipStreamIsCapturing(s, &capture));
  const bool eager = capture == hipStreamCaptureStatusNone;
  if (eager && st->recorded && st->last_stream != s) RING_HIP(hipStreamWaitEvent(s, st->last_done, 0));

  // the table, kTableChunk tensors per launch; the fused-buffer offsets are the running sum of the counts
  TableChunk chunk;
  chunk.base = 0;
  chunk.n = 0;
  uint64_t at = 0;
  for (int j = 0; j < k; j++) {
    if (counts[j] == 0) continue;
    chunk.off[chunk.n] = at;
    chunk.ptr[chunk.n] = const_cast<void*>(tensors[j]);
    chunk.n++;
    at += counts[j];
    if (chunk.n == kTableChunk || at == total) {
      chunk.end = at;
      hipLaunchKernelGGL(table_chunk_kernel, dim3(1), dim3(kBlock), 0, s, tab, chunk);
      RING_HIP(hipGetLastError());
      chunk.base += chunk.n;
      chunk.n = 0;
      if (at == total) break;  // only empty tensors can follow
    }
  }
  hipLaunchKernelGGL(table_tiles_kernel, dim3((ntiles + kBlock - 1) / kBlock), dim3(kBlock), 0, s, tab, m, ntiles,
                     tile_elems, total, static_cast<uint32_t>(esz));
  RING_HIP(hipGetLastError());
  const FusionView view{dtype, esz, ntiles, total, tab->offsets, tab->ptrs, tab->tiles, m};
  rc = fusion_run(view, fused, stream, !unpack, divisor);
  if (eager) {
    // also after a failed launch: the table kernels above are enqueued and the next call must not overtake them
    const hipError_t e = hipEventRecord(st->last_done, s);
    if (e != hipSuccess) return rc != RING_OK ? rc : hip_fail(e);
    st->last_stream = s;
    st->recorded = true;
  }
  return rc;
}

}  // extern "C"

namespace {

template <typename T, bool GATHER, bool DIV>
int launch_fusion_spans(const ring_fusion_plan* p, const FusionSpanTable& tab, uint32_t tile_lo, uint32_t tile_hi,
                        hipStream_t stream, Role role) {
  uint32_t grid = tile_hi - tile_lo;
  int nt = tuning().nt[role];
  if (nt < 0) nt = 3;
#define RING_SPANS(N)                                                                                        \
  launch(fusion_span_kernel<T, GATHER, N, DIV>, dim3(grid), dim3(kBlock), stream,                            \
         static_cast<const uint64_t*>(p->d_offsets), reinterpret_cast<T* const*>(p->d_ptrs),                 \
         static_cast<const FusionTile*>(p->d_tiles), tile_lo, tile_hi, p->total, tab)
  switch (nt & 3) {
    case 0: RING_SPANS(0); break;
    case 1: RING_SPANS(1); break;
    case 2: RING_SPANS(2); break;
    default: RING_SPANS(3); break;
  }
#undef RING_SPANS
  RING_HIP(hipGetLastError());
  return RING_OK;
}

// The finished segments of a scatter that were received in place lie in ONE buffer, each at its own offset
// (piece k at buffer + begin[k]): the scatter is then the unpack of that buffer, and takes the unpack's
// launch, in registers where the unpack would (a scatter from separate slots was built in that form twice,
// its source per round looked up in LDS or worked out on the scalar unit from the kernel arguments: 37.8 and
// 42.5 us for the ResNet-50 set against 36.6-36.9 us as tiles and 33.4 us for the unpack, because a lane's
// 112 loads then wait for a lookup each instead of going out back to back; not kept). Returns that buffer when
// the spans (empty ones aside) cover the plan's fused space end to end and every `incoming` less `begin`
// elements is the same 16-byte aligned address, else null.
const void* scatter_in_place_buffer(const ring_fusion_plan* p, const ring_fusion_span* spans, int n) {
  uintptr_t buffer = 0;
  uint64_t at = 0;
  bool any = false;
  for (int i = 0; i < n; i++) {
    const ring_fusion_span& sp = spans[i];
    if (sp.count == 0) continue;
    if (sp.begin != at || !sp.incoming) return nullptr;
    const uintptr_t base = reinterpret_cast<uintptr_t>(sp.incoming) - sp.begin * p->esz;
    if ((base & 15u) || (any && base != buffer)) return nullptr;
    buffer = base;
    any = true;
    at = sp.begin + sp.count;
  }
  return (any && at == p->total) ? reinterpret_cast<const void*>(buffer) : nullptr;
}

// Checks the spans (sorted, disjoint, inside the plan, operands present and
// element-aligned) and launches them in tables of kMaxFusionSpans.
int fusion_spans_run(const ring_fusion_plan* p, const ring_fusion_span* spans, int n, bool gather, int divisor,
                     void* stream) {
  if (!p || n < 0 || (n > 0 && !spans) || divisor < 0) return RING_ERR_ARGUMENT;
  const uint64_t tile_elems = static_cast<uint64_t>(kFusionTileVecs) * (16 / p->esz);
  hipStream_t s = static_cast<hipStream_t>(stream);
  uint64_t previous_end = 0;
  if (!gather) {
    if (const void* buffer = scatter_in_place_buffer(p, spans, n))
      return fusion_run(p, const_cast<void*>(buffer), stream, false, divisor);
  }
  int i = 0;
  while (i < n) {
    FusionSpanTable tab;
    tab.n = 0;
    tab.divisor = divisor;
    bool any_in = false;
    while (i < n && tab.n < kMaxFusionSpans) {
      const ring_fusion_span& sp = spans[i++];
      if (sp.count == 0) continue;
      const uint64_t end = sp.begin + sp.count;
      if (sp.begin < previous_end || end < sp.begin || end > p->total) return RING_ERR_ARGUMENT;
      if (gather ? !sp.out : !sp.incoming) return RING_ERR_ARGUMENT;
      if ((reinterpret_cast<uintptr_t>(sp.incoming) | reinterpret_cast<uintptr_t>(sp.out)) & (p->esz - 1))
        return RING_ERR_ARGUMENT;
      previous_end = end;
      any_in = any_in || sp.incoming != nullptr;
      tab.span[tab.n++] = FusionSpan{sp.begin, end, sp.incoming, gather ? sp.out : nullptr};
    }
    if (tab.n == 0) continue;
    const uint32_t tile_lo = static_cast<uint32_t>(tab.span[0].begin / tile_elems);
    const uint32_t tile_hi = static_cast<uint32_t>((tab.span[tab.n - 1].end + tile_elems - 1) / tile_elems);
    int rc;
    if (gather) {
      // Adds wrap on the unsigned carriers. A table with arrivals is an accumulate
      // (every byte touched once); one without is a plain pack, whose output the
      // next kernel reads.
      const Role role = any_in ? kRoleAccumulate : kRolePack;
      if (p->dtype == RING_F32 && any_in) rc = launch_fusion_spans<float, true, false>(p, tab, tile_lo, tile_hi, s, role);
      else if (p->esz == 8) rc = launch_fusion_spans<uint64_t, true, false>(p, tab, tile_lo, tile_hi, s, role);
      else rc = launch_fusion_spans<uint32_t, true, false>(p, tab, tile_lo, tile_hi, s, role);
    } else if (divisor > 0) {
      if (p->dtype == RING_F32) rc = launch_fusion_spans<float, false, true>(p, tab, tile_lo, tile_hi, s, kRoleUnpack);
      else if (p->dtype == RING_I32) rc = launch_fusion_spans<int32_t, false, true>(p, tab, tile_lo, tile_hi, s, kRoleUnpack);
      else rc = launch_fusion_spans<int64_t, false, true>(p, tab, tile_lo, tile_hi, s, kRoleUnpack);
    } else {
      if (p->esz == 8) rc = launch_fusion_spans<uint64_t, false, false>(p, tab, tile_lo, tile_hi, s, kRoleUnpack);
      else rc = launch_fusion_spans<uint32_t, false, false>(p, tab, tile_lo, tile_hi, s, kRoleUnpack);
    }
    if (rc != RING_OK) return rc;
  }
  return RING_OK;
}

}  // namespace

extern "C" {

int ring_fusion_fold_scatter(const ring_fusion_plan* plan, uint64_t fold_begin, uint64_t fold_count,
                             const void* const* staged, int m, void* wire, const ring_fusion_span* finished,
                             int n_finished, int divisor, void* stream) {
  const ring_fusion_plan* p = plan;
  if (!p || m < 0 || n_finished < 0 || divisor < 0 || (m > 0 && !staged) || (n_finished > 0 && !finished))
    return RING_ERR_ARGUMENT;
  if (m > kMaxDirectSpans || n_finished > kMaxDirectSpans) return RING_ERR_LIMIT;
  const uint64_t fold_end = fold_begin + fold_count;
  if (fold_end < fold_begin || fold_end > p->total) return RING_ERR_ARGUMENT;
  FusionDirectTable tab;
  tab.n = 0;
  tab.divisor = divisor;
  tab.m = m;
  tab.fold_begin = fold_begin;
  tab.fold_end = fold_end;
  tab.wire = wire;
  if (fold_count > 0) {
    if (!wire || (reinterpret_cast<uintptr_t>(wire) & (p->esz - 1))) return RING_ERR_ARGUMENT;
    for (int k = 0; k < m; k++)
      if (!staged[k] || (reinterpret_cast<uintptr_t>(staged[k]) & (p->esz - 1))) return RING_ERR_ARGUMENT;
  }
  for (int k = 0; k < kMaxDirectSpans; k++) tab.staged[k] = (k < m && fold_count > 0) ? staged[k] : nullptr;
  uint64_t lowest = fold_count > 0 ? fold_begin : p->total, highest = fold_count > 0 ? fold_end : 0;
  uint64_t previous_end = 0;
  for (int i = 0; i < n_finished; i++) {
    const ring_fusion_span& sp = finished[i];
    if (sp.count == 0) continue;
    const uint64_t end = sp.begin + sp.count;
    if (sp.begin < previous_end || end < sp.begin || end > p->total) return RING_ERR_ARGUMENT;
    if (fold_count > 0 && sp.begin < fold_end && fold_begin < end) return RING_ERR_ARGUMENT;  // meets the fold span
    if (!sp.incoming || (reinterpret_cast<uintptr_t>(sp.incoming) & (p->esz - 1))) return RING_ERR_ARGUMENT;
    previous_end = end;
    tab.span[tab.n++] = FusionDirectSpan{sp.begin, end, sp.incoming};
    if (sp.begin < lowest) lowest = sp.begin;
    if (end > highest) highest = end;
  }
  for (int k = tab.n; k < kMaxDirectSpans; k++) tab.span[k] = FusionDirectSpan{0, 0, nullptr};
  if (highest <= lowest) return RING_OK;  // nothing to do
  const uint64_t tile_elems = static_cast<uint64_t>(kFusionTileVecs) * (16 / p->esz);
  const uint32_t tile_lo = static_cast<uint32_t>(lowest / tile_elems);
  const uint32_t tile_hi = static_cast<uint32_t>((highest + tile_elems - 1) / tile_elems);
  int nt = tuning().nt[kRoleUnpack];
  if (nt < 0) nt = 3;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(tile_hi - tile_lo);
#define RING_DIRECT(T, D, N)                                                                                  \
  launch(fusion_direct_kernel<T, N, D>, grid, dim3(kBlock), s, static_cast<const uint64_t*>(p->d_offsets),    \
         reinterpret_cast<T* const*>(p->d_ptrs), static_cast<const FusionTile*>(p->d_tiles), tile_lo, tile_hi, \
         p->total, tab)
#define RING_DIRECT_NT(T, D)                 \
  switch (nt & 3) {                          \
    case 0: RING_DIRECT(T, D, 0); break;     \
    case 1: RING_DIRECT(T, D, 1); break;     \
    case 2: RING_DIRECT(T, D, 2); break;     \
    default: RING_DIRECT(T, D, 3); break;    \
  }
  if (divisor > 0) {
    if (p->dtype == RING_F32) { RING_DIRECT_NT(float, true) }
    else if (p->dtype == RING_I32) { RING_DIRECT_NT(int32_t, true) }
    else { RING_DIRECT_NT(int64_t, true) }
  } else {
    if (p->dtype == RING_F32) { RING_DIRECT_NT(float, false) }
    else if (p->dtype == RING_I32) { RING_DIRECT_NT(int32_t, false) }
    else { RING_DIRECT_NT(int64_t, false) }
  }
#undef RING_DIRECT_NT
#undef RING_DIRECT
  RING_HIP(hipGetLastError());
  return RING_OK;
}

int ring_fusion_allreduce_all(const ring_fusion_plan* const* in_plans, const ring_fusion_plan* const* out_plans, int n,
                              int divisor, void* stream) {
  if (n < 1 || !in_plans || !out_plans || divisor < 0) return RING_ERR_ARGUMENT;
  if (n > kMaxFusedRanks) return RING_ERR_LIMIT;
  const ring_fusion_plan* first = in_plans[0];
  if (!first) return RING_ERR_ARGUMENT;
  for (int k = 0; k < n; k++) {
    for (const ring_fusion_plan* p : {in_plans[k], out_plans[k]}) {
      // one fused space: the same element type and the same tensor sizes in the same order
      if (!p || p->dtype != first->dtype || p->h_offsets != first->h_offsets) return RING_ERR_ARGUMENT;
    }
  }
  if (first->total == 0) return RING_OK;
  FusedRanks ranks;
  ranks.n = n;
  ranks.divisor = divisor;
  ranks.total = first->total;
  ranks.seg = first->total / static_cast<uint64_t>(n);
  ranks.rem = first->total % static_cast<uint64_t>(n);
  for (int k = 0; k < kMaxFusedRanks; k++) {
    ranks.in[k] = k < n ? in_plans[k]->d_ptrs : nullptr;
    ranks.out[k] = k < n ? out_plans[k]->d_ptrs : nullptr;
    ranks.in_tiles[k] = k < n ? in_plans[k]->d_tiles : nullptr;
    ranks.out_tiles[k] = k < n ? out_plans[k]->d_tiles : nullptr;
  }
  int nt = tuning().nt[kRoleFoldAll];
  if (nt < 0) nt = 3;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint64_t items = static_cast<uint64_t>(first->ntiles) * kFusedAllSplit;
  const dim3 grid(static_cast<uint32_t>(items < 0x7fffffffull ? items : 0x7fffffffull));
#define RING_FUSED_ALL(T, D, N)                                                                              \
  launch(fusion_allreduce_kernel<T, D, N>, grid, dim3(kBlock), s, static_cast<const uint64_t*>(first->d_offsets), \
         static_cast<const FusionTile*>(first->d_tiles), first->ntiles, ranks)
#define RING_FUSED_ALL_NT(T, D)                 \
  switch (nt & 3) {                             \
    case 0: RING_FUSED_ALL(T, D, 0); break;     \
    case 1: RING_FUSED_ALL(T, D, 1); break;     \
    case 2: RING_FUSED_ALL(T, D, 2); break;     \
    default: RING_FUSED_ALL(T, D, 3); break;    \
  }
  if (divisor > 0) {
    if (first->dtype == RING_F32) { RING_FUSED_ALL_NT(float, true) }
    else if (first->dtype == RING_I32) { RING_FUSED_ALL_NT(int32_t, true) }
    else { RING_FUSED_ALL_NT(int64_t, true) }
  } else {
    if (first->dtype == RING_F32) { RING_FUSED_ALL_NT(float, false) }
    else if (first->dtype == RING_I32) { RING_FUSED_ALL_NT(int32_t, false) }
    else { RING_FUSED_ALL_NT(int64_t, false) }
  }
#undef RING_FUSED_ALL_NT
#undef RING_FUSED_ALL
  RING_HIP(hipGetLastError());
  return RING_OK;
}

int ring_describe_scatter_launch(const ring_fusion_plan* plan, const ring_fusion_span* spans, int n_spans, int divisor,
                                 int cus, int* form) {
  if (!plan || !form || n_spans < 0 || (n_spans > 0 && !spans) || divisor < 0 || cus < 1) return RING_ERR_ARGUMENT;
  *form = RING_FORM_TILES;
  if (scatter_in_place_buffer(plan, spans, n_spans))
    *form = choose_unpack_form(plan->total, plan->m, plan->esz, plan->dtype == RING_F32, divisor, tuning(), cus).form;
  return RING_OK;
}

int ring_fusion_gather(const ring_fusion_plan* plan, const ring_fusion_span* spans, int n_spans, void* stream) {
  return fusion_spans_run(plan, spans, n_spans, true, 0, stream);
}

int ring_fusion_scatter(const ring_fusion_plan* plan, const ring_fusion_span* spans, int n_spans, int divisor,
                        void* stream) {
  return fusion_spans_run(plan, spans, n_spans, false, divisor, stream);
}

}  // extern "C"
