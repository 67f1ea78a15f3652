// Launch shapes of a 56 MiB copy and accumulate on gfx950, measured.
//
// The allgather phase of a 64 MiB, N=8 ring allreduce copies 7 segments of
// 8 MiB into a rank's output; the reduce-scatter phase adds 7 such segments
// into it. This program times those two jobs in kernels that differ in ONE
// respect at a time (what a workgroup covers, how many accesses a wave keeps
// in flight, whether the grid is persistent, whether the next tile's loads
// are issued before this tile's stores, whether stores are throttled), so
// that the choices made in csrc/ring_kernels.hip rest on numbers. It does not
// use the library: every variant is a few lines here.
//
//   hipcc -O3 --offload-arch=gfx950 launch_shape_probe.hip -o launch_shape_probe
//   ./launch_shape_probe [floor|pipeline|paced|rounds|registers|timeline|all]
//
// Buffers hold random data and rotate over 8 sets (1.9 GiB), so nothing a
// launch reads is left in a cache by the one before. Durations come from HIP
// events carried in the dispatch (hipExtLaunchKernelGGL). "behind acc" means
// the timed copy is launched right after an untimed accumulate on another
// buffer set, as in a step; the copy then also pays for the accumulate's
// stores that are still draining.
#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#define CK(x)                                                                          \
  do {                                                                                 \
    hipError_t err_ = (x);                                                             \
    if (err_ != hipSuccess) {                                                          \
      printf("HIP error %s at line %d\n", hipGetErrorString(err_), __LINE__);          \
      fflush(stdout);                                                                  \
      exit(1);                                                                         \
    }                                                                                  \
  } while (0)

typedef float f4 __attribute__((ext_vector_type(4)));
constexpr int kRows = 7;
struct Rows {
  f4* dst[kRows];
  const f4* src[kRows];
};

#define LD(p) __builtin_nontemporal_load(p)
#define ST(v, p) __builtin_nontemporal_store(v, p)

enum Mode { kCopy = 0, kAcc = 1, kReadOnly = 2, kWriteOnly = 3, kEmpty = 4 };

// One workgroup per tile of 256 lanes x U vectors, grid (tiles, rows): the library's shape.
// ts != nullptr: lane 0 of every workgroup stores when it started and when its accesses had finished.
template <int MODE, int U>
__global__ void __launch_bounds__(256) k_tile(Rows r, unsigned ntiles, unsigned long long* ts) {
  unsigned long long t0 = 0;
  if (ts && threadIdx.x == 0) t0 = wall_clock64();
  if (MODE != kEmpty) {
    f4* __restrict__ dst = r.dst[blockIdx.y];
    const f4* __restrict__ src = r.src[blockIdx.y];
    for (unsigned t = blockIdx.x; t < ntiles; t += gridDim.x) {
      const size_t v0 = (size_t)t * (256 * U) + threadIdx.x;
      f4 s[U], d[U];
#pragma unroll
      for (int j = 0; j < U; j++) s[j] = MODE == kWriteOnly ? f4{1.f, 2.f, 3.f, (float)threadIdx.x} : LD(&src[v0 + j * 256]);
      if (MODE == kAcc) {
#pragma unroll
        for (int j = 0; j < U; j++) d[j] = LD(&dst[v0 + j * 256]);
#pragma unroll
        for (int j = 0; j < U; j++) s[j] = d[j] + s[j];
      }
      if (MODE == kReadOnly) {
        f4 a = s[0];
#pragma unroll
        for (int j = 1; j < U; j++) a += s[j];
        if (a.x == 12345.678f) ST(a, &dst[v0]);  // never true: keeps the loads alive
      } else {
#pragma unroll
        for (int j = 0; j < U; j++) ST(s[j], &dst[v0 + j * 256]);
      }
    }
  }
  if (ts && threadIdx.x == 0) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const unsigned wg = blockIdx.y * gridDim.x + blockIdx.x;
    ts[2 * wg] = t0;
    ts[2 * wg + 1] = wall_clock64();
  }
}

// A persistent grid over the flattened tile space (tiles_per_row * rows).
// DEPTH 2: software pipelined, the loads of the workgroup's next tile are issued before the stores of this one.
// CHUNKED: a workgroup takes a contiguous run of tiles instead of every gridDim.x-th one.
template <int MODE, int U, int DEPTH, bool CHUNKED>
__global__ void __launch_bounds__(256) k_pipe(Rows r, unsigned tiles_per_row, unsigned total) {
  unsigned t, end, stride;
  if (CHUNKED) {
    const unsigned per = (total + gridDim.x - 1) / gridDim.x;
    t = blockIdx.x * per;
    end = t + per < total ? t + per : total;
    stride = 1;
  } else {
    t = blockIdx.x;
    end = total;
    stride = gridDim.x;
  }
  f4 cur[U], curd[U];
  auto load = [&](unsigned tt, f4* s, f4* d) {
    const unsigned row = tt / tiles_per_row, tile = tt - row * tiles_per_row;
    const size_t v0 = (size_t)tile * (256 * U) + threadIdx.x;
#pragma unroll
    for (int j = 0; j < U; j++) s[j] = LD(&r.src[row][v0 + j * 256]);
    if (MODE == kAcc) {
#pragma unroll
      for (int j = 0; j < U; j++) d[j] = LD(&r.dst[row][v0 + j * 256]);
    }
  };
  auto store = [&](unsigned tt, f4* s, f4* d) {
    const unsigned row = tt / tiles_per_row, tile = tt - row * tiles_per_row;
    const size_t v0 = (size_t)tile * (256 * U) + threadIdx.x;
#pragma unroll
    for (int j = 0; j < U; j++) ST(MODE == kAcc ? d[j] + s[j] : s[j], &r.dst[row][v0 + j * 256]);
  };
  if (t >= end) return;
  load(t, cur, curd);
  while (true) {
    const unsigned nx = t + stride;
    if (DEPTH > 1 && nx < end) {
      f4 nxt[U], nxtd[U];
      load(nx, nxt, nxtd);
      store(t, cur, curd);
#pragma unroll
      for (int j = 0; j < U; j++) {
        cur[j] = nxt[j];
        if (MODE == kAcc) curd[j] = nxtd[j];
      }
    } else {
      store(t, cur, curd);
      if (nx >= end) break;
      load(nx, cur, curd);
    }
    t = nx;
  }
}

template <int K>
__device__ __forceinline__ void wait_vm() {
  if constexpr (K == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  else if constexpr (K == 1) asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
  else if constexpr (K == 3) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
}

// The paced form. R vectors per lane; WAITALL: no store before all loads have arrived;
// SMAX: at most this many stores in flight per wave (0 = no limit). LOOP: grid-stride over the
// tiles (a grid smaller than the number of tiles makes rounds); otherwise exactly one tile per workgroup.
template <int MODE, int R, int WAITALL, int SMAX>
__device__ __forceinline__ void paced_tile(const Rows& r, unsigned tiles_per_row, unsigned t) {
  const unsigned row = t / tiles_per_row, tile = t - row * tiles_per_row;
  const f4* __restrict__ src = r.src[row] + (size_t)tile * (256 * R);
  f4* __restrict__ dst = r.dst[row] + (size_t)tile * (256 * R);
  f4 s[R], d[R];
#pragma unroll
  for (int j = 0; j < R; j++) {
    s[j] = LD(&src[j * 256 + threadIdx.x]);
    if (MODE == kAcc) d[j] = LD(&dst[j * 256 + threadIdx.x]);
  }
  if (WAITALL) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int j = 0; j < R; j++) {
    ST(MODE == kAcc ? d[j] + s[j] : s[j], &dst[j * 256 + threadIdx.x]);
    if (SMAX > 0) wait_vm<SMAX - 1>();
  }
}
template <int MODE, int R, int WAITALL, int SMAX, bool LOOP>
__global__ void __launch_bounds__(256) k_paced(Rows r, unsigned tiles_per_row, unsigned total) {
  if (LOOP) {
    for (unsigned t = blockIdx.x; t < total; t += gridDim.x) paced_tile<MODE, R, WAITALL, SMAX>(r, tiles_per_row, t);
  } else {
    paced_tile<MODE, R, WAITALL, SMAX>(r, tiles_per_row, blockIdx.x);
  }
}

// The whole payload of a launch in registers between ONE read phase and ONE write phase: one
// workgroup per CU (512 registers per lane: one wave per SIMD), a lane takes vectors base,
// base + stride, ... (stride = workgroups * 256), issues all its loads, waits, stores.
// SIDE_BY_SIDE: grid (x, rows), every row swept at the same time by its own x workgroups.
// Otherwise grid (workgroups) and the rows one after the other; CHAIN: the workgroup that
// takes a row's first 256 vectors is the one after the last workgroup of the previous row's
// last round (shift[row]), so that every lane takes the same number of vectors to within one.
// OFF: the sources are read 4 * OFF bytes further on (loads that straddle 16-byte groups).
struct Shift {
  unsigned s[kRows];
};
typedef f4 f4u __attribute__((aligned(4)));
template <int PER, bool SIDE_BY_SIDE, bool CHAIN, int OFF>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
k_registers(Rows r, unsigned nvec, unsigned rounds, Shift sh) {
  constexpr int ROWS = SIDE_BY_SIDE ? 1 : kRows;
  const unsigned stride = gridDim.x * 256;
  f4 s[ROWS * PER];
#pragma unroll
  for (int k = 0; k < ROWS; k++) {
    const int row = SIDE_BY_SIDE ? blockIdx.y : k;
    const f4u* src = (const f4u*)((const char*)r.src[row] + 4 * OFF);
    unsigned w = blockIdx.x;
    if (CHAIN) {
      w += gridDim.x - sh.s[k];
      if (w >= gridDim.x) w -= gridDim.x;
    }
    const unsigned base = w * 256 + threadIdx.x;
#pragma unroll
    for (int j = 0; j < PER; j++)
      if (j < rounds && base + j * stride < nvec) s[k * PER + j] = LD(&src[base + j * stride]);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int k = 0; k < ROWS; k++) {
    const int row = SIDE_BY_SIDE ? blockIdx.y : k;
    f4* dst = r.dst[row];
    unsigned w = blockIdx.x;
    if (CHAIN) {
      w += gridDim.x - sh.s[k];
      if (w >= gridDim.x) w -= gridDim.x;
    }
    const unsigned base = w * 256 + threadIdx.x;
#pragma unroll
    for (int j = 0; j < PER; j++)
      if (j < rounds && base + j * stride < nvec) ST(s[k * PER + j], &dst[base + j * stride]);
  }
}

struct Buffers {
  static const int kSets = 8;
  size_t seg = 0;
  std::vector<char*> out;
  std::vector<std::vector<char*>> staged;
  void init(size_t seg_bytes) {
    seg = seg_bytes;
    std::vector<float> noise((8 * seg + 4096) / 4);
    unsigned x = 12345;
    for (auto& v : noise) {
      x = x * 1664525u + 1013904223u;
      v = (float)(int)(x >> 8) * (1.0f / 8388608.0f) - 1.0f;
    }
    out.resize(kSets);
    staged.assign(kSets, std::vector<char*>(kRows));
    for (int i = 0; i < kSets; i++) {
      CK(hipMalloc(&out[i], 8 * seg + 4096));
      CK(hipMemcpy(out[i], noise.data(), 8 * seg + 4096, hipMemcpyHostToDevice));
      for (int j = 0; j < kRows; j++) {
        CK(hipMalloc(&staged[i][j], seg + 4096));
        CK(hipMemcpy(staged[i][j], noise.data() + 1000 * j, seg + 4096, hipMemcpyHostToDevice));
      }
    }
  }
  void release() {
    for (auto p : out) CK(hipFree(p));
    for (auto& v : staged)
      for (auto p : v) CK(hipFree(p));
    out.clear();
    staged.clear();
  }
  // the 7 segments of set s that an allgather / reduce-scatter phase of rank s touches
  Rows rows(int s) const {
    Rows r;
    for (int j = 0; j < kRows; j++) {
      const int segment = (s + 7 - j) % 8;
      r.dst[j] = (f4*)(out[s] + (size_t)segment * seg);
      r.src[j] = (const f4*)staged[s][j];
    }
    return r;
  }
};

template <typename F>
void run(const char* name, double bytes, F launch, int iters = 168) {
  std::vector<hipEvent_t> ev(2 * iters);
  for (auto& e : ev) CK(hipEventCreate(&e));
  for (int i = 0; i < 16; i++) launch(i % Buffers::kSets, nullptr, nullptr);
  CK(hipDeviceSynchronize());
  for (int i = 0; i < iters; i++) launch(i % Buffers::kSets, ev[2 * i], ev[2 * i + 1]);
  CK(hipDeviceSynchronize());
  std::vector<float> us;
  double sum = 0;
  for (int i = 8; i < iters; i++) {
    float ms;
    CK(hipEventElapsedTime(&ms, ev[2 * i], ev[2 * i + 1]));
    us.push_back(ms * 1e3f);
    sum += ms * 1e3;
  }
  for (auto& e : ev) CK(hipEventDestroy(e));
  std::sort(us.begin(), us.end());
  const double avg = sum / us.size();
  if (bytes > 0)
    printf("%-88s med %6.2f avg %6.2f min %6.2f us  %5.0f GB/s %4.1f %%\n", name, us[us.size() / 2], avg, us[0],
           bytes / avg / 1e3, bytes / avg / 1e3 / 80.0);
  else
    printf("%-88s med %6.2f avg %6.2f min %6.2f us\n", name, us[us.size() / 2], avg, us[0]);
  fflush(stdout);
}

// When the workgroups of one launch start and finish, from their own clock reads (100 MHz).
template <typename F>
void timeline(const char* name, unsigned wgs, F launch) {
  unsigned long long* d_ts;
  CK(hipMalloc(&d_ts, wgs * 16));
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  std::vector<unsigned long long> h(2 * wgs);
  double acc[5] = {0, 0, 0, 0, 0};
  int n = 0;
  for (int i = 0; i < 24; i++) {
    launch(i % Buffers::kSets, e0, e1, d_ts);
    CK(hipDeviceSynchronize());
    if (i < 8) continue;
    float ms;
    CK(hipEventElapsedTime(&ms, e0, e1));
    CK(hipMemcpy(h.data(), d_ts, wgs * 16, hipMemcpyDeviceToHost));
    unsigned long long s0 = ~0ull, s1 = 0, f0 = ~0ull, f1 = 0;
    std::vector<unsigned long long> life(wgs);
    for (unsigned w = 0; w < wgs; w++) {
      s0 = std::min(s0, h[2 * w]);
      s1 = std::max(s1, h[2 * w]);
      f0 = std::min(f0, h[2 * w + 1]);
      f1 = std::max(f1, h[2 * w + 1]);
      life[w] = h[2 * w + 1] - h[2 * w];
    }
    std::nth_element(life.begin(), life.begin() + wgs / 2, life.end());
    acc[0] += ms * 1e3;
    acc[1] += (s1 - s0) * 0.01;
    acc[2] += (f0 - s0) * 0.01;
    acc[3] += (f1 - s0) * 0.01;
    acc[4] += life[wgs / 2] * 0.01;
    n++;
  }
  printf("%-34s dispatch %6.2f us | last workgroup starts +%5.2f | first ends +%5.2f | last ends +%6.2f | outside "
         "the workgroups %5.2f | median workgroup lives %5.2f\n",
         name, acc[0] / n, acc[1] / n, acc[2] / n, acc[3] / n, (acc[0] - acc[3]) / n, acc[4] / n);
  fflush(stdout);
  CK(hipFree(d_ts));
  CK(hipEventDestroy(e0));
  CK(hipEventDestroy(e1));
}

#define EXT(kern, grid, e0, e1, ...) hipExtLaunchKernelGGL(kern, grid, dim3(256), 0, 0, e0, e1, 0, __VA_ARGS__)
#define PLAIN(kern, grid, ...) hipLaunchKernelGGL(kern, grid, dim3(256), 0, 0, __VA_ARGS__)

int main(int argc, char** argv) {
  const char* which = argc > 1 ? argv[1] : "all";
  auto wanted = [&](const char* s) { return !strcmp(which, "all") || !strcmp(which, s); };
  int cus = 0;
  CK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0));
  printf("compute units: %d\n", cus);
  unsigned long long* no_ts = nullptr;

  Buffers B;
  B.init((size_t)8 << 20);
  const size_t seg = B.seg;
  const double cbytes = 2.0 * kRows * seg, abytes = 3.0 * kRows * seg;
  const unsigned nt4 = seg / 16 / 1024;  // 16 KiB tiles per row
  auto acc_before = [&](int s) { PLAIN((k_tile<kAcc, 4>), dim3(nt4, kRows), B.rows(s), nt4, no_ts); };

  if (wanted("floor")) {
    printf("\n-- what a launch costs, and what the chip gives one direction (7 x 8 MiB, nothing launched before)\n");
    run("copy, 16 KiB tiles, grid 512x7 (the library's shape)", cbytes,
        [&](int s, hipEvent_t a, hipEvent_t b) { EXT((k_tile<kCopy, 4>), dim3(nt4, kRows), a, b, B.rows(s), nt4, no_ts); });
    run("accumulate, same grid", abytes,
        [&](int s, hipEvent_t a, hipEvent_t b) { EXT((k_tile<kAcc, 4>), dim3(nt4, kRows), a, b, B.rows(s), nt4, no_ts); });
    run("read only (56 MiB)", cbytes / 2,
        [&](int s, hipEvent_t a, hipEvent_t b) { EXT((k_tile<kReadOnly, 4>), dim3(nt4, kRows), a, b, B.rows(s), nt4, no_ts); });
    run("write only (56 MiB)", cbytes / 2,
        [&](int s, hipEvent_t a, hipEvent_t b) { EXT((k_tile<kWriteOnly, 4>), dim3(nt4, kRows), a, b, B.rows(s), nt4, no_ts); });
    for (unsigned gx : {256u, 512u, 2048u}) {
      for (unsigned gy : {1u, 7u}) {
        char nm[96];
        snprintf(nm, sizeof nm, "empty kernel, grid %ux%u", gx, gy);
        run(nm, 0, [&](int s, hipEvent_t a, hipEvent_t b) { EXT((k_tile<kEmpty, 4>), dim3(gx, gy), a, b, B.rows(s), nt4, no_ts); });
      }
    }
    const unsigned nt2 = seg / 16 / 512, nt8 = seg / 16 / 2048, nt16 = seg / 16 / 4096;
    run("copy, 8 KiB tiles, grid 1024x7", cbytes,
        [&](int s, hipEvent_t a, hipEvent_t b) { EXT((k_tile<kCopy, 2>), dim3(nt2, kRows), a, b, B.rows(s), nt2, no_ts); });
    run("copy, 32 KiB tiles, grid 256x7", cbytes,
        [&](int s, hipEvent_t a, hipEvent_t b) { EXT((k_tile<kCopy, 8>), dim3(nt8, kRows), a, b, B.rows(s), nt8, no_ts); });
    run("copy, 64 KiB tiles, grid 128x7", cbytes,
        [&](int s, hipEvent_t a, hipEvent_t b) { EXT((k_tile<kCopy, 16>), dim3(nt16, kRows), a, b, B.rows(s), nt16, no_ts); });
  }

  if (wanted("pipeline")) {
    printf("\n-- persistent grids, with and without the next tile's loads ahead of this tile's stores\n");
    const unsigned tot4 = nt4 * kRows, nt2 = seg / 16 / 512, tot2 = nt2 * kRows;
    run("copy, one workgroup per 16 KiB tile (reference point)", cbytes,
        [&](int s, hipEvent_t a, hipEvent_t b) { EXT((k_tile<kCopy, 4>), dim3(nt4, kRows), a, b, B.rows(s), nt4, no_ts); });
    run("accumulate, one workgroup per 16 KiB tile (reference point)", abytes,
        [&](int s, hipEvent_t a, hipEvent_t b) { EXT((k_tile<kAcc, 4>), dim3(nt4, kRows), a, b, B.rows(s), nt4, no_ts); });
    for (int k : {2, 4, 8}) {
      const unsigned g = cus * k;
      char nm[128];
      snprintf(nm, sizeof nm, "copy, %d workgroups per CU, 16 KiB tiles, not pipelined", k);
      run(nm, cbytes, [&](int s, hipEvent_t a, hipEvent_t b) { EXT((k_pipe<kCopy, 4, 1, false>), dim3(g), a, b, B.rows(s), nt4, tot4); });
      snprintf(nm, sizeof nm, "copy, %d workgroups per CU, 16 KiB tiles, pipelined", k);
      run(nm, cbytes, [&](int s, hipEvent_t a, hipEvent_t b) { EXT((k_pipe<kCopy, 4, 2, false>), dim3(g), a, b, B.rows(s), nt4, tot4); });
      snprintf(nm, sizeof nm, "copy, %d workgroups per CU, 8 KiB tiles, pipelined", k);
      run(nm, cbytes, [&](int s, hipEvent_t a, hipEvent_t b) { EXT((k_pipe<kCopy, 2, 2, false>), dim3(g), a, b, B.rows(s), nt2, tot2); });
      snprintf(nm, sizeof nm, "copy, %d workgroups per CU, 16 KiB tiles, contiguous runs of tiles, pipelined", k);
      run(nm, cbytes, [&](int s, hipEvent_t a, hipEvent_t b) { EXT((k_pipe<kCopy, 4, 2, true>), dim3(g), a, b, B.rows(s), nt4, tot4); });
      snprintf(nm, sizeof nm, "accumulate, %d workgroups per CU, 16 KiB tiles, pipelined", k);
      run(nm, abytes, [&](int s, hipEvent_t a, hipEvent_t b) { EXT((k_pipe<kAcc, 4, 2, false>), dim3(g), a, b, B.rows(s), nt4, tot4); });
    }
  }

  if (wanted("paced")) {
    printf("\n-- every workgroup resident at once: loads first, stores after, stores throttled (copy timed behind an accumulate)\n");
    run("copy behind acc: 16 KiB tiles, grid 512x7 (reference point)", cbytes, [&](int s, hipEvent_t a, hipEvent_t b) {
      acc_before(s);
      EXT((k_tile<kCopy, 4>), dim3(nt4, kRows), a, b, B.rows((s + 3) % 8), nt4, no_ts);
    });
#define PACED(MODE, R, WAITALL, SMAX, bytes, before)                                                                  \
  {                                                                                                                   \
    char nm[160];                                                                                                     \
    const unsigned tpr = seg / 16 / (256 * R);                                                                        \
    snprintf(nm, sizeof nm, "%s: %d KiB tiles (%u workgroups), %s, %s", MODE == kCopy ? "copy behind acc" : "acc behind copy", \
             R * 4, tpr * kRows, WAITALL ? "stores after all loads" : "stores as loads arrive",                       \
             SMAX ? (SMAX == 1 ? "1 store in flight per wave" : "2 stores in flight per wave") : "stores not throttled"); \
    run(nm, bytes, [&](int s, hipEvent_t a, hipEvent_t b) {                                                           \
      before(s);                                                                                                      \
      EXT((k_paced<MODE, R, WAITALL, SMAX, false>), dim3(tpr * kRows), a, b, B.rows((s + 3) % 8), tpr, tpr * kRows);         \
    });                                                                                                               \
  }
    PACED(kCopy, 4, 1, 0, cbytes, acc_before) PACED(kCopy, 4, 1, 1, cbytes, acc_before)
    PACED(kCopy, 8, 0, 0, cbytes, acc_before) PACED(kCopy, 8, 1, 0, cbytes, acc_before)
    PACED(kCopy, 8, 0, 1, cbytes, acc_before) PACED(kCopy, 8, 1, 1, cbytes, acc_before) PACED(kCopy, 8, 1, 2, cbytes, acc_before)
    PACED(kCopy, 16, 0, 0, cbytes, acc_before) PACED(kCopy, 16, 1, 0, cbytes, acc_before)
    PACED(kCopy, 16, 1, 1, cbytes, acc_before) PACED(kCopy, 16, 1, 2, cbytes, acc_before)
    auto copy_before = [&](int s) { PLAIN((k_tile<kCopy, 4>), dim3(nt4, kRows), B.rows(s), nt4, no_ts); };
    run("acc behind copy: 16 KiB tiles, grid 512x7 (reference point)", abytes, [&](int s, hipEvent_t a, hipEvent_t b) {
      copy_before(s);
      EXT((k_tile<kAcc, 4>), dim3(nt4, kRows), a, b, B.rows((s + 3) % 8), nt4, no_ts);
    });
    PACED(kAcc, 4, 1, 0, abytes, copy_before) PACED(kAcc, 4, 1, 1, abytes, copy_before) PACED(kAcc, 4, 1, 2, abytes, copy_before)
    PACED(kAcc, 8, 1, 1, abytes, copy_before) PACED(kAcc, 8, 1, 2, abytes, copy_before)
  }

  if (wanted("rounds")) {
    printf("\n-- the paced form when the tiles do not all fit on the chip at once (7 x 24 MiB; copy timed behind an accumulate)\n");
    Buffers L;
    L.init((size_t)24 << 20);
    const unsigned lt4 = L.seg / 16 / 1024;
    const double lbytes = 2.0 * kRows * L.seg;
    auto acc_large = [&](int s) { PLAIN((k_tile<kAcc, 4>), dim3(lt4, kRows), L.rows(s), lt4, no_ts); };
    run("copy behind acc: 16 KiB tiles, one workgroup per tile (reference point)", lbytes, [&](int s, hipEvent_t a, hipEvent_t b) {
      acc_large(s);
      EXT((k_tile<kCopy, 4>), dim3(lt4, kRows), a, b, L.rows((s + 3) % 8), lt4, no_ts);
    });
#define ROUNDS(R, WAITALL, SMAX, PERCU)                                                                               \
  {                                                                                                                   \
    char nm[160];                                                                                                     \
    const unsigned tpr = L.seg / 16 / (256 * R), total = tpr * kRows;                                                 \
    const unsigned g = PERCU ? std::min(total, (unsigned)cus * PERCU) : total;                                        \
    snprintf(nm, sizeof nm, "copy behind acc: %d KiB tiles, %u workgroups for %u tiles, %s, %s", R * 4, g, total,     \
             WAITALL ? "stores after all loads" : "stores as loads arrive",                                           \
             SMAX ? "1 store in flight per wave" : "stores not throttled");                                           \
    run(nm, lbytes, [&](int s, hipEvent_t a, hipEvent_t b) {                                                          \
      acc_large(s);                                                                                                   \
      EXT((k_paced<kCopy, R, WAITALL, SMAX, true>), dim3(g), a, b, L.rows((s + 3) % 8), tpr, total);                        \
    });                                                                                                               \
  }
    ROUNDS(8, 1, 1, 0) ROUNDS(8, 1, 1, 7) ROUNDS(8, 1, 1, 4) ROUNDS(8, 1, 0, 4) ROUNDS(8, 0, 0, 7)
    ROUNDS(4, 1, 1, 0) ROUNDS(4, 1, 1, 8) ROUNDS(4, 0, 0, 8) ROUNDS(16, 1, 1, 0) ROUNDS(16, 1, 1, 3)
  }

  if (wanted("registers")) {
    for (size_t seg_bytes : {(size_t)8 << 20, (size_t)9 << 20, (size_t)12800 << 10}) {
      Buffers M;
      M.init(seg_bytes);
      const unsigned nvec = M.seg / 16, mt4 = (nvec + 1023) / 1024;
      const double mbytes = 2.0 * kRows * M.seg;
      printf("\n-- the payload of the launch in registers between one read phase and one write phase (7 x %.2f MiB)\n",
             M.seg / 1048576.0);
      for (int behind = 0; behind < 2; behind++) {
        const char* where = behind ? ", behind acc" : "";
        auto before = [&](int s) {
          if (behind) PLAIN((k_tile<kAcc, 4>), dim3(mt4, kRows), M.rows(s), mt4, no_ts);
        };
        char nm[160];
        snprintf(nm, sizeof nm, "copy%s: 16 KiB tiles, one workgroup per tile (reference point)", where);
        run(nm, mbytes, [&](int s, hipEvent_t a, hipEvent_t b) {
          before(s);
          EXT((k_tile<kCopy, 4>), dim3(mt4, kRows), a, b, M.rows((s + 3) % 8), mt4, no_ts);
        });
        const unsigned gx = cus / kRows, side_rounds = (nvec + gx * 256 - 1) / (gx * 256);
        snprintf(nm, sizeof nm, "copy%s: in registers, the 7 rows side by side, grid (%u, 7), %u rounds", where, gx, side_rounds);
        if (side_rounds <= 112)
          run(nm, mbytes, [&](int s, hipEvent_t a, hipEvent_t b) {
            before(s);
            EXT((k_registers<112, true, false, 0>), dim3(gx, kRows), a, b, M.rows((s + 3) % 8), nvec, side_rounds, Shift{});
          });
        const unsigned stride = cus * 256, rounds = (nvec + stride - 1) / stride;
        Shift sh{};
        unsigned at = 0;
        for (int k = 0; k < kRows; k++) {
          sh.s[k] = at;
          at = (at + (nvec % stride + 255) / 256) % cus;
        }
        if (rounds <= 16) {
          snprintf(nm, sizeof nm, "copy%s: in registers, rows one after the other, %u rounds per row", where, rounds);
          run(nm, mbytes, [&](int s, hipEvent_t a, hipEvent_t b) {
            before(s);
            EXT((k_registers<16, false, false, 0>), dim3(cus), a, b, M.rows((s + 3) % 8), nvec, rounds, sh);
          });
          snprintf(nm, sizeof nm, "copy%s: in registers, rows one after the other, rounds chained across rows", where);
          run(nm, mbytes, [&](int s, hipEvent_t a, hipEvent_t b) {
            before(s);
            EXT((k_registers<16, false, true, 0>), dim3(cus), a, b, M.rows((s + 3) % 8), nvec, rounds, sh);
          });
          snprintf(nm, sizeof nm, "copy%s: the same, sources 4 bytes off their 16-byte groups", where);
          run(nm, mbytes, [&](int s, hipEvent_t a, hipEvent_t b) {
            before(s);
            EXT((k_registers<16, false, true, 1>), dim3(cus), a, b, M.rows((s + 3) % 8), nvec, rounds, sh);
          });
        }
      }
      M.release();
    }
  }

  if (wanted("timeline")) {
    printf("\n-- inside one launch: when its workgroups start and end (nothing launched before)\n");
    const unsigned tot4 = nt4 * kRows;
    timeline("copy, grid 512x7", tot4, [&](int s, hipEvent_t a, hipEvent_t b, unsigned long long* ts) {
      EXT((k_tile<kCopy, 4>), dim3(nt4, kRows), a, b, B.rows(s), nt4, ts);
    });
    timeline("accumulate, grid 512x7", tot4, [&](int s, hipEvent_t a, hipEvent_t b, unsigned long long* ts) {
      EXT((k_tile<kAcc, 4>), dim3(nt4, kRows), a, b, B.rows(s), nt4, ts);
    });
    timeline("read only, grid 512x7", tot4, [&](int s, hipEvent_t a, hipEvent_t b, unsigned long long* ts) {
      EXT((k_tile<kReadOnly, 4>), dim3(nt4, kRows), a, b, B.rows(s), nt4, ts);
    });
    timeline("write only, grid 512x7", tot4, [&](int s, hipEvent_t a, hipEvent_t b, unsigned long long* ts) {
      EXT((k_tile<kWriteOnly, 4>), dim3(nt4, kRows), a, b, B.rows(s), nt4, ts);
    });
    timeline("empty, grid 512x7", tot4, [&](int s, hipEvent_t a, hipEvent_t b, unsigned long long* ts) {
      EXT((k_tile<kEmpty, 4>), dim3(nt4, kRows), a, b, B.rows(s), nt4, ts);
    });
    timeline("empty, grid 256x1", 256, [&](int s, hipEvent_t a, hipEvent_t b, unsigned long long* ts) {
      EXT((k_tile<kEmpty, 4>), dim3(256, 1), a, b, B.rows(s), nt4, ts);
    });
  }
  return 0;
}
