// The kernel library (csrc/ring_kernels.hip) compiled as plain C++ against the
// CPU stand-in of the HIP runtime in tests/cpp/hip_cpu_shim and run under
// AddressSanitizer and UBSan: every buffer is an exact-size heap block, so an
// index one element outside what a kernel may touch, or a 16-byte access
// through an aligned type at an address that is not, ends the run. Results
// are compared with plain loops (one add / one divide per element).
//
// This checks indexing and alignment of the device code on the CPU. It says
// nothing about speed and is not a CPU path of the product.
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <random>
#include <vector>

#include "ring_abi.h"

#define CHECK(cond)                                                            \
  do {                                                                         \
    if (!(cond)) {                                                             \
      fprintf(stderr, "%s:%d CHECK failed: %s\n", __FILE__, __LINE__, #cond);  \
      exit(1);                                                                 \
    }                                                                          \
  } while (0)
#define OK(call) CHECK((call) == RING_OK)

namespace {

std::mt19937_64 g_rng(12345);
int g_scatters_in_registers = 0;  // scatters that took the form with their payload in registers

template <typename T> int code();
template <> int code<float>() { return RING_F32; }
template <> int code<int32_t>() { return RING_I32; }
template <> int code<int64_t>() { return RING_I64; }

template <typename T> T rnd() {
  return static_cast<T>(static_cast<int64_t>(g_rng() % 2001) - 1000);
}
template <> float rnd<float>() {
  return static_cast<float>(static_cast<int64_t>(g_rng() % 2000001) - 1000000) / 1024.0f;
}

template <typename T> T add(T a, T b) { return b + a; }
template <typename T> T divide(T x, int n) {
  const T q = x / n;
  return q - ((x % n != 0) && (x < 0));
}
template <> float divide<float>(float x, int n) { return x / static_cast<float>(n); }

// An exact-size heap block holding `count` elements that start `lead` elements
// into it (lead breaks 16-byte alignment the way ragged segments do). The block
// ends with the last element, so an overrun is caught; `lead` elements before
// the data are poison that must survive.
template <typename T>
struct Buf {
  T* base = nullptr;
  T* p = nullptr;
  size_t count = 0, lead = 0;
  Buf(size_t n, size_t lead_elems, bool fill = true) : count(n), lead(lead_elems) {
    base = static_cast<T*>(malloc((n + lead_elems) * sizeof(T) + (n + lead_elems == 0)));
    p = base + lead_elems;
    for (size_t i = 0; i < lead_elems; i++) memset(&base[i], 0x5a, sizeof(T));
    for (size_t i = 0; i < n; i++) p[i] = fill ? rnd<T>() : T();
  }
  Buf(const Buf&) = delete;
  Buf(Buf&& o) : base(o.base), p(o.p), count(o.count), lead(o.lead) { o.base = nullptr; }
  ~Buf() { free(base); }
  void check_lead() const {
    for (size_t i = 0; i < lead * sizeof(T); i++) CHECK(reinterpret_cast<const unsigned char*>(base)[i] == 0x5a);
  }
};

template <typename T>
void expect_equal(const T* got, const std::vector<T>& want, const char* what) {
  if (want.empty()) return;
  if (!want.empty() && memcmp(got, want.data(), want.size() * sizeof(T)) != 0) {
    for (size_t i = 0; i < want.size(); i++)
      if (memcmp(&got[i], &want[i], sizeof(T)) != 0) {
        fprintf(stderr, "%s: element %zu of %zu differs\n", what, i, want.size());
        exit(1);
      }
  }
}

const size_t kCounts[] = {0, 1, 2, 3, 4, 5, 7, 8, 15, 16, 17, 63, 255, 1023, 1024, 1025, 4095, 4096, 4097, 4099, 8191, 12289, 20011};

template <typename T>
void test_primitives() {
  for (size_t count : kCounts)
    for (size_t dl = 0; dl < 4; dl++)
      for (size_t sl = 0; sl < 4; sl += (count > 5000 ? 3 : 1)) {
        Buf<T> dst(count, dl), src(count, sl);
        std::vector<T> want(count);
        for (size_t i = 0; i < count; i++) want[i] = add(src.p[i], dst.p[i]);
        OK(ring_accumulate(code<T>(), count ? dst.p : nullptr, count ? src.p : nullptr, count, nullptr));
        expect_equal(dst.p, want, "accumulate");
        dst.check_lead();
        Buf<T> out(count, dl, false);
        OK(ring_copy_bytes(count ? out.p : nullptr, count ? src.p : nullptr, count * sizeof(T), nullptr));
        expect_equal(out.p, std::vector<T>(src.p, src.p + count), "copy");
        out.check_lead();
        for (int divisor : {1, 3, 8}) {
          Buf<T> d(count, dl);
          std::vector<T> w(count);
          for (size_t i = 0; i < count; i++) w[i] = divide(d.p[i], divisor);
          OK(ring_scale(code<T>(), count ? d.p : nullptr, count, divisor, nullptr));
          expect_equal(d.p, w, "scale");
        }
      }
}

// The one-direction launches of the measurement hook: a write probe fills exactly the whole
// 16-byte vectors of every row (what lies behind them, and before the row, stays), a read probe
// changes nothing; what it cannot take it refuses.
template <typename T>
void test_probe() {
  constexpr size_t VEC = 16 / sizeof(T);
  const size_t counts[] = {0, 1, VEC, 5 * VEC + 1, 1024 * VEC, 1024 * VEC + VEC - 1, 3000 * VEC + 2};
  std::vector<Buf<T>> bufs;
  bufs.reserve(8);
  std::vector<ring_row> rows;
  for (size_t c : counts) {
    bufs.emplace_back(c, 4 * VEC);  // four vectors of poison ahead of an aligned row
    CHECK(reinterpret_cast<uintptr_t>(bufs.back().p) % 16 == 0);
    rows.push_back(ring_row{bufs.back().p, bufs.back().p, nullptr, c});
  }
  std::vector<std::vector<T>> before;
  for (auto& b : bufs) before.emplace_back(b.p, b.p + b.count);
  for (int mode : {0, 2}) {
    OK(ring_probe_stream(rows.data(), static_cast<int>(rows.size()), code<T>(), mode, nullptr));
    for (size_t k = 0; k < bufs.size(); k++) expect_equal(bufs[k].p, before[k], "a read probe leaves memory alone");
  }
  for (int mode : {1, 3}) {
    for (size_t k = 0; k < bufs.size(); k++)
      if (bufs[k].count) memcpy(bufs[k].p, before[k].data(), bufs[k].count * sizeof(T));
    OK(ring_probe_stream(rows.data(), static_cast<int>(rows.size()), code<T>(), mode, nullptr));
    for (size_t k = 0; k < bufs.size(); k++) {
      const size_t whole = bufs[k].count / VEC;
      const uint32_t* words = reinterpret_cast<const uint32_t*>(bufs[k].p);
      for (size_t v = 0; v < whole; v++)
        CHECK(words[4 * v] == 1u && words[4 * v + 1] == 2u && words[4 * v + 2] == 3u && words[4 * v + 3] == v % 256);
      for (size_t e = whole * VEC; e < bufs[k].count; e++) CHECK(memcmp(&bufs[k].p[e], &before[k][e], sizeof(T)) == 0);
      bufs[k].check_lead();
    }
  }
  Buf<T> odd(64, 1);  // not 16-byte aligned
  ring_row bad{odd.p, odd.p, nullptr, 64};
  CHECK(ring_probe_stream(&bad, 1, code<T>(), 0, nullptr) == RING_ERR_ARGUMENT);
  CHECK(ring_probe_stream(rows.data(), 1, code<T>(), 4, nullptr) == RING_ERR_ARGUMENT);
  std::vector<ring_row> nine(9, rows[2]);
  CHECK(ring_probe_stream(nine.data(), 9, code<T>(), 0, nullptr) == RING_ERR_ARGUMENT);
  CHECK(ring_probe_stream(rows.data(), 1, 99, 0, nullptr) == RING_ERR_DTYPE);
}

// Rows of mixed kinds and lengths in one call: in-place adds, out-of-place adds,
// copies; some divided. More rows than one table carries.
template <typename T>
void test_mixed_rows(int n_rows, int divisor, size_t max_count) {
  std::vector<Buf<T>> keep;
  keep.reserve(3 * n_rows);
  std::vector<ring_row> rows;
  std::vector<unsigned char> flags;
  std::vector<std::vector<T>> wants;
  std::vector<T*> dsts;
  for (int k = 0; k < n_rows; k++) {
    const size_t c = k == 0 ? max_count : g_rng() % max_count;
    const int kind = k % 3;
    const bool flag = divisor > 0 && ((k * 7 + 1) % 2);
    keep.emplace_back(c, k % 4);
    T* a = keep.back().p;
    T *b = nullptr, *dst;
    if (kind == 0) {
      keep.emplace_back(c, (k + 1) % 4);
      b = dst = keep.back().p;
    } else if (kind == 1) {
      keep.emplace_back(c, (k + 2) % 4);
      b = keep.back().p;
      keep.emplace_back(c, (k + 3) % 4, false);
      dst = keep.back().p;
    } else {
      keep.emplace_back(c, (k + 1) % 4, false);
      dst = keep.back().p;
    }
    std::vector<T> w(c);
    for (size_t i = 0; i < c; i++) {
      T v = b ? add(a[i], b[i]) : a[i];
      w[i] = flag ? divide(v, divisor) : v;
    }
    rows.push_back(ring_row{c ? dst : nullptr, c ? a : nullptr, c ? b : nullptr, c});
    flags.push_back(flag);
    wants.push_back(w);
    dsts.push_back(dst);
  }
  OK(ring_apply_rows_avg(rows.data(), n_rows, flags.data(), divisor, code<T>(), nullptr));
  for (int k = 0; k < n_rows; k++) expect_equal(dsts[k], wants[k], "mixed rows");
  for (auto& b : keep) b.check_lead();
}

// The step tables of one rank of a ragged allreduce: equal tile counts per row (2-D grid).
template <typename T>
void test_step_tables(size_t count, int n) {
  std::vector<size_t> sizes(n), starts(n);
  OK(ring_segment_table(count, n, sizes.data(), starts.data()));
  for (int r = 0; r < n; r += (n > 3 ? n - 1 : 1)) {
    Buf<T> in(count, 0), out(count, 0, false);
    std::vector<Buf<T>> staged;
    std::vector<ring_step> rs, ag;
    std::vector<T> want(in.p, in.p + count);
    for (int i = 0; i < n - 1; i++) {
      int snd, rcv;
      OK(ring_schedule(RING_PHASE_REDUCE_SCATTER, n, r, i, &snd, &rcv));
      staged.emplace_back(sizes[rcv], 0);
      rs.push_back(ring_step{starts[rcv], staged.back().p, sizes[rcv]});
      for (size_t e = 0; e < sizes[rcv]; e++) want[starts[rcv] + e] = add(staged.back().p[e], want[starts[rcv] + e]);
    }
    OK(ring_copy_bytes(out.p, in.p, count * sizeof(T), nullptr));
    OK(ring_reduce_scatter_steps(out.p, rs.data(), n - 1, code<T>(), nullptr));
    expect_equal(out.p, want, "reduce-scatter steps");
    // the same with the copy folded in
    Buf<T> out2(count, 0, false);
    OK(ring_reduce_scatter_steps_from(in.p, out2.p, rs.data(), n - 1, code<T>(), nullptr));
    for (int i = 0; i < n - 1; i++)
      CHECK(rs[i].count == 0 || memcmp(out2.p + rs[i].dst_offset, want.data() + rs[i].dst_offset, rs[i].count * sizeof(T)) == 0);
    for (int i = 0; i < n - 1; i++) {
      int snd, rcv;
      OK(ring_schedule(RING_PHASE_ALLGATHER, n, r, i, &snd, &rcv));
      staged.emplace_back(sizes[rcv], 0);
      ag.push_back(ring_step{starts[rcv], staged.back().p, sizes[rcv]});
      for (size_t e = 0; e < sizes[rcv]; e++) want[starts[rcv] + e] = staged.back().p[e];
    }
    OK(ring_allgather_steps(out.p, ag.data(), n - 1, code<T>(), nullptr));
    expect_equal(out.p, want, "allgather steps");
  }
}

template <typename T>
void test_fold(int m, size_t count, int divisor) {
  std::vector<Buf<T>> srcs;
  std::vector<const void*> ptrs;
  for (int k = 0; k < m; k++) {
    srcs.emplace_back(count, k % 4);
    ptrs.push_back(srcs.back().p);
  }
  Buf<T> dst(count, 1, false);
  std::vector<T> want(count);
  for (size_t i = 0; i < count; i++) {
    T acc = srcs[0].p[i];
    for (int k = 1; k < m; k++) acc = add(acc, srcs[k].p[i]);
    want[i] = divisor ? divide(acc, divisor) : acc;
  }
  ring_fold_row row{dst.p, ptrs.data(), count};
  Buf<T> csrc(count / 2 + 3, 2), cdst(count / 2 + 3, 3, false);
  ring_row copy{cdst.p, csrc.p, nullptr, csrc.count};
  OK(ring_fold_and_copy_rows(&row, 1, m, divisor, &copy, 1, code<T>(), nullptr));
  expect_equal(dst.p, want, "fold");
  expect_equal(cdst.p, std::vector<T>(csrc.p, csrc.p + csrc.count), "copy row beside a fold");
  dst.check_lead();
  cdst.check_lead();
}

// The fold of m sources stored to n_dst destinations of any element alignment, two rows of
// different lengths in one call; then the same in place (every destination is a source).
template <typename T>
void test_fold_to_all(int m, int n_dst, size_t count, int divisor) {
  std::vector<Buf<T>> keep;
  keep.reserve(2 * (m + n_dst) + 4 * m);
  std::vector<std::vector<const void*>> srcs(2);
  std::vector<std::vector<void*>> dsts(2);
  std::vector<std::vector<T>> wants(2);
  const size_t counts[2] = {count, count / 3 + 1};
  std::vector<ring_fold_to_all_row> rows;
  for (int q = 0; q < 2; q++) {
    for (int k = 0; k < m; k++) {
      keep.emplace_back(counts[q], (k + q) % 4);
      srcs[q].push_back(keep.back().p);
    }
    for (int d = 0; d < n_dst; d++) {
      keep.emplace_back(counts[q], (d + 2 * q + 1) % 4, false);
      dsts[q].push_back(keep.back().p);
    }
    wants[q].resize(counts[q]);
    for (size_t i = 0; i < counts[q]; i++) {
      T acc = static_cast<const T*>(srcs[q][0])[i];
      for (int k = 1; k < m; k++) acc = add(acc, static_cast<const T*>(srcs[q][k])[i]);
      wants[q][i] = divisor ? divide(acc, divisor) : acc;
    }
    rows.push_back(ring_fold_to_all_row{dsts[q].data(), srcs[q].data(), counts[q]});
  }
  OK(ring_fold_to_all_rows(rows.data(), 2, m, n_dst, divisor, code<T>(), nullptr));
  for (int q = 0; q < 2; q++)
    for (int d = 0; d < n_dst; d++) expect_equal(static_cast<T*>(dsts[q][d]), wants[q], "fold stored to every destination");
  for (auto& b : keep) b.check_lead();
  // in place: an allreduce of m ranks whose outputs are their inputs
  std::vector<const void*> in_place_src;
  std::vector<void*> in_place_dst;
  for (int k = 0; k < m; k++) {
    keep.emplace_back(count, k % 4);
    in_place_src.push_back(keep.back().p);
    in_place_dst.push_back(keep.back().p);
  }
  std::vector<T> want(count);
  for (size_t i = 0; i < count; i++) {
    T acc = static_cast<const T*>(in_place_src[0])[i];
    for (int k = 1; k < m; k++) acc = add(acc, static_cast<const T*>(in_place_src[k])[i]);
    want[i] = divisor ? divide(acc, divisor) : acc;
  }
  ring_fold_to_all_row row{in_place_dst.data(), in_place_src.data(), count};
  OK(ring_fold_to_all_rows(&row, 1, m, m, divisor, code<T>(), nullptr));
  for (int k = 0; k < m; k++) expect_equal(static_cast<T*>(in_place_dst[k]), want, "fold to all, in place");
}

// The fused allreduce of n resident ranks without a fused buffer, into fresh tensors and in
// place: every tensor element equals the ring's fold of the packed layout's segment it lies in.
template <typename T>
void test_fused_allreduce_of_all_ranks(const std::vector<size_t>& counts, int divisor, int n) {
  size_t total = 0;
  for (size_t c : counts) total += c;
  std::vector<std::vector<Buf<T>>> in(n), out(n);
  std::vector<std::vector<const void*>> in_ptrs(n), out_ptrs(n);
  std::vector<std::vector<T>> packed(n);
  std::vector<ring_fusion_plan*> in_plans(n), out_plans(n);
  for (int r = 0; r < n; r++) {
    in[r].reserve(counts.size());
    out[r].reserve(counts.size());
    for (size_t j = 0; j < counts.size(); j++) {
      in[r].emplace_back(counts[j], (j + r) % 4);
      out[r].emplace_back(counts[j], (j + 2 * r + 1) % 4, false);
      in_ptrs[r].push_back(counts[j] ? in[r].back().p : nullptr);
      out_ptrs[r].push_back(counts[j] ? out[r].back().p : nullptr);
      packed[r].insert(packed[r].end(), in[r].back().p, in[r].back().p + counts[j]);
    }
    OK(ring_fusion_plan_create(in_ptrs[r].data(), counts.data(), static_cast<int>(counts.size()), code<T>(), &in_plans[r]));
    OK(ring_fusion_plan_create(out_ptrs[r].data(), counts.data(), static_cast<int>(counts.size()), code<T>(), &out_plans[r]));
  }
  std::vector<size_t> sizes(n), starts(n);
  OK(ring_segment_table(total, n, sizes.data(), starts.data()));
  std::vector<T> want(total);
  for (int sg = 0; sg < n; sg++)
    for (size_t e = starts[sg]; e < starts[sg] + sizes[sg]; e++) {
      T acc = packed[sg][e];
      for (int k = 1; k < n; k++) acc = add(acc, packed[(sg + k) % n][e]);
      want[e] = divisor ? divide(acc, divisor) : acc;
    }
  auto check = [&](std::vector<std::vector<Buf<T>>>& got, const char* what) {
    for (int r = 0; r < n; r++) {
      size_t at = 0;
      for (auto& t : got[r]) {
        CHECK(t.count == 0 || memcmp(t.p, want.data() + at, t.count * sizeof(T)) == 0 ||
              (fprintf(stderr, "%s, rank %d\n", what, r), false));
        t.check_lead();
        at += t.count;
      }
    }
  };
  OK(ring_fusion_allreduce_all(in_plans.data(), out_plans.data(), n, divisor, nullptr));
  check(out, "fused allreduce of all ranks");
  OK(ring_fusion_allreduce_all(in_plans.data(), in_plans.data(), n, divisor, nullptr));
  check(in, "fused allreduce of all ranks, in place");
  // plans over different tensor sizes do not describe one fused space
  if (counts.size() >= 2 && counts[0] != counts[1] && counts[0] && counts[1] && n >= 2) {
    std::vector<size_t> swapped(counts);
    std::swap(swapped[0], swapped[1]);
    std::vector<const void*> p(in_ptrs[1]);
    std::swap(p[0], p[1]);
    ring_fusion_plan* other = nullptr;
    OK(ring_fusion_plan_create(p.data(), swapped.data(), static_cast<int>(swapped.size()), code<T>(), &other));
    std::vector<ring_fusion_plan*> mixed(in_plans);
    mixed[1] = other;
    CHECK(ring_fusion_allreduce_all(mixed.data(), out_plans.data(), n, divisor, nullptr) == RING_ERR_ARGUMENT);
    OK(ring_fusion_plan_destroy(other));
  }
  CHECK(ring_fusion_allreduce_all(in_plans.data(), out_plans.data(), 17, divisor, nullptr) == RING_ERR_LIMIT);
  for (int r = 0; r < n; r++) {
    OK(ring_fusion_plan_destroy(in_plans[r]));
    OK(ring_fusion_plan_destroy(out_plans[r]));
  }
}

// Pack, unpack (divided or not), gather and scatter over a tensor set, through a
// plan and through the static device table.
template <typename T>
void test_fusion(const std::vector<size_t>& counts, int divisor, int n_ranks) {
  std::vector<Buf<T>> tensors;
  std::vector<const void*> ptrs;
  size_t total = 0;
  for (size_t j = 0; j < counts.size(); j++) {
    tensors.emplace_back(counts[j], j % 4);
    ptrs.push_back(counts[j] ? tensors.back().p : nullptr);
    total += counts[j];
  }
  std::vector<T> packed;
  for (auto& t : tensors) packed.insert(packed.end(), t.p, t.p + t.count);
  ring_fusion_plan* plan = nullptr;
  OK(ring_fusion_plan_create(ptrs.data(), counts.data(), static_cast<int>(counts.size()), code<T>(), &plan));
  CHECK(ring_fusion_plan_elements(plan) == total);
  // the fused buffer must be 16-byte aligned: malloc'd blocks are
  Buf<T> fused(total, 0, false), fused2(total, 0, false);
  OK(ring_fusion_pack(plan, total ? fused.p : nullptr, nullptr));
  expect_equal(fused.p, packed, "pack");
  OK(ring_fusion_run_static(0, ptrs.data(), counts.data(), static_cast<int>(counts.size()), code<T>(),
                            total ? fused2.p : nullptr, 0, nullptr));
  expect_equal(fused2.p, packed, "static pack");

  // unpack into fresh tensors
  auto fresh = [&](std::vector<Buf<T>>& out, std::vector<const void*>& out_ptrs) {
    for (size_t j = 0; j < counts.size(); j++) {
      out.emplace_back(counts[j], (j + 1) % 4, false);
      out_ptrs.push_back(counts[j] ? out.back().p : nullptr);
    }
  };
  auto check_tensors = [&](std::vector<Buf<T>>& out, const std::vector<T>& flat, const char* what) {
    size_t at = 0;
    for (auto& t : out) {
      CHECK(t.count == 0 || memcmp(t.p, flat.data() + at, t.count * sizeof(T)) == 0 || (fprintf(stderr, "%s\n", what), false));
      t.check_lead();
      at += t.count;
    }
  };
  std::vector<T> divided(packed);
  if (divisor)
    for (auto& v : divided) v = divide(v, divisor);
  // as tiles, and with the payload in registers wherever that form takes the set (up to 512 tensors,
  // 112 rounds of the chip, no divisor or a power of two)
  for (int phased : {-1, 1}) {
    CHECK(ring_set_option("phased_copy", phased) == RING_OK);
    {
      std::vector<Buf<T>> out;
      std::vector<const void*> out_ptrs;
      fresh(out, out_ptrs);
      ring_fusion_plan* p2 = nullptr;
      OK(ring_fusion_plan_create(out_ptrs.data(), counts.data(), static_cast<int>(counts.size()), code<T>(), &p2));
      if (divisor) OK(ring_fusion_unpack_scaled(p2, fused.p, divisor, nullptr));
      else OK(ring_fusion_unpack(p2, fused.p, nullptr));
      check_tensors(out, divided, phased > 0 ? "unpack, payload in registers" : "unpack");
      OK(ring_fusion_plan_destroy(p2));
    }
    {
      std::vector<Buf<T>> out;
      std::vector<const void*> out_ptrs;
      fresh(out, out_ptrs);
      OK(ring_fusion_run_static(1, out_ptrs.data(), counts.data(), static_cast<int>(counts.size()), code<T>(),
                                total ? fused.p : nullptr, divisor, nullptr));
      check_tensors(out, divided, phased > 0 ? "static unpack, payload in registers" : "static unpack");
    }
  }
  CHECK(ring_set_option("phased_copy", -1) == RING_OK);
  // gather: wire[seg] = tensors[seg] + incoming (one segment only packed); scatter the result back
  if (total >= static_cast<size_t>(n_ranks)) {
    std::vector<size_t> sizes(n_ranks), starts(n_ranks);
    OK(ring_segment_table(total, n_ranks, sizes.data(), starts.data()));
    Buf<T> wire(total, 0, false);
    std::vector<Buf<T>> incoming;
    std::vector<ring_fusion_span> spans;
    std::vector<T> want(packed);
    for (int g = 0; g < n_ranks; g++) {
      incoming.emplace_back(sizes[g], g % 4);
      const bool plain = g == 1;
      spans.push_back(ring_fusion_span{starts[g], sizes[g], plain ? nullptr : incoming.back().p, wire.p + starts[g]});
      if (!plain)
        for (size_t e = 0; e < sizes[g]; e++) want[starts[g] + e] = add(incoming.back().p[e], want[starts[g] + e]);
    }
    OK(ring_fusion_gather(plan, spans.data(), n_ranks, nullptr));
    expect_equal(wire.p, want, "gather");
    std::vector<Buf<T>> out;
    std::vector<const void*> out_ptrs;
    fresh(out, out_ptrs);
    ring_fusion_plan* p2 = nullptr;
    OK(ring_fusion_plan_create(out_ptrs.data(), counts.data(), static_cast<int>(counts.size()), code<T>(), &p2));
    std::vector<T> scattered(total);
    for (int g = 0; g < n_ranks; g++) {
      spans[g].incoming = incoming[g].p;
      spans[g].out = nullptr;
      for (size_t e = 0; e < sizes[g]; e++)
        scattered[starts[g] + e] = divisor ? divide(incoming[g].p[e], divisor) : incoming[g].p[e];
    }
    OK(ring_fusion_scatter(p2, spans.data(), n_ranks, divisor, nullptr));
    check_tensors(out, scattered, "scatter");
    OK(ring_fusion_plan_destroy(p2));
    {
      // the finished segments received in place, all in one buffer at their own offsets: the scatter is
      // the unpack of that buffer and takes its launch (here forced into the form with the payload in registers)
      Buf<T> arrivals(total, 0, false);
      std::vector<ring_fusion_span> in_place;
      for (int g = 0; g < n_ranks; g++) {
        memcpy(arrivals.p + starts[g], incoming[g].p, sizes[g] * sizeof(T));
        in_place.push_back(ring_fusion_span{starts[g], sizes[g], arrivals.p + starts[g], nullptr});
      }
      std::vector<Buf<T>> out2;
      std::vector<const void*> out2_ptrs;
      fresh(out2, out2_ptrs);
      ring_fusion_plan* p4 = nullptr;
      OK(ring_fusion_plan_create(out2_ptrs.data(), counts.data(), static_cast<int>(counts.size()), code<T>(), &p4));
      CHECK(ring_set_option("phased_copy", 1) == RING_OK);
      int form = -1;
      OK(ring_describe_scatter_launch(p4, in_place.data(), n_ranks, divisor, 4, &form));
      if (form != RING_FORM_TILES) g_scatters_in_registers++;
      OK(ring_fusion_scatter(p4, in_place.data(), n_ranks, divisor, nullptr));
      CHECK(ring_set_option("phased_copy", -1) == RING_OK);
      check_tensors(out2, scattered, "scatter of segments received in place");
      OK(ring_fusion_plan_destroy(p4));
    }
    // the direct form in one launch: segment `own` folded from staged copies and the tensors (last), its sum
    // to the wire buffer, the quotient into the tensors; the other segments scattered
    for (int own : {n_ranks / 2, n_ranks - 1}) {
      std::vector<Buf<T>> work;
      std::vector<const void*> work_ptrs;
      fresh(work, work_ptrs);
      size_t at = 0;
      for (auto& t : work) {
        memcpy(t.p, packed.data() + at, t.count * sizeof(T));
        at += t.count;
      }
      ring_fusion_plan* p3 = nullptr;
      OK(ring_fusion_plan_create(work_ptrs.data(), counts.data(), static_cast<int>(counts.size()), code<T>(), &p3));
      std::vector<Buf<T>> staged;
      std::vector<const void*> staged_ptrs;
      for (int k = 0; k < n_ranks - 1; k++) {
        staged.emplace_back(sizes[own], (k + 1) % 4);
        staged_ptrs.push_back(staged.back().p);
      }
      std::vector<T> sum(sizes[own]);
      for (size_t e = 0; e < sizes[own]; e++) {
        T acc = n_ranks > 1 ? staged[0].p[e] : packed[starts[own] + e];
        for (int k = 1; k < n_ranks - 1; k++) acc = add(staged[k].p[e], acc);
        if (n_ranks > 1) acc = add(packed[starts[own] + e], acc);
        sum[e] = acc;
      }
      std::vector<ring_fusion_span> others;
      std::vector<T> want_tensors(scattered);
      for (int g = 0; g < n_ranks; g++)
        if (g != own) others.push_back(ring_fusion_span{starts[g], sizes[g], incoming[g].p, nullptr});
      for (size_t e = 0; e < sizes[own]; e++) want_tensors[starts[own] + e] = divisor ? divide(sum[e], divisor) : sum[e];
      Buf<T> wire2(sizes[own], 1, false);
      OK(ring_fusion_fold_scatter(p3, starts[own], sizes[own], staged_ptrs.data(), n_ranks - 1, wire2.p, others.data(),
                                  n_ranks - 1, divisor, nullptr));
      expect_equal(wire2.p, sum, "fold_scatter wire");
      check_tensors(work, want_tensors, "fold_scatter tensors");
      OK(ring_fusion_plan_destroy(p3));
    }
  }
  OK(ring_fusion_plan_destroy(plan));
  for (auto& t : tensors) t.check_lead();
  test_fused_allreduce_of_all_ranks<T>(counts, divisor, n_ranks);
}

template <typename T>
void run_all(const char* name) {
  printf("%s: primitives\n", name); fflush(stdout);
  test_primitives<T>();
  test_probe<T>();
  printf("%s: mixed rows\n", name); fflush(stdout);
  test_mixed_rows<T>(1, 1, 20011);
  test_mixed_rows<T>(4, 8, 9000);
  test_mixed_rows<T>(7, 3, 9000);
  test_mixed_rows<T>(70, 6, 5000);
  test_mixed_rows<T>(9, 0, 12000);
  printf("%s: step tables\n", name); fflush(stdout);
  test_step_tables<T>(100003, 6);   // ragged: segments alternate between 0 and 8 / 4 bytes mod 16
  test_step_tables<T>(65536, 8);
  test_step_tables<T>(5, 8);        // fewer elements than ranks
  test_step_tables<T>(40013, 3);
  CHECK(ring_set_option("paced_copy", 1) == RING_OK);   // the allgather copies in their paced form
  test_step_tables<T>(100003, 6);
  test_step_tables<T>(70001, 3);
  CHECK(ring_set_option("paced_copy", -1) == RING_OK);
  CHECK(ring_set_option("phased_copy", 1) == RING_OK);  // ... and with the payload of the launch in registers
  test_step_tables<T>(40013, 3);
  test_step_tables<T>(100003, 4);
  test_step_tables<T>(5, 4);
  test_step_tables<T>(70001, 2);
  test_step_tables<T>(65536, 8);
  test_step_tables<T>(100003, 6);
  test_step_tables<T>(900001, 9);   // 8 rows beyond their share of the registers: falls back to tiles
  test_step_tables<T>(300007, 4);   // one workgroup per CU (more than 224 KiB per CU)
  test_step_tables<T>(400003, 8);
  CHECK(ring_set_option("phased_copy", -1) == RING_OK);
  printf("%s: fold\n", name); fflush(stdout);
  test_fold<T>(8, 10007, 0);
  test_fold<T>(3, 4096, 3);
  test_fold<T>(17, 777, 8);
  test_fold_to_all<T>(8, 8, 10007, 8);
  test_fold_to_all<T>(3, 5, 4099, 0);
  test_fold_to_all<T>(1, 2, 700, 3);
  test_fold_to_all<T>(1, 3, 700, 0);  // one source stored to several destinations as it is
  printf("%s: fusion\n", name); fflush(stdout);
  test_fusion<T>({5, 0, 4099, 1, 64, 0, 3}, 0, 3);
  test_fusion<T>({20000, 64, 64, 36864, 64, 64, 9001, 2, 12288}, 8, 8);
  std::vector<size_t> tiny(600);
  for (auto& c : tiny) c = g_rng() % 40;
  tiny[77] = 9000;
  test_fusion<T>(tiny, 8, 4);  // (a divisor the unpack that holds its payload in registers takes, here on 600 tensors)
  test_fusion<T>({17}, 3, 2);
  test_fusion<T>({}, 0, 2);
  test_fusion<T>({100003, 1, 2, 50001, 0, 4096, 3}, 4, 2);  // tensor ends that cut 16-byte groups, divided by a power of two
  // segments whose ends cut 16-byte groups (19,107 elements in 3, 5 and 7 segments), received in place and scattered from there
  test_fusion<T>({10003, 1, 2, 5001, 0, 4096, 3, 1}, 0, 3);
  test_fusion<T>({10003, 1, 2, 5001, 0, 4096, 3, 1}, 2, 5);
  test_fusion<T>({7, 10003, 1, 2, 5001, 0, 4096, 1}, 4, 7);
}

}  // namespace

// Without an argument all three element types, one after the other; with
// "float32", "int32" or "int64" that one alone (the test runner starts one
// process per type side by side).
int main(int argc, char** argv) {
  CHECK(ring_abi_version() == RING_ABI_VERSION);
  const char* only = argc > 1 ? argv[1] : nullptr;
  int types = 0;
  if (!only || !strcmp(only, "float32")) { run_all<float>("float32"); types++; }
  if (!only || !strcmp(only, "int32")) { run_all<int32_t>("int32"); types++; }
  if (!only || !strcmp(only, "int64")) { run_all<int64_t>("int64"); types++; }
  CHECK(types >= 1);                             // an argument that names no type runs nothing
  CHECK(g_scatters_in_registers >= 3 * types);  // the three cases made for it, per element type, at least
  printf("kernel emulation: ok\n");
  return 0;
}
