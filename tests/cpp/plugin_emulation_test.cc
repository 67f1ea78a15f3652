// The whole plugin on the CPU: csrc/host/*.cc over csrc/ring_kernels.hip
// compiled as plain C++ against tests/cpp/hip_cpu_shim, under
// -fsanitize=address,undefined. The coordinator's paths that end in a launch
// (a tick of separate rings, fused groups in the direct form and through the
// fusion buffer, prepared batches run several steps, allgather of unequal
// rows, a bad node among good ones, ranks submitting from threads of their
// own) otherwise only run where there is a GPU and no sanitizer. "Device"
// memory is host memory here; results are compared bit for bit with the C
// oracle (oracle/ring_oracle.c). Built and run by tests/test_kernels_on_cpu.py;
// prints "plugin emulation: ok".
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include "mpi_collectives.h"

extern "C" {
#include "ring_oracle.h"
}

#define CHECK(cond)                                                                 \
  do {                                                                              \
    if (!(cond)) {                                                                  \
      std::fprintf(stderr, "%s:%d: CHECK failed: %s\n", __FILE__, __LINE__, #cond); \
      std::exit(1);                                                                 \
    }                                                                               \
  } while (0)

namespace {

struct Type {
  int mpic;    // mpic_dtype
  int oracle;  // the oracle's code: 0 float32, 1 int32, 2 int64
  size_t size;
};
const Type kF32 = {MPIC_DT_FLOAT, 0, 4}, kI32 = {MPIC_DT_INT32, 1, 4}, kI64 = {MPIC_DT_INT64, 2, 8};

// 16-byte aligned, as device allocations are
void* device_alloc(size_t bytes) {
  void* p = nullptr;
  CHECK(posix_memalign(&p, 256, bytes ? bytes : 16) == 0);
  std::memset(p, 0xAB, bytes ? bytes : 16);
  return p;
}

uint64_t g_seed = 0x9e3779b97f4a7c15ull;
uint64_t next_random() {
  g_seed ^= g_seed << 13;
  g_seed ^= g_seed >> 7;
  g_seed ^= g_seed << 17;
  return g_seed;
}

// values whose sum depends on the order of the additions (float32) or wraps nowhere (ints)
void fill(const Type& t, void* p, size_t count) {
  for (size_t i = 0; i < count; i++) {
    const uint64_t x = next_random();
    if (t.mpic == MPIC_DT_FLOAT) {
      const float mantissa = static_cast<float>(static_cast<int64_t>(x % 2000001) - 1000000) / 1000000.0f;
      static_cast<float*>(p)[i] = std::ldexp(mantissa, static_cast<int>((x >> 32) % 24) - 12);
    } else if (t.mpic == MPIC_DT_INT32) {
      static_cast<int32_t*>(p)[i] = static_cast<int32_t>(x % 2001) - 1000;
    } else {
      static_cast<int64_t*>(p)[i] = static_cast<int64_t>(x % 2001) - 1000;
    }
  }
}

// tf.div(sum, n): true division for float32, floor division for the integers
void divide(const Type& t, void* p, size_t count, int n) {
  for (size_t i = 0; i < count; i++) {
    if (t.mpic == MPIC_DT_FLOAT) {
      static_cast<float*>(p)[i] = static_cast<float*>(p)[i] / static_cast<float>(n);
    } else if (t.mpic == MPIC_DT_INT32) {
      int32_t& v = static_cast<int32_t*>(p)[i];
      v = static_cast<int32_t>(std::floor(static_cast<double>(v) / n));
    } else {
      int64_t& v = static_cast<int64_t*>(p)[i];
      v = static_cast<int64_t>(std::floor(static_cast<double>(v) / n));
    }
  }
}

// the oracle's ring over the n ranks' tensors; out[r] is rank r's result
std::vector<std::vector<char>> oracle_allreduce(const Type& t, int n, size_t count,
                                                const std::vector<const void*>& inputs) {
  std::vector<std::vector<char>> out(static_cast<size_t>(n), std::vector<char>(count * t.size + 1));
  std::vector<void*> outs;
  for (auto& o : out) outs.push_back(o.data());
  CHECK(oracle_ring_allreduce_threads(n, t.oracle, count, inputs.data(), outs.data(), nullptr) == 0);
  return out;
}

bool same_bytes(const void* a, const void* b, size_t bytes) { return bytes == 0 || std::memcmp(a, b, bytes) == 0; }

void init_world(mpic_world* w, int rank = 0) {
  mpic_context* c = nullptr;
  CHECK(mpic_context_create(w, rank, "MPIInit", "MPIInit", "GPU", nullptr, nullptr, &c) == MPIC_OK);
  CHECK(mpic_context_compute(c) == MPIC_OK);
  CHECK(mpic_context_wait(c) == MPIC_OK);
  CHECK(mpic_context_destroy(c) == MPIC_OK);
}

struct TensorSet {
  std::vector<Type> types;
  std::vector<size_t> counts;
  std::vector<std::string> names;
  // per rank
  std::vector<std::vector<void*>> in, out;

  TensorSet(int n, std::vector<Type> ts, std::vector<size_t> cs, const char* prefix)
      : types(std::move(ts)), counts(std::move(cs)), in(static_cast<size_t>(n)), out(static_cast<size_t>(n)) {
    for (size_t j = 0; j < counts.size(); j++) names.push_back(std::string(prefix) + "/gradient_" + std::to_string(j));
    for (int r = 0; r < n; r++)
      for (size_t j = 0; j < counts.size(); j++) {
        in[static_cast<size_t>(r)].push_back(device_alloc(counts[j] * types[j].size));
        out[static_cast<size_t>(r)].push_back(device_alloc(counts[j] * types[j].size));
      }
  }
  void refill() {
    for (size_t r = 0; r < in.size(); r++)
      for (size_t j = 0; j < counts.size(); j++) fill(types[j], in[r][j], counts[j]);
  }
  ~TensorSet() {
    for (auto& v : in) for (void* p : v) std::free(p);
    for (auto& v : out) for (void* p : v) std::free(p);
  }
  size_t k() const { return counts.size(); }
  std::vector<const char*> name_ptrs() const {
    std::vector<const char*> v;
    for (auto& s : names) v.push_back(s.c_str());
    return v;
  }
  std::vector<int> dtypes() const {
    std::vector<int> v;
    for (auto& t : types) v.push_back(t.mpic);
    return v;
  }
  std::vector<int64_t> dims() const { return std::vector<int64_t>(counts.begin(), counts.end()); }
};

// every tensor on its own: the oracle's ring per tensor, divided where asked
void check_separate(const TensorSet& s, int n, int divisor, const char* what) {
  for (size_t j = 0; j < s.k(); j++) {
    std::vector<const void*> ins;
    for (int r = 0; r < n; r++) ins.push_back(s.in[static_cast<size_t>(r)][j]);
    auto want = oracle_allreduce(s.types[j], n, s.counts[j], ins);
    for (int r = 0; r < n; r++) {
      if (divisor) divide(s.types[j], want[static_cast<size_t>(r)].data(), s.counts[j], divisor);
      if (!same_bytes(want[static_cast<size_t>(r)].data(), s.out[static_cast<size_t>(r)][j], s.counts[j] * s.types[j].size)) {
        std::fprintf(stderr, "%s: tensor %zu of rank %d differs from the oracle\n", what, j, r);
        std::exit(1);
      }
    }
  }
}

// tensors [first, last) fused: the oracle's ring on the concatenation, divided where asked
// divisors[j - first] divides tensor j of the group (0: the sum stays)
void check_fused(const TensorSet& s, int n, size_t first, size_t last, const std::vector<int>& divisors,
                 const char* what) {
  const Type& t = s.types[first];
  size_t total = 0;
  for (size_t j = first; j < last; j++) total += s.counts[j];
  std::vector<std::vector<char>> packed(static_cast<size_t>(n), std::vector<char>(total * t.size + 1));
  std::vector<const void*> ins;
  for (int r = 0; r < n; r++) {
    size_t at = 0;
    for (size_t j = first; j < last; j++) {
      std::memcpy(packed[static_cast<size_t>(r)].data() + at, s.in[static_cast<size_t>(r)][j], s.counts[j] * t.size);
      at += s.counts[j] * t.size;
    }
    ins.push_back(packed[static_cast<size_t>(r)].data());
  }
  auto want = oracle_allreduce(t, n, total, ins);
  for (int r = 0; r < n; r++) {
    size_t at = 0;
    for (size_t j = first; j < last; j++) {
      if (divisors[j - first]) divide(t, want[static_cast<size_t>(r)].data() + at, s.counts[j], divisors[j - first]);
      if (!same_bytes(want[static_cast<size_t>(r)].data() + at, s.out[static_cast<size_t>(r)][j], s.counts[j] * t.size)) {
        std::fprintf(stderr, "%s: fused tensor %zu of rank %d differs from the oracle on the packed buffer\n", what, j, r);
        std::exit(1);
      }
      at += s.counts[j] * t.size;
    }
  }
}

void check_fused(const TensorSet& s, int n, size_t first, size_t last, int divisor, const char* what) {
  check_fused(s, n, first, last, std::vector<int>(last - first, divisor), what);
}

void submit_batches(mpic_world* w, const TensorSet& s, int n, int divisor, std::vector<std::vector<mpic_context*>>* ctx,
                    bool threads) {
  auto names = s.name_ptrs();
  auto dtypes = s.dtypes();
  auto dims = s.dims();
  std::vector<int> ndims(s.k(), 1);
  ctx->assign(static_cast<size_t>(n), std::vector<mpic_context*>(s.k(), nullptr));
  auto one = [&](int r) {
    CHECK(mpic_allreduce_batch(w, r, static_cast<int>(s.k()), names.data(), dtypes.data(), ndims.data(), dims.data(),
                               s.in[static_cast<size_t>(r)].data(), s.out[static_cast<size_t>(r)].data(), divisor,
                               (*ctx)[static_cast<size_t>(r)].data()) == MPIC_OK);
  };
  if (threads) {
    std::vector<std::thread> ts;
    for (int r = 0; r < n; r++) ts.emplace_back(one, r);
    for (auto& t : ts) t.join();
  } else {
    for (int r = 0; r < n; r++) one(r);
  }
}

void wait_all_ok(std::vector<std::vector<mpic_context*>>* ctx) {
  for (auto& v : *ctx) {
    const int rc = mpic_context_wait_batch(v.data(), static_cast<int>(v.size()), 1, nullptr);
    if (rc != MPIC_OK) {
      for (mpic_context* c : v)
        if (c) std::fprintf(stderr, "node failed: %s\n", mpic_context_message(c));
      CHECK(rc == MPIC_OK);
    }
  }
}

void* malloc_output(void*, int dtype, int ndims, const int64_t* dims, int) {
  size_t n = 1;
  for (int i = 0; i < ndims; i++) n *= static_cast<size_t>(dims[i]);
  return device_alloc(n * (dtype == MPIC_DT_INT64 ? 8 : 4));  // freed by the test that reads it
}

}  // namespace

int main() {
  // ---- a tick of separate rings, every form of the ring, ranks on one thread and on threads of their own ----
  for (int n : {1, 3, 4}) {
    mpic_world* w = nullptr;
    CHECK(mpic_world_create(n, &w) == MPIC_OK);
    init_world(w);
    TensorSet s(n, {kF32, kF32, kI32, kI64, kF32, kF32}, {1000, 0, 20011, 5, 8192, 2}, "separate");
    struct { int direct, batched, fuse_copy, divisor; bool threads; } forms[] = {
        {1, 1, 1, 0, false}, {1, 1, 1, n, true}, {0, 1, 1, 0, true}, {0, 0, 0, 0, false}, {0, 1, 0, 3, false}};
    for (auto& f : forms) {
      CHECK(mpic_world_set_option(w, "direct", f.direct) == MPIC_OK);
      CHECK(mpic_world_set_option(w, "batched", f.batched) == MPIC_OK);
      CHECK(mpic_world_set_option(w, "fuse_copy", f.fuse_copy) == MPIC_OK);
      s.refill();
      std::vector<std::vector<mpic_context*>> ctx;
      submit_batches(w, s, n, f.divisor, &ctx, f.threads);
      wait_all_ok(&ctx);
      check_separate(s, n, f.divisor, "separate rings");
    }
    CHECK(mpic_world_destroy(w) == MPIC_OK);
  }

  // ---- one bad node among good ones: it fails alone, on every rank, with the reference's message ----
  {
    const int n = 3;
    mpic_world* w = nullptr;
    CHECK(mpic_world_create(n, &w) == MPIC_OK);
    init_world(w);
    TensorSet s(n, {kF32, kI32, kF32}, {300, 40, 77}, "bad");
    s.refill();
    auto names = s.name_ptrs();
    auto dtypes = s.dtypes();
    std::vector<int> ndims(s.k(), 1);
    std::vector<std::vector<mpic_context*>> ctx(static_cast<size_t>(n), std::vector<mpic_context*>(s.k(), nullptr));
    for (int r = 0; r < n; r++) {
      auto dims = s.dims();
      if (r == 1) dims[1] = 39;  // rank 1 announces another shape for the middle tensor
      CHECK(mpic_allreduce_batch(w, r, static_cast<int>(s.k()), names.data(), dtypes.data(), ndims.data(), dims.data(),
                                 s.in[static_cast<size_t>(r)].data(), s.out[static_cast<size_t>(r)].data(), 0,
                                 ctx[static_cast<size_t>(r)].data()) == MPIC_OK);
    }
    for (int r = 0; r < n; r++) {
      std::vector<int> codes(s.k(), -1);
      CHECK(mpic_context_wait_batch(ctx[static_cast<size_t>(r)].data(), static_cast<int>(s.k()), 1, codes.data()) ==
            MPIC_FAILED_PRECONDITION);
      CHECK(codes[0] == MPIC_OK && codes[1] == MPIC_FAILED_PRECONDITION && codes[2] == MPIC_OK);
      mpic_context* bad = ctx[static_cast<size_t>(r)][1];
      CHECK(bad && std::strstr(mpic_context_message(bad), "Mismatched allreduce tensor shapes") != nullptr);
      CHECK(std::strstr(mpic_context_message(bad), "[40]") && std::strstr(mpic_context_message(bad), "[39]"));
      CHECK(mpic_context_destroy(bad) == MPIC_OK);
    }
    // the good ones are the oracle's
    s.counts[1] = 0;  // nothing of the bad one is compared
    check_separate(s, n, 0, "good nodes beside a bad one");
    CHECK(mpic_world_destroy(w) == MPIC_OK);
  }

  // ---- coordinator fusion: prepared batches run three steps, direct form and through the fusion buffer ----
  for (int direct : {1, 0}) {
    const int n = 4;
    mpic_world* w = nullptr;
    CHECK(mpic_world_create(n, &w) == MPIC_OK);
    init_world(w);
    CHECK(mpic_world_set_option(w, "direct", direct) == MPIC_OK);
    const size_t per_rank = 64 << 10;
    void* buffer = device_alloc(per_rank * n);
    CHECK(mpic_world_set_fusion_buffer(w, buffer, per_rank) == MPIC_OK);
    // six float32 tensors (one empty, ends that cut 16-byte groups), then two int32: two groups
    TensorSet s(n, {kF32, kF32, kF32, kF32, kF32, kF32, kI32, kI32}, {1, 17, 4099, 0, 256, 1023, 333, 12}, "fused");
    auto names = s.name_ptrs();
    auto dtypes = s.dtypes();
    auto dims = s.dims();
    std::vector<int> ndims(s.k(), 1);
    std::vector<mpic_batch*> batches(static_cast<size_t>(n), nullptr);
    for (int r = 0; r < n; r++) {
      CHECK(mpic_batch_create(w, r, static_cast<int>(s.k()), names.data(), dtypes.data(), ndims.data(), dims.data(),
                              s.in[static_cast<size_t>(r)].data(), s.out[static_cast<size_t>(r)].data(), n,
                              &batches[static_cast<size_t>(r)]) == MPIC_OK);
      CHECK(mpic_batch_size(batches[static_cast<size_t>(r)]) == static_cast<int>(s.k()));
    }
    for (int step = 0; step < 3; step++) {
      s.refill();
      for (int r = 0; r < n; r++) CHECK(mpic_batch_submit(batches[static_cast<size_t>(r)]) == MPIC_OK);
      CHECK(mpic_batch_submit(batches[0]) == MPIC_FAILED_PRECONDITION);  // still running: nothing was flushed yet
      CHECK(mpic_batch_busy(batches[0]) == 1);
      CHECK(mpic_world_flush(w) == MPIC_OK);
      for (int r = 0; r < n; r++) {
        std::vector<int> codes(s.k(), -1);
        const int rc = mpic_batch_wait(batches[static_cast<size_t>(r)], codes.data());
        if (rc != MPIC_OK) std::fprintf(stderr, "fused node failed: %s\n", mpic_batch_message(batches[static_cast<size_t>(r)], 0));
        CHECK(rc == MPIC_OK);
        for (int code : codes) CHECK(code == MPIC_OK);
      }
      check_fused(s, n, 0, 6, n, direct ? "fusion, direct form" : "fusion through the buffer");
      check_fused(s, n, 6, 8, n, direct ? "fusion, direct form (int32)" : "fusion through the buffer (int32)");
    }
    // one group whose tensors ask for different divisions (an averaged gradient next to a summed one): it is
    // still one ring on the packed buffer, and only the tensors that asked are divided
    {
      TensorSet mixed(n, {kF32, kF32, kF32, kF32, kF32}, {700, 3, 1025, 64, 333}, "mixed");
      mixed.refill();
      auto mnames = mixed.name_ptrs();
      auto mdtypes = mixed.dtypes();
      auto mdims = mixed.dims();
      std::vector<int> mndims(mixed.k(), 1);
      std::vector<std::vector<mpic_context*>> ctx(static_cast<size_t>(n), std::vector<mpic_context*>(mixed.k(), nullptr));
      for (int r = 0; r < n; r++) {
        const size_t rr = static_cast<size_t>(r);
        CHECK(mpic_allreduce_batch(w, r, 2, mnames.data(), mdtypes.data(), mndims.data(), mdims.data(), mixed.in[rr].data(),
                                   mixed.out[rr].data(), n, ctx[rr].data()) == MPIC_OK);
        CHECK(mpic_allreduce_batch(w, r, 3, mnames.data() + 2, mdtypes.data() + 2, mndims.data() + 2, mdims.data() + 2,
                                   mixed.in[rr].data() + 2, mixed.out[rr].data() + 2, 0, ctx[rr].data() + 2) == MPIC_OK);
      }
      CHECK(mpic_world_flush(w) == MPIC_OK);
      wait_all_ok(&ctx);
      check_fused(mixed, n, 0, 5, std::vector<int>{n, n, 0, 0, 0}, "a group of mixed divisors");
    }
    // a group that does not fit the buffer is cut where it is full: 3 x 5000 float32 against 64 KiB per rank
    {
      TensorSet big(n, {kF32, kF32, kF32, kF32}, {5000, 5000, 5000, 5000}, "cut");
      big.refill();
      std::vector<std::vector<mpic_context*>> ctx;
      submit_batches(w, big, n, 0, &ctx, false);
      CHECK(mpic_world_flush(w) == MPIC_OK);
      wait_all_ok(&ctx);
      check_fused(big, n, 0, 3, 0, "first group of a cut set");   // 60,000 bytes fit, 80,000 do not
      // the fourth tensor is alone in its group: its own ring
      std::vector<const void*> ins;
      for (int r = 0; r < n; r++) ins.push_back(big.in[static_cast<size_t>(r)][3]);
      auto want = oracle_allreduce(kF32, n, 5000, ins);
      for (int r = 0; r < n; r++)
        CHECK(same_bytes(want[static_cast<size_t>(r)].data(), big.out[static_cast<size_t>(r)][3], 20000));
    }
    for (mpic_batch* b : batches) CHECK(mpic_batch_destroy(b) == MPIC_OK);
    CHECK(mpic_world_destroy(w) == MPIC_OK);
    std::free(buffer);
  }

  // ---- allgather of unequal rows (the second phase of mpi_ops.py:152-160: sizes known) ----
  {
    const int n = 4;
    mpic_world* w = nullptr;
    CHECK(mpic_world_create(n, &w) == MPIC_OK);
    init_world(w);
    const int64_t rows[4] = {3, 0, 17, 1}, cols = 37;
    int64_t total = 0;
    for (int64_t r : rows) total += r;
    std::vector<void*> ins;
    std::vector<float> want;
    for (int r = 0; r < n; r++) {
      ins.push_back(device_alloc(static_cast<size_t>(rows[r] * cols) * 4));
      fill(kF32, ins.back(), static_cast<size_t>(rows[r] * cols));
      const float* p = static_cast<const float*>(ins.back());
      want.insert(want.end(), p, p + rows[r] * cols);
    }
    std::vector<mpic_context*> ctx(static_cast<size_t>(n), nullptr);
    for (int r = 0; r < n; r++) {
      CHECK(mpic_context_create(w, r, "MPIAllgather", "gather", "GPU", malloc_output, nullptr, &ctx[static_cast<size_t>(r)]) == MPIC_OK);
      const int64_t dims[2] = {rows[r], cols}, sizes_dims[1] = {n};
      CHECK(mpic_context_add_input(ctx[static_cast<size_t>(r)], MPIC_DT_FLOAT, 2, dims, ins[static_cast<size_t>(r)], 0) == MPIC_OK);
      CHECK(mpic_context_add_input(ctx[static_cast<size_t>(r)], MPIC_DT_INT64, 1, sizes_dims, rows, 1) == MPIC_OK);
      CHECK(mpic_context_compute(ctx[static_cast<size_t>(r)]) == MPIC_OK);
    }
    for (int r = 0; r < n; r++) {
      CHECK(mpic_context_wait(ctx[static_cast<size_t>(r)]) == MPIC_OK);
      int dtype = 0, ndims = 0;
      int64_t dims[8] = {0};
      void* data = nullptr;
      CHECK(mpic_context_num_outputs(ctx[static_cast<size_t>(r)]) == 1);
      CHECK(mpic_context_output(ctx[static_cast<size_t>(r)], 0, &dtype, &ndims, dims, &data) == MPIC_OK);
      CHECK(dtype == MPIC_DT_FLOAT && ndims == 2 && dims[0] == total && dims[1] == cols);
      CHECK(same_bytes(data, want.data(), want.size() * 4));
      std::free(data);
      CHECK(mpic_context_destroy(ctx[static_cast<size_t>(r)]) == MPIC_OK);
    }
    for (void* p : ins) std::free(p);
    CHECK(mpic_world_destroy(w) == MPIC_OK);
  }

  // ---- a world of ONE real rank whose peers' segments are pre-staged: what every rank received in the
  // oracle's threaded ring is staged for it, and the op gives that rank's output; fuse_copy on and off,
  // the average after the collective as the reference has it; nothing staged is an error, not a hang ----
  for (const Type& t : {kF32, kI64}) {
    const int n = 4;
    const size_t count = 10007, slot = oracle_temp_elements(count, n);
    std::vector<void*> ins;
    std::vector<const void*> cins;
    for (int r = 0; r < n; r++) {
      ins.push_back(device_alloc(count * t.size));
      fill(t, ins.back(), count);
      cins.push_back(ins.back());
    }
    std::vector<std::vector<char>> outs(static_cast<size_t>(n), std::vector<char>(count * t.size));
    std::vector<std::vector<char>> rs(static_cast<size_t>(n), std::vector<char>((n - 1) * slot * t.size));
    std::vector<std::vector<char>> ag(static_cast<size_t>(n), std::vector<char>((n - 1) * slot * t.size));
    std::vector<void*> out_ptrs;
    std::vector<oracle_tap> taps(static_cast<size_t>(n));
    for (int r = 0; r < n; r++) {
      out_ptrs.push_back(outs[static_cast<size_t>(r)].data());
      taps[static_cast<size_t>(r)] = oracle_tap{rs[static_cast<size_t>(r)].data(), ag[static_cast<size_t>(r)].data(), slot};
    }
    CHECK(oracle_ring_allreduce_threads(n, t.oracle, count, cins.data(), out_ptrs.data(), taps.data()) == 0);
    for (int r = 0; r < n; r++) {
      const size_t rr = static_cast<size_t>(r);
      // the same from the oracle's rank run alone on these segments (its fourth way to run)
      std::vector<const void*> rs_ptrs, ag_ptrs;
      std::vector<void*> staged;  // "device" copies of the segments
      for (int i = 0; i < n - 1; i++) {
        for (auto* from : {&rs, &ag}) {
          staged.push_back(device_alloc(slot * t.size));
          std::memcpy(staged.back(), (*from)[rr].data() + static_cast<size_t>(i) * slot * t.size, slot * t.size);
          (from == &rs ? rs_ptrs : ag_ptrs).push_back(staged.back());
        }
      }
      std::vector<char> alone(count * t.size);
      CHECK(oracle_ring_allreduce_rank_prestaged(n, r, t.oracle, ins[rr], alone.data(), count, rs_ptrs.data(),
                                                 ag_ptrs.data()) == 0);
      CHECK(same_bytes(alone.data(), outs[rr].data(), count * t.size));
      for (int fuse_copy : {1, 0}) {
        mpic_world* w = nullptr;
        CHECK(mpic_world_create_prestaged(n, r, &w) == MPIC_OK);
        init_world(w, r);
        CHECK(mpic_world_set_option(w, "fuse_copy", fuse_copy) == MPIC_OK);
        for (int staged_first : {1, 0}) {
          if (staged_first) CHECK(mpic_stage_peers(w, "grad", rs_ptrs.data(), ag_ptrs.data()) == MPIC_OK);
          mpic_context* c = nullptr;
          CHECK(mpic_context_create(w, r, "MPIAllreduce", "grad", "GPU", malloc_output, nullptr, &c) == MPIC_OK);
          const int64_t dims[1] = {static_cast<int64_t>(count)};
          CHECK(mpic_context_add_input(c, t.mpic, 1, dims, ins[rr], 0) == MPIC_OK);
          CHECK(mpic_context_compute(c) == MPIC_OK);
          void* data = nullptr;
          if (staged_first) {
            CHECK(mpic_context_wait(c) == MPIC_OK);
            CHECK(mpic_context_output(c, 0, nullptr, nullptr, nullptr, &data) == MPIC_OK);
            CHECK(same_bytes(data, outs[rr].data(), count * t.size));
          } else {
            CHECK(mpic_context_wait(c) == MPIC_FAILED_PRECONDITION);  // the staged segments were consumed
            CHECK(std::strstr(mpic_context_message(c), "No pre-staged peer segments") != nullptr);
            CHECK(mpic_context_num_outputs(c) == 1 && mpic_context_output(c, 0, nullptr, nullptr, nullptr, &data) == MPIC_OK);
          }
          std::free(data);
          CHECK(mpic_context_destroy(c) == MPIC_OK);
        }
        CHECK(mpic_world_destroy(w) == MPIC_OK);
      }
      for (void* p : staged) std::free(p);
    }
    for (void* p : ins) std::free(p);
  }

  // ---- the ring over a transport, one thread per rank (the reference's loop with its MPI calls behind the
  // loopback transport): whole segments, pieces, a temp of two segments, the average, allgather of unequal rows ----
  for (const Type& t : {kF32, kI32}) {
    const int n = 3;
    const size_t count = 2003, seg = oracle_temp_elements(count, n);
    struct { int chunks; size_t temp; int divisor; } forms[] = {{1, seg, 0}, {4, seg, 0}, {3, 2 * seg, n}, {16, 2 * seg, 0}};
    for (auto& f : forms) {
      std::vector<void*> ins, outs, temps;
      std::vector<const void*> cins;
      for (int r = 0; r < n; r++) {
        ins.push_back(device_alloc(count * t.size));
        fill(t, ins.back(), count);
        cins.push_back(ins.back());
        outs.push_back(device_alloc(count * t.size));
        temps.push_back(device_alloc(f.temp * t.size));
      }
      auto want = oracle_allreduce(t, n, count, cins);
      mpic_loopback* lb = nullptr;
      CHECK(mpic_loopback_create(n, 60.0, &lb) == MPIC_OK);
      std::vector<std::thread> ranks;
      std::vector<int> rcs(static_cast<size_t>(n), -1);
      for (int r = 0; r < n; r++) {
        ranks.emplace_back([&, r] {
          mpic_transport tp;
          CHECK(mpic_loopback_endpoint(lb, r, &tp) == MPIC_OK);
          const int flags = ((f.chunks - 1) << 4) | (f.divisor << 8);
          rcs[static_cast<size_t>(r)] = mpic_ring_allreduce_transport(n, r, t.mpic, ins[static_cast<size_t>(r)],
                                                                      outs[static_cast<size_t>(r)], temps[static_cast<size_t>(r)],
                                                                      f.temp, count, &tp, nullptr, flags);
          if (rcs[static_cast<size_t>(r)] != MPIC_OK) std::fprintf(stderr, "rank %d: %s\n", r, mpic_last_error());
        });
      }
      for (auto& th : ranks) th.join();
      for (int r = 0; r < n; r++) {
        if (rcs[static_cast<size_t>(r)] != MPIC_OK) std::fprintf(stderr, "transport ring, rank %d: %d\n", r, rcs[static_cast<size_t>(r)]);
        CHECK(rcs[static_cast<size_t>(r)] == MPIC_OK);
        if (f.divisor) divide(t, want[static_cast<size_t>(r)].data(), count, f.divisor);
        CHECK(same_bytes(want[static_cast<size_t>(r)].data(), outs[static_cast<size_t>(r)], count * t.size));
      }
      // allgather of unequal rows over the same transport
      const size_t rows[3] = {5, 0, 2}, cols = 129;
      std::vector<char> gathered_want;
      std::vector<void*> gin, gout;
      for (int r = 0; r < n; r++) {
        gin.push_back(device_alloc(rows[r] * cols * t.size));
        fill(t, gin.back(), rows[r] * cols);
        gathered_want.insert(gathered_want.end(), static_cast<char*>(gin.back()),
                             static_cast<char*>(gin.back()) + rows[r] * cols * t.size);
        gout.push_back(device_alloc(7 * cols * t.size));
      }
      ranks.clear();
      for (int r = 0; r < n; r++) {
        ranks.emplace_back([&, r] {
          mpic_transport tp;
          CHECK(mpic_loopback_endpoint(lb, r, &tp) == MPIC_OK);
          rcs[static_cast<size_t>(r)] = mpic_ring_allgather_transport(n, r, t.mpic, gin[static_cast<size_t>(r)], rows, cols,
                                                                      gout[static_cast<size_t>(r)], &tp, nullptr,
                                                                      (f.chunks - 1) << 4);
        });
      }
      for (auto& th : ranks) th.join();
      for (int r = 0; r < n; r++) {
        CHECK(rcs[static_cast<size_t>(r)] == MPIC_OK);
        CHECK(same_bytes(gathered_want.data(), gout[static_cast<size_t>(r)], gathered_want.size()));
      }
      CHECK(mpic_loopback_destroy(lb) == MPIC_OK);
      for (auto* v : {&ins, &outs, &temps, &gin, &gout})
        for (void* p : *v) std::free(p);
    }
  }

  // ---- the same on random rings: ranks, element type, count (fewer elements than ranks among them), pieces,
  // size of the temp buffer between one and two segments, the average ----
  for (int iteration = 0; iteration < 10; iteration++) {
    const Type types[3] = {kF32, kI32, kI64};
    const Type t = types[next_random() % 3];
    const int n = 1 + static_cast<int>(next_random() % 6);
    const size_t count = next_random() % 4 == 0 ? next_random() % 8 : next_random() % 6000;
    const size_t seg = oracle_temp_elements(count, n);
    const int chunks = 1 + static_cast<int>(next_random() % 16);
    const size_t temp = next_random() % 3 == 0 ? 2 * seg : (next_random() % 2 ? seg : seg + next_random() % (seg + 1));
    const int divisor = next_random() % 2 ? 0 : 1 + static_cast<int>(next_random() % 9);
    std::vector<void*> ins, outs, temps;
    std::vector<const void*> cins;
    for (int r = 0; r < n; r++) {
      ins.push_back(device_alloc(count * t.size));
      fill(t, ins.back(), count);
      cins.push_back(ins.back());
      outs.push_back(device_alloc(count * t.size));
      temps.push_back(device_alloc(temp * t.size));
    }
    auto want = oracle_allreduce(t, n, count, cins);
    mpic_loopback* lb = nullptr;
    CHECK(mpic_loopback_create(n, 60.0, &lb) == MPIC_OK);
    std::vector<std::thread> ranks;
    std::vector<int> rcs(static_cast<size_t>(n), -1);
    for (int r = 0; r < n; r++) {
      ranks.emplace_back([&, r] {
        mpic_transport tp;
        CHECK(mpic_loopback_endpoint(lb, r, &tp) == MPIC_OK);
        const size_t rr = static_cast<size_t>(r);
        rcs[rr] = mpic_ring_allreduce_transport(n, r, t.mpic, ins[rr], outs[rr], temps[rr], temp, count, &tp, nullptr,
                                                ((chunks - 1) << 4) | (divisor << 8));
        if (rcs[rr] != MPIC_OK) std::fprintf(stderr, "rank %d: %s\n", r, mpic_last_error());
      });
    }
    for (auto& th : ranks) th.join();
    for (int r = 0; r < n; r++) {
      const size_t rr = static_cast<size_t>(r);
      if (divisor) divide(t, want[rr].data(), count, divisor);
      if (rcs[rr] != MPIC_OK || !same_bytes(want[rr].data(), outs[rr], count * t.size)) {
        std::fprintf(stderr, "random ring %d: %zu-byte elements, n=%d, count=%zu, %d pieces, temp %zu of segment %zu, divisor %d, rank %d\n",
                     iteration, t.size, n, count, chunks, temp, seg, divisor, r);
        std::exit(1);
      }
    }
    CHECK(mpic_loopback_destroy(lb) == MPIC_OK);
    for (auto* v : {&ins, &outs, &temps})
      for (void* p : *v) std::free(p);
  }

  // ---- fusion scheduling on random gradient sets: which tensors are reduced together follows from the
  // submission order, the element types and the buffer size alone (consecutive ready allreduces of one
  // type while they fit; a group of one is a ring of its own), in both forms of the fused reduction ----
  for (int iteration = 0; iteration < 24; iteration++) {
    const int n = 2 + static_cast<int>(next_random() % 4);
    const size_t k = 1 + next_random() % 12;
    const size_t per_rank = 16 * (1 + next_random() % 1024);  // 16 B .. 16 KiB
    const int direct = static_cast<int>(next_random() % 2);
    const int divisor = (next_random() % 3 == 0) ? 0 : n;
    std::vector<Type> types;
    std::vector<size_t> counts;
    for (size_t j = 0; j < k; j++) {
      const uint64_t x = next_random();
      types.push_back(x % 8 < 5 ? kF32 : (x % 8 < 7 ? kI32 : kI64));  // runs of one type are common
      counts.push_back((x >> 8) % 5 == 0 ? (x >> 16) % 3 : (x >> 16) % 1500);
    }
    mpic_world* w = nullptr;
    CHECK(mpic_world_create(n, &w) == MPIC_OK);
    init_world(w);
    CHECK(mpic_world_set_option(w, "direct", direct) == MPIC_OK);
    void* buffer = device_alloc(per_rank * static_cast<size_t>(n));
    CHECK(mpic_world_set_fusion_buffer(w, buffer, per_rank) == MPIC_OK);
    TensorSet s(n, types, counts, "random");
    s.refill();
    // one tensor in six is announced with another shape by one of the ranks: that node fails on every rank,
    // and a run of tensors that would have been reduced together ends in front of it
    std::vector<bool> bad(k, false);
    std::vector<int> liar(k, 0);
    for (size_t j = 0; j < k; j++) {
      bad[j] = next_random() % 6 == 0;
      liar[j] = static_cast<int>(next_random() % static_cast<uint64_t>(n));
    }
    auto names = s.name_ptrs();
    auto dtypes = s.dtypes();
    std::vector<int> ndims(k, 1);
    std::vector<std::vector<mpic_context*>> ctx(static_cast<size_t>(n), std::vector<mpic_context*>(k, nullptr));
    for (int r = 0; r < n; r++) {
      auto dims = s.dims();
      for (size_t j = 0; j < k; j++)
        if (bad[j] && liar[j] == r) dims[j] += 1;
      const size_t rr = static_cast<size_t>(r);
      CHECK(mpic_allreduce_batch(w, r, static_cast<int>(k), names.data(), dtypes.data(), ndims.data(), dims.data(),
                                 s.in[rr].data(), s.out[rr].data(), divisor, ctx[rr].data()) == MPIC_OK);
    }
    CHECK(mpic_world_flush(w) == MPIC_OK);
    for (int r = 0; r < n; r++) {
      const size_t rr = static_cast<size_t>(r);
      std::vector<int> codes(k, -1);
      mpic_context_wait_batch(ctx[rr].data(), static_cast<int>(k), 1, codes.data());
      for (size_t j = 0; j < k; j++) {
        CHECK(codes[j] == (bad[j] ? MPIC_FAILED_PRECONDITION : MPIC_OK));
        if (bad[j]) {
          CHECK(std::strstr(mpic_context_message(ctx[rr][j]), "Mismatched allreduce tensor shapes") != nullptr);
          CHECK(mpic_context_destroy(ctx[rr][j]) == MPIC_OK);
        }
      }
    }
    char what[128];
    std::snprintf(what, sizeof what, "random set %d (n=%d, k=%zu, buffer %zu, direct=%d, divisor=%d)", iteration, n, k,
                  per_rank, direct, divisor);
    size_t i = 0;
    while (i < k) {
      if (bad[i]) {
        i++;
        continue;
      }
      size_t j = i, bytes = 0;
      while (j < k && !bad[j] && types[j].mpic == types[i].mpic && bytes + counts[j] * types[j].size <= per_rank) {
        bytes += counts[j] * types[j].size;
        j++;
      }
      if (j - i >= 2) {
        check_fused(s, n, i, j, divisor, what);
        i = j;
      } else {
        std::vector<const void*> ins;
        for (int r = 0; r < n; r++) ins.push_back(s.in[static_cast<size_t>(r)][i]);
        auto want = oracle_allreduce(types[i], n, counts[i], ins);
        for (int r = 0; r < n; r++) {
          if (divisor) divide(types[i], want[static_cast<size_t>(r)].data(), counts[i], divisor);
          if (!same_bytes(want[static_cast<size_t>(r)].data(), s.out[static_cast<size_t>(r)][i], counts[i] * types[i].size)) {
            std::fprintf(stderr, "%s: tensor %zu (a ring of its own) of rank %d differs from the oracle\n", what, i, r);
            std::exit(1);
          }
        }
        i++;
      }
    }
    CHECK(mpic_world_destroy(w) == MPIC_OK);
    std::free(buffer);
  }

  std::printf("plugin emulation: ok\n");
  return 0;
}
