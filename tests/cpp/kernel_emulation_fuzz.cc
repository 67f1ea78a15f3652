// Random shapes, element types and launch options through the cases of
// kernel_emulation_test.cc, on the CPU build of the kernel library under
// AddressSanitizer and UBSan: rows of mixed kinds, step tables of ragged
// rings, folds to one and to many destinations, fusion plans (pack, unpack,
// spans, the direct form, the allocation-free entry point) and the fused
// allreduce of resident ranks. Every case prints its parameters before it
// runs, so a failure names itself.
//
//   kernel_emulation_fuzz [seed] [cases]      (tests/test_kernels_on_cpu.py runs a short, fixed sweep)
#define main kernel_emulation_main
#include "kernel_emulation_test.cc"
#undef main

namespace {

template <typename T>
void one_case(std::mt19937_64& r, int index) {
  auto pick = [&](uint64_t n) { return static_cast<size_t>(r() % n); };
  const int paced = static_cast<int>(pick(3)) - 1, phased = static_cast<int>(pick(3)) - 1;
  const int unroll = 1 << (1 + pick(3));
  CHECK(ring_set_option("paced_copy", paced) == RING_OK);
  CHECK(ring_set_option("phased_copy", phased) == RING_OK);
  CHECK(ring_set_option("unroll", unroll) == RING_OK);
  CHECK(ring_set_option("flat_grid", static_cast<int>(pick(2))) == RING_OK);
  const int per_cu_choices[] = {0, 0, 1, 2, 8};  // 0: one workgroup per tile; else a grid of that many per CU that loops
  const int per_cu = per_cu_choices[pick(5)];
  CHECK(ring_set_option("blocks_per_cu", per_cu) == RING_OK);
  const int what = static_cast<int>(pick(6));
  const size_t big = pick(4) == 0 ? 1 + pick(600000) : 1 + pick(30000);
  printf("[%d] %zu-byte elements, paced_copy=%d phased_copy=%d unroll=%d blocks_per_cu=%d: ", index, sizeof(T), paced,
         phased, unroll, per_cu);
  switch (what) {
    case 0: {
      const int rows = 1 + static_cast<int>(pick(80)), divisor = static_cast<int>(pick(9));
      printf("%d mixed rows of up to %zu elements, divisor %d\n", rows, 1 + big % 20000, divisor);
      fflush(stdout);
      test_mixed_rows<T>(rows, divisor, 1 + big % 20000);
      break;
    }
    case 1: {
      const int n = 1 + static_cast<int>(pick(12));
      printf("step tables of %zu elements in a ring of %d\n", big, n);
      fflush(stdout);
      test_step_tables<T>(big, n);
      break;
    }
    case 2: {
      const int m = 1 + static_cast<int>(pick(20)), divisor = static_cast<int>(pick(9));
      printf("fold of %d sources, %zu elements, divisor %d\n", m, 1 + big % 40000, divisor);
      fflush(stdout);
      test_fold<T>(m, 1 + big % 40000, divisor);
      break;
    }
    case 3: {
      const int m = 1 + static_cast<int>(pick(10)), n_dst = 1 + static_cast<int>(pick(10)), divisor = static_cast<int>(pick(9));
      printf("fold of %d sources to %d destinations, %zu elements, divisor %d\n", m, n_dst, 1 + big % 40000, divisor);
      fflush(stdout);
      test_fold_to_all<T>(m, n_dst, 1 + big % 40000, divisor);
      break;
    }
    default: {
      std::vector<size_t> counts(pick(40));
      for (auto& c : counts) c = pick(5) == 0 ? pick(3) : (pick(6) == 0 ? pick(60000) : pick(3000));
      const int divisors[] = {0, 2, 3, 4, 6, 8};
      const int divisor = divisors[pick(6)], n = 1 + static_cast<int>(pick(9));
      printf("fusion of %zu tensors, divisor %d, %d ranks%s\n", counts.size(), divisor, n,
             what == 5 ? ", and the fused allreduce of resident ranks" : "");
      fflush(stdout);
      test_fusion<T>(counts, divisor, n);
      if (what == 5 && !counts.empty() && n <= 8) test_fused_allreduce_of_all_ranks<T>(counts, divisor, n);
    }
  }
}

}  // namespace

int main(int argc, char** argv) {
  const uint64_t seed = argc > 1 ? strtoull(argv[1], nullptr, 10) : 1;
  const int cases = argc > 2 ? atoi(argv[2]) : 30;
  std::mt19937_64 r(seed);
  g_rng.seed(seed * 7919);
  for (int i = 0; i < cases; i++) {
    switch (r() % 3) {
      case 0: one_case<float>(r, i); break;
      case 1: one_case<int32_t>(r, i); break;
      default: one_case<int64_t>(r, i);
    }
  }
  printf("kernel emulation fuzz, seed %llu: %d cases ok\n", static_cast<unsigned long long>(seed), cases);
  return 0;
}
