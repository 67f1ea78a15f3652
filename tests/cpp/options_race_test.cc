// ring_set_option on one thread while another launches: the options are
// atomic cells and a launch works on the snapshot it took at entry, so this is
// no data race (built with -fsanitize=thread against the CPU stand-in of the
// HIP runtime, like kernel_emulation_test.cc) and, since every form a copy can
// take gives the same bytes, every launch's output is right whichever options
// it happened to see. TEST CODE: not part of the product.
#include <atomic>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <thread>
#include <vector>

#include "ring_abi.h"

int main() {
  std::atomic<bool> done{false};
  std::atomic<long> sets{0};
  std::thread setter([&] {
    const char* names[] = {"paced_copy", "phased_copy", "unroll", "nontemporal_allgather", "nontemporal", "blocks_per_cu"};
    const int values[6][3] = {{-1, 0, 1}, {-1, 0, 1}, {2, 4, 8}, {3, 0, -1}, {-1, 3, 1}, {0, 2, 0}};
    long i = 0;
    while (!done.load()) {
      for (int k = 0; k < 6; k++)
        if (ring_set_option(names[k], values[k][i % 3]) != RING_OK) abort();
      i++;
      sets.fetch_add(1);
    }
    for (int k = 0; k < 6; k++) ring_set_option(names[k], values[k][0] == 2 ? 4 : values[k][0]);
  });

  const size_t counts[3] = {3001, 2049, 777};
  std::vector<uint32_t> src[3];
  for (int k = 0; k < 3; k++) {
    src[k].resize(counts[k]);
    for (size_t i = 0; i < counts[k]; i++) src[k][i] = static_cast<uint32_t>(i * 2654435761u + k);
  }
  const size_t total = counts[0] + counts[1] + counts[2];
  // the fused layout of a small unpack, and a plan over three tensors
  std::vector<uint32_t> t0(counts[0]), t1(counts[1]), t2(counts[2]);
  const void* tensors[3] = {t0.data(), t1.data(), t2.data()};
  ring_fusion_plan* plan = nullptr;
  if (ring_fusion_plan_create(tensors, counts, 3, RING_I32, &plan) != RING_OK) return 2;
  uint32_t* fused = nullptr;
  if (posix_memalign(reinterpret_cast<void**>(&fused), 16, total * 4)) return 2;
  for (size_t i = 0; i < total; i++) fused[i] = static_cast<uint32_t>(i * 40503u + 7);

  int bad = 0;
  for (int it = 0; it < 60 && !bad; it++) {
    std::vector<uint32_t> out(total + 3, 0xdeadbeefu);
    ring_step steps[3];
    size_t at = 1 + (it & 1);  // the destination's alignment alternates
    for (int k = 0; k < 3; k++) {
      steps[k] = ring_step{at, src[k].data(), counts[k]};
      at += counts[k];
    }
    if (ring_allgather_steps(out.data(), steps, 3, RING_I32, nullptr) != RING_OK) bad = 1;
    at = 1 + (it & 1);
    for (int k = 0; k < 3 && !bad; k++) {
      for (size_t i = 0; i < counts[k]; i++)
        if (out[at + i] != src[k][i]) { bad = 1; break; }
      at += counts[k];
    }
    if (out[0] != 0xdeadbeefu || out[at] != 0xdeadbeefu) bad = 1;
    std::vector<uint32_t> acc(counts[0], 5u);
    if (ring_accumulate(RING_I32, acc.data(), src[0].data(), counts[0], nullptr) != RING_OK) bad = 1;
    for (size_t i = 0; i < counts[0] && !bad; i++)
      if (acc[i] != src[0][i] + 5u) bad = 1;
    if (ring_fusion_unpack(plan, fused, nullptr) != RING_OK) bad = 1;
    size_t f = 0;
    for (size_t i = 0; i < counts[0] && !bad; i++) bad = t0[i] != fused[f++];
    for (size_t i = 0; i < counts[1] && !bad; i++) bad = t1[i] != fused[f++];
    for (size_t i = 0; i < counts[2] && !bad; i++) bad = t2[i] != fused[f++];
  }
  done.store(true);
  setter.join();
  ring_fusion_plan_destroy(plan);
  free(fused);
  if (bad) {
    printf("options race test: wrong output\n");
    return 1;
  }
  printf("options race test: ok (%ld rounds of option changes while launching)\n", sets.load());
  return 0;
}
