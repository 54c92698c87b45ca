// Shutdown while other threads are inside the communicator (CPU only; built with ThreadSanitizer or
// AddressSanitizer by tests/test_host_shutdown.py).
//
// The inference <-> training queues and the info board live in a shared-memory mapping.  Threads of the
// training process sit inside it all the time: a stub's control thread and the stand-in peer's receiver wait in
// tch_mq_timed_get, command threads call tch_mq_put / tch_train_info_set_field.  tch_TorchColShutdown from the
// main thread must not unmap the segment under any of them: every entry point holds a counted reference for
// its own duration, and blocked waits return within 50 ms of the shutdown.  Under the sanitizers a
// use-after-unmap is a SEGV / a reported race, and the program exits non-zero.
#include <stdio.h>
#include <stdlib.h>
#include <unistd.h>

#include <atomic>
#include <chrono>
#include <thread>
#include <vector>

#include "torch_col_host.h"

int main(int argc, char** argv) {
  const int rounds = argc > 1 ? atoi(argv[1]) : 20;
  char port[32];
  snprintf(port, sizeof(port), "%d", 40000 + static_cast<int>(getpid() % 20000));
  setenv("SIRIUS_PORT", port, 1);
  setenv("COLTRAIN_HAS_INFER_SERVER", "1", 1);
  setenv("COLTRAIN_MODE", "colocate-l1", 1);
  int failures = 0;
  for (int r = 0; r < rounds; ++r) {
    // this process plays both sides: it creates the segment (server side), then initialises the trainer
    if (tch_InfTraCommunicator_Init(1, 1, 1) != 0) {
      fprintf(stderr, "communicator init failed: %s\n", tch_host_last_error());
      return 2;
    }
    if (tch_TorchColInit(0, 1, 0) != 0) {
      fprintf(stderr, "runtime init failed: %s\n", tch_host_last_error());
      return 2;
    }
    tch_stub* stub = tch_stub_create(2, 64);   // control thread: timed_get(1000) in a loop
    std::atomic<bool> stop{false};
    std::atomic<long> got{0}, put{0}, refused{0};
    std::vector<std::thread> ts;
    ts.emplace_back([&] {                       // the peer's receiver: short timed waits (10 ms), as DebugServer
      tch_ctrl_msg m;
      while (!stop.load()) {
        int rc = tch_mq_timed_get(1, 0, 10, &m);
        if (rc == 1) got++;
        if (rc < 0) refused++;
      }
    });
    ts.emplace_back([&] {                       // a waiter with a long timeout: must come back soon after shutdown
      tch_ctrl_msg m;
      const auto t0 = std::chrono::steady_clock::now();
      int rc = tch_mq_timed_get(1, 0, 30000, &m);
      while (rc == 1) rc = tch_mq_timed_get(1, 0, 30000, &m);
      const double s = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
      if (s > 5.0) {
        fprintf(stderr, "a blocked timed_get took %.1f s to notice the shutdown\n", s);
        refused += 1000000;
      }
    });
    ts.emplace_back([&] {                       // command threads: put + board updates
      tch_ctrl_msg m{1, 6 /* kReportBatchSize */, 64};
      while (!stop.load()) {
        if (tch_mq_put(1, 0, &m) == 0) put++;
        tch_train_info_set_field(0, 5 /* target batch size */, 16);
        tch_infer_required_cus_set(0, 32);
      }
    });
    std::this_thread::sleep_for(std::chrono::milliseconds(5 + 3 * (r % 5)));
    tch_TorchColShutdown();                     // stops the stub threads, drops the communicator, the pools
    std::this_thread::sleep_for(std::chrono::milliseconds(20));
    stop.store(true);
    for (auto& t : ts) t.join();
    tch_stub_destroy(stub);
    if (refused.load() >= 1000000) failures++;
    if (r == 0) fprintf(stderr, "round 0: %ld got, %ld put, %ld calls refused after the shutdown\n", got.load(), put.load(), refused.load());
  }
  if (failures) return 1;
  printf("shutdown race: %d rounds clean\n", rounds);
  return 0;
}
