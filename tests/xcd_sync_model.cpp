// Host model of the XCD-local barrier protocol (lightseq_amd/csrc/xcd_sync.h): one thread per
// workgroup, std atomics in place of the L2.  Built and run by tests/test_xcd_sync_model.py.
// Prints one line per scenario, "ok" or what went wrong; exit status 0 only if all are ok.
#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <thread>
#include <vector>

#include "../lightseq_amd/csrc/xcd_sync.h"

struct HostMem {
  static unsigned load(const unsigned* p) { return __atomic_load_n(p, __ATOMIC_ACQUIRE); }
  static void add(unsigned* p, unsigned v) { __atomic_fetch_add(p, v, __ATOMIC_ACQ_REL); }
  static void fetch_or(unsigned* p, unsigned v) { __atomic_fetch_or(p, v, __ATOMIC_ACQ_REL); }
  static void pause() { std::this_thread::yield(); }
};

using namespace lsh;

struct Result {
  int gave_up = 0;       // workgroups whose wait returned false
  int bad_reads = 0;     // neighbour data that was not what the round should show
  int rounds_done = 0;   // rounds completed, summed over the workgroups
};

// `absent`: index of a workgroup (xcd 0) that never starts -- as if it were not resident
static Result run(std::vector<unsigned>& counters, unsigned* error, unsigned base, int wgs_per_xcd,
                  int rounds, int spin_limit, int absent) {
  const int total = kXcdCount * wgs_per_xcd;
  std::vector<unsigned> data(2 * total, 0xffffffffu);
  std::atomic<int> gave_up{0}, bad{0}, done{0};
  std::vector<std::thread> th;
  for (int wg = 0; wg < total; ++wg) {
    if (wg == absent) continue;
    th.emplace_back([&, wg] {
      const int xcd = wg % kXcdCount, slot = wg / kXcdCount;
      const int nb = ((slot + 1) % wgs_per_xcd) * kXcdCount + xcd;
      unsigned* ctr = counters.data() + xcd * kXcdCounterStride;
      for (int r = 0; r < rounds; ++r) {
        __atomic_store_n(&data[(r & 1) * total + wg], (unsigned)(r * 1000 + wg), __ATOMIC_RELEASE);
        if (!xcd_arrive_and_wait<HostMem>(ctr, base + (unsigned)wgs_per_xcd * (unsigned)(r + 1), error,
                                          spin_limit)) {
          ++gave_up;
          return;  // the whole workgroup leaves
        }
        if (__atomic_load_n(&data[(r & 1) * total + nb], __ATOMIC_ACQUIRE) != (unsigned)(r * 1000 + nb))
          ++bad;
        ++done;
      }
    });
  }
  for (auto& t : th) t.join();
  Result res;
  res.gave_up = gave_up;
  res.bad_reads = bad;
  res.rounds_done = done;
  return res;
}

static int fails = 0;
static void report(const char* name, bool ok, const char* detail = "") {
  std::printf("%s: %s %s\n", name, ok ? "ok" : "FAILED", detail);
  if (!ok) ++fails;
}

int main() {
  const int W = 8, R = 50;  // 64 threads
  char buf[200];
  {
    std::vector<unsigned> c(kXcdCount * kXcdCounterStride, 0u);
    unsigned err = 0;
    Result a = run(c, &err, 0u, W, R, 1 << 22, -1);
    bool ok = a.gave_up == 0 && a.bad_reads == 0 && a.rounds_done == kXcdCount * W * R && err == 0;
    for (int x = 0; x < kXcdCount; ++x) ok = ok && c[x * kXcdCounterStride] == (unsigned)(W * R);
    // a second launch goes on from where the counters stand
    Result b = run(c, &err, (unsigned)(W * R), W, R, 1 << 22, -1);
    ok = ok && b.gave_up == 0 && b.bad_reads == 0 && b.rounds_done == kXcdCount * W * R && err == 0;
    std::snprintf(buf, sizeof buf, "(gave up %d/%d, bad reads %d/%d)", a.gave_up, b.gave_up, a.bad_reads,
                  b.bad_reads);
    report("two launches in a row", ok, buf);
  }
  {
    // counters about to wrap around 2^32
    const unsigned base = 0xffffffffu - 37u;
    std::vector<unsigned> c(kXcdCount * kXcdCounterStride, base);
    unsigned err = 0;
    Result a = run(c, &err, base, W, R, 1 << 22, -1);
    report("counter wrap-around", a.gave_up == 0 && a.bad_reads == 0 && err == 0 &&
                                      a.rounds_done == kXcdCount * W * R);
  }
  {
    // one workgroup of XCD 0 never arrives: its XCD gives up at the first round after a bounded
    // number of polls, the other XCDs see the error word at their next wait; nobody hangs
    std::vector<unsigned> c(kXcdCount * kXcdCounterStride, 0u);
    unsigned err = 0;
    const auto t0 = std::chrono::steady_clock::now();
    Result a = run(c, &err, 0u, W, 1 << 20, 2000, 0);
    const double s = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    std::snprintf(buf, sizeof buf, "(gave up %d of %d, error word %u, %.2f s)", a.gave_up,
                  kXcdCount * W - 1, err, s);
    report("a workgroup that never arrives", a.gave_up == kXcdCount * W - 1 && (err & kXcdErrTimeout) &&
                                                 a.bad_reads == 0 && s < 60.0, buf);
  }
  {
    // the error word is already set (a mapping error, an earlier time-out): nobody waits
    std::vector<unsigned> c(kXcdCount * kXcdCounterStride, 0u);
    unsigned err = kXcdErrMapping;
    Result a = run(c, &err, 0u, W, R, 1 << 22, -1);
    bool ok = a.gave_up == kXcdCount * W && a.rounds_done == 0 && err == kXcdErrMapping;
    for (int x = 0; x < kXcdCount; ++x) ok = ok && c[x * kXcdCounterStride] == 0u;  // nobody even arrived
    report("error word set before the launch", ok);
  }
  return fails == 0 ? 0 : 1;
}
