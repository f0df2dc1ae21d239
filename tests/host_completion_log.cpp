// Host-side unit test of csrc/hpx_completion_log.h (compiled and run by tests/test_completion_log.py).
// Marks are integers; `done` holds the marks that have been reached, `flag` stands for the expiry flag.
#include <cstdio>
#include <cstdlib>
#include <set>
#include <vector>

#include "hpx_completion_log.h"

#define CHECK(c)                                                   \
  do {                                                             \
    if (!(c)) {                                                    \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #c);   \
      std::exit(1);                                                \
    }                                                              \
  } while (0)

int main() {
  hpx::CompletionLog<int, int> log;
  std::set<int> done;
  std::vector<int> pool;
  bool flag = false;
  int health_checks = 0;
  auto reached = [&](int m) { return done.count(m) != 0; };
  auto healthy = [&] { health_checks++; return !flag; };
  auto recycle = [&](int m) { pool.push_back(m); };
  std::vector<int> order;

  // a mark with nothing to cover is handed back at once
  log.mark(100, recycle);
  CHECK(pool.size() == 1 && pool[0] == 100 && log.pending_marks() == 0);
  pool.clear();

  // three calls: records 1,2 | 3 | 4,5,6
  log.add(1); log.add(2); log.mark(10, recycle);
  log.add(3); log.mark(11, recycle);
  log.add(4); log.add(5); log.add(6); log.mark(12, recycle);
  CHECK(log.size() == 6 && log.pending_marks() == 3);

  // nothing reached: nothing dropped, and the health of the stream is not even asked
  CHECK(log.prune(reached, healthy, recycle) == 0 && log.size() == 6 && health_checks == 0);

  // a later mark reached while an earlier one is not (cannot happen on one stream, but the log must not
  // skip): stops at the first unreached mark
  done.insert(11);
  CHECK(log.prune(reached, healthy, recycle) == 0 && log.size() == 6);

  // first two calls finished well: their records go, the third call's stay
  done.insert(10);
  CHECK(log.prune(reached, healthy, recycle) == 3);
  CHECK(log.size() == 3 && log.records()[0] == 4 && log.records()[2] == 6 && log.pending_marks() == 1);
  CHECK(pool.size() == 2 && pool[0] == 10 && pool[1] == 11);
  pool.clear();

  // the third call's mark is reached but the flag is up: nothing may be dropped - these are the records to repair
  done.insert(12); flag = true;
  CHECK(log.prune(reached, healthy, recycle) == 0 && log.size() == 3 && log.pending_marks() == 1);
  // a fourth call queued behind the failure is part of the repair too
  log.add(7); log.mark(13, recycle);
  CHECK(log.size() == 4 && log.pending_marks() == 2);
  // the repair takes the records over
  order.assign(log.records().begin(), log.records().end());
  CHECK(order == std::vector<int>({4, 5, 6, 7}));
  log.clear(recycle);
  CHECK(log.empty() && log.pending_marks() == 0 && pool.size() == 2);
  pool.clear();

  // positions stay right after a clear: a new call, marked twice (the second mark covers nothing new)
  flag = false;
  log.add(8); log.mark(14, recycle); log.mark(15, recycle);
  CHECK(log.pending_marks() == 1 && pool.size() == 1 && pool[0] == 15);
  done.insert(14);
  CHECK(log.prune(reached, healthy, recycle) == 1 && log.empty() && log.pending_marks() == 0);

  // records added without a mark (event creation failed) are covered by the next call's mark
  log.add(9);
  log.add(10); log.mark(16, recycle);
  done.insert(16);
  CHECK(log.prune(reached, healthy, recycle) == 2 && log.empty());

  std::printf("OK\n");
  return 0;
}
