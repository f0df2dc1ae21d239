// Task scheduler over the codecs of hpx.h (see include/hpx_sched.h for what it
// replaces and what it does differently).
//
// One worker thread owns a compute stream and a data stream.  It sleeps on a
// condition variable, takes everything that is queued as one batch (like
// TaskQueue::GetTasksFromQueue, hp_cuda.cpp:122-133) and turns the batch into a
// few multi-tensor codec calls.  Transfers and codec calls are cut into runs of
// growing size (1 MB of messages, then 2, 4 ... 16 MB) so that the link and the
// kernels work at the same time:
//
//   data stream     H2D run 1 ── a_1 ── H2D run 2 ── a_2 ...      D2H run 1 ── d_1 ── D2H run 2 ── d_2 ...
//   compute stream  (waits a_1) decode run 1, (waits a_2) decode run 2 ... encode run 1 ── e_1 ── encode run 2 ── e_2 ...
//                                                                  (D2H run k waits e_k)
//   worker          between runs, and at the end: publishes every run whose event has passed
//
// A transfer run is one launch of the range-copy kernel over all its messages (the GPU reads or
// writes the pinned host buffers itself): with a copy call per message the host spent longer
// issuing 200 copies than the copies and the encode take together.
//
// Group order per algorithm, as in the reference:
//   terngrad  encode(COMP) | decode(DECOMP + root slots) | encode(ROOT)     hp_cuda.cpp:464-477
//   tbq       decode(all)  | encode(COMP + ROOT)                            hp_cuda.cpp:610-611
//   graddrop  decode(all)  | encode(COMP + ROOT)                            hp_cuda.cpp:284-301
//   powersgd  encode1 | encode2 | decode                                    hp_cuda.cpp:729-752
// A root task decodes the `size - 1` gathered slots of C other than its own
// rank's into the gradient (all slots of a tensor in one fused pass, see the
// multi-message decoders) and then re-encodes it.
#include <hip/hip_runtime.h>

#include <atomic>
#include <chrono>
#include <cmath>
#include <condition_variable>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <deque>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "hpx.h"
#include "hpx_sched.h"

#define HPX_API extern "C" __attribute__((visibility("default")))

namespace hpx {
// hpx_runtime.hip: all ranges in one kernel launch (device memory or pinned host memory on either side)
int copy_ranges(int count, uint8_t* const* dst, const uint8_t* const* src, const int64_t* bytes, hipStream_t st);
}

namespace {

enum Alg { kTerngrad, kTbq, kGraddrop, kPowersgd };

struct Params {  // CompAlg, hp_cuda.h:54-66
  Alg alg = kTbq;
  int enable_random = 0;
  int bitwidth = 2;
  float threshold = 0.f;
  double sample_rate = 0.0, drop_ratio = 0.0;
  int rank_r = 0;
  bool has_seed = false;
  uint64_t seed = 0;
  int device = 0, rank = 0, size = 1;
};

struct Task {
  std::string name;
  uint64_t serial = 0;
  hpx_task_t t{};
  mutable bool published = false;
};

struct Sched {
  std::mutex mu;                  // queue, params, running flags
  std::condition_variable cv;     // work arrived / shutdown
  std::deque<Task> queue;
  Params params;
  bool running = false, stop = false, ready = false;
  int init_rc = 0;
  std::thread worker;
  uint64_t next_serial = 1;

  std::mutex fmu;                 // finished queues, done serials
  std::condition_variable fcv;
  std::deque<std::string> finished[3];  // COMP, DECOMP, ROOT (FinishedQueues, hp_cuda.h:128-132)
  std::deque<uint64_t> done;

  std::mutex emu;
  std::string last_error;
  std::atomic<int64_t> errors{0};
};
Sched g;

void fail(const char* fmt, ...) {
  char buf[600];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  {
    std::lock_guard<std::mutex> l(g.emu);
    g.last_error = buf;
  }
  g.errors++;
  fprintf(stderr, "%s\n", buf);  // the reference prints and carries on
}

int queue_of(int task_id) {  // getResults, hp_cuda.cpp:1045-1061
  switch (task_id) {
    case HPX_COMP_TASK: case HPX_POWERSGD_ENCODE1: return 0;
    case HPX_DECOMP_TASK: case HPX_POWERSGD_DECODE: return 1;
    case HPX_ROOT_DECOMP_COMP_TASK: case HPX_POWERSGD_ENCODE2: return 2;
    default: return -1;
  }
}

// ---- worker-side resources ----------------------------------------------------
struct Arena {  // grow-only block, re-used from offset 0 by every batch
  uint8_t* base = nullptr;
  size_t cap = 0, used = 0;
  bool pinned = false;
  bool reserve(size_t bytes) {  // only while nothing in flight uses the block
    used = 0;
    if (bytes <= cap) return true;
    release();
    const size_t want = bytes + bytes / 4 + (1 << 20);
    hipError_t e = pinned ? hipHostMalloc(reinterpret_cast<void**>(&base), want, hipHostMallocDefault)
                          : hipMalloc(reinterpret_cast<void**>(&base), want);
    if (e != hipSuccess) { base = nullptr; cap = 0; fail("scheduler: cannot allocate %zu bytes of %s memory: %s", want, pinned ? "pinned" : "device", hipGetErrorString(e)); return false; }
    cap = want;
    return true;
  }
  uint8_t* take(size_t bytes) {
    uint8_t* p = base + used;
    used += (bytes + 255) & ~size_t(255);
    return p;
  }
  void release() {
    if (base) (void)(pinned ? hipHostFree(base) : hipFree(base));
    base = nullptr; cap = 0; used = 0;
  }
};

struct Worker {
  hipStream_t compute = nullptr, data = nullptr;
  Arena pinned_arena, device_arena;
  std::vector<hipEvent_t> events;
  size_t next_event = 0;
  struct Pending { uint8_t* dst; const uint8_t* src; size_t bytes; };
  hipEvent_t event() {
    if (next_event == events.size()) {
      hipEvent_t e = nullptr;
      if (hipEventCreateWithFlags(&e, hipEventDisableTiming) != hipSuccess) { fail("scheduler: hipEventCreate failed"); return nullptr; }
      events.push_back(e);
    }
    return events[next_event++];
  }
};

// The address under which the GPU can reach host memory `p` (pinned and mapped), or null for
// pageable memory, which has to go through the bounce buffer.
uint8_t* device_alias(const void* p) {
  hipPointerAttribute_t a;
  if (hipPointerGetAttributes(&a, p) != hipSuccess) {
    (void)hipGetLastError();  // pageable memory: not an error for us, do not leave it behind
    return nullptr;
  }
  if (a.type != hipMemoryTypeHost) return nullptr;
  return static_cast<uint8_t*>(a.devicePointer);
}

#define SCHED_HIP(call)                                                                            \
  do {                                                                                             \
    hipError_t e__ = (call);                                                                       \
    if (e__ != hipSuccess) fail("scheduler: %s failed: %s", #call, hipGetErrorString(e__));         \
  } while (0)

void codec(int rc, const char* what) {  // "Call ... failed, ret = ..." (hp_cuda_kernel.cu:63)
  if (rc != HPX_OK) fail("Call %s failed, ret = %d. %s", what, rc, hpx_last_error());
}

// The bytes one message of task t occupies in B and in one slot of C.
int64_t message_bytes(const Params& p, const hpx_task_t& t) {
  if (p.alg == kGraddrop)  // hp_cuda.cpp:230
    return 4 + int64_t(int(2 * std::ceil(double(t.tensor_numel) * (1 - p.drop_ratio)))) * 4;
  return t.B_bytes;        // compressed_size = t.B->numel(), hp_cuda.cpp:411, :558
}

// Message bytes per run of a batch (see run_codec_batch).  The first run is short so that the link starts
// early (1 MB is 4 Mi elements of 2-bit codes: about 10 us of encode, 20 us on the link); each run is twice
// as long as the one before, up to 16 MB, because every run costs its own launches and event hand-overs.
constexpr int64_t kPipeFirstBytes = int64_t(1) << 20;
constexpr int64_t kPipeMaxBytes = int64_t(16) << 20;

struct Group {  // tasks published together once `landed` has passed
  std::vector<const Task*> tasks;
  int queue = 0;
  hipEvent_t landed = nullptr;
  std::vector<Worker::Pending> host_copies;  // pinned bounce buffer -> pageable C
};

// Copies gathered for one phase and issued as one kernel launch on the data stream.
struct CopyList {
  std::vector<uint8_t*> dst;
  std::vector<const uint8_t*> src;
  std::vector<int64_t> bytes;
  void add(uint8_t* d, const uint8_t* s, int64_t b) { dst.push_back(d); src.push_back(s); bytes.push_back(b); }
  void issue(Worker& w) {
    if (dst.empty()) return;
    const int rc = hpx::copy_ranges(int(dst.size()), dst.data(), src.data(), bytes.data(), w.data);
    if (rc != HPX_OK) fail("scheduler: staging copy failed, ret = %d. %s", rc, hpx_last_error());
    dst.clear(); src.clear(); bytes.clear();
  }
};

// Device -> host of one message: straight into C when it is pinned, else into the pinned bounce
// buffer, from where the worker copies it to C once the data stream has passed.
void copy_out(Worker& w, CopyList& cl, Group& grp, const hpx_task_t& t, int64_t bytes) {
  if (bytes <= 0) return;
  if (bytes > t.C_bytes || bytes > t.B_bytes) { fail("scheduler: task buffers too small for a %lld-byte message (B %lld, C %lld)", (long long)bytes, (long long)t.B_bytes, (long long)t.C_bytes); return; }
  if (uint8_t* c = device_alias(t.C)) {
    cl.add(c, t.B, bytes);
  } else {
    uint8_t* bounce = w.pinned_arena.take(size_t(bytes));
    cl.add(bounce, t.B, bytes);
    grp.host_copies.push_back({t.C, bounce, size_t(bytes)});
  }
}

// Host -> device of `bytes` from `src` to device `dst` (through the bounce buffer when src is pageable).
void copy_in(Worker& w, CopyList& cl, uint8_t* dst, const uint8_t* src, int64_t bytes) {
  if (bytes <= 0) return;
  if (const uint8_t* c = device_alias(src)) {
    cl.add(dst, c, bytes);
  } else {
    uint8_t* bounce = w.pinned_arena.take(size_t(bytes));
    std::memcpy(bounce, src, size_t(bytes));
    cl.add(dst, bounce, bytes);
  }
}

void publish(Group& grp) {
  if (grp.tasks.empty()) return;
  if (grp.landed) SCHED_HIP(hipEventSynchronize(grp.landed));
  for (const auto& c : grp.host_copies) std::memcpy(c.dst, c.src, c.bytes);
  {
    std::lock_guard<std::mutex> l(g.fmu);
    for (const Task* t : grp.tasks) {
      g.finished[grp.queue].push_back(t->name);
      g.done.push_back(t->serial);
      t->published = true;
    }
  }
  g.fcv.notify_all();
}

// after `producer` has reached this point, `consumer` may go on
hipEvent_t chain(Worker& w, hipStream_t producer, hipStream_t consumer) {
  hipEvent_t e = w.event();
  if (!e) return nullptr;
  SCHED_HIP(hipEventRecord(e, producer));
  if (consumer) SCHED_HIP(hipStreamWaitEvent(consumer, e, 0));
  return e;
}

// ---- the three quantiser / sparsifier algorithms ---------------------------------
void run_codec_batch(Worker& w, const Params& p, const std::vector<Task>& batch) {
  std::vector<const Task*> comp, decomp, root;
  for (const Task& t : batch) {
    switch (t.t.task_id) {
      case HPX_COMP_TASK: comp.push_back(&t); break;
      case HPX_DECOMP_TASK: decomp.push_back(&t); break;
      case HPX_ROOT_DECOMP_COMP_TASK: root.push_back(&t); break;
      default: fail("error find task_id != 10 20 30 where task_id is %d", t.t.task_id); break;
    }
  }
  // staging memory for the whole batch, sized before anything is in flight
  size_t pinned_need = 0, device_need = 0;
  auto pad = [](int64_t b) { return (size_t(b > 0 ? b : 0) + 255) & ~size_t(255); };
  for (const Task* t : comp) pinned_need += pad(message_bytes(p, t->t));
  for (const Task* t : decomp) pinned_need += pad(message_bytes(p, t->t));
  for (const Task* t : root) {
    const int64_t slots = int64_t(p.size) * message_bytes(p, t->t);
    pinned_need += pad(slots) + pad(message_bytes(p, t->t));
    device_need += pad(slots);
  }
  if (!w.pinned_arena.reserve(pinned_need) || !w.device_arena.reserve(device_need)) return;
  w.next_event = 0;

  // Transfers and codec calls are cut into runs so that the PCIe transfer of one run overlaps the kernels of
  // the next (a 200-tensor TBQ bucket spends 2.5 times as long on the link as in its encode kernel).
  // GradDrop messages are tiny and its encode has a large fixed cost per call, so a GradDrop batch stays
  // one run.
  const bool one_run = p.alg == kGraddrop;
  auto next_run_bytes = [one_run](int64_t b) {
    if (one_run) return INT64_MAX;
    return b == 0 ? kPipeFirstBytes : (b * 2 < kPipeMaxBytes ? b * 2 : kPipeMaxBytes);
  };

  // ---- messages in (data stream): every run's copy is queued now, its decode later ----
  struct DecodeRun {
    std::vector<float*> out;           // decode argument lists (hp_cuda.cpp:420-461)
    std::vector<int32_t> out_size, in_size, add;
    std::vector<const uint8_t*> in;
    std::vector<const Task*> decomp;   // the DECOMP tasks among them: published once the decode has run
    hipEvent_t arrived = nullptr;
    int64_t bytes = 0;
  };
  std::vector<DecodeRun> dec_runs;
  std::vector<const Task*> root_ok;
  {
    CopyList cl_in;
    DecodeRun run;
    int64_t pipe_bytes = next_run_bytes(0);
    auto close_run = [&]() {
      if (run.out.empty()) return;
      cl_in.issue(w);
      run.arrived = chain(w, w.data, nullptr);
      dec_runs.push_back(std::move(run));
      run = DecodeRun();
      pipe_bytes = next_run_bytes(pipe_bytes);
    };
    for (const Task* t : decomp) {
      const int64_t bytes = message_bytes(p, t->t);
      if (bytes > t->t.C_bytes || bytes > t->t.B_bytes) { fail("scheduler: decode task '%s': message of %lld bytes does not fit B (%lld) / C (%lld)", t->name.c_str(), (long long)bytes, (long long)t->t.B_bytes, (long long)t->t.C_bytes); continue; }
      copy_in(w, cl_in, t->t.B, t->t.C, bytes);  // t.B->copy_(t.C->slice(0,0,compressed_size,1), true)
      run.out.push_back(t->t.tensor); run.out_size.push_back(int32_t(t->t.tensor_numel));
      run.in.push_back(t->t.B); run.in_size.push_back(int32_t(bytes)); run.add.push_back(t->t.is_root);
      run.decomp.push_back(t);
      run.bytes += bytes;
      if (run.bytes >= pipe_bytes) close_run();
    }
    for (const Task* t : root) {
      const int64_t bytes = message_bytes(p, t->t);
      const int64_t slots = int64_t(p.size) * bytes;
      if (slots > t->t.C_bytes) { fail("scheduler: root task '%s': C holds %lld bytes, %d slots of %lld needed", t->name.c_str(), (long long)t->t.C_bytes, p.size, (long long)bytes); continue; }
      uint8_t* tmp = w.device_arena.take(size_t(slots));  // temp_cuda_tensors_for_c, hp_cuda.cpp:149-158
      copy_in(w, cl_in, tmp, t->t.C, slots);
      for (int i = 0; i < p.size; i++) {
        if (i == p.rank) continue;
        run.out.push_back(t->t.tensor); run.out_size.push_back(int32_t(t->t.tensor_numel));
        run.in.push_back(tmp + int64_t(i) * bytes); run.in_size.push_back(int32_t(bytes)); run.add.push_back(t->t.is_root);
      }
      root_ok.push_back(t);
      run.bytes += slots;
      if (run.bytes >= pipe_bytes) close_run();  // all slots of a tensor stay in one run: one fused pass over it
    }
    close_run();
  }
  root = root_ok;

  // Groups in the order they were queued; names go out as their events pass.
  std::deque<Group> sent;
  size_t next_pub = 0;
  auto publish_landed = [&](bool wait) {
    for (; next_pub < sent.size(); next_pub++) {
      Group& grp = sent[next_pub];
      if (!wait && grp.landed && hipEventQuery(grp.landed) != hipSuccess) {
        (void)hipGetLastError();  // "not ready" must not be taken for a failed launch later on
        return;
      }
      publish(grp);
    }
  };

  // ---- compute ----
  auto encode = [&](const std::vector<const Task*>& ts, const char* what) {
    if (ts.empty()) return;
    const int n = int(ts.size());
    std::vector<const float*> in(n);
    std::vector<float*> res(n);
    std::vector<uint8_t*> out(n);
    std::vector<int32_t> in_size(n), out_size(n);
    for (int i = 0; i < n; i++) {
      in[i] = ts[i]->t.tensor; in_size[i] = int32_t(ts[i]->t.tensor_numel);
      res[i] = ts[i]->t.residual; out[i] = ts[i]->t.B; out_size[i] = int32_t(ts[i]->t.B_bytes);
    }
    std::vector<uint64_t> seeds(n, p.seed);
    if (p.alg == kTerngrad) {
      std::vector<uint8_t> bw(n, uint8_t(p.bitwidth));
      std::vector<int32_t> rnd(n, p.enable_random);
      codec(hpx_terngrad_encode(n, in.data(), in_size.data(), out.data(), out_size.data(), bw.data(), rnd.data(),
                                p.has_seed ? seeds.data() : nullptr, w.compute), what);
      // Before the messages leave B: a launch that waits at a grid barrier is the one kind that can fail to
      // write its message.  Returns at once when the run took none; otherwise waits for the compute stream
      // and encodes again what an expired barrier left unwritten.
      codec(hpx_terngrad_encode_status(w.compute), "hpx_terngrad_encode_status");
    } else if (p.alg == kTbq) {
      std::vector<float> thr(n, p.threshold);
      codec(hpx_tbq_encode(n, in.data(), in_size.data(), res.data(), out.data(), thr.data(), w.compute), what);
    } else {
      std::vector<double> sr(n, p.sample_rate), dr(n, p.drop_ratio);
      codec(hpx_gd_encode(n, in.data(), in_size.data(), res.data(), out.data(), sr.data(), dr.data(),
                          p.has_seed ? seeds.data() : nullptr, w.compute), what);
    }
  };
  auto decode = [&]() {
    for (DecodeRun& r : dec_runs) {
      if (r.arrived) SCHED_HIP(hipStreamWaitEvent(w.compute, r.arrived, 0));
      const int n = int(r.out.size());
      if (p.alg == kTerngrad) {
        codec(hpx_terngrad_decode(n, r.out.data(), r.out_size.data(), r.in.data(), r.in_size.data(), r.add.data(), w.compute), "hp_cuda_terngradr");
      } else if (p.alg == kTbq) {
        std::vector<float> thr(n, p.threshold);
        codec(hpx_tbq_decode(n, r.out.data(), r.out_size.data(), r.in.data(), thr.data(), r.add.data(), w.compute), "hp_cuda_tbqr");
      } else {
        codec(hpx_gd_decode(n, r.in.data(), r.in_size.data(), r.out.data(), r.out_size.data(), r.add.data(), w.compute), "hp_cuda_gdr");
      }
      if (!r.decomp.empty()) {
        sent.emplace_back();
        Group& grp = sent.back();
        grp.queue = 1;
        grp.tasks = std::move(r.decomp);
        grp.landed = chain(w, w.compute, nullptr);
      }
      publish_landed(false);
    }
  };
  // Encodes `ts` run by run; each run's messages go out behind it:
  // t.C->slice(0,0,compressed_size,1).copy_(*(t.B)).
  auto encode_and_send = [&](const std::vector<const Task*>& ts, const char* what) {
    size_t i = 0;
    int64_t pipe_bytes = 0;
    while (i < ts.size()) {
      std::vector<const Task*> run;
      int64_t bytes = 0;
      pipe_bytes = next_run_bytes(pipe_bytes);
      while (i < ts.size() && bytes < pipe_bytes) {
        bytes += message_bytes(p, ts[i]->t);
        run.push_back(ts[i++]);
      }
      encode(run, what);
      chain(w, w.compute, w.data);
      CopyList cl;
      const size_t first_group = sent.size();
      for (const Task* t : run) {
        const int q = queue_of(t->t.task_id);
        if (sent.size() == first_group || sent.back().queue != q) {
          sent.emplace_back();
          sent.back().queue = q;
        }
        sent.back().tasks.push_back(t);
        copy_out(w, cl, sent.back(), t->t, message_bytes(p, t->t));
      }
      cl.issue(w);
      hipEvent_t landed = chain(w, w.data, nullptr);
      for (size_t k = first_group; k < sent.size(); k++) sent[k].landed = landed;
      publish_landed(false);
    }
  };

  if (p.alg == kTerngrad) {
    encode_and_send(comp, "hp_cuda_terngrad");
    decode();
    encode_and_send(root, "hp_cuda_terngrad");
  } else {
    decode();
    std::vector<const Task*> both = root;  // root first, then comp (hp_cuda.cpp:304-314, :614-622)
    both.insert(both.end(), comp.begin(), comp.end());
    encode_and_send(both, p.alg == kTbq ? "hp_cuda_tbq" : "hp_cuda_gd");
  }
  publish_landed(true);
}

// ---- PowerSGD --------------------------------------------------------------------
void run_powersgd_batch(Worker& w, const Params&, const std::vector<Task>& batch) {
  std::vector<const Task*> e1, e2, dec;
  for (const Task& t : batch) {
    switch (t.t.task_id) {
      case HPX_POWERSGD_ENCODE1: e1.push_back(&t); break;
      case HPX_POWERSGD_ENCODE2: e2.push_back(&t); break;
      case HPX_POWERSGD_DECODE: dec.push_back(&t); break;
      default: fail("error find task_id != 40 50 60 where task_id is %d", t.t.task_id); break;
    }
  }
  w.next_event = 0;
  auto lists = [](const std::vector<const Task*>& ts, std::vector<float*>& G, std::vector<float*>& R, std::vector<float*>& M,
                  std::vector<float*>& P, std::vector<float*>& Q, std::vector<int64_t>& numel, std::vector<int32_t>& n,
                  std::vector<int32_t>& m, std::vector<int32_t>& r) {
    for (const Task* t : ts) {
      G.push_back(t->t.tensor); R.push_back(t->t.residual); M.push_back(t->t.M); P.push_back(t->t.P); Q.push_back(t->t.Q);
      numel.push_back(t->t.tensor_numel); n.push_back(t->t.n); m.push_back(t->t.m); r.push_back(t->t.r);
    }
  };
  Group g1, g2, g3;
  g1.queue = 0; g2.queue = 2; g3.queue = 1;  // hp_cuda.cpp:756-769
  g1.tasks = e1; g2.tasks = e2; g3.tasks = dec;
  {
    std::vector<float*> G, R, M, P, Q; std::vector<int64_t> numel; std::vector<int32_t> n, m, r;
    lists(e1, G, R, M, P, Q, numel, n, m, r);
    if (!e1.empty())
      codec(hpx_powersgd_encode1(int(e1.size()), G.data(), numel.data(), R.data(), Q.data(), M.data(), P.data(), n.data(),
                                 m.data(), r.data(), w.compute), "hp_cuda_powersgd_encode1");
    g1.landed = chain(w, w.compute, nullptr);
  }
  {
    std::vector<float*> G, R, M, P, Q; std::vector<int64_t> numel; std::vector<int32_t> n, m, r;
    lists(e2, G, R, M, P, Q, numel, n, m, r);
    if (!e2.empty())
      codec(hpx_powersgd_encode2(int(e2.size()), P.data(), M.data(), Q.data(), n.data(), m.data(), r.data(), w.compute),
            "hp_cuda_powersgd_encode2");
    g2.landed = chain(w, w.compute, nullptr);
  }
  {
    std::vector<float*> G, R, M, P, Q; std::vector<int64_t> numel; std::vector<int32_t> n, m, r;
    lists(dec, G, R, M, P, Q, numel, n, m, r);
    if (!dec.empty())
      codec(hpx_powersgd_decode(int(dec.size()), P.data(), Q.data(), M.data(), R.data(), G.data(), numel.data(), n.data(),
                                m.data(), r.data(), w.compute), "hp_cuda_powersgd_decode");
    g3.landed = chain(w, w.compute, nullptr);
  }
  publish(g3);  // decode, encode1, encode2: the reference's publication order
  publish(g1);
  publish(g2);
}

void worker_main() {
  Worker w;
  w.pinned_arena.pinned = true;
  int rc = 0;
  Params p0;
  {
    std::lock_guard<std::mutex> l(g.mu);
    p0 = g.params;
  }
  if (hipSetDevice(p0.device) != hipSuccess || hipStreamCreateWithFlags(&w.compute, hipStreamNonBlocking) != hipSuccess ||
      hipStreamCreateWithFlags(&w.data, hipStreamNonBlocking) != hipSuccess) {
    fail("scheduler: cannot set up device %d: %s", p0.device, hipGetErrorString(hipGetLastError()));
    rc = HPX_ERR_HIP;
  }
  {
    std::lock_guard<std::mutex> l(g.mu);
    g.init_rc = rc;
    g.ready = true;
  }
  g.cv.notify_all();
  if (rc != 0) return;

  for (;;) {
    std::vector<Task> batch;
    Params p;
    {
      std::unique_lock<std::mutex> l(g.mu);
      g.cv.wait(l, [] { return g.stop || !g.queue.empty(); });
      if (g.queue.empty() && g.stop) break;
      batch.assign(std::make_move_iterator(g.queue.begin()), std::make_move_iterator(g.queue.end()));
      g.queue.clear();
      p = g.params;
    }
    for (Task& t : batch) t.t.name = t.name.c_str();
    if (p.alg == kPowersgd) run_powersgd_batch(w, p, batch); else run_codec_batch(w, p, batch);
    // A task that failed its checks was skipped (the failure is counted and kept for hpx_sched_error); its
    // name is published all the same, once the batch has drained, so that a caller polling for it does not
    // wait for ever: the reference publishes every task of a batch (hp_cuda.cpp:626-636).
    SCHED_HIP(hipStreamSynchronize(w.compute));
    SCHED_HIP(hipStreamSynchronize(w.data));
    {
      bool any = false;
      std::lock_guard<std::mutex> l(g.fmu);
      for (const Task& t : batch) {
        if (t.published) continue;
        const int q = queue_of(t.t.task_id);
        if (q >= 0) { g.finished[q].push_back(t.name); any = true; }
        g.done.push_back(t.serial);
      }
      if (any) g.fcv.notify_all();
    }
  }
  (void)hipStreamSynchronize(w.compute);
  (void)hipStreamSynchronize(w.data);
  for (hipEvent_t e : w.events) (void)hipEventDestroy(e);
  w.pinned_arena.release();
  w.device_arena.release();
  // The codec workspaces of the two streams go with them, and with the compute stream's its claim on the
  // grid-barrier kernels: the worker of a later init() gets the resident TernGrad encode again.
  (void)hpx_release_stream(w.compute);
  (void)hpx_release_stream(w.data);
  (void)hipStreamDestroy(w.compute);
  (void)hipStreamDestroy(w.data);
}

}  // namespace

HPX_API int hpx_sched_init(const char* alg, const char* const* keys, const double* values, int nparams, int device,
                           int rank, int size) {
  if (!alg || nparams < 0 || (nparams > 0 && (!keys || !values)) || size < 1 || rank < 0 || rank >= size) {
    fail("hpx_sched_init: bad argument");
    return HPX_ERR_ARG;
  }
  auto get = [&](const char* k, double def) {
    for (int i = 0; i < nparams; i++)
      if (keys[i] && std::strcmp(keys[i], k) == 0) return values[i];
    return def;  // the reference's unordered_map::operator[] yields 0 for a missing key
  };
  Params p;
  const std::string a(alg);
  if (a == "terngrad") {
    p.alg = kTerngrad; p.enable_random = int(get("enable_random", 0)); p.bitwidth = int(get("bitwidth", 0));
  } else if (a == "tbq") {
    p.alg = kTbq; p.threshold = float(get("threshold", 0));
  } else if (a == "graddrop") {
    p.alg = kGraddrop; p.drop_ratio = get("drop_ratio", 0); p.sample_rate = get("sample_rate", 0);
  } else if (a == "powersgd") {
    p.alg = kPowersgd; p.rank_r = int(get("matrix_approximation_rank", 0));
  } else {
    fail("only support terngrad, tbq, graddrop and powersgd now");
    return HPX_ERR_ARG;
  }
  for (int i = 0; i < nparams; i++)
    if (keys[i] && std::strcmp(keys[i], "seed") == 0) { p.has_seed = true; p.seed = uint64_t(values[i]); }
  p.device = device; p.rank = rank; p.size = size;

  std::unique_lock<std::mutex> l(g.mu);
  g.params = p;
  if (g.running) return HPX_OK;  // threads already started are kept (hp_cuda.cpp:814)
  if (g.worker.joinable()) g.worker.join();
  g.stop = false; g.ready = false; g.init_rc = 0;
  g.errors = 0;
  g.worker = std::thread(worker_main);
  g.cv.wait(l, [] { return g.ready; });
  if (g.init_rc != 0) {
    l.unlock();
    g.worker.join();
    return g.init_rc;
  }
  g.running = true;
  return HPX_OK;
}

HPX_API int hpx_sched_end(void) {
  {
    std::lock_guard<std::mutex> l(g.mu);
    if (!g.running && !g.worker.joinable()) return HPX_OK;
    g.stop = true;
  }
  g.cv.notify_all();
  if (g.worker.joinable()) g.worker.join();
  std::lock_guard<std::mutex> l(g.mu);
  g.running = false;
  return HPX_OK;
}

HPX_API int hpx_sched_submit(const hpx_task_t* task, uint64_t* serial) {
  if (!task || !task->name) { fail("hpx_sched_submit: null task"); return HPX_ERR_ARG; }
  std::lock_guard<std::mutex> l(g.mu);
  if (!g.running || g.stop) { fail("hpx_sched_submit: the scheduler is not running (call init first)"); return HPX_ERR_ARG; }
  const bool psgd = g.params.alg == kPowersgd;
  const int id = task->task_id;
  if (psgd) {
    if (id != HPX_POWERSGD_ENCODE1 && id != HPX_POWERSGD_ENCODE2 && id != HPX_POWERSGD_DECODE) {
      fail("'submit_task' : powersgd task_id should be 40 (encode1) or 50 (encode2) or 60 (decode), find task_id is %d", id);
      return HPX_ERR_ARG;
    }
    if (!task->tensor || !task->residual || !task->M || !task->P || !task->Q || task->n <= 0 || task->m <= 0 ||
        task->r <= 0 || task->tensor_numel <= 0 || task->tensor_numel > int64_t(task->n) * task->m) {
      fail("hpx_sched_submit: powersgd task '%s' has a null tensor or inconsistent shapes", task->name);
      return HPX_ERR_ARG;
    }
  } else {
    if (task->is_root != 0 && task->is_root != 1) {
      fail("is_root should be 0 (~root) or 1 (root), find is_root is %d", task->is_root);
      return HPX_ERR_ARG;
    }
    if (id != HPX_COMP_TASK && id != HPX_DECOMP_TASK && id != HPX_ROOT_DECOMP_COMP_TASK) {
      fail("'submit_task' : task_id should be 10 (comp) or 20 (decomp) or 30 (root decomp and comp), find task_id is %d", id);
      return HPX_ERR_ARG;
    }
    const bool needs_residual = g.params.alg != kTerngrad && id != HPX_DECOMP_TASK;
    if (!task->tensor || !task->B || !task->C || task->tensor_numel <= 0 || task->tensor_numel > INT32_MAX ||
        task->B_bytes <= 0 || task->B_bytes > INT32_MAX || task->C_bytes <= 0 || (needs_residual && !task->residual)) {
      fail("hpx_sched_submit: task '%s' has a null or empty buffer", task->name);
      return HPX_ERR_ARG;
    }
  }
  Task t;
  t.name = task->name;
  t.t = *task;
  t.serial = g.next_serial++;
  if (serial) *serial = t.serial;
  g.queue.push_back(std::move(t));
  g.cv.notify_one();
  return HPX_OK;
}

HPX_API int64_t hpx_sched_get_results(int task_id, char* buf, int64_t cap) {
  const int q = queue_of(task_id);
  if (q < 0) { fail("not invalid task_id in getResults: %d", task_id); return HPX_ERR_ARG; }
  if (!buf || cap <= 0) return 0;
  std::lock_guard<std::mutex> l(g.fmu);
  int64_t n = 0, off = 0;
  while (!g.finished[q].empty()) {
    const std::string& s = g.finished[q].front();
    if (off + int64_t(s.size()) + 1 > cap) break;
    std::memcpy(buf + off, s.c_str(), s.size() + 1);
    off += int64_t(s.size()) + 1;
    g.finished[q].pop_front();
    n++;
  }
  return n;
}

HPX_API int hpx_sched_wait(int task_id, int timeout_ms) {
  const int q = queue_of(task_id);
  if (q < 0) { fail("not invalid task_id in getResults: %d", task_id); return HPX_ERR_ARG; }
  std::unique_lock<std::mutex> l(g.fmu);
  const bool ok = g.fcv.wait_for(l, std::chrono::milliseconds(timeout_ms < 0 ? 0 : timeout_ms), [q] { return !g.finished[q].empty(); });
  return ok ? 1 : 0;
}

HPX_API int64_t hpx_sched_take_done(uint64_t* serials, int64_t cap) {
  if (!serials || cap <= 0) return 0;
  std::lock_guard<std::mutex> l(g.fmu);
  int64_t n = 0;
  while (n < cap && !g.done.empty()) {
    serials[n++] = g.done.front();
    g.done.pop_front();
  }
  return n;
}

HPX_API int64_t hpx_sched_error_count(void) { return g.errors.load(); }

HPX_API const char* hpx_sched_error(void) {
  static thread_local std::string copy;
  std::lock_guard<std::mutex> l(g.emu);
  copy = g.last_error;
  return copy.c_str();
}
