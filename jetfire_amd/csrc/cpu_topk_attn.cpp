// Host side of the hand-off: exact softmax attention over the top-k slots from the bf16 shadow
// (restates the contract of jetfire_vllm/csrc/cpu_topk_attn.cpp:602-690,854-956; AVX2+FMA and AVX-512-BF16 rows
// selected at run time, :316-479), a persistent worker pool (spin, then sleep on a condition variable), and the
// pinned hand-off: a small kernel stores q and the winners' slots into pinned host memory and raises a flag
// there, a host thread that polls the flag runs the correction, and the result comes back either after a
// host-blocking wait or through a kernel that waits on the device (graph-capturable).  No hipMemcpyAsync and
// no stream callbacks anywhere.
#include <hip/hip_runtime.h>

#include <atomic>
#include <chrono>
#include <cmath>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

#include <pthread.h>
#include <sched.h>

#if defined(__x86_64__)
#include <immintrin.h>
#endif

#include "common.h"

namespace jf {

// ------------------------------------------------------------------ error string
static thread_local char g_err[512] = "";
void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

// ------------------------------------------------------------------ worker pool
// One job at a time (like the reference's single-flight pool, jetfire_pool.h:270-305).  A job is a range
// [0, n) of rows handed out in small chunks from a shared counter; the submitting thread either blocks in
// run() or returns immediately from start() and later calls join().
//
// A job is finished when all of its ROWS are, not when every worker has checked in: a worker that has lost
// its core (more busy threads than cores) or is still asleep takes no rows and holds nobody up; it only
// matters while it sits on a claimed row.  The counter carries the job's epoch in its upper half, so a worker
// that wakes up late with an old job in hand cannot claim rows of a newer one.
struct CpuJob {
  const uint16_t *q, *k_shadow, *v_shadow;
  const int64_t *head_map, *ts_buf;  // head_map may be null (kv-head = query head / (H_q / H_kv)); ts_buf or ts32
  uint16_t* o_new;
  int B, H_q, K, H_kv;
  int64_t num_slots;
  float scale;
  const int32_t* ts32 = nullptr;     // 32-bit slots instead of ts_buf
};
// One row (sequence, query head) of the job into `out` (128 bf16 values of the caller's choosing).
static void compute_row(const CpuJob& j, int64_t r, uint16_t* out);

#ifdef JF_DEBUG_HOOKS
// Test aid: the worker that claims this row of the next job sleeps first (one shot); see jf_debug_pool_stall.
static std::atomic<int64_t> g_stall_row{-1};
static std::atomic<int> g_stall_us{0};
#endif
// Whether a synchronous call returns only after every worker has left its rows (default; the caller may free its
// tensors right after the call).  Jobs over buffers that outlive them (the hand-off contexts) never wait.
static std::atomic<int> g_wait_stragglers{1};

// Backup copies of straggling rows: a worker that finds no unclaimed row left waits a grace period
// (JETFIRE_POOL_BACKUP_US, default 30; negative: never) and then recomputes rows that are claimed but not yet
// committed.  Every row is computed into a buffer of the worker and committed by the first one to finish
// (compare-and-swap on the row's epoch tag, then the copy to o_new, then the count), so a worker that has lost its
// core in the middle of a row (a scheduler time slice is milliseconds, a row ten microseconds) delays the job by
// the grace period instead of by its absence, and whatever it does when it comes back is discarded.
class Pool {
 public:
  static Pool& instance() {
    static Pool p;
    return p;
  }
  int threads() {
    std::lock_guard<std::mutex> g(cfg_mu_);
    return resolve_threads();
  }
  void set_threads(int n) {
    std::lock_guard<std::mutex> g(cfg_mu_);
    override_ = n;
  }
  // Start the rows [0, n) of `job` asynchronously.  Returns false if a job is already in flight.
  bool start(const CpuJob& job, int64_t n) {
    ensure_workers();
    std::unique_lock<std::mutex> lk(mu_);
    if (busy_) return false;
    if (n > tag_cap_) {  // grow the tags only while no worker can be looking at them
      lk.unlock();
      quiesce();
      lk.lock();
      if (busy_) return false;
      int64_t cap = tag_cap_ > 0 ? tag_cap_ : 1024;
      while (cap < n) cap *= 2;
      tags_.reset(new std::atomic<uint64_t>[(size_t)cap]);
      const uint64_t now = epoch_.load(std::memory_order_relaxed);
      for (int64_t i = 0; i < cap; ++i) tags_[i].store(now, std::memory_order_relaxed);
      tag_cap_ = cap;
    }
    busy_ = true;
    const uint64_t e = epoch_.load(std::memory_order_relaxed) + 1;
    Job& jb = jobs_[e & 1];
    jb.cj = job;
    jb.n = n;
    const int w = (int)workers_.size();
    jb.chunk = std::max<int64_t>(1, n / ((int64_t)w * 8));
    n_ = n;
    done_rows_.store(0, std::memory_order_relaxed);
    next_.store(e << 32, std::memory_order_relaxed);
    epoch_.store(e, std::memory_order_release);
    lk.unlock();
    cv_work_.notify_all();
    return true;
  }
  // Wait for the job started with start().  timeout_s <= 0: wait forever.  On a timeout the job is withdrawn
  // (no further rows can be claimed or committed, rows in flight are waited for) and the pool is free again.
  bool join(double timeout_s, bool wait_stragglers) {
    const auto t0 = std::chrono::steady_clock::now();
    for (int spin = 0; spin < 20000; ++spin) {
      if (done_rows_.load(std::memory_order_acquire) >= n_) break;
#if defined(__x86_64__)
      _mm_pause();
#endif
    }
    std::unique_lock<std::mutex> lk(mu_);
    while (done_rows_.load(std::memory_order_acquire) < n_) {
      if (timeout_s > 0) {
        const double el = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
        if (el > timeout_s) {
          // withdraw: a counter value of a later epoch stops every claim and every commit; then let the rows in
          // flight drain
          const uint64_t e = epoch_.load(std::memory_order_relaxed) + 1;
          next_.store(e << 32, std::memory_order_release);
          jobs_[e & 1].n = 0;
          epoch_.store(e, std::memory_order_release);
          lk.unlock();
          quiesce();
          lk.lock();
          busy_ = false;
          return false;
        }
      }
      cv_done_.wait_for(lk, std::chrono::milliseconds(1));
    }
    lk.unlock();
    if (wait_stragglers) quiesce();
    lk.lock();
    busy_ = false;
    return true;
  }
  // `persistent`: the job's buffers outlive it (a straggler may still read them after the call has returned).
  bool run(const CpuJob& job, int64_t n, bool persistent) {
    if (n <= 0) return true;
    while (!start(job, n)) std::this_thread::yield();
    return join(0, !persistent && g_wait_stragglers.load(std::memory_order_relaxed) != 0);
  }
  // Starts (or resizes) the workers without running anything.
  void warm() { ensure_workers(); }
  // Sleeping workers go back to spinning for the next job (for JETFIRE_POOL_SPIN_US): called when a decode step
  // is known to be on its way, so that its first layer does not pay the wake-up of the whole pool.
  void wake() {
    ensure_workers();
    wake_gen_.fetch_add(1, std::memory_order_acq_rel);
    { std::lock_guard<std::mutex> g(mu_); }
    cv_work_.notify_all();
  }
  int64_t jobs_done() const { return jobs_done_.load(std::memory_order_relaxed); }
  int worker_count() {
    std::lock_guard<std::mutex> g(mu_);
    return (int)workers_.size();
  }
  // Returns when no worker is inside a job (between its first claim and its last look at the rows).
  void quiesce() {
    while (active_.load(std::memory_order_acquire) != 0) std::this_thread::sleep_for(std::chrono::microseconds(20));
  }

 private:
  struct Job {
    CpuJob cj{};
    int64_t n = 0, chunk = 1;
  };
  Pool() = default;
  ~Pool() {
    {
      std::lock_guard<std::mutex> g(mu_);
      stop_ = true;
    }
    cv_work_.notify_all();
    for (auto& t : workers_) t.join();
  }
  int resolve_threads() {
    if (override_ > 0) return override_;
    if (const char* e = std::getenv("JETFIRE_CPU_ATTN_THREADS")) {
      const int n = std::atoi(e);
      if (n > 0) return n;
    }
    // default: all cores but two (the thread that launches the GPU work and the hand-off's dispatcher spin
    // while a layer is in flight; workers that share a core with them stretch every job)
    unsigned hc = std::thread::hardware_concurrency();
    if (hc == 0) hc = 1;
    if (hc > 4) hc -= 2;
    return (int)(hc < 64 ? hc : 64);
  }
  void ensure_workers() {
    // one resize at a time: a second submitter must not join the same thread objects
    std::lock_guard<std::mutex> rg(resize_mu_);
    int want;
    {
      std::lock_guard<std::mutex> g(cfg_mu_);
      want = resolve_threads();
    }
    std::unique_lock<std::mutex> lk(mu_);
    if ((int)workers_.size() == want || busy_) return;
    // resize: stop the old set, start a new one
    if (!workers_.empty()) {
      stop_ = true;
      lk.unlock();
      cv_work_.notify_all();
      for (auto& t : workers_) t.join();
      lk.lock();
      workers_.clear();
      stop_ = false;
    }
    const uint64_t e0 = epoch_.load(std::memory_order_acquire);
    for (int i = 0; i < want; ++i) workers_.emplace_back([this, e0, i] { worker(e0, i); });
  }
  static double spin_seconds() {
    // how long an idle worker spins for the next job before it sleeps: the gap between two layers of a decode
    // step (and between two steps of a running decode loop) is shorter than a futex wake-up of the whole pool,
    // which costs the first job after it several hundred microseconds (JETFIRE_POOL_SPIN_US, default 2000)
    static const double s = [] {
      const char* e = std::getenv("JETFIRE_POOL_SPIN_US");
      const double us = e ? std::atof(e) : 2000.0;
      return (us >= 0.0 && us <= 1e6 ? us : 2000.0) * 1e-6;
    }();
    return s;
  }
  static double backup_seconds() {
    static const double s = [] {
      const char* e = std::getenv("JETFIRE_POOL_BACKUP_US");
      const double us = e ? std::atof(e) : 30.0;
      return (us <= 1e6 ? us : 30.0) * 1e-6;  // negative: no backup copies
    }();
    return s;
  }
  // Computes row r of the job of epoch e and commits it unless somebody else has.  The caller (worker) holds
  // `active_` raised from before it claims a row or scans the tags until it has left the job, so quiesce() also
  // waits for a worker that sits between a claim and its row.
  void do_row(const Job& jb, uint64_t e, int64_t r, bool claimed) {
    uint16_t local[D];
#ifdef JF_DEBUG_HOOKS
    if (claimed) {
      int64_t sr = g_stall_row.load(std::memory_order_relaxed);
      if (sr == r && g_stall_row.compare_exchange_strong(sr, -1))
        std::this_thread::sleep_for(std::chrono::microseconds(g_stall_us.load(std::memory_order_relaxed)));
    }
#else
    (void)claimed;
#endif
    compute_row(jb.cj, r, local);
    // the row's tag holds the epoch of the last job that committed it: a tag below e means that the job of epoch e
    // is still current and the row is open; the worker that moves it to e owns the row's output
    uint64_t old = tags_[r].load(std::memory_order_acquire);
    // (a job that has been withdrawn, or followed by a newer one, commits nothing: its output buffer and the row
    // count now belong to somebody else)
    while (old < e && epoch_.load(std::memory_order_acquire) == e) {
      if (tags_[r].compare_exchange_weak(old, e, std::memory_order_acq_rel, std::memory_order_acquire)) {
        memcpy(jb.cj.o_new + r * D, local, sizeof(local));
        if (done_rows_.fetch_add(1, std::memory_order_acq_rel) + 1 >= jb.n) {
          jobs_done_.fetch_add(1, std::memory_order_relaxed);
          std::lock_guard<std::mutex> g(mu_);
          cv_done_.notify_all();
        }
        break;
      }
    }
  }
  // JETFIRE_CPU_ATTN_PIN=1 (jetfire_vllm/csrc/cpu_topk_attn.cpp:895-905, jetfire_pool.h:141-149): worker i stays on
  // one core.  The reference binds it to core i; here it is the i-th core the process may run on (the same core
  // when every core is allowed, and still a valid one inside a restricted cpu set).  More workers than allowed
  // cores: the surplus stays unpinned.
  static bool pin_workers() {
    static const bool on = [] {
      const char* e = std::getenv("JETFIRE_CPU_ATTN_PIN");
      return e != nullptr && std::atoi(e) == 1;
    }();
    return on;
  }
  static void pin_to_allowed_core(int index) {
    cpu_set_t allowed;
    CPU_ZERO(&allowed);
    if (sched_getaffinity(0, sizeof(allowed), &allowed) != 0) return;
    int seen = 0;
    for (int c = 0; c < CPU_SETSIZE; ++c) {
      if (!CPU_ISSET(c, &allowed)) continue;
      if (seen++ == index) {
        cpu_set_t one;
        CPU_ZERO(&one);
        CPU_SET(c, &one);
        (void)pthread_setaffinity_np(pthread_self(), sizeof(one), &one);
        return;
      }
    }
  }
  void worker(uint64_t seen, int index) {
    if (pin_workers()) pin_to_allowed_core(index);
    for (;;) {
      bool got = false;
      const auto t0 = std::chrono::steady_clock::now();
      for (uint32_t spin = 0;; ++spin) {
        if (epoch_.load(std::memory_order_acquire) != seen || stop_flag()) { got = true; break; }
#if defined(__x86_64__)
        _mm_pause();
#endif
        if ((spin & 0x3ff) == 0x3ff &&
            std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() > spin_seconds()) break;
      }
      if (!got) {
        std::unique_lock<std::mutex> lk(mu_);
        const uint64_t wg = wake_gen_.load(std::memory_order_acquire);
        cv_work_.wait(lk, [&] {
          return stop_ || epoch_.load(std::memory_order_acquire) != seen || wake_gen_.load(std::memory_order_acquire) != wg;
        });
      }
      if (stop_flag()) return;
      const uint64_t e = epoch_.load(std::memory_order_acquire);
      if (e == seen) continue;  // woken ahead of a job (wake()): back to spinning for it
      seen = e;
      // from here until this worker has left the job it counts as active: quiesce() waits for it
      struct ActiveScope {
        std::atomic<int>& a;
        explicit ActiveScope(std::atomic<int>& x) : a(x) { a.fetch_add(1, std::memory_order_acq_rel); }
        ~ActiveScope() { a.fetch_sub(1, std::memory_order_acq_rel); }
      } in_job(active_);
      // A private copy of the job: its slot is rewritten by the job after next at the earliest, so the copy is
      // whole if the epoch has moved by at most one since it was read.
      const Job jb = jobs_[e & 1];
      if (epoch_.load(std::memory_order_acquire) - e > 1) continue;
      uint64_t v = next_.load(std::memory_order_acquire);
      for (;;) {
        if ((v >> 32) != (e & 0xffffffffu)) break;  // a newer job: this one is finished or withdrawn
        const int64_t b = (int64_t)(v & 0xffffffffu);
        if (b >= jb.n) break;
        if (!next_.compare_exchange_weak(v, v + (uint64_t)jb.chunk, std::memory_order_acq_rel, std::memory_order_acquire)) continue;
        const int64_t end = std::min<int64_t>(jb.n, b + jb.chunk);
        for (int64_t r = b; r < end; ++r) do_row(jb, e, r, true);
        v = next_.load(std::memory_order_acquire);
      }
      // no unclaimed row left: after the grace period, back up rows that are still open
      const double grace = backup_seconds();
      if (grace < 0.0 || jb.n <= 0) continue;
      const auto t_idle = std::chrono::steady_clock::now();
      bool waited = false;
      while (done_rows_.load(std::memory_order_acquire) < jb.n && epoch_.load(std::memory_order_acquire) == e &&
             !stop_flag()) {
        if (!waited) {
          if (std::chrono::duration<double>(std::chrono::steady_clock::now() - t_idle).count() < grace) {
#if defined(__x86_64__)
            _mm_pause();
#endif
            continue;
          }
          waited = true;
        }
        int64_t open = -1;
        const int64_t first = ((int64_t)index * 7919) % jb.n;  // idle workers start their search at different rows
        for (int64_t k = 0; k < jb.n; ++k) {
          const int64_t r = first + k < jb.n ? first + k : first + k - jb.n;
          if (tags_[r].load(std::memory_order_acquire) < e) { open = r; break; }
        }
        if (open < 0) break;
        do_row(jb, e, open, false);
      }
    }
  }
  bool stop_flag() {
    return __atomic_load_n(&stop_, __ATOMIC_ACQUIRE);
  }

  std::mutex mu_, cfg_mu_, resize_mu_;
  std::atomic<int> active_{0};          // workers inside a job (from before their first claim until they leave it)
  std::atomic<uint64_t> wake_gen_{0};   // bumped by wake()
  std::atomic<int64_t> jobs_done_{0};   // jobs whose last row has been committed
  std::condition_variable cv_work_, cv_done_;
  std::vector<std::thread> workers_;
  Job jobs_[2];
  int64_t n_ = 0;
  std::atomic<uint64_t> next_{0};       // (epoch << 32) | first unclaimed row
  std::atomic<int64_t> done_rows_{0};   // committed rows of the current job
  std::unique_ptr<std::atomic<uint64_t>[]> tags_;  // per row: epoch of the last job that committed it
  int64_t tag_cap_ = 0;
  int override_ = 0;
  bool busy_ = false, stop_ = false;
  std::atomic<uint64_t> epoch_{0};
};

// ------------------------------------------------------------------ row kernel
static inline float bf(uint16_t b) { return bf16_to_f32(b); }

// One (sequence, query head) row.  fp32 accumulation in ascending channel / slot order.
// SlotT: int64 (the operator's ts_buf) or int32 (the hand-off's own pinned buffer).  head_map == nullptr: every
// slot of the row reads kv-head `fixed_h`.
template <typename SlotT>
static void topk_attn_row(const uint16_t* q, const uint16_t* k_shadow, const uint16_t* v_shadow, int64_t num_slots,
                          const int64_t* head_map, int64_t fixed_h, const SlotT* slots, int K, int H_kv, float scale,
                          uint16_t* out, float* score_buf) {
  float qf[D];
  for (int i = 0; i < D; ++i) qf[i] = bf(q[i]);
  float mx = -INFINITY;
  bool any = false;
  for (int k = 0; k < K; ++k) {
    const int64_t s = slots[k], h = head_map ? head_map[k] : fixed_h;
    if (s < 0 || s >= num_slots || h < 0 || h >= H_kv) {
      score_buf[k] = -INFINITY;
      continue;
    }
    any = true;
    const uint16_t* kr = k_shadow + ((size_t)h * num_slots + s) * D;
    float lanes[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int i = 0; i < D; i += 8)
      for (int j = 0; j < 8; ++j) lanes[j] += qf[i + j] * bf(kr[i + j]);
    const float dot = ((lanes[0] + lanes[4]) + (lanes[2] + lanes[6])) + ((lanes[1] + lanes[5]) + (lanes[3] + lanes[7]));
    const float sc = dot * scale;
    score_buf[k] = sc;
    if (sc > mx) mx = sc;
  }
  if (!any) {
    memset(out, 0, D * sizeof(uint16_t));
    return;
  }
  float den = 0.0f;
  for (int k = 0; k < K; ++k) {
    score_buf[k] = std::exp(score_buf[k] - mx);
    den += score_buf[k];
  }
  if (!(den > 0.0f) || !std::isfinite(den)) {
    memset(out, 0, D * sizeof(uint16_t));
    return;
  }
  const float inv = 1.0f / den;
  float o[D];
  for (int i = 0; i < D; ++i) o[i] = 0.0f;
  for (int k = 0; k < K; ++k) {
    const int64_t s = slots[k], h = head_map ? head_map[k] : fixed_h;
    if (s < 0 || s >= num_slots || h < 0 || h >= H_kv) continue;
    const uint16_t* vr = v_shadow + ((size_t)h * num_slots + s) * D;
    const float w = score_buf[k] * inv;
    for (int i = 0; i < D; ++i) o[i] += w * bf(vr[i]);
  }
  for (int i = 0; i < D; ++i) out[i] = f32_to_bf16(o[i]);
}

#if defined(__x86_64__)
// AVX2 + FMA form of the same row (selected at run time when the host supports it): eight fp32 lanes per
// step, the rows of the next slots requested ahead of their use (the gather is DRAM-latency bound).
__attribute__((target("avx2,fma"))) static inline __m256 bf16x8_to_f32(const uint16_t* p) {
  return _mm256_castsi256_ps(_mm256_slli_epi32(_mm256_cvtepu16_epi32(_mm_loadu_si128(reinterpret_cast<const __m128i*>(p))), 16));
}
template <typename SlotT>
__attribute__((target("avx2,fma"))) static void topk_attn_row_avx2(const uint16_t* q, const uint16_t* k_shadow,
                                                                   const uint16_t* v_shadow, int64_t num_slots,
                                                                   const int64_t* head_map, int64_t fixed_h,
                                                                   const SlotT* slots, int K, int H_kv, float scale,
                                                                   uint16_t* out, float* score_buf) {
  // rows requested ahead of their use: measured on a 16-core EPYC share, 8 rows leave the gather at 3/4 of the
  // rate that 24 to 64 rows reach (110 against 148 us for 32768 row pairs on 14 threads)
  constexpr int AHEAD = 32;
  __m256 qv[D / 8];
  for (int i = 0; i < D / 8; ++i) qv[i] = bf16x8_to_f32(q + 8 * i);
  auto row_of = [&](const uint16_t* base, int k) -> const uint16_t* {
    const int64_t s = slots[k], h = head_map ? head_map[k] : fixed_h;
    if (s < 0 || s >= num_slots || h < 0 || h >= H_kv) return nullptr;
    return base + ((size_t)h * num_slots + s) * D;
  };
  auto prefetch_row = [](const uint16_t* r) {
    if (r) {
      for (int b = 0; b < D * 2; b += 64) _mm_prefetch(reinterpret_cast<const char*>(r) + b, _MM_HINT_T0);
    }
  };
  for (int k = 0; k < K && k < AHEAD; ++k) prefetch_row(row_of(k_shadow, k));
  float mx = -INFINITY;
  bool any = false;
  for (int k = 0; k < K; ++k) {
    if (k + AHEAD < K) prefetch_row(row_of(k_shadow, k + AHEAD));
    const uint16_t* kr = row_of(k_shadow, k);
    if (!kr) {
      score_buf[k] = -INFINITY;
      continue;
    }
    any = true;
    __m256 a0 = _mm256_setzero_ps(), a1 = _mm256_setzero_ps();
    for (int i = 0; i < D / 8; i += 2) {
      a0 = _mm256_fmadd_ps(qv[i], bf16x8_to_f32(kr + 8 * i), a0);
      a1 = _mm256_fmadd_ps(qv[i + 1], bf16x8_to_f32(kr + 8 * i + 8), a1);
    }
    const __m256 a = _mm256_add_ps(a0, a1);
    __m128 r = _mm_add_ps(_mm256_castps256_ps128(a), _mm256_extractf128_ps(a, 1));
    r = _mm_add_ps(r, _mm_movehl_ps(r, r));
    r = _mm_add_ss(r, _mm_shuffle_ps(r, r, 1));
    const float sc = _mm_cvtss_f32(r) * scale;
    score_buf[k] = sc;
    if (sc > mx) mx = sc;
  }
  if (!any) {
    memset(out, 0, D * sizeof(uint16_t));
    return;
  }
  for (int k = 0; k < K && k < AHEAD; ++k) prefetch_row(row_of(v_shadow, k));
  float den = 0.0f;
  for (int k = 0; k < K; ++k) {
    score_buf[k] = std::exp(score_buf[k] - mx);
    den += score_buf[k];
  }
  if (!(den > 0.0f) || !std::isfinite(den)) {
    memset(out, 0, D * sizeof(uint16_t));
    return;
  }
  const float inv = 1.0f / den;
  __m256 o[D / 8];
  for (int i = 0; i < D / 8; ++i) o[i] = _mm256_setzero_ps();
  for (int k = 0; k < K; ++k) {
    if (k + AHEAD < K) prefetch_row(row_of(v_shadow, k + AHEAD));
    const uint16_t* vr = row_of(v_shadow, k);
    if (!vr) continue;
    const __m256 w = _mm256_set1_ps(score_buf[k] * inv);
    for (int i = 0; i < D / 8; ++i) o[i] = _mm256_fmadd_ps(w, bf16x8_to_f32(vr + 8 * i), o[i]);
  }
  float of[D];
  for (int i = 0; i < D / 8; ++i) _mm256_storeu_ps(of + 8 * i, o[i]);
  for (int i = 0; i < D; ++i) out[i] = f32_to_bf16(of[i]);
}
static bool host_has_avx2_fma() {
  static const bool ok = __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma");
  return ok;
}

// AVX-512-BF16 form (jetfire_vllm/csrc/cpu_topk_attn.cpp:316-479): the K dot products run on vdpbf16ps, which
// multiplies the bf16 operands directly (four instructions per 128-channel row, pairs of products summed in
// fp32); V is accumulated in eight 16-lane fp32 registers and converted with vcvtneps2bf16.  Rows are
// requested 32 slots ahead like the AVX2 form (the gather is DRAM-latency bound on this host; the reference's
// packing of the V rows into a contiguous buffer trades that latency for a second pass over 256 bytes per slot).
#define JF_AVX512BF16_TARGET __attribute__((target("avx512f,avx512bw,avx512vl,avx512dq,avx512bf16")))
template <typename SlotT>
JF_AVX512BF16_TARGET static void topk_attn_row_avx512bf16(const uint16_t* q, const uint16_t* k_shadow,
                                                          const uint16_t* v_shadow, int64_t num_slots,
                                                          const int64_t* head_map, int64_t fixed_h,
                                                          const SlotT* slots, int K, int H_kv, float scale,
                                                          uint16_t* out, float* score_buf) {
  constexpr int AHEAD = 32;
  __m512bh qv[4];
  for (int i = 0; i < 4; ++i) qv[i] = (__m512bh)_mm512_loadu_si512(reinterpret_cast<const void*>(q + 32 * i));
  auto row_of = [&](const uint16_t* base, int k) -> const uint16_t* {
    const int64_t s = slots[k], h = head_map ? head_map[k] : fixed_h;
    if (s < 0 || s >= num_slots || h < 0 || h >= H_kv) return nullptr;
    return base + ((size_t)h * num_slots + s) * D;
  };
  auto prefetch_row = [](const uint16_t* r) {
    if (r) {
      for (int b = 0; b < D * 2; b += 64) _mm_prefetch(reinterpret_cast<const char*>(r) + b, _MM_HINT_T0);
    }
  };
  for (int k = 0; k < K && k < AHEAD; ++k) prefetch_row(row_of(k_shadow, k));
  float mx = -INFINITY;
  bool any = false;
  for (int k = 0; k < K; ++k) {
    if (k + AHEAD < K) prefetch_row(row_of(k_shadow, k + AHEAD));
    const uint16_t* kr = row_of(k_shadow, k);
    if (!kr) {
      score_buf[k] = -INFINITY;
      continue;
    }
    any = true;
    __m512 acc = _mm512_setzero_ps();
    for (int i = 0; i < 4; ++i)
      acc = _mm512_dpbf16_ps(acc, qv[i], (__m512bh)_mm512_loadu_si512(reinterpret_cast<const void*>(kr + 32 * i)));
    const float sc = _mm512_reduce_add_ps(acc) * scale;
    score_buf[k] = sc;
    if (sc > mx) mx = sc;
  }
  if (!any) {
    memset(out, 0, D * sizeof(uint16_t));
    return;
  }
  for (int k = 0; k < K && k < AHEAD; ++k) prefetch_row(row_of(v_shadow, k));
  float den = 0.0f;
  for (int k = 0; k < K; ++k) {
    score_buf[k] = std::exp(score_buf[k] - mx);
    den += score_buf[k];
  }
  if (!(den > 0.0f) || !std::isfinite(den)) {
    memset(out, 0, D * sizeof(uint16_t));
    return;
  }
  const float inv = 1.0f / den;
  __m512 o[D / 16];
  for (int i = 0; i < D / 16; ++i) o[i] = _mm512_setzero_ps();
  for (int k = 0; k < K; ++k) {
    if (k + AHEAD < K) prefetch_row(row_of(v_shadow, k + AHEAD));
    const uint16_t* vr = row_of(v_shadow, k);
    if (!vr) continue;
    const __m512 w = _mm512_set1_ps(score_buf[k] * inv);
    for (int i = 0; i < D / 16; ++i) {
      const __m512i u = _mm512_slli_epi32(_mm512_cvtepu16_epi32(_mm256_loadu_si256(reinterpret_cast<const __m256i*>(vr + 16 * i))), 16);
      o[i] = _mm512_fmadd_ps(w, _mm512_castsi512_ps(u), o[i]);
    }
  }
  for (int i = 0; i < D / 16; ++i)
    _mm256_storeu_si256(reinterpret_cast<__m256i*>(out + 16 * i), (__m256i)_mm512_cvtneps_pbh(o[i]));
}
static bool host_has_avx512bf16() {
  static const bool ok = __builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw") &&
                        __builtin_cpu_supports("avx512vl") && __builtin_cpu_supports("avx512dq") &&
                        __builtin_cpu_supports("avx512bf16");
  return ok;
}
#else
static bool host_has_avx2_fma() { return false; }
static bool host_has_avx512bf16() { return false; }
#endif

// Row implementation in use: 0 scalar, 1 AVX2+FMA, 2 AVX-512-BF16.  The widest the host supports, unless
// JETFIRE_CPU_ATTN_ISA (scalar | avx2 | avx512bf16) or jf_set_cpu_attn_isa asks for a narrower one.
static std::atomic<int> g_isa_override{-1};
static int resolve_isa() {
  int best = host_has_avx512bf16() ? 2 : (host_has_avx2_fma() ? 1 : 0);
  int want = g_isa_override.load(std::memory_order_relaxed);
  if (want < 0) {
    static const int env = [] {
      const char* e = std::getenv("JETFIRE_CPU_ATTN_ISA");
      if (!e) return -1;
      if (!strcmp(e, "scalar")) return 0;
      if (!strcmp(e, "avx2")) return 1;
      if (!strcmp(e, "avx512bf16")) return 2;
      return -1;
    }();
    want = env;
  }
  if (want >= 0 && want < best) best = want;
  return best;
}

// Rows whose output came out non-finite (jetfire_vllm/csrc/cpu_topk_attn.cpp:809-826, 839-846): a vector row
// is recomputed by the scalar row, and a row that is still non-finite is zeroed, so that one bad correction
// cannot poison the layers after it.  The counter is what get_cpu_topk_sanitize_count reports.
static std::atomic<int64_t> g_sanitize_count{0};
static inline bool bf16_row_has_nonfinite(const uint16_t* r) {
  for (int i = 0; i < D; ++i)
    if ((r[i] & 0x7f80u) == 0x7f80u) return true;
  return false;
}

template <typename SlotT>
static void compute_row_t(const CpuJob& j, const SlotT* ts, int64_t r, uint16_t* out, float* buf) {
  const int G = j.H_q / j.H_kv;
  const int isa = resolve_isa();
  const uint16_t* q = j.q + r * D;
  const int64_t* hm = j.head_map ? j.head_map + r * j.K : nullptr;
  const int64_t fixed_h = (r % j.H_q) / G;
#if defined(__x86_64__)
  if (isa == 2) topk_attn_row_avx512bf16<SlotT>(q, j.k_shadow, j.v_shadow, j.num_slots, hm, fixed_h, ts + r * j.K, j.K, j.H_kv, j.scale, out, buf);
  else if (isa == 1) topk_attn_row_avx2<SlotT>(q, j.k_shadow, j.v_shadow, j.num_slots, hm, fixed_h, ts + r * j.K, j.K, j.H_kv, j.scale, out, buf);
  else
#endif
    topk_attn_row<SlotT>(q, j.k_shadow, j.v_shadow, j.num_slots, hm, fixed_h, ts + r * j.K, j.K, j.H_kv, j.scale, out, buf);
  if (bf16_row_has_nonfinite(out)) {
    g_sanitize_count.fetch_add(1, std::memory_order_acq_rel);
    if (isa != 0) topk_attn_row<SlotT>(q, j.k_shadow, j.v_shadow, j.num_slots, hm, fixed_h, ts + r * j.K, j.K, j.H_kv, j.scale, out, buf);
    if (isa == 0 || bf16_row_has_nonfinite(out)) memset(out, 0, D * sizeof(uint16_t));
  }
}

static void compute_row(const CpuJob& j, int64_t r, uint16_t* out) {
  static thread_local std::vector<float> buf;
  if (buf.size() < (size_t)j.K) buf.resize((size_t)j.K);
  if (j.ts32) compute_row_t<int32_t>(j, j.ts32, r, out, buf.data());
  else compute_row_t<int64_t>(j, j.ts_buf, r, out, buf.data());
}

}  // namespace jf

using namespace jf;

extern "C" const char* jf_last_error(void) { return g_err; }
#ifndef JF_BUILD_ID
#define JF_BUILD_ID "unknown"
#endif
#ifdef JF_DEBUG_HOOKS
#define JF_HOOKS_TAG " +debug-hooks"
#else
#define JF_HOOKS_TAG ""
#endif
// "jetfire_amd <release> (gfx950) build <id>[ +debug-hooks]": the id is a digest of the sources and flags the library
// was built from (jetfire_amd/build.py), so a measurement can be tied to the exact code that ran
extern "C" const char* jf_version(void) { return "jetfire_amd 0.3 (gfx950) build " JF_BUILD_ID JF_HOOKS_TAG; }

extern "C" int jf_set_cpu_attn_threads(int n) {
  Pool::instance().set_threads(n);
  return JF_OK;
}
extern "C" int jf_get_cpu_attn_threads(void) { return Pool::instance().threads(); }

extern "C" int jf_set_cpu_attn_isa(int isa) {
  JF_CHECK_ARG(isa >= -1 && isa <= 2, "set_cpu_attn_isa: isa must be -1 (widest), 0 (scalar), 1 (avx2) or 2 (avx512bf16)");
  g_isa_override.store(isa);
  return JF_OK;
}
extern "C" int jf_get_cpu_attn_isa(void) { return resolve_isa(); }
extern "C" int64_t jf_cpu_topk_sanitize_count(void) { return g_sanitize_count.load(); }

#ifdef JF_DEBUG_HOOKS
extern "C" int jf_debug_pool_stall(int64_t row, int microseconds) {
  JF_CHECK_ARG(microseconds >= 0 && microseconds <= 10000000, "debug_pool_stall: bad duration");
  g_stall_us.store(microseconds);
  g_stall_row.store(row);
  return JF_OK;
}
extern "C" int jf_debug_pool_wait_stragglers(int on) {
  g_wait_stragglers.store(on ? 1 : 0);
  if (on) Pool::instance().quiesce();
  return JF_OK;
}
#endif  // JF_DEBUG_HOOKS

extern "C" int jf_cpu_topk_attn(const uint16_t* q, const uint16_t* k_shadow, const uint16_t* v_shadow,
                                const int64_t* head_map, const int64_t* ts_buf, uint16_t* o_new, int B, int H_q, int K,
                                int H_kv, int64_t num_slots, float scale, int64_t* done_flag) {
  JF_CHECK_ARG(B >= 0 && H_q > 0 && K > 0 && H_kv > 0 && num_slots > 0, "cpu_topk_attn: bad shape");
  if (B > 0) {
    JF_CHECK_ARG(q && k_shadow && v_shadow && head_map && ts_buf && o_new, "cpu_topk_attn: null pointer");
    CpuJob j{q, k_shadow, v_shadow, head_map, ts_buf, o_new, B, H_q, K, H_kv, num_slots, scale};
    Pool::instance().run(j, (int64_t)B * H_q, false);
  }
  std::atomic_thread_fence(std::memory_order_release);
  if (done_flag) reinterpret_cast<std::atomic<int64_t>*>(done_flag)->store(1, std::memory_order_release);
  return JF_OK;
}

// ------------------------------------------------------------------ pinned hand-off
// submit: one small kernel, in stream order behind the merge, copies q and the winners' slots into pinned
// host memory and then raises a sequence flag there (last workgroup, after a system-scope fence).  A
// dispatcher thread of the context polls the flag while a submit is outstanding (it sleeps on a condition
// variable otherwise), runs the correction on the worker pool and publishes the finished sequence number.
// wait: the calling host thread waits for that number (the reference blocks on its future the same way,
// decode_path.py:3082-3114) and then enqueues a small kernel that brings o_new from the pinned buffer to the
// device.  No stream callbacks and no hipMemcpyAsync: on this runtime each costs tens of microseconds per layer.
struct jf_handoff {
  int B, H_q, H_kv, K;
  int64_t num_slots;
  const uint16_t *k_shadow, *v_shadow;
  float scale;
  uint16_t* q_pin = nullptr;       // (B, H_q, D) bf16
  int32_t* ts_pin = nullptr;       // (B, H_q, K) slots, narrowed to 32 bits by the publish kernel (half the PCIe bytes)
  uint16_t* o_pin = nullptr;       // (B, H_q, D) bf16
  int64_t* flag_pin = nullptr;     // [0]: sequence number of the last published (q, slots); [8]: sequence number of
                                   // the last finished correction; [16]: status raised by the device-side wait
  unsigned* counter_dev = nullptr; // [0]: workgroups of the publish kernel that have finished; bytes 8..15: the
                                   // device's own sequence counter (stream mode)
  std::atomic<int> mode{0};        // 0 = not used yet, 1 = host-blocking wait, 2 = stream mode (device-side wait)
  std::atomic<int> paused{0};      // test aid: published flags are ignored
  std::atomic<int> sanitize{0};    // stream_wait_blend writes zero for non-finite outputs
  int64_t stream_seen = 0;         // stream mode: last sequence number the shared poller has served
  bool registered = false;         // stream mode: known to the shared poller
  uint64_t device_wait_ticks = 0;  // bound of the device-side wait, in ticks of the 100 MHz wall clock
  std::atomic<int64_t> submits{0};
  std::atomic<int64_t> host_seq{0};  // submits enqueued by the host
  std::atomic<int64_t> done_seq{0};  // corrections finished by the dispatcher
  std::atomic<int> failed{0};
  std::atomic<int> stop{0};
  std::mutex mu;
  std::condition_variable cv;
  std::thread dispatcher;
  double timeout_s = 30.0;         // JETFIRE_CPU_FUTURE_TIMEOUT_S in the reference (decode_path.py:3082-3098)
  // submit contexts over the caller's own pinned buffers (jf_submit_ctx_create): nothing is copied by a kernel,
  // the correction reads q / head_map / slots from and writes o_new to these, then raises ext_flag
  const uint16_t* ext_q = nullptr;
  const int64_t* ext_head_map = nullptr;
  const int64_t* ext_ts = nullptr;
  uint16_t* ext_o = nullptr;
  int64_t* ext_flag = nullptr;
};

namespace {

__global__ __launch_bounds__(256) void handoff_publish_kernel(const uint4* __restrict__ q_src, uint4* q_dst, int nq16,
                                                              const uint4* __restrict__ s_src, uint4* s_dst, int ns16,
                                                              unsigned* counter, int64_t* flag, int64_t seq,
                                                              int64_t* seq_dev) {
  // q: 16 bytes per item; slots: item i narrows four int64 slots (two 16-byte loads) to one 16-byte store
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < nq16 + ns16; i += gridDim.x * blockDim.x) {
    if (i < nq16) {
      q_dst[i] = q_src[i];
    } else {
      const int j = i - nq16;
      const uint4 a = s_src[2 * j], b = s_src[2 * j + 1];
      s_dst[j] = make_uint4(a.x, a.z, b.x, b.z);  // low words: slots are < 2^31, -1 stays -1
    }
  }
  __threadfence_system();  // this thread's stores to host memory are ordered before the counter update
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned done = atomicAdd(counter, 1u);
    if (done == gridDim.x - 1) {  // every workgroup's stores are out: raise the flag
      *counter = 0u;
      if (seq_dev) {  // stream mode: the device numbers the submits itself, so a graph replay needs no new argument
        seq = *seq_dev + 1;
        *seq_dev = seq;
      }
      __threadfence_system();
      __hip_atomic_store(flag, seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
  }
}

__global__ __launch_bounds__(256) void handoff_fetch_kernel(const uint4* __restrict__ src, uint4* dst, int n16) {
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += gridDim.x * blockDim.x) dst[i] = src[i];
}

// Stream mode: ONE workgroup.  Its first lane polls the finished-sequence word in pinned host memory until the
// correction of the device's current sequence number is done or `limit_ticks` of the constant 100 MHz clock have
// passed (then the status word is raised and o_new is zero-filled: the kernel always ends), the workgroup then
// copies o_new to the device.
__global__ __launch_bounds__(1024) void handoff_wait_fetch_kernel(const int64_t* done, const int64_t* seq_dev,
                                                                  int64_t* status, uint64_t limit_ticks,
                                                                  const uint4* __restrict__ src, uint4* dst, int n16,
                                                                  const float* __restrict__ o_hat,
                                                                  const float* __restrict__ o_old,
                                                                  const float* __restrict__ W, uint4* out, int sanitize,
                                                                  int64_t* wait_log, int wait_log_cap) {
  // Each lane owns up to U items per pass (item = eight bf16 elements).  What does not depend on the CPU -- the
  // o_hat / o_old rows and W of the first pass -- is loaded before the wait, and the U reads from pinned host
  // memory of a pass are issued together, so that one PCIe round trip covers them.
  constexpr int U = 4;
  __shared__ int ok_sh;
  float4 H[U][2], O[U][2];
  float Wv[U];
  auto load_gpu_side = [&](int base) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = base + (int)threadIdx.x + u * (int)blockDim.x;
      if (out && i < n16) {
        H[u][0] = reinterpret_cast<const float4*>(o_hat)[2 * i];
        H[u][1] = reinterpret_cast<const float4*>(o_hat)[2 * i + 1];
        O[u][0] = reinterpret_cast<const float4*>(o_old)[2 * i];
        O[u][1] = reinterpret_cast<const float4*>(o_old)[2 * i + 1];
        Wv[u] = W[i >> 4];  // 16 items per 128-element row
      }
    }
  };
  load_gpu_side(0);
  if (threadIdx.x == 0) {
    const int64_t want = *seq_dev;
    const uint64_t t0 = wall_clock64();
    // a context that has failed once does not wait again: every later launch falls through at once
    int ok = __hip_atomic_load(status, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_SYSTEM) == 0;
    while (ok && __hip_atomic_load(done, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_SYSTEM) < want) {
      if (wall_clock64() - t0 > limit_ticks) {
        ok = 0;
        break;
      }
      __builtin_amdgcn_s_sleep(16);
    }
    if (!ok && __hip_atomic_load(status, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_SYSTEM) == 0)
      __hip_atomic_store(status, (int64_t)1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    if (wait_log) {  // measurement aid: how long this launch waited, in ticks of the 100 MHz clock
      const unsigned long long slot = atomicAdd(reinterpret_cast<unsigned long long*>(wait_log), 1ull);
      wait_log[1 + (int64_t)(slot % (unsigned long long)wait_log_cap)] = (int64_t)(wall_clock64() - t0);
    }
    ok_sh = ok;
  }
  __syncthreads();
  const bool ok = ok_sh != 0;
  for (int base = 0; base < n16; base += U * (int)blockDim.x) {
    if (base > 0) load_gpu_side(base);
    uint4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = base + (int)threadIdx.x + u * (int)blockDim.x;
      v[u] = (ok && i < n16) ? src[i] : make_uint4(0u, 0u, 0u, 0u);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = base + (int)threadIdx.x + u * (int)blockDim.x;
      if (i >= n16) continue;
      if (dst) dst[i] = v[u];
      if (out) {  // the blend of jf_blend_unnorm on the eight elements this lane has just fetched
        const uint32_t n[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
        const float hh[8] = {H[u][0].x, H[u][0].y, H[u][0].z, H[u][0].w, H[u][1].x, H[u][1].y, H[u][1].z, H[u][1].w};
        const float dd[8] = {O[u][0].x, O[u][0].y, O[u][0].z, O[u][0].w, O[u][1].x, O[u][1].y, O[u][1].z, O[u][1].w};
        uint32_t r[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float lo = __builtin_fmaf(Wv[u], bf16_to_f32((uint16_t)(n[e] & 0xffffu)), hh[2 * e]) - dd[2 * e];
          float hi = __builtin_fmaf(Wv[u], bf16_to_f32((uint16_t)(n[e] >> 16)), hh[2 * e + 1]) - dd[2 * e + 1];
          if (sanitize) {  // non-finite outputs become zero (decode_path.py:1133-1149)
            lo = isfinite(lo) ? lo : 0.0f;
            hi = isfinite(hi) ? hi : 0.0f;
          }
          r[e] = (uint32_t)f32_to_bf16(lo) | ((uint32_t)f32_to_bf16(hi) << 16);
        }
        out[i] = make_uint4(r[0], r[1], r[2], r[3]);
      }
    }
  }
}

inline void cpu_relax() {
#if defined(__x86_64__)
  _mm_pause();
#endif
}

std::atomic<int64_t> g_graph_submits{0};   // stream-mode submits served by the poller (get_graph_submit_count)
// what get_graph_timing_stats reports (jetfire_vllm/csrc/cpu_topk_attn.cpp:2361-2434): the corrections the poller ran
// and the host-blocking joins, count / total / longest in nanoseconds
std::atomic<int64_t> g_topk_jobs{0}, g_topk_ns{0}, g_topk_max_ns{0};
std::atomic<int64_t> g_join_jobs{0}, g_join_ns{0}, g_join_max_ns{0};
inline void stat_add(std::atomic<int64_t>& n, std::atomic<int64_t>& tot, std::atomic<int64_t>& mx, int64_t dt) {
  n.fetch_add(1, std::memory_order_relaxed);
  tot.fetch_add(dt, std::memory_order_relaxed);
  int64_t cur = mx.load(std::memory_order_relaxed);
  while (dt > cur && !mx.compare_exchange_weak(cur, dt, std::memory_order_relaxed)) {}
}
inline int64_t steady_ns() {
  return std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now().time_since_epoch()).count();
}
// Doorbell of the pool: a word in pinned host memory that a one-lane kernel at the head of a decode step (or of its
// HIP graph) bumps; the poller thread sees the change and wakes the pool's workers ahead of the first layer's job.
// measurement aid (jf_debug_wait_log): device buffer the device-side waits record their waiting times in
std::atomic<int64_t*> g_wait_log{nullptr};
std::atomic<int> g_wait_log_cap{0};
int64_t* g_doorbell_pin = nullptr;   // [0]: the word the kernel bumps
int64_t* g_doorbell_dev = nullptr;   // the same word as the device sees it
int64_t g_doorbell_seen = 0;         // (poller thread only)
std::mutex g_doorbell_mu;

bool run_correction(jf_handoff* h) {
  if (h->ext_q) {  // the caller's buffers, its head map and 64-bit slots
    CpuJob j{h->ext_q, h->k_shadow, h->v_shadow, h->ext_head_map, h->ext_ts, h->ext_o,
             h->B, h->H_q, h->K, h->H_kv, h->num_slots, h->scale};
    const bool ok = Pool::instance().run(j, (int64_t)h->B * h->H_q, true);  // the context's buffers outlive the job
    std::atomic_thread_fence(std::memory_order_release);
    if (h->ext_flag) __atomic_store_n(h->ext_flag, (int64_t)1, __ATOMIC_RELEASE);
    return ok;
  }
  // kv-head of a row = query head / (H_q / H_kv) (decode_path.py:400-408): no head map is read
  CpuJob j{h->q_pin, h->k_shadow, h->v_shadow, nullptr, nullptr, h->o_pin,
           h->B, h->H_q, h->K, h->H_kv, h->num_slots, h->scale, h->ts_pin};
  return Pool::instance().run(j, (int64_t)h->B * h->H_q, true);
}

// Raises the sequence flag of a context whose buffers the caller fills itself (stream-ordered behind its copies).
__global__ void handoff_signal_kernel(int64_t* flag, int64_t* seq_dev) {
  const int64_t seq = *seq_dev + 1;
  *seq_dev = seq;
  __threadfence_system();
  __hip_atomic_store(flag, seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Stream value operations as kernels (the reference uses cuStreamWriteValue64 / cuStreamWaitValue64,
// jetfire_vllm/csrc/cpu_topk_attn.cpp:1293-1344): one lane writes, or polls until the word equals `value` or the
// limit has passed (then *timeouts is incremented: every kernel ends).
__global__ void stream_write_value64_kernel(int64_t* p, int64_t value) {
  __threadfence_system();
  __hip_atomic_store(p, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}
__global__ void stream_wait_value64_kernel(const int64_t* p, int64_t value, uint64_t limit_ticks, int64_t* timeouts) {
  const uint64_t t0 = wall_clock64();
  while (__hip_atomic_load(p, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_SYSTEM) != value) {
    if (wall_clock64() - t0 > limit_ticks) {
      __hip_atomic_fetch_add(timeouts, (int64_t)1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      break;
    }
    __builtin_amdgcn_s_sleep(16);
  }
}

// Host mode: the context's own thread, asleep unless a submit is outstanding.
void handoff_dispatch(jf_handoff* h) {
  int64_t seen = 0;
  for (;;) {
    {  // nothing outstanding: sleep until a submit (or the end)
      std::unique_lock<std::mutex> lk(h->mu);
      h->cv.wait(lk, [&] { return h->stop.load() || h->host_seq.load() > seen; });
    }
    if (h->stop.load()) return;
    // a submit is in the stream: poll the flag the publish kernel raises
    const auto t0 = std::chrono::steady_clock::now();
    int64_t f = seen;
    for (uint64_t spin = 0;; ++spin) {
      f = __atomic_load_n(h->flag_pin, __ATOMIC_ACQUIRE);
      if (f != seen || h->stop.load(std::memory_order_relaxed)) break;
      cpu_relax();
      if ((spin & 0xfff) == 0xfff) {
        const double el = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
        if (el > h->timeout_s) { h->failed.store(1); break; }
        if (el > 0.002) std::this_thread::sleep_for(std::chrono::microseconds(50));  // a long GPU queue: stop burning a core
      }
    }
    if (h->stop.load()) return;
    if (f == seen) {  // timed out: give up on the outstanding submits
      seen = h->host_seq.load();
      h->done_seq.store(seen, std::memory_order_release);
      continue;
    }
    seen = f;
    const int64_t t_job = steady_ns();
    if (!run_correction(h)) h->failed.store(1);
    stat_add(g_topk_jobs, g_topk_ns, g_topk_max_ns, steady_ns() - t_job);
    h->submits.fetch_add(1, std::memory_order_relaxed);
    h->done_seq.store(seen, std::memory_order_release);
  }
}

// Stream mode: submits arrive from kernels (graph replays included) without any host call, so somebody has to
// keep looking at the flags.  ONE thread of the process does that for every stream-mode context (a model has a
// context per layer and batch size; a spinning thread each would eat the cores the correction needs): it walks
// the registered contexts, serves a raised flag at once, and sleeps between walks, longer and longer, while the
// GPU stays silent.  It is created on first use and lives until the process ends.
struct StreamPoller {
  std::mutex mu;
  std::condition_variable cv;
  std::vector<jf_handoff*> ctxs;

  static StreamPoller& instance() {
    static StreamPoller* p = [] {
      StreamPoller* sp = new StreamPoller();
      std::thread([sp] { sp->loop(); }).detach();
      return sp;
    }();
    return *p;
  }
  void add(jf_handoff* h) {
    {
      std::lock_guard<std::mutex> g(mu);
      ctxs.push_back(h);
    }
    cv.notify_one();
  }
  void remove(jf_handoff* h) {  // on return the poller does not touch h any more
    std::lock_guard<std::mutex> g(mu);
    for (size_t i = 0; i < ctxs.size(); ++i)
      if (ctxs[i] == h) {
        ctxs[i] = ctxs.back();
        ctxs.pop_back();
        break;
      }
  }
  void loop() {
    auto idle_since = std::chrono::steady_clock::now();
    for (uint64_t walk = 0;; ++walk) {
      bool served = false;
      {
        std::unique_lock<std::mutex> lk(mu);
        if (ctxs.empty() && __atomic_load_n(&g_doorbell_pin, __ATOMIC_ACQUIRE) == nullptr) {
          cv.wait(lk, [&] { return !ctxs.empty() || __atomic_load_n(&g_doorbell_pin, __ATOMIC_ACQUIRE) != nullptr; });
          idle_since = std::chrono::steady_clock::now();
        }
        for (jf_handoff* h : ctxs) {
          if (h->paused.load(std::memory_order_relaxed)) continue;
          const int64_t f = __atomic_load_n(h->flag_pin, __ATOMIC_ACQUIRE);
          if (f == h->stream_seen) continue;
          h->stream_seen = f;
          const int64_t t_job = steady_ns();
          if (!run_correction(h)) {
            h->failed.store(1);
            __atomic_store_n(h->flag_pin + 16, (int64_t)2, __ATOMIC_RELEASE);
          }
          h->submits.fetch_add(1, std::memory_order_relaxed);
          g_graph_submits.fetch_add(1, std::memory_order_relaxed);
          __atomic_store_n(h->flag_pin + 8, f, __ATOMIC_RELEASE);  // what the device-side wait polls
          stat_add(g_topk_jobs, g_topk_ns, g_topk_max_ns, steady_ns() - t_job);
          served = true;
        }
      }
      if (int64_t* db = __atomic_load_n(&g_doorbell_pin, __ATOMIC_ACQUIRE)) {
        const int64_t v = __atomic_load_n(db, __ATOMIC_ACQUIRE);
        if (v != g_doorbell_seen) {  // a step is on its way: have the workers spinning when its first job arrives
          g_doorbell_seen = v;
          Pool::instance().wake();
          served = true;
        }
      }
      if (served) {
        idle_since = std::chrono::steady_clock::now();
        continue;
      }
      cpu_relax();
      if ((walk & 0x3ff) == 0x3ff) {
        const double el = std::chrono::duration<double>(std::chrono::steady_clock::now() - idle_since).count();
        // a decode loop raises a flag every few hundred microseconds; only a GPU that has been silent for a while
        // (no step in flight) is worth sleeping on: a sleep costs the next submit its wake-up latency
        if (el > 0.05) std::this_thread::sleep_for(std::chrono::microseconds(el > 1.0 ? 200 : 50));
      }
    }
  }
};

bool claim_mode(jf_handoff* h, int mode) {
  int expected = 0;
  return h->mode.compare_exchange_strong(expected, mode) || expected == mode;
}

}  // namespace

extern "C" jf_handoff* jf_handoff_create(int B, int H_q, int H_kv, int K, int64_t num_slots,
                                         const uint16_t* k_shadow_host, const uint16_t* v_shadow_host, float scale) {
  if (B <= 0 || H_q <= 0 || H_kv <= 0 || K <= 0 || K % 4 != 0 || num_slots <= 0 || num_slots > 0x7fffffffLL || H_q % H_kv != 0 ||
      !k_shadow_host || !v_shadow_host) {
    set_error("handoff_create: bad arguments");
    return nullptr;
  }
  jf_handoff* h = new jf_handoff();
  h->B = B; h->H_q = H_q; h->H_kv = H_kv; h->K = K; h->num_slots = num_slots;
  h->k_shadow = k_shadow_host; h->v_shadow = v_shadow_host; h->scale = scale;
  if (const char* e = std::getenv("JETFIRE_CPU_FUTURE_TIMEOUT_S")) {
    const double t = std::atof(e);
    if (t > 0) h->timeout_s = t;
  }
  const size_t nq = (size_t)B * H_q * D * sizeof(uint16_t), nt = (size_t)B * H_q * K * sizeof(int32_t);
  if (hipHostMalloc((void**)&h->q_pin, nq, hipHostMallocDefault) != hipSuccess ||
      hipHostMalloc((void**)&h->ts_pin, nt, hipHostMallocDefault) != hipSuccess ||
      hipHostMalloc((void**)&h->o_pin, nq, hipHostMallocDefault) != hipSuccess ||
      hipHostMalloc((void**)&h->flag_pin, 256, hipHostMallocDefault) != hipSuccess ||
      hipMalloc((void**)&h->counter_dev, 64) != hipSuccess || hipMemset(h->counter_dev, 0, 64) != hipSuccess) {
    set_error("handoff_create: allocation failed");
    jf_handoff_destroy(h);
    return nullptr;
  }
  h->flag_pin[0] = h->flag_pin[8] = h->flag_pin[16] = 0;
  h->device_wait_ticks = (uint64_t)((h->timeout_s < 10.0 ? h->timeout_s : 10.0) * 1e8);
  h->dispatcher = std::thread(handoff_dispatch, h);
  return h;
}

extern "C" int jf_handoff_submit(jf_handoff* h, const uint16_t* q_dev, const int64_t* topk_slots_dev, void* stream) {
  JF_CHECK_ARG(h && q_dev && topk_slots_dev, "handoff_submit: null argument");
  JF_CHECK_ARG(((uintptr_t)q_dev & 15) == 0 && ((uintptr_t)topk_slots_dev & 15) == 0, "handoff_submit: q and topk_slots must be 16-byte aligned");
  if (h->failed.load()) { set_error("handoff: an earlier CPU correction job failed or timed out"); return JF_ERR_TIMEOUT; }
  JF_CHECK_ARG(claim_mode(h, 1), "handoff_submit: the context is in stream mode (use jf_handoff_stream_submit)");
  JF_CHECK_ARG(h->host_seq.load() == h->done_seq.load(), "handoff_submit: the previous correction is still in flight (wait for it first)");
  hipStream_t st = (hipStream_t)stream;
  const int nq16 = (int)((size_t)h->B * h->H_q * D * sizeof(uint16_t) / 16);
  const int ns16 = (int)((size_t)h->B * h->H_q * h->K * sizeof(int32_t) / 16);
  const int64_t seq = h->host_seq.load() + 1;
  int blocks = (nq16 + ns16 + 255) / 256;
  if (blocks > 32) blocks = 32;
  hipLaunchKernelGGL(handoff_publish_kernel, dim3(blocks), dim3(256), 0, st, reinterpret_cast<const uint4*>(q_dev),
                     reinterpret_cast<uint4*>(h->q_pin), nq16, reinterpret_cast<const uint4*>(topk_slots_dev),
                     reinterpret_cast<uint4*>(h->ts_pin), ns16, h->counter_dev, h->flag_pin, seq, (int64_t*)nullptr);
  JF_CHECK_HIP(hipGetLastError());
  {
    std::lock_guard<std::mutex> g(h->mu);
    h->host_seq.store(seq);
  }
  h->cv.notify_one();
  return JF_OK;
}

extern "C" int jf_handoff_stream_submit(jf_handoff* h, const uint16_t* q_dev, const int64_t* topk_slots_dev, void* stream) {
  JF_CHECK_ARG(h && q_dev && topk_slots_dev, "handoff_stream_submit: null argument");
  JF_CHECK_ARG(((uintptr_t)q_dev & 15) == 0 && ((uintptr_t)topk_slots_dev & 15) == 0, "handoff_stream_submit: q and topk_slots must be 16-byte aligned");
  if (h->failed.load() || __atomic_load_n(h->flag_pin + 16, __ATOMIC_ACQUIRE) != 0) {
    set_error("handoff: an earlier CPU correction job failed or timed out");
    return JF_ERR_TIMEOUT;
  }
  JF_CHECK_ARG(claim_mode(h, 2), "handoff_stream_submit: the context is in host mode (use jf_handoff_submit)");
  if (!h->registered) {  // the shared poller looks at this context's flag from now on
    h->registered = true;
    StreamPoller::instance().add(h);
  }
  const int nq16 = (int)((size_t)h->B * h->H_q * D * sizeof(uint16_t) / 16);
  const int ns16 = (int)((size_t)h->B * h->H_q * h->K * sizeof(int32_t) / 16);
  int blocks = (nq16 + ns16 + 255) / 256;
  if (blocks > 32) blocks = 32;
  hipLaunchKernelGGL(handoff_publish_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                     reinterpret_cast<const uint4*>(q_dev), reinterpret_cast<uint4*>(h->q_pin), nq16,
                     reinterpret_cast<const uint4*>(topk_slots_dev), reinterpret_cast<uint4*>(h->ts_pin), ns16,
                     h->counter_dev, h->flag_pin, (int64_t)0, reinterpret_cast<int64_t*>(h->counter_dev + 2));
  JF_CHECK_HIP(hipGetLastError());
  return JF_OK;
}

extern "C" int jf_handoff_stream_wait(jf_handoff* h, uint16_t* o_new_dev, void* stream) {
  JF_CHECK_ARG(h && o_new_dev, "handoff_stream_wait: null argument");
  JF_CHECK_ARG(((uintptr_t)o_new_dev & 15) == 0, "handoff_stream_wait: o_new must be 16-byte aligned");
  JF_CHECK_ARG(h->mode.load() == 2, "handoff_stream_wait: no jf_handoff_stream_submit precedes it");
  const int n16 = (int)((size_t)h->B * h->H_q * D * sizeof(uint16_t) / 16);
  hipLaunchKernelGGL(handoff_wait_fetch_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, h->flag_pin + 8,
                     reinterpret_cast<const int64_t*>(h->counter_dev + 2), h->flag_pin + 16, h->device_wait_ticks,
                     reinterpret_cast<const uint4*>(h->o_pin), reinterpret_cast<uint4*>(o_new_dev), n16,
                     (const float*)nullptr, (const float*)nullptr, (const float*)nullptr, (uint4*)nullptr, 0,
                     g_wait_log.load(), g_wait_log_cap.load());
  JF_CHECK_HIP(hipGetLastError());
  return JF_OK;
}

extern "C" int jf_handoff_set_output_sanitize(jf_handoff* h, int on) {
  JF_CHECK_ARG(h, "handoff_set_output_sanitize: null argument");
  h->sanitize.store(on ? 1 : 0);
  return JF_OK;
}

extern "C" int jf_handoff_stream_wait_blend(jf_handoff* h, const float* o_hat, const float* o_old_unnorm, const float* W,
                                            uint16_t* out, uint16_t* o_new_dev, void* stream) {
  JF_CHECK_ARG(h && o_hat && o_old_unnorm && W && out, "handoff_stream_wait_blend: null argument");
  JF_CHECK_ARG((((uintptr_t)o_hat | (uintptr_t)o_old_unnorm | (uintptr_t)out | (uintptr_t)o_new_dev) & 15) == 0,
               "handoff_stream_wait_blend: tensors must be 16-byte aligned");
  JF_CHECK_ARG(h->mode.load() == 2, "handoff_stream_wait_blend: no jf_handoff_stream_submit precedes it");
  const int n16 = (int)((size_t)h->B * h->H_q * D * sizeof(uint16_t) / 16);
  hipLaunchKernelGGL(handoff_wait_fetch_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, h->flag_pin + 8,
                     reinterpret_cast<const int64_t*>(h->counter_dev + 2), h->flag_pin + 16, h->device_wait_ticks,
                     reinterpret_cast<const uint4*>(h->o_pin), reinterpret_cast<uint4*>(o_new_dev), n16, o_hat,
                     o_old_unnorm, W, reinterpret_cast<uint4*>(out), h->sanitize.load(), g_wait_log.load(), g_wait_log_cap.load());
  JF_CHECK_HIP(hipGetLastError());
  return JF_OK;
}

extern "C" int jf_handoff_status(jf_handoff* h) {
  JF_CHECK_ARG(h, "handoff_status: null argument");
  const int64_t st = __atomic_load_n(h->flag_pin + 16, __ATOMIC_ACQUIRE);
  if (st == 1) { set_error("handoff: the device-side wait for the CPU correction ran into its limit"); return JF_ERR_TIMEOUT; }
  if (st != 0 || h->failed.load()) { set_error("handoff: a CPU correction job failed or timed out"); return JF_ERR_TIMEOUT; }
  return JF_OK;
}

extern "C" int jf_handoff_set_device_wait_limit_us(jf_handoff* h, int64_t us) {
  JF_CHECK_ARG(h && us > 0 && us <= 60000000, "handoff_set_device_wait_limit_us: limit must be in (0, 60 s]");
  h->device_wait_ticks = (uint64_t)us * 100u;
  return JF_OK;
}

#ifdef JF_DEBUG_HOOKS
extern "C" int jf_debug_wait_log(void* device_buffer, int capacity) {
  JF_CHECK_ARG(device_buffer == nullptr || capacity > 0, "debug_wait_log: capacity must be positive");
  g_wait_log_cap.store(device_buffer ? capacity : 0);
  g_wait_log.store(reinterpret_cast<int64_t*>(device_buffer));
  return JF_OK;
}

extern "C" int jf_handoff_debug_pause(jf_handoff* h, int on) {
  JF_CHECK_ARG(h, "handoff_debug_pause: null argument");
  h->paused.store(on ? 1 : 0);
  return JF_OK;
}
#endif  // JF_DEBUG_HOOKS

extern "C" int jf_handoff_wait(jf_handoff* h, uint16_t* o_new_dev, void* stream) {
  JF_CHECK_ARG(h && o_new_dev, "handoff_wait: null argument");
  JF_CHECK_ARG(((uintptr_t)o_new_dev & 15) == 0, "handoff_wait: o_new must be 16-byte aligned");
  JF_CHECK_ARG(h->mode.load() != 2, "handoff_wait: the context is in stream mode (use jf_handoff_stream_wait)");
  hipStream_t st = (hipStream_t)stream;
  const int64_t want = h->host_seq.load();
  const auto t0 = std::chrono::steady_clock::now();
  for (uint64_t spin = 0; h->done_seq.load(std::memory_order_acquire) < want; ++spin) {
    cpu_relax();
    if ((spin & 0xfff) == 0xfff) {
      const double el = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
      if (el > h->timeout_s + 1.0) { h->failed.store(1); break; }
      if (el > 0.002) std::this_thread::sleep_for(std::chrono::microseconds(50));
    }
  }
  stat_add(g_join_jobs, g_join_ns, g_join_max_ns,
           std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now() - t0).count());
  if (h->failed.load()) { set_error("handoff: CPU correction job failed or timed out"); return JF_ERR_TIMEOUT; }
  const int n16 = (int)((size_t)h->B * h->H_q * D * sizeof(uint16_t) / 16);
  hipLaunchKernelGGL(handoff_fetch_kernel, dim3((n16 + 255) / 256 < 8 ? (n16 + 255) / 256 : 8), dim3(256), 0, st,
                     reinterpret_cast<const uint4*>(h->o_pin), reinterpret_cast<uint4*>(o_new_dev), n16);
  JF_CHECK_HIP(hipGetLastError());
  return JF_OK;
}

extern "C" int64_t jf_handoff_submit_count(const jf_handoff* h) { return h ? h->submits.load() : -1; }

extern "C" void jf_handoff_destroy(jf_handoff* h) {
  Pool::instance().quiesce();  // a straggling worker may still be reading a finished job's buffers
  if (!h) return;
  // stream mode: kernels that poll or fill the pinned buffers may still be queued; they need the dispatcher alive
  if (h->mode.load() == 2) (void)hipDeviceSynchronize();
  if (h->registered) StreamPoller::instance().remove(h);
  // a submit that was never waited for: its kernel still writes the pinned buffers and its job reads them
  if (h->dispatcher.joinable() && !h->failed.load()) {
    const auto t0 = std::chrono::steady_clock::now();
    while (h->done_seq.load(std::memory_order_acquire) < h->host_seq.load()) {
      std::this_thread::sleep_for(std::chrono::microseconds(100));
      if (std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() > h->timeout_s + 1.0) break;
    }
  }
  {
    std::lock_guard<std::mutex> g(h->mu);
    h->stop.store(1);
  }
  h->cv.notify_all();
  if (h->dispatcher.joinable()) h->dispatcher.join();
  if (h->q_pin) (void)hipHostFree(h->q_pin);
  if (h->ts_pin) (void)hipHostFree(h->ts_pin);
  if (h->o_pin) (void)hipHostFree(h->o_pin);
  if (h->flag_pin) (void)hipHostFree(h->flag_pin);
  if (h->counter_dev) (void)hipFree(h->counter_dev);
  delete h;
}

// ------------------------------------------------------------------ submit contexts, the reference's way
// create_cpu_topk_submit_ctx / stream_submit_cpu_topk_attn / stream_wait_cpu_topk_attn
// (jetfire_vllm/csrc/cpu_topk_attn.cpp:2054-2163, 2239, 2302): the caller owns the pinned q / slots / o_new
// buffers and fills them with its own stream-ordered copies; a context only remembers the pointers.  Contexts
// are integer handles that live until clear_graph_contexts.
namespace {
std::mutex g_ctx_mu;
std::vector<jf_handoff*> g_ctxs;             // handle = index + 1
int64_t* g_wait_timeouts = nullptr;          // pinned counter of stream_wait_value64 waits that hit their limit

jf_handoff* ctx_of(int64_t handle) {
  std::lock_guard<std::mutex> g(g_ctx_mu);
  if (handle <= 0 || handle > (int64_t)g_ctxs.size()) return nullptr;
  return g_ctxs[(size_t)handle - 1];
}
double future_timeout_s() {
  double t = 30.0;
  if (const char* e = std::getenv("JETFIRE_CPU_FUTURE_TIMEOUT_S")) {
    const double v = std::atof(e);
    if (v > 0) t = v;
  }
  return t;
}

// submit_cpu_topk_attn_async (cpu_topk_attn.cpp:1184-1205): one executor thread takes the jobs in order
struct AsyncExecutor {
  std::mutex mu;
  std::condition_variable cv;
  std::vector<std::pair<CpuJob, int64_t*>> queue;
  bool started = false;
  static AsyncExecutor& instance() {
    static AsyncExecutor* e = new AsyncExecutor();
    return *e;
  }
  void submit(const CpuJob& j, int64_t* flag) {
    {
      std::lock_guard<std::mutex> g(mu);
      if (!started) {
        started = true;
        std::thread([this] { loop(); }).detach();
      }
      queue.emplace_back(j, flag);
    }
    cv.notify_one();
  }
  void loop() {
    for (;;) {
      std::pair<CpuJob, int64_t*> item;
      {
        std::unique_lock<std::mutex> lk(mu);
        cv.wait(lk, [&] { return !queue.empty(); });
        item = queue.front();
        queue.erase(queue.begin());
      }
      const CpuJob j = item.first;
      Pool::instance().run(j, (int64_t)j.B * j.H_q, false);
      std::atomic_thread_fence(std::memory_order_release);
      __atomic_store_n(item.second, (int64_t)1, __ATOMIC_RELEASE);
    }
  }
};
}  // namespace

extern "C" int64_t jf_submit_ctx_create(const uint16_t* q_host, const uint16_t* k_shadow_host, const uint16_t* v_shadow_host,
                                        const int64_t* head_map_host, const int64_t* ts_buf_host, uint16_t* o_new_host,
                                        int B, int H_q, int K, int H_kv, int64_t num_slots, float scale,
                                        int64_t* flag_host) {
  if (!q_host || !k_shadow_host || !v_shadow_host || !head_map_host || !ts_buf_host || !o_new_host || B <= 0 || H_q <= 0 ||
      K <= 0 || H_kv <= 0 || num_slots <= 0) {
    set_error("submit_ctx_create: bad arguments");
    return 0;
  }
  jf_handoff* h = new jf_handoff();
  h->B = B; h->H_q = H_q; h->H_kv = H_kv; h->K = K; h->num_slots = num_slots;
  h->k_shadow = k_shadow_host; h->v_shadow = v_shadow_host; h->scale = scale;
  h->ext_q = q_host; h->ext_head_map = head_map_host; h->ext_ts = ts_buf_host; h->ext_o = o_new_host; h->ext_flag = flag_host;
  h->timeout_s = future_timeout_s();
  if (hipHostMalloc((void**)&h->flag_pin, 256, hipHostMallocDefault) != hipSuccess ||
      hipMalloc((void**)&h->counter_dev, 64) != hipSuccess || hipMemset(h->counter_dev, 0, 64) != hipSuccess) {
    set_error("submit_ctx_create: allocation failed");
    jf_handoff_destroy(h);
    return 0;
  }
  h->flag_pin[0] = h->flag_pin[8] = h->flag_pin[16] = 0;
  h->device_wait_ticks = (uint64_t)((h->timeout_s < 10.0 ? h->timeout_s : 10.0) * 1e8);
  h->mode.store(2);
  std::lock_guard<std::mutex> g(g_ctx_mu);
  g_ctxs.push_back(h);
  return (int64_t)g_ctxs.size();
}

extern "C" int jf_submit_ctx_stream_submit(int64_t ctx, void* stream) {
  jf_handoff* h = ctx_of(ctx);
  if (!h || !h->ext_q) { set_error("stream_submit_cpu_topk_attn: unknown context handle %lld", (long long)ctx); return JF_ERR_STATE; }
  if (h->failed.load() || __atomic_load_n(h->flag_pin + 16, __ATOMIC_ACQUIRE) != 0) {
    set_error("handoff: an earlier CPU correction job failed or timed out");
    return JF_ERR_TIMEOUT;
  }
  if (!h->registered) {
    h->registered = true;
    StreamPoller::instance().add(h);
  }
  hipLaunchKernelGGL(handoff_signal_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, h->flag_pin,
                     reinterpret_cast<int64_t*>(h->counter_dev + 2));
  JF_CHECK_HIP(hipGetLastError());
  return JF_OK;
}

extern "C" int jf_submit_ctx_stream_wait(int64_t ctx, void* stream) {
  jf_handoff* h = ctx_of(ctx);
  if (!h || !h->ext_q) { set_error("stream_wait_cpu_topk_attn: unknown context handle %lld", (long long)ctx); return JF_ERR_STATE; }
  hipLaunchKernelGGL(handoff_wait_fetch_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, h->flag_pin + 8,
                     reinterpret_cast<const int64_t*>(h->counter_dev + 2), h->flag_pin + 16, h->device_wait_ticks,
                     (const uint4*)nullptr, (uint4*)nullptr, 0, (const float*)nullptr, (const float*)nullptr,
                     (const float*)nullptr, (uint4*)nullptr, 0, g_wait_log.load(), g_wait_log_cap.load());
  JF_CHECK_HIP(hipGetLastError());
  return JF_OK;
}

extern "C" int jf_submit_ctx_status(int64_t ctx) {
  jf_handoff* h = ctx_of(ctx);
  if (!h) { set_error("submit_ctx_status: unknown context handle %lld", (long long)ctx); return JF_ERR_STATE; }
  return jf_handoff_status(h);
}

extern "C" int jf_stream_write_value64(void* stream, int64_t* flag_device, int64_t value) {
  JF_CHECK_ARG(flag_device, "stream_write_value64: null flag");
  hipLaunchKernelGGL(stream_write_value64_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, flag_device, value);
  JF_CHECK_HIP(hipGetLastError());
  return JF_OK;
}

extern "C" int jf_stream_wait_value64(void* stream, const int64_t* flag_device, int64_t value) {
  JF_CHECK_ARG(flag_device, "stream_wait_value64: null flag");
  {
    std::lock_guard<std::mutex> g(g_ctx_mu);
    if (!g_wait_timeouts) {
      JF_CHECK_HIP(hipHostMalloc((void**)&g_wait_timeouts, 64, hipHostMallocDefault));
      *g_wait_timeouts = 0;
    }
  }
  const double t = future_timeout_s();
  hipLaunchKernelGGL(stream_wait_value64_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, flag_device, value,
                     (uint64_t)((t < 10.0 ? t : 10.0) * 1e8), g_wait_timeouts);
  JF_CHECK_HIP(hipGetLastError());
  return JF_OK;
}

extern "C" int64_t jf_stream_wait_timeouts(void) {
  std::lock_guard<std::mutex> g(g_ctx_mu);
  return g_wait_timeouts ? __atomic_load_n(g_wait_timeouts, __ATOMIC_ACQUIRE) : 0;
}

extern "C" int jf_cpu_topk_attn_async(const uint16_t* q, const uint16_t* k_shadow, const uint16_t* v_shadow,
                                      const int64_t* head_map, const int64_t* ts_buf, uint16_t* o_new, int B, int H_q, int K,
                                      int H_kv, int64_t num_slots, float scale, int64_t* flag) {
  JF_CHECK_ARG(B > 0 && H_q > 0 && K > 0 && H_kv > 0 && num_slots > 0, "submit_cpu_topk_attn_async: bad shape");
  JF_CHECK_ARG(q && k_shadow && v_shadow && head_map && ts_buf && o_new && flag, "submit_cpu_topk_attn_async: null pointer");
  CpuJob j{q, k_shadow, v_shadow, head_map, ts_buf, o_new, B, H_q, K, H_kv, num_slots, scale};
  AsyncExecutor::instance().submit(j, flag);
  return JF_OK;
}

extern "C" int jf_wait_for_flag(const int64_t* flag, double timeout_s) {
  JF_CHECK_ARG(flag, "wait_for_flag: null flag");
  const auto t0 = std::chrono::steady_clock::now();
  for (uint64_t spin = 0; __atomic_load_n(flag, __ATOMIC_ACQUIRE) == 0; ++spin) {
    cpu_relax();
    if ((spin & 0xfff) == 0xfff) {
      const double el = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
      if (timeout_s > 0 && el > timeout_s) { set_error("wait_for_flag: timed out after %.1f s", el); return JF_ERR_TIMEOUT; }
      if (el > 0.002) std::this_thread::sleep_for(std::chrono::microseconds(50));
    }
  }
  return JF_OK;
}

extern "C" int jf_graph_pool_warmup(int n_threads) {
  if (n_threads > 0) Pool::instance().set_threads(n_threads);
  Pool::instance().warm();  // starts (or resizes) the workers
  return JF_OK;
}

extern "C" int64_t jf_graph_submit_count(void) { return g_graph_submits.load(); }

extern "C" int jf_graph_timing_stats(double* out, int n) {
  JF_CHECK_ARG(out && n >= JF_GRAPH_TIMING_FIELDS, "graph_timing_stats: room for %d values needed", JF_GRAPH_TIMING_FIELDS);
  const int64_t jobs = g_topk_jobs.load(), joins = g_join_jobs.load();
  int64_t appends = 0;
  (void)jf_shadow_append_count(&appends, 0);
  out[0] = (double)jobs;
  out[1] = jobs > 0 ? (double)g_topk_ns.load() / (double)jobs / 1000.0 : 0.0;
  out[2] = (double)g_topk_max_ns.load() / 1000.0;
  out[3] = (double)appends;
  out[4] = (double)joins;
  out[5] = joins > 0 ? (double)g_join_ns.load() / (double)joins / 1000.0 : 0.0;
  out[6] = (double)g_join_max_ns.load() / 1000.0;
  out[7] = (double)Pool::instance().worker_count();
  out[8] = (double)Pool::instance().jobs_done();
  return JF_OK;
}

extern "C" int jf_reset_graph_submit_count(void) {
  g_graph_submits.store(0);
  g_sanitize_count.store(0);
  for (std::atomic<int64_t>* c : {&g_topk_jobs, &g_topk_ns, &g_topk_max_ns, &g_join_jobs, &g_join_ns, &g_join_max_ns}) c->store(0);
  int64_t unused = 0;
  return jf_shadow_append_count(&unused, 1);
}

// One lane bumps the doorbell word (system scope: the poller thread reads it from host memory).
__global__ void pool_doorbell_kernel(int64_t* word) {
  __hip_atomic_fetch_add(word, (int64_t)1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

extern "C" int jf_pool_wake(void) {
  Pool::instance().wake();
  return JF_OK;
}

extern "C" int jf_pool_doorbell(void* stream) {
  {
    std::lock_guard<std::mutex> g(g_doorbell_mu);
    if (g_doorbell_dev == nullptr) {  // once per process: the word, its device address, the poller
      int64_t* pin = nullptr;
      JF_CHECK_HIP(hipHostMalloc(reinterpret_cast<void**>(&pin), 64, hipHostMallocMapped));
      memset(pin, 0, 64);
      void* dev = nullptr;
      JF_CHECK_HIP(hipHostGetDevicePointer(&dev, pin, 0));
      g_doorbell_dev = reinterpret_cast<int64_t*>(dev);
      __atomic_store_n(&g_doorbell_pin, pin, __ATOMIC_RELEASE);
      StreamPoller::instance().cv.notify_one();
    }
  }
  hipLaunchKernelGGL(pool_doorbell_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, g_doorbell_dev);
  JF_CHECK_LAUNCH();
  return JF_OK;
}

extern "C" int jf_reset_graph_runtime_state(void) {
  Pool::instance().quiesce();  // a straggling worker may still be reading a finished job's buffers
  g_graph_submits.store(0);
  g_sanitize_count.store(0);
  std::lock_guard<std::mutex> g(g_ctx_mu);
  if (g_wait_timeouts) __atomic_store_n(g_wait_timeouts, (int64_t)0, __ATOMIC_RELEASE);
  return JF_OK;
}

extern "C" int jf_clear_graph_contexts(void) {
  Pool::instance().quiesce();  // a straggling worker may still be reading a finished job's buffers
  std::vector<jf_handoff*> old;
  {
    std::lock_guard<std::mutex> g(g_ctx_mu);
    old.swap(g_ctxs);
  }
  for (jf_handoff* h : old) jf_handoff_destroy(h);
  g_graph_submits.store(0);
  return JF_OK;
}
