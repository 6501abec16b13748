// feeder.hip — pipelined upload of training batches that live in pageable host memory.
//
// network::fit hands every mini-batch over as host vectors (tiny_dnn/network.h:866-879,
// layer::set_in_data, tiny_dnn/layers/layer.h:230-251). Uploading them synchronously in front
// of each step leaves the GPU idle for the copy and the host idle for the step. The feeder
// owns three slots of pinned host memory and three of device memory and a worker thread. Up to
// two batches may be staged ahead of the one being computed on: for each, the worker copies the
// caller's arrays into the pinned slot, waits (on the host, polling) until the device slot is
// free, and queues the upload on a copy stream itself, so a batch is on its way to the device
// as early as it can be, whatever the caller's thread is doing (queueing a step, capturing a
// graph: the step's capture is thread-local; the worker queues work on the copy stream only
// and never makes a stream depend on an event of the compute stream, which the runtime would
// take for a dependency on captured work while the caller captures).
// tdh_feeder_acquire then only makes the compute stream wait for an upload that was queued a
// step earlier. A device slot is never overwritten while a queued step still reads it: behind
// the steps on a slot the compute stream sets a word in pinned memory, and the worker queues the
// next upload into that slot only after it has seen the word change (a slot comes round again
// after three batches).
#include <algorithm>
#include <condition_variable>
#include <cstdint>
#include <cstring>
#include <mutex>
#include <string>
#include <thread>

#include "common.h"

namespace {
constexpr int kSlots = 3;     // device and pinned buffers
constexpr int kAhead = 2;     // batches that may be staged and not yet acquired
// A batch of a megabyte and more takes one core longer to copy into pinned memory than a small
// net's step lasts (about 10 GB/s: 150 us for 128 CIFAR images against a 190 us step, and the
// worker also queues the upload), so copies above kSplitBytes are cut into kCopyThreads pieces:
// the worker takes the first, helper threads of the feeder the others.
constexpr int kCopyThreads = 4;
constexpr size_t kSplitBytes = 256u << 10;
}  // namespace

struct tdh_feeder {
  size_t x_len = 0, t_len = 0;  // floats per sample
  int max_batch = 0;
  float *pin_x[kSlots] = {}, *pin_t[kSlots] = {};
  float *dev_x[kSlots] = {}, *dev_t[kSlots] = {};
  hipEvent_t uploaded[kSlots] = {};  // on the copy stream: the slot holds its batch
  // A word of pinned host memory per slot that a one-thread kernel on the compute stream sets
  // to consumed_seq[s] once every step that reads the slot has run. The worker polls the word:
  // it must not touch an event of the compute stream (a query or a wait from another thread
  // while the caller's thread captures a step on that stream invalidates the capture).
  uint32_t *consumed_flag = nullptr;
  uint32_t consumed_seq[kSlots] = {};  // value of the last mark queued for the slot
  int batch[kSlots] = {};
  int next_slot = 0;                 // slot of the next tdh_feeder_stage
  int staged_n = 0;                  // staged and not yet acquired
  int staged_slot[kAhead] = {};      // their slots, oldest first
  int current = -1;                  // slot handed out by the last tdh_feeder_acquire
  hipStream_t copy = nullptr;
  int device = 0;
  // worker thread: jobs in order, one per staged batch
  struct Job {
    int slot = 0, batch = 0;
    const float *x = nullptr, *t = nullptr;
    uint32_t wait_consumed = 0;      // value consumed_flag[slot] must have reached
  };
  std::thread worker;
  std::mutex mu;
  std::condition_variable cv;
  bool quit = false;
  Job jobs[kAhead];
  int jobs_n = 0;                    // queued for the worker (jobs[0] is next)
  bool slot_done[kSlots] = {};       // the slot's job has run (its upload is queued)
  hipError_t slot_error[kSlots] = {};
  // helper threads: each copies its piece of the worker's current copy
  std::thread helpers[kCopyThreads - 1];
  std::mutex hmu;
  std::condition_variable hcv;
  uint64_t copy_gen = 0;             // bumped by the worker for every split copy
  int copy_left = 0;                 // helpers that have not finished the current one
  char *copy_dst = nullptr;
  const char *copy_src = nullptr;
  size_t copy_bytes = 0;
  bool hquit = false;
};

namespace tdh {
namespace {
// piece `part` of kCopyThreads of a copy (whole 4 KiB pages, the last piece takes the rest)
void copy_piece(char *dst, const char *src, size_t bytes, int part) {
  const size_t per = ((bytes / kCopyThreads) + 4095) & ~size_t(4095);
  const size_t beg = std::min(bytes, per * part);
  const size_t end = part == kCopyThreads - 1 ? bytes : std::min(bytes, per * (part + 1));
  if (end > beg) std::memcpy(dst + beg, src + beg, end - beg);
}

void feeder_helper(tdh_feeder *f, int part) {
  uint64_t seen = 0;
  std::unique_lock<std::mutex> lock(f->hmu);
  for (;;) {
    f->hcv.wait(lock, [f, seen] { return f->hquit || f->copy_gen != seen; });
    if (f->hquit) return;
    seen = f->copy_gen;
    char *dst = f->copy_dst;
    const char *src = f->copy_src;
    const size_t bytes = f->copy_bytes;
    lock.unlock();
    copy_piece(dst, src, bytes, part);
    lock.lock();
    if (--f->copy_left == 0) f->hcv.notify_all();
  }
}

// host copy on the worker thread, shared with the helpers when it is large
void feeder_copy(tdh_feeder *f, void *dst, const void *src, size_t bytes) {
  if (bytes < kSplitBytes) {
    std::memcpy(dst, src, bytes);
    return;
  }
  {
    std::lock_guard<std::mutex> lock(f->hmu);
    f->copy_dst = static_cast<char *>(dst);
    f->copy_src = static_cast<const char *>(src);
    f->copy_bytes = bytes;
    f->copy_left = kCopyThreads - 1;
    ++f->copy_gen;
  }
  f->hcv.notify_all();
  copy_piece(static_cast<char *>(dst), static_cast<const char *>(src), bytes, 0);
  std::unique_lock<std::mutex> lock(f->hmu);
  f->hcv.wait(lock, [f] { return f->copy_left == 0; });
}

// behind the steps that read a device slot, on the compute stream: tells the worker (through
// pinned host memory) that the slot may be overwritten
__global__ void feeder_mark_kernel(uint32_t *flag, uint32_t value) { *flag = value; }

// Waits on the worker thread until an event OF THE COPY STREAM has completed, polling.
hipError_t feeder_poll_event(hipEvent_t event) {
  for (;;) {
    const hipError_t e = hipEventQuery(event);
    if (e == hipSuccess) return hipSuccess;
    (void)hipGetLastError();
    if (e != hipErrorNotReady) return e;
    std::this_thread::yield();
  }
}

// one staged batch: pinned copy + upload, all on the worker thread
hipError_t feeder_run_job(tdh_feeder *f, const tdh_feeder::Job &j) {
  const int s = j.slot;
  // the pinned slot is free once its previous upload has left it (three batches ago)
  hipError_t e = feeder_poll_event(f->uploaded[s]);
  if (e != hipSuccess) return e;
  feeder_copy(f, f->pin_x[s], j.x, f->x_len * j.batch * sizeof(float));
  feeder_copy(f, f->pin_t[s], j.t, f->t_len * j.batch * sizeof(float));
  // The device slot is free once every step that reads it has run (the mark that the caller's
  // thread queued behind them before this batch was staged). The worker waits for that here, on the host:
  // a stream-side wait queued on the copy stream would also hold back whatever upload lands
  // behind it, and a batch whose upload waits for the step before it is not overlapped with
  // anything. When the wait ends the upload starts at once.
  while (*const_cast<volatile uint32_t *>(&f->consumed_flag[s]) != j.wait_consumed) std::this_thread::yield();
  e = hipMemcpyAsync(f->dev_x[s], f->pin_x[s], f->x_len * j.batch * sizeof(float), hipMemcpyHostToDevice, f->copy);
  if (e != hipSuccess) return e;
  e = hipMemcpyAsync(f->dev_t[s], f->pin_t[s], f->t_len * j.batch * sizeof(float), hipMemcpyHostToDevice, f->copy);
  if (e != hipSuccess) return e;
  return hipEventRecord(f->uploaded[s], f->copy);
}

void feeder_worker(tdh_feeder *f) {
  (void)hipSetDevice(f->device);
  std::unique_lock<std::mutex> lock(f->mu);
  for (;;) {
    f->cv.wait(lock, [f] { return f->quit || f->jobs_n > 0; });
    if (f->quit) return;
    const tdh_feeder::Job j = f->jobs[0];
    lock.unlock();
    const hipError_t e = feeder_run_job(f, j);
    lock.lock();
    for (int i = 1; i < f->jobs_n; ++i) f->jobs[i - 1] = f->jobs[i];
    --f->jobs_n;
    f->slot_error[j.slot] = e;
    f->slot_done[j.slot]  = true;
    f->cv.notify_all();
  }
}

// waits until the worker has dealt with the batch staged into `slot`; returns its status
hipError_t feeder_wait_slot(tdh_feeder *f, int slot) {
  std::unique_lock<std::mutex> lock(f->mu);
  f->cv.wait(lock, [f, slot] { return f->slot_done[slot]; });
  return f->slot_error[slot];
}

void feeder_wait_idle(tdh_feeder *f) {
  std::unique_lock<std::mutex> lock(f->mu);
  f->cv.wait(lock, [f] { return f->jobs_n == 0; });
}

void feeder_release(tdh_feeder *f) {
  if (f->worker.joinable()) {
    {
      std::lock_guard<std::mutex> lock(f->mu);
      f->quit = true;
    }
    f->cv.notify_all();
    f->worker.join();
  }
  {
    std::lock_guard<std::mutex> lock(f->hmu);
    f->hquit = true;
  }
  f->hcv.notify_all();
  for (std::thread &h : f->helpers)
    if (h.joinable()) h.join();
  for (int s = 0; s < kSlots; ++s) {
    if (f->pin_x[s]) (void)hipHostFree(f->pin_x[s]);
    if (f->pin_t[s]) (void)hipHostFree(f->pin_t[s]);
    if (f->dev_x[s]) (void)hipFree(f->dev_x[s]);
    if (f->dev_t[s]) (void)hipFree(f->dev_t[s]);
    if (f->uploaded[s]) (void)hipEventDestroy(f->uploaded[s]);
  }
  if (f->consumed_flag) (void)hipHostFree(f->consumed_flag);
  if (f->copy) (void)hipStreamDestroy(f->copy);
  delete f;
}
}  // namespace
}  // namespace tdh

using namespace tdh;

extern "C" {

int tdh_feeder_create(size_t x_len, size_t t_len, int max_batch, tdh_feeder **out) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(out && x_len > 0 && t_len > 0 && max_batch > 0, "tdh_feeder_create: bad argument");
  tdh_feeder *f = new tdh_feeder();
  f->x_len = x_len; f->t_len = t_len; f->max_batch = max_batch;
  const size_t xb = x_len * max_batch * sizeof(float), tb = t_len * max_batch * sizeof(float);
  hipError_t e = hipStreamCreateWithFlags(&f->copy, hipStreamNonBlocking);
  if (e == hipSuccess)
    e = hipHostMalloc(reinterpret_cast<void **>(&f->consumed_flag), kSlots * sizeof(uint32_t), hipHostMallocDefault);
  if (e == hipSuccess) std::memset(f->consumed_flag, 0, kSlots * sizeof(uint32_t));
  for (int s = 0; s < kSlots && e == hipSuccess; ++s) {
    if (e == hipSuccess) e = hipHostMalloc(reinterpret_cast<void **>(&f->pin_x[s]), xb, hipHostMallocDefault);
    if (e == hipSuccess) e = hipHostMalloc(reinterpret_cast<void **>(&f->pin_t[s]), tb, hipHostMallocDefault);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&f->dev_x[s]), xb);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&f->dev_t[s]), tb);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&f->uploaded[s], hipEventDisableTiming);
  }
  if (e != hipSuccess) {
    (void)hipGetLastError();
    feeder_release(f);
    return set_error(TDH_ERR_HIP, "tdh_feeder_create: %s", hipGetErrorString(e));
  }
  f->device = ctx().device;
  f->worker = std::thread(feeder_worker, f);
  if (xb >= kSplitBytes)
    for (int i = 0; i < kCopyThreads - 1; ++i) f->helpers[i] = std::thread(feeder_helper, f, i + 1);
  *out = f;
  return TDH_OK;
}

int tdh_feeder_destroy(tdh_feeder *f) {
  TDH_REQUIRE_INIT();
  if (!f) return TDH_OK;
  feeder_wait_idle(f);
  TDH_HIP(hipStreamSynchronize(f->copy));
  TDH_HIP(hipStreamSynchronize(ctx().stream));
  feeder_release(f);
  return TDH_OK;
}

int tdh_feeder_stage(tdh_feeder *f, int batch, const float *x_host, const float *t_host) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(f && x_host && t_host && batch > 0 && batch <= f->max_batch,
                "tdh_feeder_stage: bad argument");
  TDH_CHECK_ARG(f->staged_n < kAhead, "tdh_feeder_stage: %d batches are staged and have not been acquired", kAhead);
  const int s = f->next_slot;
  f->next_slot = (s + 1) % kSlots;
  {
    std::lock_guard<std::mutex> lock(f->mu);
    tdh_feeder::Job &j = f->jobs[f->jobs_n++];
    j.slot = s; j.batch = batch; j.x = x_host; j.t = t_host;
    // the slot's last mark was queued by this thread before this call (the slot was handed out
    // three batches ago and another batch has been acquired since): the worker waits for it
    j.wait_consumed   = f->consumed_seq[s];
    f->slot_done[s]   = false;
    f->slot_error[s]  = hipSuccess;
  }
  f->cv.notify_all();
  f->batch[s] = batch;
  f->staged_slot[f->staged_n++] = s;
  return TDH_OK;
}

int tdh_feeder_acquire(tdh_feeder *f, const float **x_dev, const float **t_dev, int *batch) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(f && x_dev && t_dev, "tdh_feeder_acquire: bad argument");
  TDH_CHECK_ARG(f->staged_n > 0, "tdh_feeder_acquire: nothing has been staged");
  const int s = f->staged_slot[0];
  for (int i = 1; i < f->staged_n; ++i) f->staged_slot[i - 1] = f->staged_slot[i];
  --f->staged_n;
  const hipError_t staged_status = feeder_wait_slot(f, s);  // (its upload has been queued)
  if (staged_status != hipSuccess)
    return set_error(TDH_ERR_HIP, "tdh_feeder_acquire: staging failed: %s", hipGetErrorString(staged_status));
  hipStream_t compute = ctx().stream;
  if (f->current >= 0) {  // everything queued so far may still read the slot handed out before
    const int c = f->current;
    ++f->consumed_seq[c];
    hipLaunchKernelGGL(feeder_mark_kernel, dim3(1), dim3(1), 0, compute, f->consumed_flag + c, f->consumed_seq[c]);
    TDH_HIP(hipGetLastError());
  }
  TDH_HIP(hipStreamWaitEvent(compute, f->uploaded[s], 0));
  *x_dev = f->dev_x[s];
  *t_dev = f->dev_t[s];
  if (batch) *batch = f->batch[s];
  f->current = s;
  return TDH_OK;
}

}  // extern "C"
