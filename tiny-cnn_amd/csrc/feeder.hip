// feeder.hip — double-buffered upload of training batches that live in pageable host memory.
//
// network::fit hands every mini-batch over as host vectors (tiny_dnn/network.h:866-879,
// layer::set_in_data, tiny_dnn/layers/layer.h:230-251). Uploading them synchronously in front
// of each step leaves the GPU idle for the copy and the host idle for the step. The feeder
// owns two slots of pinned host memory and two of device memory: while step k computes from
// slot k%2, the caller's batch k+1 is copied into the other pinned slot and uploaded on a copy
// stream. Events order the two streams in both directions, so no call blocks the host longer
// than it takes to hand the batch over, and a slot is never overwritten while a queued step
// still reads it. The host-side copy into pinned memory runs on a worker thread of the feeder,
// so that it also overlaps the caller's own launch work; every HIP call stays on the caller's
// thread (a stream capture in progress there tolerates no stream work from other threads).
#include <condition_variable>
#include <cstring>
#include <mutex>
#include <string>
#include <thread>

#include "common.h"

struct tdh_feeder {
  size_t x_len = 0, t_len = 0;  // floats per sample
  int max_batch = 0;
  float *pin_x[2] = {nullptr, nullptr}, *pin_t[2] = {nullptr, nullptr};
  float *dev_x[2] = {nullptr, nullptr}, *dev_t[2] = {nullptr, nullptr};
  hipEvent_t uploaded[2] = {nullptr, nullptr};  // on the copy stream: slot holds its batch
  hipEvent_t consumed[2] = {nullptr, nullptr};  // on the compute stream: every step that reads the slot is queued
  bool used[2]   = {false, false};              // consumed[s] has been recorded at least once
  int batch[2]   = {0, 0};
  int staged     = -1;                          // slot filled by the last tdh_feeder_stage, or -1
  int current    = -1;                          // slot handed out by the last tdh_feeder_acquire
  hipStream_t copy = nullptr;
  // worker thread: one job at a time (the batch being staged)
  int device = 0;
  std::thread worker;
  std::mutex mu;
  std::condition_variable cv;
  bool quit = false, job_pending = false, job_done = true;
  int job_slot = 0, job_batch = 0;
  const float *job_x = nullptr, *job_t = nullptr;
  hipError_t job_error = hipSuccess;
};

namespace tdh {
namespace {
// copies the job's batch into its pinned slot (host work only)
hipError_t feeder_run_job(tdh_feeder *f) {
  const int s = f->job_slot, batch = f->job_batch;
  std::memcpy(f->pin_x[s], f->job_x, f->x_len * batch * sizeof(float));
  std::memcpy(f->pin_t[s], f->job_t, f->t_len * batch * sizeof(float));
  return hipSuccess;
}

void feeder_worker(tdh_feeder *f) {
  std::unique_lock<std::mutex> lock(f->mu);
  for (;;) {
    f->cv.wait(lock, [f] { return f->quit || f->job_pending; });
    if (f->quit) return;
    f->job_pending = false;
    lock.unlock();
    const hipError_t e = feeder_run_job(f);
    lock.lock();
    f->job_error = e;
    f->job_done  = true;
    f->cv.notify_all();
  }
}

// waits for the batch being staged; returns its status
hipError_t feeder_wait_job(tdh_feeder *f) {
  std::unique_lock<std::mutex> lock(f->mu);
  f->cv.wait(lock, [f] { return f->job_done; });
  return f->job_error;
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
  for (int s = 0; s < 2; ++s) {
    if (f->pin_x[s]) (void)hipHostFree(f->pin_x[s]);
    if (f->pin_t[s]) (void)hipHostFree(f->pin_t[s]);
    if (f->dev_x[s]) (void)hipFree(f->dev_x[s]);
    if (f->dev_t[s]) (void)hipFree(f->dev_t[s]);
    if (f->uploaded[s]) (void)hipEventDestroy(f->uploaded[s]);
    if (f->consumed[s]) (void)hipEventDestroy(f->consumed[s]);
  }
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
  for (int s = 0; s < 2 && e == hipSuccess; ++s) {
    if (e == hipSuccess) e = hipHostMalloc(reinterpret_cast<void **>(&f->pin_x[s]), xb, hipHostMallocDefault);
    if (e == hipSuccess) e = hipHostMalloc(reinterpret_cast<void **>(&f->pin_t[s]), tb, hipHostMallocDefault);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&f->dev_x[s]), xb);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&f->dev_t[s]), tb);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&f->uploaded[s], hipEventDisableTiming);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&f->consumed[s], hipEventDisableTiming);
  }
  if (e != hipSuccess) {
    (void)hipGetLastError();
    feeder_release(f);
    return set_error(TDH_ERR_HIP, "tdh_feeder_create: %s", hipGetErrorString(e));
  }
  f->device = ctx().device;
  f->worker = std::thread(feeder_worker, f);
  *out = f;
  return TDH_OK;
}

int tdh_feeder_destroy(tdh_feeder *f) {
  TDH_REQUIRE_INIT();
  if (!f) return TDH_OK;
  (void)feeder_wait_job(f);
  TDH_HIP(hipStreamSynchronize(f->copy));
  TDH_HIP(hipStreamSynchronize(ctx().stream));
  feeder_release(f);
  return TDH_OK;
}

int tdh_feeder_stage(tdh_feeder *f, int batch, const float *x_host, const float *t_host) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(f && x_host && t_host && batch > 0 && batch <= f->max_batch,
                "tdh_feeder_stage: bad argument");
  TDH_CHECK_ARG(f->staged < 0, "tdh_feeder_stage: the batch staged before has not been acquired");
  const int s = f->current < 0 ? 0 : 1 - f->current;
  // the pinned slot is free once its previous upload has left it
  TDH_HIP(hipEventSynchronize(f->uploaded[s]));
  {
    std::lock_guard<std::mutex> lock(f->mu);
    f->job_slot = s; f->job_batch = batch; f->job_x = x_host; f->job_t = t_host;
    f->job_error = hipSuccess;
    f->job_done = false;
    f->job_pending = true;
  }
  f->cv.notify_all();
  f->batch[s] = batch;
  f->staged   = s;
  return TDH_OK;
}

int tdh_feeder_acquire(tdh_feeder *f, const float **x_dev, const float **t_dev, int *batch) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(f && x_dev && t_dev, "tdh_feeder_acquire: bad argument");
  TDH_CHECK_ARG(f->staged >= 0, "tdh_feeder_acquire: nothing has been staged");
  const hipError_t staged_status = feeder_wait_job(f);
  if (staged_status != hipSuccess) {
    f->staged = -1;
    return set_error(TDH_ERR_HIP, "tdh_feeder_acquire: staging failed: %s", hipGetErrorString(staged_status));
  }
  hipStream_t compute = ctx().stream;
  if (f->current >= 0) {  // everything queued so far may still read the slot handed out before
    TDH_HIP(hipEventRecord(f->consumed[f->current], compute));
    f->used[f->current] = true;
  }
  const int s = f->staged;
  // the device slot is free once every step that reads it has run; then the upload may start,
  // usually while the step queued last is still running
  if (f->used[s]) TDH_HIP(hipStreamWaitEvent(f->copy, f->consumed[s], 0));
  TDH_HIP(hipMemcpyAsync(f->dev_x[s], f->pin_x[s], f->x_len * f->batch[s] * sizeof(float),
                         hipMemcpyHostToDevice, f->copy));
  TDH_HIP(hipMemcpyAsync(f->dev_t[s], f->pin_t[s], f->t_len * f->batch[s] * sizeof(float),
                         hipMemcpyHostToDevice, f->copy));
  TDH_HIP(hipEventRecord(f->uploaded[s], f->copy));
  TDH_HIP(hipStreamWaitEvent(compute, f->uploaded[s], 0));
  *x_dev = f->dev_x[s];
  *t_dev = f->dev_t[s];
  if (batch) *batch = f->batch[s];
  f->current = s;
  f->staged  = -1;
  return TDH_OK;
}

}  // extern "C"
