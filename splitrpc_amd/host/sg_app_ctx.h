// sg_app_ctx.h -- the execution contexts and small-object pool of the reference
// for one HIP device: MetaAppCtx<T> / AppCtx / CopyCtx and the application
// callback types (src/p2p_rpc_app_ctx.h:24-112), g_copy_params and the
// sg_on_gpu C entry points (src/transport/g_copy_ng.cuh:21-37), BufItemPool<T>
// (src/p2p_buf_pool.h:12-78).  Same names and members, so code written against
// the reference's headers compiles.  The doorbell of a context is a word in
// pinned host memory.  Where the reference makes the stream wait on such a word
// or write it (cuStreamWaitValue32 / cuStreamWriteValue32,
// src/utils/g_utils.cu:42-53), the waiting is done by the calling host thread
// before it queues anything further, and the writing by a host function queued
// on the stream: no kernel and no stream ever spins on memory.
#pragma once

#include <hip/hip_runtime.h>

#include <chrono>
#include <climits>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <unordered_map>

#include "sg_hip.h"
#include "sg_tables.h"

template <class T>
class MetaAppCtx {
 public:
  MetaAppCtx() : curr_batch_size(1), next_batch_size(1) {}

  // Work queued after this call runs once *d_state == value (src/p2p_rpc_app_ctx.h:35-37).  The
  // reference queues a wait on the stream and returns; here the CALLING THREAD waits for the word
  // (it lives in pinned host memory) and only then goes on queueing.  So the word has to be set by
  // somebody else -- another thread, or work that is already queued: a thread that calls this and
  // means to set the word itself afterwards, as it may with the reference's queued wait, would wait
  // for itself.  The wait is therefore bounded: after notify_timeout_ns (default 2 s; 0 = no
  // bound) it gives up, reports, and returns false; notify_timeouts counts such returns.
  inline bool AppRrRunNotify(volatile uint32_t *d_state, int value)
  {
    if (*d_state == (uint32_t)value) return true;
    const auto t0 = std::chrono::steady_clock::now();
    for (uint32_t spins = 0;; spins++) {
      if (*d_state == (uint32_t)value) return true;
      __builtin_ia32_pause();
      if ((spins & 1023u) == 1023u && notify_timeout_ns) {
        const auto waited = std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now() - t0).count();
        if ((uint64_t)waited > notify_timeout_ns) {
          notify_timeouts++;
          std::printf("MetaAppCtx: waited %llu ns for a state word to become %d (it holds %u): giving up\n",
                      (unsigned long long)waited, value, *d_state);
          return false;
        }
      }
    }
  }
  // the same on this context's doorbell (:40-42)
  inline bool AppRunNotify(int value) { return AppRrRunNotify(d_door_bell, value); }
  // the same without waiting: true when the word holds the value now
  inline bool AppRrRunReady(volatile uint32_t *d_state, int value) const { return *d_state == (uint32_t)value; }
  uint64_t notify_timeout_ns = 2000000000ull;
  uint64_t notify_timeouts = 0;
  // the doorbell is set once what was queued before is done (:45-47)
  inline void AppCompleteNotify(uint32_t value = 2)
  {
    // the value travels with the queued call (a later notification must not change what this one writes)
    Ring *r = new Ring{door_bell, value};
    if (hipLaunchHostFunc(work_stream, &MetaAppCtx::ring_door_bell, r) != hipSuccess) delete r;
  }
  inline void NotifyAppRunStart()
  {
    *(volatile uint32_t *)door_bell = (uint32_t)curr_batch_size;
    __sync_synchronize();
  }
  inline bool IsAppRunComplete() { return *(volatile uint32_t *)door_bell == 1; }
  inline void ResetAppRunStatus()
  {
    *(volatile uint32_t *)door_bell = UINT_MAX;
    __sync_synchronize();
  }
  // No launch type spins here: waiting is waiting for the stream (:62-70).
  inline void WaitForAppRunComplete() { (void)hipStreamSynchronize(work_stream); }

  // what the application is told
  T *h_stub = nullptr;
  T *d_stub = nullptr;
  // doorbell (pinned host memory: one address for both sides)
  uint32_t *door_bell = nullptr;
  uint32_t *d_door_bell = nullptr;
  void *app_ctx_internal = nullptr;  // whatever the owner wants to keep (the copy engine keeps its sg_hip_ctx here)
  int curr_batch_size;
  int next_batch_size;
  hipStream_t work_stream = nullptr;
  hipEvent_t work_complete = nullptr;
  void *curr_rr = nullptr;
  uint8_t launch_type = 1;  // 1 = kernel launch per call; the persistent-kernel types of the reference do not exist here
  int device_id = 0;
  bool graphCreated = false;
  hipGraph_t graph = nullptr;
  hipGraphExec_t instance = nullptr;

 private:
  struct Ring {
    uint32_t *bell;
    uint32_t value;
  };
  static void ring_door_bell(void *ring)
  {
    Ring *r = static_cast<Ring *>(ring);
    *(volatile uint32_t *)r->bell = r->value;
    delete r;
  }
};

typedef MetaAppCtx<g_params> AppCtx;
using AppInitCB = int (*)(AppCtx *);
using AppRunCB = int (*)(AppCtx *);
using AppCleanupCB = int (*)(AppCtx *);
using AppRunAsyncCB = int (*)(AppCtx *);
using AppRunWaitCB = int (*)(AppCtx *);
using AppCompleteCB = int (*)(AppCtx *);

// src/transport/g_copy_ng.cuh:25-26
typedef p2p_sk_buf g_copy_params;
typedef MetaAppCtx<g_copy_params> CopyCtx;

// Bring a copy context up: the reference starts its persistent kernel here
// (src/transport/g_copy_ng.cu:169-184); this creates the engine context on the
// context's device and stream.  Returns 1 on success, 0 on failure, as there.
static inline int sg_on_gpu_entry(CopyCtx *ctx)
{
  if (!ctx) return 0;
  sg_hip_cfg cfg{sizeof(sg_hip_cfg), 0, 0, 0, ctx->work_stream};
  sg_hip_ctx *c = sg_hip_create(ctx->device_id, &cfg);
  if (!c) {
    std::printf("sg_on_gpu_entry: %s\n", sg_hip_last_error(nullptr));
    return 0;
  }
  ctx->app_ctx_internal = c;
  if (!ctx->work_stream) ctx->work_stream = static_cast<hipStream_t>(sg_hip_stream(c));
  return 1;
}

// Copy every run of a run table (src/transport/g_copy_ng.cu:186-223): 1 / 0.
static inline int sg_on_gpu(CopyCtx *ctx, p2p_sk_buf *skb)
{
  if (!ctx || !ctx->app_ctx_internal) return 0;
  return sg_hip_gather(static_cast<sg_hip_ctx *>(ctx->app_ctx_internal), reinterpret_cast<const sg_sk_buf *>(skb)) == SG_OK;
}

static inline void sg_on_gpu_exit(CopyCtx *ctx)
{
  if (ctx && ctx->app_ctx_internal) sg_hip_destroy(static_cast<sg_hip_ctx *>(ctx->app_ctx_internal));
  if (ctx) ctx->app_ctx_internal = nullptr;
}

// Small objects both sides can reach (src/p2p_buf_pool.h:12-78).  The reference
// maps GPU memory into the host with GDRCopy; here type >= 0 gives pinned host
// memory mapped into device `type`'s address space, type < 0 plain host memory.
// Not thread safe, and not a pool, as the reference says of its own.
template <class T>
class BufItemPool {
  static std::unordered_map<T *, T *> &info()
  {
    static std::unordered_map<T *, T *> m;  // host pointer -> device pointer (nullptr: host only)
    return m;
  }

 public:
  static T *create_buf_item_pool(int num, int type = -1)
  {
    T *h = nullptr, *d = nullptr;
    if (type >= 0) {
      int prev = -1;
      (void)hipGetDevice(&prev);
      if (hipSetDevice(type) != hipSuccess ||
          hipHostMalloc((void **)&h, sizeof(T) * (size_t)num, hipHostMallocMapped) != hipSuccess ||
          hipHostGetDevicePointer((void **)&d, h, 0) != hipSuccess) {
        std::printf("BufItemPool: no pinned memory for %d items on device %d\n", num, type);
        if (h) (void)hipHostFree(h);
        if (prev >= 0) (void)hipSetDevice(prev);
        return nullptr;
      }
      if (prev >= 0) (void)hipSetDevice(prev);
    } else {
      h = static_cast<T *>(std::malloc(sizeof(T) * (size_t)num));
      if (!h) return nullptr;
    }
    info()[h] = d;
    std::memset(h, 0, sizeof(T) * (size_t)num);
    return h;
  }

  static void delete_buf_item_pool(T *h, int /*type*/ = -1)
  {
    auto it = info().find(h);
    if (it == info().end()) return;
    if (it->second) (void)hipHostFree(h);
    else std::free(h);
    info().erase(it);
  }

  static T *get_dev_ptr(T *h)
  {
    auto it = info().find(h);
    if (it == info().end()) return nullptr;
    if (it->second) return it->second;
    std::printf("Warning! BufItem does not have a dev mapping\n");
    return h;
  }
};
