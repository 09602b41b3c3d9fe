// sg_app_rr.h -- application-side buffers of the reference, for one GPU:
// P2pRpcTring (src/p2p_rpc_tring.h), P2pRpcAppRr / P2pRpcAppRrPool
// (src/p2p_rpc_app_rr.h) and the arena pool behind them
// (src/p2p_rpc_app_rr_mem_pool.h), with HIP virtual-memory calls where the
// reference uses the CUDA driver API.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <numeric>

#include "sg_tables.h"

// Bump ring over an address range (src/p2p_rpc_tring.h:9-33).
class P2pRpcTring {
  uintptr_t base_addr_range;
  size_t ring_capacity;
  size_t prev_offset;
  uintptr_t prev_addr;

 public:
  P2pRpcTring(void *base_addr, size_t capacity)
      : base_addr_range((uintptr_t)base_addr), ring_capacity(capacity), prev_offset(0),
        prev_addr((uintptr_t)base_addr)
  {
  }

  inline void *get_next(size_t req_size)
  {
    void *ret = (void *)prev_addr;
    prev_offset = (prev_offset + req_size) % ring_capacity;
    prev_addr = base_addr_range + prev_offset;
    return ret;
  }

  size_t offset() const { return prev_offset; }
  size_t capacity() const { return ring_capacity; }
};

// src/p2p_rpc_app_ctx.h:22
enum APP_RR_STATUS { FREE, RX_COMPLETE, WORK_COMPLETE, TX_COMPLETE };

#define SG_HIP_OK(call)                                                                      \
  do {                                                                                       \
    hipError_t e_ = (call);                                                                  \
    if (e_ != hipSuccess) {                                                                  \
      std::printf("%s failed: %s (%s:%d)\n", #call, hipGetErrorString(e_), __FILE__, __LINE__); \
      std::exit(1);                                                                          \
    }                                                                                        \
  } while (0)

// Request and response arenas of pool_size slots each, padded to a common
// multiple of the slot bytes and the allocation granularity and mapped TWICE
// back to back, so that a batch that wraps the ring end is still one
// contiguous address range (src/p2p_rpc_app_rr_mem_pool.h:268-316).  Where the
// device cannot map one allocation twice the arenas are plain allocations and
// mirrored() says so; the copy kernels then split the one run that crosses
// the end.  Slot states live in pinned host memory both sides can see
// (the reference's doorbells, :318-335).
class P2pRpcAppRrMemPool {
  int device_id;
  size_t req_bytes = 0, resp_bytes = 0;
  void *req_va = nullptr, *resp_va = nullptr;
  hipMemGenericAllocationHandle_t req_h{}, resp_h{};
  bool mirrored_ = false;
  volatile uint32_t *states = nullptr;

  static size_t lcm(size_t a, size_t b) { return a / std::gcd(a, b) * b; }

  bool map_twice(size_t bytes, void **va, hipMemGenericAllocationHandle_t *h)
  {
    hipMemAllocationProp prop{};
    prop.type = hipMemAllocationTypePinned;
    prop.location.type = hipMemLocationTypeDevice;
    prop.location.id = device_id;
    if (hipMemCreate(h, bytes, &prop, 0) != hipSuccess) return false;
    if (hipMemAddressReserve(va, 2 * bytes, 0, nullptr, 0) != hipSuccess) {
      (void)hipMemRelease(*h);
      return false;
    }
    hipMemAccessDesc acc{};
    acc.location = prop.location;
    acc.flags = hipMemAccessFlagsProtReadWrite;
    bool ok = hipMemMap(*va, bytes, 0, *h, 0) == hipSuccess;
    ok = ok && hipMemMap((uint8_t *)*va + bytes, bytes, 0, *h, 0) == hipSuccess;
    ok = ok && hipMemSetAccess(*va, 2 * bytes, &acc, 1) == hipSuccess;
    if (!ok) {
      (void)hipMemUnmap(*va, 2 * bytes);
      (void)hipMemAddressFree(*va, 2 * bytes);
      (void)hipMemRelease(*h);
      *va = nullptr;
    }
    return ok;
  }

 public:
  P2pRpcAppRrMemPool(int pool_size, int _device_id, size_t req_size, size_t resp_size, bool want_mirror = true)
      : device_id(_device_id)
  {
    SG_HIP_OK(hipSetDevice(device_id));
    size_t gran = 1 << 21;
    hipMemAllocationProp prop{};
    prop.type = hipMemAllocationTypePinned;
    prop.location.type = hipMemLocationTypeDevice;
    prop.location.id = device_id;
    bool vmm = want_mirror &&
               hipMemGetAllocationGranularity(&gran, &prop, hipMemAllocationGranularityRecommended) == hipSuccess;
    req_bytes = vmm ? lcm(req_size * pool_size, gran) : req_size * pool_size;
    resp_bytes = vmm ? lcm(resp_size * pool_size, gran) : resp_size * pool_size;
    if (vmm && map_twice(req_bytes, &req_va, &req_h)) {
      if (map_twice(resp_bytes, &resp_va, &resp_h)) {
        mirrored_ = true;
      } else {
        (void)hipMemUnmap(req_va, 2 * req_bytes);
        (void)hipMemAddressFree(req_va, 2 * req_bytes);
        (void)hipMemRelease(req_h);
        req_va = nullptr;
      }
    }
    (void)hipGetLastError();
    if (!mirrored_) {
      req_bytes = req_size * pool_size;
      resp_bytes = resp_size * pool_size;
      SG_HIP_OK(hipMalloc(&req_va, req_bytes));
      SG_HIP_OK(hipMalloc(&resp_va, resp_bytes));
    }
    void *st = nullptr;
    SG_HIP_OK(hipHostMalloc(&st, sizeof(uint32_t) * pool_size, hipHostMallocDefault));
    states = static_cast<volatile uint32_t *>(st);
    for (int i = 0; i < pool_size; i++) states[i] = FREE;
  }

  ~P2pRpcAppRrMemPool()
  {
    (void)hipSetDevice(device_id);
    if (mirrored_) {
      (void)hipMemUnmap(req_va, 2 * req_bytes);
      (void)hipMemAddressFree(req_va, 2 * req_bytes);
      (void)hipMemRelease(req_h);
      (void)hipMemUnmap(resp_va, 2 * resp_bytes);
      (void)hipMemAddressFree(resp_va, 2 * resp_bytes);
      (void)hipMemRelease(resp_h);
    } else {
      (void)hipFree(req_va);
      (void)hipFree(resp_va);
    }
    if (states) (void)hipHostFree((void *)states);
  }

  bool mirrored() const { return mirrored_; }
  void *get_req_addr_range() const { return req_va; }
  void *get_resp_addr_range() const { return resp_va; }
  size_t get_req_addr_pool_size() const { return req_bytes; }
  size_t get_resp_addr_pool_size() const { return resp_bytes; }
  volatile uint32_t *get_doorbells_host() const { return states; }
  volatile uint32_t *get_doorbells_device() const { return states; }  // pinned: one address for both
};

// One application slot (src/p2p_rpc_app_rr.h:15-46).
class P2pRpcAppRr {
 public:
  g_params *h_stub = nullptr;
  g_params *d_stub = nullptr;
  volatile uint32_t *h_state = nullptr;
  volatile uint32_t *d_state = nullptr;
  size_t req_size = 0, resp_size = 0;
  void *rpc_rr = nullptr;  // valid in RX_COMPLETE / WORK_COMPLETE
  int rr_idx = 0;

  void print_app_rr_info() const
  {
    std::printf("app_rr: %p, rr_idx: %d, h_stub: %p, req: %p, resp: %p\n", (const void *)this, rr_idx,
                (void *)h_stub, (void *)h_stub->req, (void *)h_stub->resp);
  }
};

// Slot table over the two arenas: get_next() hands out consecutive request and
// response addresses, so the requests of one batch form one tensor
// (src/p2p_rpc_app_rr.h:82-191).
class P2pRpcAppRrPool {
  int pool_size;
  int device_id;
  g_params *h_stubs;
  g_params *d_stubs;
  P2pRpcTring *req_pool, *resp_pool;
  volatile uint32_t *h_states;
  volatile uint32_t *d_states;
  size_t app_rr_pi_idx;

 public:
  size_t req_size, resp_size;
  P2pRpcAppRr *rr_pool;
  P2pRpcAppRrMemPool *rr_mem_pool;

  P2pRpcAppRrPool(int _pool_size, int _device_id, size_t _req_size, size_t _resp_size, bool want_mirror = true)
      : pool_size(_pool_size), device_id(_device_id), app_rr_pi_idx(0), req_size(_req_size),
        resp_size(_resp_size)
  {
    rr_pool = new P2pRpcAppRr[pool_size];
    rr_mem_pool = new P2pRpcAppRrMemPool(pool_size, device_id, req_size, resp_size, want_mirror);
    req_pool = new P2pRpcTring(rr_mem_pool->get_req_addr_range(), rr_mem_pool->get_req_addr_pool_size());
    resp_pool = new P2pRpcTring(rr_mem_pool->get_resp_addr_range(), rr_mem_pool->get_resp_addr_pool_size());
    h_states = rr_mem_pool->get_doorbells_host();
    d_states = rr_mem_pool->get_doorbells_device();
    h_stubs = new g_params[pool_size];
    d_stubs = h_stubs;
    for (int i = 0; i < pool_size; i++) {
      P2pRpcAppRr *a = &rr_pool[i];
      a->req_size = req_size;
      a->resp_size = resp_size;
      a->h_stub = &h_stubs[i];
      a->d_stub = &d_stubs[i];
      a->h_state = &h_states[i];
      a->d_state = &d_states[i];
      *a->h_state = FREE;
      a->rr_idx = i;
      a->h_stub->req = nullptr;
      a->h_stub->resp = nullptr;
    }
  }

  ~P2pRpcAppRrPool()
  {
    delete req_pool;
    delete resp_pool;
    delete rr_mem_pool;
    delete[] rr_pool;
    delete[] h_stubs;
  }

  inline int get_pool_size() const { return pool_size; }
  inline P2pRpcAppRr *get_app_rr_pool() { return rr_pool; }
  inline P2pRpcAppRr *get_app_rr(int idx) { return idx >= 0 && idx < pool_size ? &rr_pool[idx] : nullptr; }
  inline void init_pool() { app_rr_pi_idx = 0; }

  // not thread-safe, as in the reference (:126-134)
  inline P2pRpcAppRr *get_next()
  {
    P2pRpcAppRr *a = &rr_pool[app_rr_pi_idx];
    a->h_stub->req = (uint8_t *)req_pool->get_next(req_size);
    a->h_stub->resp = (uint8_t *)resp_pool->get_next(resp_size);
    app_rr_pi_idx = (app_rr_pi_idx + 1) % pool_size;
    return a;
  }
};

// The worker's view of the slot ring: the window logic of
// dynamic_batching_sync_worker_loop and sync_worker_loop
// (src/p2p_rpc_async_app_server.h:173-206, 220-263) as steps a loop calls.
// collect() extends the window over consecutive RX_COMPLETE slots from the
// consumer index, up to max_batch; the batch's requests are contiguous from
// get_app_rr(start())->h_stub (the model reads curr_batch_size requests from
// there, :213-218).  complete() publishes WORK_COMPLETE for the window and
// moves on.
struct SgBatchWindow {
  int rr_si_idx = 0;  // first slot of the window
  int rr_ci_idx = 0;  // next slot to look at
  int rr_win_size = 0;

  inline int collect(P2pRpcAppRrPool *pool, int max_batch)
  {
    const int n = pool->get_pool_size();
    while (rr_win_size < max_batch && rr_win_size < n &&
           *pool->get_app_rr(rr_ci_idx)->h_state == RX_COMPLETE) {
      rr_win_size++;
      rr_ci_idx = (rr_ci_idx + 1) % n;
    }
    return rr_win_size;
  }
  inline int start() const { return rr_si_idx; }
  inline void complete(P2pRpcAppRrPool *pool)
  {
    const int n = pool->get_pool_size();
    int i = rr_si_idx;
    for (int k = 0; k < rr_win_size; k++, i = (i + 1) % n) *pool->get_app_rr(i)->h_state = WORK_COMPLETE;
    rr_si_idx = rr_ci_idx;
    rr_win_size = 0;
  }
};

