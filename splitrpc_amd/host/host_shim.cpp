// host_shim.cpp -- C entry points over the C++ host layer, for the tests and
// for callers that cannot include C++ headers.  Built into libsg_host.so next
// to libsg_hip.so.  Functions whose name ends in _gpu touch the device; the
// others are pure host logic.
#include <hip/hip_runtime.h>

#include <chrono>
#include <cstring>
#include <thread>
#include <vector>

#include "sg_app_ctx.h"
#include "sg_app_rr.h"
#include "sg_engine.h"
#include "sg_rr.h"
#include "sg_tables.h"
#include "sg_wire.h"

extern "C" {

// Layout facts, numbered like the reference probe's table (tests compare the two).
uint64_t sgh_layout(int what)
{
  switch (what) {
    case 0: return sizeof(p2p_hbufs);
    case 1: return sizeof(p2p_bufs);
    case 2: return sizeof(p2p_sk_buf);
    case 3: return sizeof(g_params);
    case 4: return sizeof(g_params_v2);
    case 5: return sizeof(eth_hdr);
    case 6: return sizeof(ipv4_hdr);
    case 7: return sizeof(udp_hdr);
    case 8: return UDP_HEADER_LEN;
    case 9: return MAX_BI_SIZE;
    case 10: return offsetof(p2p_hbufs, num_items);
    case 11: return offsetof(p2p_bufs, item_size);
    case 12: return offsetof(p2p_bufs, num_items);
    case 13: return offsetof(p2p_sk_buf, o_buf);
    case 14: return offsetof(p2p_sk_buf, len);
    case 15: return offsetof(p2p_sk_buf, num_items);
    case 16: return offsetof(g_params, resp);
    case 17: return offsetof(g_params_v2, outputs);
    case 18: return offsetof(g_params_v2, input_tensor_size);
    case 19: return offsetof(g_params_v2, output_tensor_size);
    case 20: return offsetof(ipv4_hdr, tot_len);
    case 21: return offsetof(ipv4_hdr, check);
    case 22: return offsetof(ipv4_hdr, src_ip);
    case 23: return offsetof(ipv4_hdr, dst_ip);
    case 24: return offsetof(udp_hdr, len);
    case 25: return offsetof(udp_hdr, check);
    case 26: return offsetof(ipv4_hdr, protocol);
    case 27: return sizeof(p2p_rpc_hdr);
    case 28: return offsetof(p2p_rpc_hdr, req_token);
    case 29: return offsetof(p2p_rpc_hdr, sock_perf_header);
    case 30: return offsetof(p2p_rpc_hdr, seq_num);
    default: return ~0ull;
  }
}

// gather_skbs / scatter_skbs on a caller-supplied fragment table.
uint64_t sgh_skbs(int scatter, const uint64_t *ptrs, const uint64_t *sizes, uint32_t n, uint64_t app_buf,
                  uint64_t *i_out, uint64_t *o_out, uint64_t *len_out)
{
  p2p_bufs *b = new p2p_bufs;
  p2p_sk_buf *s = new p2p_sk_buf;
  for (uint32_t i = 0; i < n && i < MAX_BI_SIZE; i++) {
    b->burst_items[i] = ptrs[i];
    b->item_size[i] = sizes[i];
  }
  if (n == 0) {  // entry 0 is read even then
    b->burst_items[0] = ptrs[0];
    b->item_size[0] = sizes[0];
  }
  b->num_items = (uint16_t)n;
  if (scatter) scatter_skbs(s, b, (uint8_t *)app_buf);
  else gather_skbs(s, b, (uint8_t *)app_buf);
  const uint64_t k = s->num_items;
  for (uint64_t i = 0; i < k; i++) {
    i_out[i] = s->i_buf[i];
    o_out[i] = s->o_buf[i];
    len_out[i] = s->len[i];
  }
  delete b;
  delete s;
  return k;
}

void sgh_tring_replay(uint64_t base, uint64_t capacity, const uint64_t *sizes, uint32_t n, uint64_t *out)
{
  P2pRpcTring t((void *)base, capacity);
  for (uint32_t i = 0; i < n; i++) out[i] = (uint64_t)(uintptr_t)t.get_next(sizes[i]);
}

// Feed `n` ring slots, in arrival order, through P2pRpcRRPool::append_to_rr the
// way the receive loop does (src/transport/dpdk_transport_ng.h:221-252), then
// drain the rx-ready ring and emit the completed requests' tables.  `ring` is a
// host image of the packet ring; payload pointers are formed on `dev_base`
// (only their arithmetic matters here).  Returns completed requests or -1.
int64_t sgh_pool_replay(const uint8_t *ring, uint32_t n_slots, uint32_t slot_size, uint32_t profile,
                        uint64_t dev_base, const uint32_t *arrivals, uint32_t n, const uint32_t *len_nic,
                        uint64_t req_size, int pool_size, uint32_t *frag_slot_out, uint32_t *frag_len_out,
                        uint32_t *req_first_out, uint64_t *req_token_out, uint64_t *leftover_out)
{
  const uint32_t hl = rpc_header_len(profile);
  P2pRpcRRPool pool(pool_size, profile);
  p2p_rpc_conn_info *srv = initialize_src_conn_info("b8:ce:f6:cc:6a:52,192.168.25.1,50051");
  pool.setup_and_init_rr_pool(srv, req_size);
  release_conn_info(srv);
  SgRingView view{sg_ring_desc{(void *)dev_base, n_slots, slot_size, profile, 0}};
  for (uint32_t a = 0; a < n; a++) {
    const uint32_t s = arrivals[a];
    if (s >= n_slots) return -1;
    uint8_t hdr[64];
    std::memcpy(hdr, ring + (size_t)s * slot_size, sizeof hdr);
    p2p_rpc_hdr *h = reinterpret_cast<p2p_rpc_hdr *>(hdr);
    if (h->req_token == 0) continue;  // dropped, as the reference does (:231,247)
    const size_t len = len_nic ? len_nic[s] : reinterpret_cast<bl58_rpc_hdr *>(hdr)->payload_len;
    const uintptr_t slot_addr = (uintptr_t)dev_base + (uintptr_t)s * slot_size;
    pool.append_to_rr(h, slot_addr, slot_addr, slot_addr + hl, len);
  }
  int64_t done = 0;
  uint32_t f = 0;
  req_first_out[0] = 0;
  P2pRpcRr *rr;
  while (pool.get_next_rx_ready_rr(&rr)) {
    req_token_out[done] = rr->req_token;
    for (int i = 0; i < rr->payload_bufs->num_items; i++, f++) {
      const int64_t s = view.slot_of_payload(rr->payload_bufs->burst_items[i]);
      if (s < 0) return -1;
      frag_slot_out[f] = (uint32_t)s;
      frag_len_out[f] = (uint32_t)rr->payload_bufs->item_size[i];
    }
    done++;
    req_first_out[done] = f;
    pool.reap_rr(rr);
  }
  if (leftover_out) *leftover_out = pool.in_flight();
  return done;
}

// Pool exhaustion: more concurrent requests than rrs grows the pool, as the
// reference does.  Returns the container size afterwards.
uint64_t sgh_pool_exhaust(int pool_size, uint32_t n_tokens)
{
  P2pRpcRRPool pool(pool_size, SG_HDR_REF64);
  p2p_rpc_conn_info *srv = initialize_src_conn_info("b8:ce:f6:cc:6a:52,192.168.25.1,50051");
  pool.setup_and_init_rr_pool(srv, 1 << 20);
  release_conn_info(srv);
  p2p_rpc_hdr h;
  std::memset(&h, 0, sizeof h);
  for (uint32_t t = 1; t <= n_tokens; t++) {
    h.req_token = t;
    h.seq_num = 0;
    pool.append_to_rr(&h, 0, 0, 0x1000, 16);
  }
  return pool.get_rr_pool_container().size();
}

// Several producers and consumers hammer one SgPtrRing; returns 1 when every
// value came out exactly once.
int sgh_ring_stress(uint32_t n_threads, uint32_t per_thread, uint32_t capacity)
{
  SgPtrRing ring(capacity);
  std::vector<std::atomic<uint32_t>> seen(n_threads * per_thread);
  for (auto &s : seen) s.store(0);
  std::atomic<uint32_t> consumed{0};
  const uint32_t total = n_threads * per_thread;
  std::vector<std::thread> th;
  for (uint32_t t = 0; t < n_threads; t++) {
    th.emplace_back([&, t] {
      for (uint32_t i = 0; i < per_thread; i++) {
        void *p = (void *)(uintptr_t)(t * per_thread + i + 1);
        while (ring.enqueue(p) != 0) std::this_thread::yield();
      }
    });
    th.emplace_back([&] {
      while (consumed.load() < total) {
        void *p;
        if (ring.dequeue(&p) == 0) {
          seen[(uintptr_t)p - 1].fetch_add(1);
          consumed.fetch_add(1);
        } else {
          std::this_thread::yield();
        }
      }
    });
  }
  for (auto &x : th) x.join();
  for (auto &s : seen)
    if (s.load() != 1) return 0;
  void *p;
  return ring.dequeue(&p) == -ENOENT ? 1 : 0;
}

// The shunter's work for one burst (src/splitrpc_server/p2p_rpc_dpdk_server.cc:
// 117-189) on one GPU: file the arrivals under their requests, take a slot of
// the application ring per ready request, gather, and -- for the responses the
// caller describes -- set up the response buffers, rewrite their headers and
// scatter.  per_request == 1 uses the reference's one-request calls; 0 the
// batched gather with per-request TX; 2 the batched gather and the batched TX
// (headers from the connections' templates, written by the scatter kernel),
// with the application slots' state words published by the device and walked
// by the worker's batching window on the host; 3 the same with the requests'
// fragment tables kept where the device reads them, so that the batched calls
// walk no fragment on the host (the form large calls take, forced here); 4 is 2
// with the walked tables copied to the device instead of read in place.  The request arena
// (n_done * req_size bytes) and the TX ring are copied back for inspection.
// Fixed-size requests (req_size) as in the reference.  Returns completed
// requests or a negative error.
int64_t sgh_serve_gpu(int device_id, const uint8_t *ring_host, uint32_t n_slots, uint32_t slot_size,
                      uint32_t profile, const uint32_t *arrivals, uint32_t n_arr, const uint32_t *len_nic,
                      uint64_t req_size, uint64_t resp_size, uint32_t mtu, uint32_t flags, int per_request,
                      int want_mirror, const uint8_t *resp_host, uint8_t *tx_ring_host, uint32_t tx_n_slots,
                      const uint32_t *tx_slot, const uint32_t *hdr_src_slot, uint8_t *req_out,
                      int *mirrored_out)
{
  if (hipSetDevice(device_id) != hipSuccess) return -1;
  const uint32_t hl = rpc_header_len(profile);
  const size_t ring_bytes = (size_t)n_slots * slot_size, tx_bytes = (size_t)tx_n_slots * slot_size;
  uint8_t *d_ring = nullptr, *d_tx = nullptr;
  if (hipMalloc(&d_ring, ring_bytes) != hipSuccess || hipMalloc(&d_tx, tx_bytes) != hipSuccess) return -2;
  (void)hipMemcpy(d_ring, ring_host, ring_bytes, hipMemcpyHostToDevice);
  (void)hipMemcpy(d_tx, tx_ring_host, tx_bytes, hipMemcpyHostToDevice);

  int64_t done = 0;
  bool tables_pulled = false;
  {
    P2pRpcRRPool pool(-1, profile);
    p2p_rpc_conn_info *srv = initialize_src_conn_info("b8:ce:f6:cc:6a:52,192.168.25.1,50051");
    pool.setup_and_init_rr_pool(srv, req_size);
    release_conn_info(srv);
    P2pRpcSgHipEngine engine(device_id);
    if (per_request == 4) {
      // the tables the thread walks brought over by a kernel, as calls too large to be read in place are
      engine.in_place_max_bytes = 0;
      per_request = 2;
    }
    if (per_request == 3) {
      // the requests' fragment tables where the device reads them: written below as fragments are
      // filed, pulled by the batched calls
      sg_frag_table *t = engine.frag_tables((uint32_t)pool.get_pool_size());
      if (!t) return -18;
      pool.attach_frag_tables(t, (size_t)pool.get_pool_size(), (uintptr_t)d_ring & ~(uintptr_t)1);
      engine.pull_min_items = 0;  // every call of this (small) run pulls its tables
      tables_pulled = true;
      per_request = 2;
    }
    for (uint32_t a = 0; a < n_arr; a++) {
      const uint32_t s = arrivals[a];
      uint8_t hdr[64];
      std::memcpy(hdr, ring_host + (size_t)s * slot_size, sizeof hdr);
      p2p_rpc_hdr *h = reinterpret_cast<p2p_rpc_hdr *>(hdr);
      if (h->req_token == 0) continue;
      const size_t len = len_nic ? len_nic[s] : reinterpret_cast<bl58_rpc_hdr *>(hdr)->payload_len;
      const uintptr_t slot_addr = (uintptr_t)d_ring + (uintptr_t)s * slot_size;
      pool.append_to_rr(h, slot_addr, slot_addr, slot_addr + hl, len);
    }
    std::vector<P2pRpcRr *> ready;
    P2pRpcRr *rr;
    while (pool.get_next_rx_ready_rr(&rr)) ready.push_back(rr);
    done = (int64_t)ready.size();
    const int n_app = (int)ready.size() + 3;  // the application ring wraps after a few slots
    P2pRpcAppRrPool app_pool(n_app, device_id, req_size, resp_size, want_mirror != 0);
    if (mirrored_out) *mirrored_out = app_pool.rr_mem_pool->mirrored() ? 1 : 0;
    std::vector<P2pRpcAppRr *> slots;
    for (size_t k = 0; k < ready.size(); k++) slots.push_back(app_pool.get_next());

    // ---- RX half: gather ----
    if (per_request) {
      for (size_t k = 0; k < ready.size(); k++) {
        engine.gather(ready[k], slots[k]->h_stub);
        if (engine.last_rc != SG_OK) return -10;
        *slots[k]->h_state = RX_COMPLETE;
      }
    } else if (!ready.empty()) {
      SgRingView view{sg_ring_desc{d_ring, n_slots, slot_size, profile, 0}};
      sg_app_desc app;
      std::memset(&app, 0, sizeof app);
      app.arena = app_pool.rr_mem_pool->get_req_addr_range();
      app.arena_cap = app_pool.rr_mem_pool->get_req_addr_pool_size();
      app.arena_mirrored = app_pool.rr_mem_pool->mirrored();
      uint32_t *states = per_request == 2 ? (uint32_t *)app_pool.rr_mem_pool->get_doorbells_device() : nullptr;
      if (engine.gather_batch(ready.data(), (uint32_t)ready.size(), view, app, nullptr, req_size,
                              len_nic ? 0 : mtu, 0, states, states ? (uint32_t)n_app : 0) != SG_OK)
        return -11;
      if (states) {
        // RX_COMPLETE was published by the device, behind the copy
        for (auto *s : slots)
          if (*s->h_state != RX_COMPLETE) return -14;
      } else {
        for (auto *s : slots) *s->h_state = RX_COMPLETE;
      }
    }
    for (size_t k = 0; k < ready.size(); k++)
      (void)hipMemcpy(req_out + k * req_size, slots[k]->h_stub->req, req_size, hipMemcpyDeviceToHost);

    // ---- the model: responses land in the slots' resp buffers ----
    for (size_t k = 0; k < ready.size(); k++)
      (void)hipMemcpy(slots[k]->h_stub->resp, resp_host + k * resp_size, resp_size, hipMemcpyHostToDevice);
    if (per_request == 2) {
      // the worker's window over the very words the device wrote
      SgBatchWindow win;
      if (win.collect(&app_pool, (int)ready.size()) != (int)ready.size()) return -15;
      win.complete(&app_pool);
    } else {
      for (size_t k = 0; k < ready.size(); k++) *slots[k]->h_state = WORK_COMPLETE;
    }

    // ---- TX half: response buffers, headers, scatter ----
    const uint32_t per = (uint32_t)((resp_size + mtu - 1) / mtu);
    if (per_request == 2) {
      for (size_t k = 0; k < ready.size(); k++) {
        // rr_alloc_mbufs: fresh response buffers take the place of the request's
        P2pRpcRr *r = ready[k];
        r->transport_mbufs->num_items = r->hdr_bufs->num_items = r->payload_bufs->num_items = 0;
        r->payload_size = 0;
        // the response buffers lie in another allocation than the request's: its table counts from there now
        if (tables_pulled) r->pkt_base = (uintptr_t)d_tx & ~(uintptr_t)1;
        size_t rem = resp_size;
        for (uint32_t i = 0; i < per; i++) {
          uint8_t *slot = d_tx + (size_t)tx_slot[(uint32_t)k * per + i] * slot_size;
          const size_t cur = rem <= mtu ? rem : mtu;
          rem -= cur;
          r->rr_append_mbuf((uintptr_t)slot, (uintptr_t)slot, (uintptr_t)(slot + hl), cur);
        }
      }
      SgRingView txv{sg_ring_desc{d_tx, tx_n_slots, slot_size, profile, 0}};
      sg_app_desc rapp;
      std::memset(&rapp, 0, sizeof rapp);
      rapp.arena = app_pool.rr_mem_pool->get_resp_addr_range();
      rapp.arena_cap = app_pool.rr_mem_pool->get_resp_addr_pool_size();
      rapp.arena_mirrored = app_pool.rr_mem_pool->mirrored();
      uint32_t *states = (uint32_t *)app_pool.rr_mem_pool->get_doorbells_device();
      if (!ready.empty() &&
          engine.scatter_batch(ready.data(), (uint32_t)ready.size(), txv, rapp, mtu, flags, states, (uint32_t)n_app) != SG_OK)
        return -16;
      for (auto *s : slots)
        if (*s->h_state != FREE) return -17;  // freed by the device, behind the copy
      for (auto *r : ready) pool.reap_rr(r);
    }
    for (size_t k = 0; per_request != 2 && k < ready.size(); k++) {
      P2pRpcRr *r = ready[k];
      r->transport_mbufs->num_items = r->hdr_bufs->num_items = r->payload_bufs->num_items = 0;
      r->payload_size = 0;
      size_t rem = resp_size;
      for (uint32_t i = 0; i < per; i++) {
        const uint32_t f = (uint32_t)k * per + i;
        uint8_t *slot = d_tx + (size_t)tx_slot[f] * slot_size;
        // the response buffer starts out holding the request header it answers
        (void)hipMemcpy(slot, d_ring + (size_t)hdr_src_slot[f] * slot_size, hl, hipMemcpyDeviceToDevice);
        const size_t cur = rem <= mtu ? rem : mtu;
        rem -= cur;
        r->rr_append_mbuf((uintptr_t)slot, (uintptr_t)slot, (uintptr_t)(slot + hl), cur);
      }
      // device-to-device copies do not make the host wait: the engine's stream does not know of them
      (void)hipStreamSynchronize(nullptr);
      engine.swap_hdrs(r, profile, resp_size, mtu, flags & ~SG_F_UDP_CSUM_FULL);
      if (engine.last_rc != SG_OK) return -12;
      engine.scatter(r, slots[k]->h_stub);
      if (engine.last_rc != SG_OK) return -13;
      *slots[k]->h_state = FREE;
      pool.reap_rr(r);
    }
    (void)hipMemcpy(tx_ring_host, d_tx, tx_bytes, hipMemcpyDeviceToHost);
  }
  (void)hipFree(d_ring);
  (void)hipFree(d_tx);
  return done;
}

// Replays the worker's batching window over a slot ring.  ops[k] > 0: the
// shunter publishes ops[k] more requests (get_next + RX_COMPLETE, a slot is
// reused once the transmit side has set it FREE); ops[k] < 0: the worker
// collects a window of at most -ops[k] slots, "runs" it and completes it, and
// the transmit side frees those slots.  out gets (start, size) per collect.
// Returns the number of windows, or negative on error.
int64_t sgh_window_replay(int device_id, int pool_size, const int32_t *ops, uint32_t n_ops, int32_t *out)
{
  if (hipSetDevice(device_id) != hipSuccess) return -1;
  P2pRpcAppRrPool pool(pool_size, device_id, 64, 64, false);
  SgBatchWindow win;
  int64_t n_win = 0;
  for (uint32_t k = 0; k < n_ops; k++) {
    if (ops[k] > 0) {
      for (int i = 0; i < ops[k]; i++) {
        P2pRpcAppRr *a = pool.get_next();
        if (*a->h_state != FREE) return -2;  // the caller overran the ring
        *a->h_state = RX_COMPLETE;
      }
    } else {
      const int got = win.collect(&pool, -ops[k]);
      out[2 * n_win] = win.start();
      out[2 * n_win + 1] = got;
      n_win++;
      const int s0 = win.start();
      win.complete(&pool);
      for (int i = 0, s = s0; i < got; i++, s = (s + 1) % pool_size) {
        if (*pool.get_app_rr(s)->h_state != WORK_COMPLETE) return -3;
        *pool.get_app_rr(s)->h_state = FREE;
      }
    }
  }
  return n_win;
}

// P2pRpcSgZcEngine (src/p2p_rpc_sg_engine.h:109-134): gather hands out the
// first payload pointer as request and response buffer, scatter does nothing.
// Returns 1 when it behaves so.
int sgh_zc_engine(uint64_t payload_ptr)
{
  P2pRpcSgEngine *e = new P2pRpcSgZcEngine();
  P2pRpcRr rr;
  rr.rr_append_mbuf(payload_ptr - 64, payload_ptr - 64, payload_ptr, 1024);
  g_params stub{nullptr, nullptr};
  e->gather(&rr, &stub);
  const bool ok = (uint64_t)(uintptr_t)stub.req == payload_ptr && (uint64_t)(uintptr_t)stub.resp == payload_ptr;
  g_params before = stub;
  e->scatter(&rr, &stub);
  e->gather(&rr, (uint8_t *)nullptr);
  e->scatter(&rr, (uint8_t *)nullptr);
  const bool same = stub.req == before.req && stub.resp == before.resp && e->num_instances == 1;
  delete e;
  return ok && same ? 1 : 0;
}

// The reference's copy context and its C entry points (CopyCtx,
// sg_on_gpu_entry, sg_on_gpu; src/transport/g_copy_ng.cuh:21-37) moving one
// run on the device, its doorbell in a BufItemPool object
// (src/p2p_buf_pool.h:12-78).  Returns a bit per step that went as it should.
int sgh_copy_ctx_gpu(int device_id, uint64_t src, uint64_t dst, uint64_t len)
{
  if (hipSetDevice(device_id) != hipSuccess) return -1;
  int ok = 0;
  CopyCtx c;
  c.device_id = device_id;
  c.door_bell = BufItemPool<uint32_t>::create_buf_item_pool(1, device_id);
  if (!c.door_bell) return -2;
  c.d_door_bell = BufItemPool<uint32_t>::get_dev_ptr(c.door_bell);
  if (c.d_door_bell) ok |= 1;
  g_copy_params *skb = BufItemPool<g_copy_params>::create_buf_item_pool(1);  // host memory
  if (BufItemPool<g_copy_params>::get_dev_ptr(skb) == skb) ok |= 2;          // "no dev mapping": the host pointer
  if (sg_on_gpu_entry(&c) == 1) ok |= 4;
  skb->i_buf[0] = src;
  skb->o_buf[0] = dst;
  skb->len[0] = len;
  skb->num_items = 1;
  if (sg_on_gpu(&c, skb) == 1) ok |= 8;
  c.ResetAppRunStatus();
  if (!c.IsAppRunComplete()) ok |= 16;
  c.AppCompleteNotify(1);
  c.WaitForAppRunComplete();
  if (c.IsAppRunComplete()) ok |= 32;
  c.AppRunNotify(1);  // the doorbell holds 1 already: returns at once
  sg_on_gpu_exit(&c);
  BufItemPool<g_copy_params>::delete_buf_item_pool(skb);
  BufItemPool<uint32_t>::delete_buf_item_pool(c.door_bell, device_id);
  if (BufItemPool<uint32_t>::get_dev_ptr(c.door_bell) == nullptr) ok |= 64;
  return ok;
}

// MetaAppCtx::AppRrRunNotify with the word set by ANOTHER thread `delay_us` later, against a bound
// of `timeout_ns`.  Bit 0: the wait saw the value; bit 1: it gave up (and counted the timeout).
int sgh_notify_wait(uint32_t delay_us, uint64_t timeout_ns)
{
  AppCtx c;
  c.notify_timeout_ns = timeout_ns;
  volatile uint32_t word = 0;
  std::thread setter([&] {
    std::this_thread::sleep_for(std::chrono::microseconds(delay_us));
    word = RX_COMPLETE;
  });
  const bool seen = c.AppRrRunNotify(&word, RX_COMPLETE);
  setter.join();
  return (seen ? 1 : 0) | (c.notify_timeouts ? 2 : 0) | (c.AppRrRunReady(&word, RX_COMPLETE) ? 4 : 0);
}

// A double-mapped arena for callers outside C++ (the tests): the request
// range of a P2pRpcAppRrMemPool.  Returns a handle, or NULL.
void *sgh_mempool_create(int device_id, int n, uint64_t req_size, uint64_t resp_size, int want_mirror)
{
  if (hipSetDevice(device_id) != hipSuccess) return nullptr;
  try {
    return new P2pRpcAppRrMemPool(n, device_id, req_size, resp_size, want_mirror != 0);
  } catch (...) {
    return nullptr;
  }
}
void sgh_mempool_destroy(void *p) { delete static_cast<P2pRpcAppRrMemPool *>(p); }
int sgh_mempool_mirrored(void *p) { return static_cast<P2pRpcAppRrMemPool *>(p)->mirrored() ? 1 : 0; }
void *sgh_mempool_req_base(void *p) { return static_cast<P2pRpcAppRrMemPool *>(p)->get_req_addr_range(); }
uint64_t sgh_mempool_req_bytes(void *p) { return static_cast<P2pRpcAppRrMemPool *>(p)->get_req_addr_pool_size(); }
void *sgh_mempool_resp_base(void *p) { return static_cast<P2pRpcAppRrMemPool *>(p)->get_resp_addr_range(); }
uint64_t sgh_mempool_resp_bytes(void *p) { return static_cast<P2pRpcAppRrMemPool *>(p)->get_resp_addr_pool_size(); }

// `steps` steps of the batched hot path from a native loop, as a shunter thread would issue
// them: step i is one asynchronous gather call on `g` and one asynchronous scatter call on `s`
// (the same context, or one per direction) with the i-th of `n` prepared argument sets, taken
// in turns; both contexts are waited for at the end.  Returns the seconds the loop took, or a
// negative error code.
double sgh_step_loop_gpu(sg_hip_ctx *g, sg_hip_ctx *s, const sg_gather_args *const *ga,
                         const sg_scatter_args *const *sa, uint32_t n, uint32_t steps)
{
  if (!g || !s || !ga || !sa || n == 0) return (double)SG_E_INVAL;
  int rc = sg_hip_sync(g);
  if (rc == SG_OK && s != g) rc = sg_hip_sync(s);
  if (rc != SG_OK) return (double)rc;
  const auto t0 = std::chrono::steady_clock::now();
  for (uint32_t i = 0; i < steps; i++) {
    rc = sg_hip_gather_batch(g, ga[i % n]);
    if (rc != SG_OK) return (double)rc;
    rc = sg_hip_scatter_batch(s, sa[i % n]);
    if (rc != SG_OK) return (double)rc;
  }
  rc = sg_hip_sync(g);
  if (rc == SG_OK && s != g) rc = sg_hip_sync(s);
  if (rc != SG_OK) return (double)rc;
  return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
}

// The C++ engine's calls as a shunter thread issues them, timed: `n_req` requests of `per_req`
// fragments each (request r's fragment i in slot frag_slot[r * per_req + i] of the item's RX
// ring) held as P2pRpcRr objects, and as many responses of `per_resp` frames in the item's TX
// ring.  `items` are ring copies taken in turns (bases[4 * k + 0..3]: RX ring, TX ring, request
// arena, response arena of item k).
//   mode 0  batched: gather_batch(P2pRpcRr **) + scatter_batch(P2pRpcRr **) per step, the engine
//           walking every fragment on the host
//   mode 1  the same with the requests' fragment tables kept where the device reads them: calls of
//           engine.pull_min_items fragments (frames) or more have them pulled by the device
//   mode 2  the reference's call: one synchronous gather(rr, stub) per request, `steps` calls
// out[0]: seconds per step (per call in mode 2) over the whole loop, the device drained at the
// end; out[1..7] / out[8..14]: [N, mean, p90, p95, p99, min, max] of the nanoseconds the
// calling thread spent inside each gather / scatter call.  Returns 0 or a negative error.
int sgh_engine_loop_gpu(int device_id, int mode, uint32_t n_items, const uint64_t *bases, uint32_t n_slots,
                        uint32_t slot_size, uint32_t profile, const uint32_t *frag_slot, const uint32_t *frag_len,
                        uint32_t n_req, uint32_t per_req, uint64_t req_size, uint64_t req_cap, uint32_t mtu,
                        uint32_t tx_n_slots, const uint32_t *tx_slot, uint32_t per_resp, uint64_t resp_size,
                        uint64_t resp_cap, uint32_t flags, uint32_t steps, double *out)
{
  if (hipSetDevice(device_id) != hipSuccess) return -1;
  if (!n_items || !n_req || !steps) return -2;
  const uint32_t hl = rpc_header_len(profile);
  const uint32_t n_rr = 2 * n_items * n_req;
  P2pRpcSgHipEngine engine(device_id, n_req, n_req * (per_req > per_resp ? per_req : per_resp));
  P2pRpcRRPool pool((int)n_rr + 1, profile);
  p2p_rpc_conn_info *srv = initialize_src_conn_info("b8:ce:f6:cc:6a:52,192.168.25.1,50051");
  pool.setup_and_init_rr_pool(srv, req_size);
  release_conn_info(srv);
  if (mode == 1) {
    sg_frag_table *t = engine.frag_tables(n_rr);
    if (!t) return -3;
    pool.attach_frag_tables(t, n_rr, 0);
  }
  std::vector<std::vector<P2pRpcRr *>> rx(n_items), tx(n_items);
  for (uint32_t k = 0; k < n_items; k++) {
    const uintptr_t ring = (uintptr_t)bases[4 * k], txr = (uintptr_t)bases[4 * k + 1];
    for (uint32_t r = 0; r < n_req; r++) {
      // the receive thread's work: every fragment filed at its sequence number
      P2pRpcRr *q = pool.consume_rr();
      q->pkt_base = ring & ~(uintptr_t)1;
      q->req_token = ((uint64_t)k << 32) | (r + 1);
      for (uint32_t i = 0; i < per_req; i++) {
        const uintptr_t slot = ring + (uintptr_t)frag_slot[r * per_req + i] * slot_size;
        q->rr_emplace_mbuf(slot, slot, slot + hl, frag_len[r * per_req + i], (int)i);
      }
      rx[k].push_back(q);
      // rr_alloc_mbufs: the response's buffers
      P2pRpcRr *p = pool.consume_rr();
      p->pkt_base = txr & ~(uintptr_t)1;
      p->req_token = q->req_token;
      size_t rem = resp_size;
      for (uint32_t i = 0; i < per_resp; i++) {
        const uintptr_t slot = txr + (uintptr_t)tx_slot[r * per_resp + i] * slot_size;
        const size_t cur = rem <= mtu ? rem : mtu;
        rem -= cur;
        p->rr_append_mbuf(slot, slot, slot + hl, cur);
      }
      tx[k].push_back(p);
    }
  }
  auto fill = [&](const std::vector<uint64_t> &v, double *o) {
    const SgStatLine s = sg_stat_line(v);
    for (int i = 0; i < 7; i++) o[i] = s.v[i];
  };
  int rc = 0;
  if (mode == 2) {
    for (uint32_t i = 0; i < 20 && i < steps; i++) engine.gather(rx[0][i % n_req], (uint8_t *)(uintptr_t)bases[2] + (i % n_req) * req_size);
    engine.GDelay.clear();
    engine.numSkbs.clear();
    const uint64_t t0 = getCurNs();
    for (uint32_t i = 0; i < steps; i++) {
      const uint32_t k = i % n_items, r = (i / n_items) % n_req;
      engine.gather(rx[k][r], (uint8_t *)(uintptr_t)bases[4 * k + 2] + r * req_size);
      if (engine.last_rc != SG_OK) rc = -10;
    }
    out[0] = (double)(getCurNs() - t0) * 1e-9 / steps;
    fill(engine.GDelay, out + 1);
    fill(std::vector<uint64_t>(), out + 8);
    engine.GDelay.clear();
    engine.numSkbs.clear();
  } else {
    auto step = [&](uint32_t i) {
      const uint32_t k = i % n_items;
      SgRingView rv{sg_ring_desc{(void *)(uintptr_t)bases[4 * k], n_slots, slot_size, profile, 0}};
      SgRingView tv{sg_ring_desc{(void *)(uintptr_t)bases[4 * k + 1], tx_n_slots, slot_size, profile, 0}};
      sg_app_desc ra, ta;
      std::memset(&ra, 0, sizeof ra);
      std::memset(&ta, 0, sizeof ta);
      ra.arena = (void *)(uintptr_t)bases[4 * k + 2];
      ra.arena_cap = req_cap;
      ta.arena = (void *)(uintptr_t)bases[4 * k + 3];
      ta.arena_cap = resp_cap;
      if (engine.gather_batch(rx[k].data(), n_req, rv, ra, nullptr, req_size, profile == SG_HDR_BL58 || frag_len ? mtu : 0,
                              SG_F_ASYNC) != SG_OK)
        rc = -11;
      if (engine.scatter_batch(tx[k].data(), n_req, tv, ta, mtu, flags | SG_F_ASYNC) != SG_OK) rc = -12;
    };
    for (uint32_t i = 0; i < 2 * n_items && rc == 0; i++) step(i);
    if (engine.sync() != SG_OK) rc = -13;
    engine.GBatchHostNs.clear();
    engine.SBatchHostNs.clear();
    const uint64_t t0 = getCurNs();
    for (uint32_t i = 0; i < steps && rc == 0; i++) step(i);
    if (engine.sync() != SG_OK && rc == 0) rc = -14;
    out[0] = (double)(getCurNs() - t0) * 1e-9 / steps;
    fill(engine.GBatchHostNs, out + 1);
    fill(engine.SBatchHostNs, out + 8);
    engine.GBatchHostNs.clear();
    engine.SBatchHostNs.clear();
  }
  for (auto &v : rx)
    for (auto *q : v) pool.reap_rr(q);
  for (auto &v : tx)
    for (auto *q : v) pool.reap_rr(q);
  return rc;
}

// `steps` passes of the shunter's loop as one sg_hip_shunt_batch call each, from a native loop
// over `n_ctx` contexts (streams) taken in turns, so that up to n_ctx calls are in flight; pass i
// uses the i-th of `n` prepared argument sets.  Returns the seconds the loop took (device drained
// at the end) or a negative error code.  `lat_ns` (steps entries, or NULL): with n_ctx == 1 every
// call is made synchronous and its nanoseconds are left there.
double sgh_shunt_loop_gpu(sg_hip_ctx *const *ctxs, uint32_t n_ctx, const sg_gather_args *const *ga,
                          const sg_scatter_args *const *sa, uint32_t n, uint32_t steps, uint64_t *lat_ns)
{
  if (!ctxs || !n_ctx || !ga || !sa || n == 0) return (double)SG_E_INVAL;
  int rc = SG_OK;
  for (uint32_t c = 0; c < n_ctx && rc == SG_OK; c++) rc = sg_hip_sync(ctxs[c]);
  if (rc != SG_OK) return (double)rc;
  const uint64_t t0 = getCurNs();
  if (lat_ns && n_ctx == 1) {
    for (uint32_t i = 0; i < steps; i++) {
      const uint64_t a = getCurNs();
      rc = sg_hip_shunt_batch(ctxs[0], ga[i % n], sa[i % n]);
      if (rc == SG_OK) rc = sg_hip_sync(ctxs[0]);
      if (rc != SG_OK) return (double)rc;
      lat_ns[i] = getCurNs() - a;
    }
  } else {
    for (uint32_t i = 0; i < steps; i++) {
      rc = sg_hip_shunt_batch(ctxs[i % n_ctx], ga[i % n], sa[i % n]);
      if (rc != SG_OK) return (double)rc;
    }
  }
  for (uint32_t c = 0; c < n_ctx && rc == SG_OK; c++) rc = sg_hip_sync(ctxs[c]);
  if (rc != SG_OK) return (double)rc;
  return (double)(getCurNs() - t0) * 1e-9;
}

// The receive path on the device, burst after burst, from a native loop and without a host wait:
// burst k is filed by sg_hip_reassemble(ra, ras[k]) and the requests it completed are gathered and
// answered by sg_hip_shunt_batch(sg, ga[k], sa[k]) (their counts stay on the device).  With
// `overlapped` the two contexts are different ones (a stream each), the reassembly's output tables
// are two sets taken in turns (ras[k], ga[k], sa[k] name set k & 1) and events order the streams:
// the copy of burst k waits for its tables, the reassembly of burst k + 2 for the copy of burst k
// to have read them -- so burst k + 1 is filed while burst k is copied.  Returns the seconds the
// loop took, both contexts drained, or a negative error code.
double sgh_pipeline_loop_gpu(sg_hip_ctx *ra, sg_hip_ctx *sg, const sg_reassemble_args *const *ras,
                             const sg_gather_args *const *ga, const sg_scatter_args *const *sa, uint32_t n_bursts,
                             int overlapped)
{
  if (!ra || !sg || !ras || !ga || !sa) return (double)SG_E_INVAL;
  if (overlapped && ra == sg) return (double)SG_E_INVAL;
  hipStream_t s_ra = static_cast<hipStream_t>(sg_hip_stream(ra)), s_sg = static_cast<hipStream_t>(sg_hip_stream(sg));
  hipEvent_t filled[2] = {nullptr, nullptr}, drained[2] = {nullptr, nullptr};
  bool have_drained[2] = {false, false};
  for (int j = 0; j < 2 && overlapped; j++)
    if (hipEventCreateWithFlags(&filled[j], hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&drained[j], hipEventDisableTiming) != hipSuccess)
      return (double)SG_E_HIP;
  int rc = sg_hip_sync(ra);
  if (rc == SG_OK && sg != ra) rc = sg_hip_sync(sg);
  const uint64_t t0 = getCurNs();
  // files burst k on the reassembly's stream (once the copy that last read its table set is through)
  auto file = [&](uint32_t k) {
    const int j = k & 1;
    if (overlapped && have_drained[j] && hipStreamWaitEvent(s_ra, drained[j], 0) != hipSuccess) return SG_E_HIP;
    int r = sg_hip_reassemble(ra, ras[k], nullptr);
    if (r == SG_OK && overlapped && hipEventRecord(filled[j], s_ra) != hipSuccess) r = SG_E_HIP;
    return r;
  };
  if (overlapped && n_bursts) rc = file(0);
  for (uint32_t k = 0; k < n_bursts && rc == SG_OK; k++) {
    const int j = k & 1;
    if (overlapped) {
      // burst k + 1 is queued ahead of the copy of burst k: when both become runnable together, the
      // reassembly's few large workgroups are placed before the copy's many small ones fill the chip
      if (k + 1 < n_bursts) rc = file(k + 1);
      if (rc == SG_OK && hipStreamWaitEvent(s_sg, filled[j], 0) != hipSuccess) rc = SG_E_HIP;
    } else {
      rc = file(k);
    }
    if (rc == SG_OK) rc = sg_hip_shunt_batch(sg, ga[k], sa[k]);
    if (rc == SG_OK && overlapped) {
      if (hipEventRecord(drained[j], s_sg) != hipSuccess) rc = SG_E_HIP;
      have_drained[j] = true;
    }
    // a caller takes the counts in now and then; it also keeps the queues from growing without bound
    if (rc == SG_OK && (k & 255u) == 255u) rc = sg_hip_sync(sg);
  }
  if (rc == SG_OK) rc = sg_hip_sync(ra);
  if (rc == SG_OK && sg != ra) rc = sg_hip_sync(sg);
  const double dt = (double)(getCurNs() - t0) * 1e-9;
  for (int j = 0; j < 2; j++) {
    if (filled[j]) (void)hipEventDestroy(filled[j]);
    if (drained[j]) (void)hipEventDestroy(drained[j]);
  }
  return rc == SG_OK ? dt : (double)rc;
}

// Slot indices of `n` payload pointers of a ring, by the walk the batched calls make (a shift for
// slots of a power of two bytes) and by the single-pointer form (a division): both into their
// output, -1 where a pointer is no payload start of the ring.  Host only.
void sgh_slots_of_payloads(uint64_t base, uint32_t n_slots, uint32_t slot_size, uint32_t profile,
                           const uint64_t *payloads, uint32_t n, int64_t *by_walk, int64_t *by_division)
{
  SgRingView view{sg_ring_desc{(void *)(uintptr_t)base, n_slots, slot_size, profile, 0}};
  const SgRingView::Walk slot_of = view.walk();
  for (uint32_t i = 0; i < n; i++) {
    by_walk[i] = slot_of((uintptr_t)payloads[i]);
    by_division[i] = view.slot_of_payload((uintptr_t)payloads[i]);
  }
}

// Several receive queues side by side, each with a context (stream, reassembly table, cursors) of
// its own, as a NIC spreads flows over its RX queues and the reference keeps an rr pool per queue:
// every burst of a queue is filed and its completed requests gathered and answered
// (sg_hip_reassemble + sg_hip_shunt_batch on the queue's context), without a host wait.  ras / ga /
// sa hold n_queues * n_bursts entries, queue q's burst k at [q * n_bursts + k].  Small bursts are a
// chain of short dependent launches per queue; the queues' chains run beside each other on the
// device.  threaded == 0: this thread queues burst k of every queue before burst k + 1 of any;
// else a thread per queue, as the reference runs a shunter thread per transport.  Returns the
// seconds the loop took, every context drained, or a negative error code.
double sgh_pipeline_queues_gpu(sg_hip_ctx *const *ctxs, uint32_t n_queues, const sg_reassemble_args *const *ras,
                               const sg_gather_args *const *ga, const sg_scatter_args *const *sa, uint32_t n_bursts,
                               int threaded)
{
  if (!ctxs || !ras || !ga || !sa || n_queues == 0) return (double)SG_E_INVAL;
  int rc = SG_OK;
  for (uint32_t q = 0; q < n_queues && rc == SG_OK; q++) rc = ctxs[q] ? sg_hip_sync(ctxs[q]) : SG_E_INVAL;
  if (rc != SG_OK) return (double)rc;
  auto burst = [&](uint32_t q, uint32_t k) {
    const size_t at = (size_t)q * n_bursts + k;
    int r = sg_hip_reassemble(ctxs[q], ras[at], nullptr);
    if (r == SG_OK) r = sg_hip_shunt_batch(ctxs[q], ga[at], sa[at]);
    // a caller takes the counts in now and then; it also keeps the queues from growing without bound
    if (r == SG_OK && (k & 255u) == 255u) r = sg_hip_sync(ctxs[q]);
    return r;
  };
  const uint64_t t0 = getCurNs();
  if (threaded) {
    std::vector<int> rcs(n_queues, SG_OK);
    std::vector<std::thread> threads;
    for (uint32_t q = 0; q < n_queues; q++)
      threads.emplace_back([&, q] {
        int r = SG_OK;
        for (uint32_t k = 0; k < n_bursts && r == SG_OK; k++) r = burst(q, k);
        if (r == SG_OK) r = sg_hip_sync(ctxs[q]);
        rcs[q] = r;
      });
    for (auto &t : threads) t.join();
    for (int r : rcs)
      if (r != SG_OK && rc == SG_OK) rc = r;
  } else {
    for (uint32_t k = 0; k < n_bursts && rc == SG_OK; k++)
      for (uint32_t q = 0; q < n_queues && rc == SG_OK; q++) rc = burst(q, k);
    for (uint32_t q = 0; q < n_queues && rc == SG_OK; q++) rc = sg_hip_sync(ctxs[q]);
  }
  const double dt = (double)(getCurNs() - t0) * 1e-9;
  return rc == SG_OK ? dt : (double)rc;
}

}  // extern "C"
