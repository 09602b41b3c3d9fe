// CPU-only exercise of the host layer's request pool and its rings, built by
// tests/test_host_layer.py with the thread sanitizer and with the address +
// undefined-behaviour sanitizers: the rings are shared between the receive and
// the shunter threads of a server (src/p2p_rpc_rr_pool_ng.h:27-45 creates them
// multi-producer / multi-consumer).
#include <algorithm>
#include <atomic>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <random>
#include <thread>
#include <vector>

#include "sg_rr.h"

static int ring_stress(uint32_t n_threads, uint32_t per_thread, uint32_t capacity)
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
    if (s.load() != 1) return 1;
  return 0;
}

// One thread files arrivals (the receive thread), another takes completed
// requests off the rx-ready ring and reaps them (the shunter thread).
static int pool_two_threads(uint32_t n_req, uint32_t frags_per_req)
{
  P2pRpcRRPool pool(64, SG_HDR_BL58);
  p2p_rpc_conn_info *srv = initialize_src_conn_info("b8:ce:f6:cc:6a:52,192.168.25.1,50051");
  pool.setup_and_init_rr_pool(srv, (size_t)frags_per_req * 100);
  release_conn_info(srv);
  std::atomic<uint32_t> reaped{0};
  std::atomic<uint64_t> bytes{0};
  std::thread shunter([&] {
    P2pRpcRr *rr;
    while (reaped.load() < n_req) {
      if (pool.get_next_rx_ready_rr(&rr)) {
        uint64_t b = 0;
        for (int i = 0; i < rr->payload_bufs->num_items; i++) b += rr->payload_bufs->item_size[i];
        bytes.fetch_add(b);
        pool.reap_rr(rr);
        reaped.fetch_add(1);
      } else {
        std::this_thread::yield();
      }
    }
  });
  std::mt19937 rng(3);
  // requests arrive four at a time, their fragments interleaved and out of order
  for (uint32_t base = 0; base < n_req; base += 4) {
    // stay inside the pool: growing and shrinking it is the receive thread's business alone
    while (base - reaped.load() > 40) std::this_thread::yield();
    std::vector<std::pair<uint32_t, uint32_t>> arrivals;
    for (uint32_t r = base; r < base + 4 && r < n_req; r++)
      for (uint32_t i = 0; i < frags_per_req; i++) arrivals.push_back({r, i});
    std::shuffle(arrivals.begin(), arrivals.end(), rng);
    for (auto &a : arrivals) {
      uint8_t hdr[64];
      std::memset(hdr, 0, sizeof hdr);
      bl58_rpc_hdr *h = reinterpret_cast<bl58_rpc_hdr *>(hdr);
      h->req_id = 1000 + a.first;
      h->frag_idx = (uint16_t)a.second;
      h->num_frags = (uint16_t)frags_per_req;
      h->payload_len = 100;
      const uintptr_t slot = 0x10000000u + (uintptr_t)(a.first * frags_per_req + a.second) * 2048;
      pool.append_to_rr(reinterpret_cast<p2p_rpc_hdr *>(hdr), slot, slot, slot + 58, 100);
    }
  }
  shunter.join();
  return bytes.load() == (uint64_t)n_req * frags_per_req * 100 ? 0 : 1;
}

int main()
{
  int bad = 0;
  bad |= ring_stress(4, 20000, 8);
  bad |= ring_stress(2, 50000, 1024);
  bad |= pool_two_threads(400, 7);
  std::printf(bad ? "host sanitize: FAILED\n" : "host sanitize: ok\n");
  return bad;
}
