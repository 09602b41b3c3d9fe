// sg_rr.h -- request reassembly state on the host: P2pRpcRr (src/p2p_rpc_rr_ng.h)
// and P2pRpcRRPool (src/p2p_rpc_rr_pool_ng.h), same names, members and
// behaviour.  The three DPDK rte_rings of the reference become bounded
// multi-producer / multi-consumer pointer rings of this file.
#pragma once

#include <atomic>
#include <cerrno>
#include <cstdio>
#include <cstdlib>
#include <memory>
#include <unordered_map>
#include <vector>

#include "sg_hip.h"
#include "sg_tables.h"
#include "sg_wire.h"

enum P2P_RPC_RR_STATES { RR_CREATE, RR_PROCESS, RR_READY, RR_FINISH, RR_UNUSED };

// Holder of one request / response (src/p2p_rpc_rr_ng.h:13-127).
class P2pRpcRr {
 public:
  // application
  uint64_t req_token;
  size_t payload_size;
  size_t max_payload_size;
  p2p_rpc_conn_info _client_conn_info;
  // pool
  uint32_t rr_state;
  // transport: one entry per fragment, indexed by the fragment's seq_num
  p2p_hbufs *transport_mbufs;
  p2p_hbufs *hdr_bufs;
  p2p_bufs *payload_bufs;
  // copy engine scratch
  p2p_sk_buf *payload_sk_bufs;
  // The payload table once more, in the form the device reads (sg_frag_table: 32-bit offsets from
  // pkt_base and lengths), written entry for entry with payload_bufs where a table is attached.
  // The table lives in memory the GPU can read (the copy engine allocates it, pinned), so a batched
  // gather or scatter names the table and walks no fragment on the host.  No counterpart in the
  // reference; nullptr: not kept.
  sg_frag_table *frag_table = nullptr;
  uintptr_t pkt_base = 0;

  explicit P2pRpcRr(p2p_rpc_conn_info *template_conn_info = nullptr, size_t _max_payload_size = 0)
      : req_token(0), payload_size(0), max_payload_size(_max_payload_size), rr_state(RR_CREATE),
        transport_mbufs(new p2p_hbufs), hdr_bufs(new p2p_hbufs), payload_bufs(new p2p_bufs),
        payload_sk_bufs(new p2p_sk_buf)
  {
    std::memset(&_client_conn_info, 0, sizeof _client_conn_info);
    if (template_conn_info)
      std::memcpy(&_client_conn_info.hdr_template, &template_conn_info->hdr_template, RPC_HEADER_LEN);
    transport_mbufs->num_items = 0;
    hdr_bufs->num_items = 0;
    payload_bufs->num_items = 0;
  }

  ~P2pRpcRr()
  {
    delete transport_mbufs;
    delete hdr_bufs;
    delete payload_bufs;
    delete payload_sk_bufs;
  }

  P2pRpcRr(const P2pRpcRr &) = delete;
  P2pRpcRr &operator=(const P2pRpcRr &) = delete;

  // entry idx of all three tables, counts bumped (src/p2p_rpc_rr_ng.h:65-81)
  inline void rr_merge_mbuf(uintptr_t transport_mbuf, uintptr_t hdr_buf, uintptr_t payload_buf,
                            size_t item_size, int idx)
  {
    transport_mbufs->burst_items[idx] = transport_mbuf;
    transport_mbufs->num_items++;
    hdr_bufs->burst_items[idx] = hdr_buf;
    hdr_bufs->num_items++;
    payload_bufs->burst_items[idx] = payload_buf;
    payload_bufs->item_size[idx] = item_size;
    payload_bufs->num_items++;
    if (frag_table) {
      // an address the 32-bit form cannot hold becomes an entry the device refuses
      const uintptr_t d = payload_buf - pkt_base;
      const bool fits = payload_buf >= pkt_base && !(d & 1u) && (d >> 33) == 0 && (d >> 1) != 0xffffffffu;
      frag_table->off[idx] = fits ? (uint32_t)(d >> 1) : 0xffffffffu;
      frag_table->len[idx] = (uint32_t)item_size;
    }
  }

  // at the end, whatever the frame id (src/p2p_rpc_rr_ng.h:85-93)
  inline void rr_append_mbuf(uintptr_t transport_mbuf, uintptr_t hdr_buf, uintptr_t payload_buf, size_t item_size)
  {
    rr_merge_mbuf(transport_mbuf, hdr_buf, payload_buf, item_size, transport_mbufs->num_items);
    payload_size += item_size;
  }

  // at its sequence number: absorbs out-of-order arrival (src/p2p_rpc_rr_ng.h:96-105)
  inline void rr_emplace_mbuf(uintptr_t transport_mbuf, uintptr_t hdr_buf, uintptr_t payload_buf,
                              size_t item_size, int seq_num)
  {
    rr_merge_mbuf(transport_mbuf, hdr_buf, payload_buf, item_size, seq_num);
    payload_size += item_size;
  }

  // src/p2p_rpc_rr_ng.h:107-110
  inline bool is_rr_ready() const { return payload_size == max_payload_size; }

  void rr_print_bufs() const
  {
    std::printf("Req: %p, num_bufs: %d\n", (const void *)this, payload_bufs->num_items);
    for (int i = 0; i < payload_bufs->num_items; i++)
      std::printf("  start: %p, size: %zu\n", (void *)payload_bufs->burst_items[i], (size_t)payload_bufs->item_size[i]);
  }
};

// New rr with the same request size and header template, no buffers (src/p2p_rpc_rr_ng.h:130-140)
static inline P2pRpcRr *rr_clone_alloc(const P2pRpcRr *rr)
{
  P2pRpcRr *n = new P2pRpcRr();
  n->max_payload_size = rr->max_payload_size;
  n->req_token = 0;
  std::memcpy(&n->_client_conn_info.hdr_template, &rr->_client_conn_info.hdr_template, RPC_HEADER_LEN);
  return n;
}

// Bounded multi-producer / multi-consumer ring of pointers: per-cell sequence
// numbers, no locks.  Stands in for rte_ring with RING_F_MP_RTS_ENQ |
// RING_F_MC_RTS_DEQ (src/p2p_rpc_rr_pool_ng.h:34-35).  Holds at least
// `min_capacity` entries.
class SgPtrRing {
  struct Cell {
    std::atomic<size_t> seq;
    void *ptr;
  };
  std::unique_ptr<Cell[]> cells_;
  size_t mask_;
  alignas(64) std::atomic<size_t> head_{0};
  alignas(64) std::atomic<size_t> tail_{0};

 public:
  explicit SgPtrRing(size_t min_capacity)
  {
    size_t cap = 2;
    while (cap < min_capacity) cap <<= 1;
    cells_.reset(new Cell[cap]);
    mask_ = cap - 1;
    for (size_t i = 0; i < cap; i++) cells_[i].seq.store(i, std::memory_order_relaxed);
  }

  // 0, or -ENOBUFS when full (rte_ring_enqueue's convention)
  int enqueue(void *p)
  {
    size_t pos = tail_.load(std::memory_order_relaxed);
    for (;;) {
      Cell &c = cells_[pos & mask_];
      const size_t seq = c.seq.load(std::memory_order_acquire);
      const intptr_t dif = (intptr_t)seq - (intptr_t)pos;
      if (dif == 0) {
        if (tail_.compare_exchange_weak(pos, pos + 1, std::memory_order_relaxed)) {
          c.ptr = p;
          c.seq.store(pos + 1, std::memory_order_release);
          return 0;
        }
      } else if (dif < 0) {
        return -ENOBUFS;
      } else {
        pos = tail_.load(std::memory_order_relaxed);
      }
    }
  }

  // 0, or -ENOENT when empty (rte_ring_dequeue's convention)
  int dequeue(void **out)
  {
    size_t pos = head_.load(std::memory_order_relaxed);
    for (;;) {
      Cell &c = cells_[pos & mask_];
      const size_t seq = c.seq.load(std::memory_order_acquire);
      const intptr_t dif = (intptr_t)seq - (intptr_t)(pos + 1);
      if (dif == 0) {
        if (head_.compare_exchange_weak(pos, pos + 1, std::memory_order_relaxed)) {
          *out = c.ptr;
          c.seq.store(pos + mask_ + 1, std::memory_order_release);
          return 0;
        }
      } else if (dif < 0) {
        return -ENOENT;
      } else {
        pos = head_.load(std::memory_order_relaxed);
      }
    }
  }
};

static const int RR_POOL_SIZE = 4096 - 1;  // src/p2p_rpc_rr_pool_ng.h:12

// Token -> rr map of the in-flight requests plus free / rx-ready / tx-ready
// rings (src/p2p_rpc_rr_pool_ng.h:14-188).  As in the reference, get_rr /
// append_to_rr / mark_rx_ready_rr belong to the single receive thread; the
// rings may be used from several threads.
class P2pRpcRRPool {
  std::unordered_map<uint64_t, P2pRpcRr *> rr_cache;
  SgPtrRing *free_rr_pool;
  SgPtrRing *rx_ready_rr_pool;
  SgPtrRing *tx_ready_rr_pool;
  std::vector<P2pRpcRr *> rr_pool;
  P2pRpcRr *proto_rr;
  int pool_size;
  uint32_t hdr_profile;
  uintptr_t frag_pkt_base = 0;  // what the rrs' fragment tables count from when they file a request

 public:
  // _pool_size == -1: RR_POOL_SIZE rrs; else _pool_size - 1 (as the reference counts)
  explicit P2pRpcRRPool(int _pool_size = -1, uint32_t _hdr_profile = SG_HDR_REF64)
      : proto_rr(nullptr), hdr_profile(_hdr_profile)
  {
    pool_size = _pool_size == -1 ? RR_POOL_SIZE : _pool_size - 1;
    free_rr_pool = new SgPtrRing(pool_size + 1);
    rx_ready_rr_pool = new SgPtrRing(pool_size + 1);
    tx_ready_rr_pool = new SgPtrRing(pool_size + 1);
  }

  ~P2pRpcRRPool()
  {
    if (!rr_cache.empty()) {
      std::printf("Cleaning up RR Pool: %zu requests never completed\n", rr_cache.size());
      for (auto &e : rr_cache)
        if (e.second)
          std::printf("  token %llu: payload_size %zu, %d fragments\n", (unsigned long long)e.first,
                      e.second->payload_size, e.second->payload_bufs->num_items);
    }
    delete proto_rr;
    for (P2pRpcRr *rr : rr_pool) delete rr;
    delete free_rr_pool;
    delete rx_ready_rr_pool;
    delete tx_ready_rr_pool;
  }

  std::vector<P2pRpcRr *> &get_rr_pool_container() { return rr_pool; }
  P2pRpcRr **get_rr_pool() { return rr_pool.data(); }
  int get_pool_size() const { return pool_size; }
  size_t in_flight() const { return rr_cache.size(); }

  void setup_and_init_rr_pool(p2p_rpc_conn_info *template_conn_info, size_t payload_size)
  {
    proto_rr = new P2pRpcRr(template_conn_info, payload_size);
    for (int i = 0; i < pool_size; i++) rr_pool.push_back(rr_clone_alloc(proto_rr));
    for (int i = 0; i < pool_size; i++)
      if (free_rr_pool->enqueue(rr_pool[i]) != 0) std::printf("P2pRpcRRPool: Free pool full!\n");
  }

  // Gives rr i of the pool table i of `tables` (n of them, in memory the GPU reads; see
  // P2pRpcSgHipEngine::frag_tables) and the address its 32-bit offsets count from.  Rrs beyond n,
  // and rrs the pool allocates later when it runs dry, keep none: batched calls walk those on the host.
  // The 32-bit offsets reach 8 GiB: where response buffers come from memory further than that
  // from the request buffers, whoever hands an rr its response buffers sets rr->pkt_base to that
  // memory's base first (reap_rr sets it back).
  void attach_frag_tables(sg_frag_table *tables, size_t n, uintptr_t pkt_base)
  {
    frag_pkt_base = pkt_base;
    for (size_t i = 0; i < rr_pool.size(); i++) {
      if (!rr_pool[i]) continue;
      rr_pool[i]->frag_table = i < n ? tables + i : nullptr;
      rr_pool[i]->pkt_base = pkt_base;
    }
  }

  // cached rr of this token, or a fresh one filed under it (:97-109)
  inline P2pRpcRr *get_rr(p2p_rpc_hdr *rpc_hdr)
  {
    const uint64_t req_token = get_req_token(rpc_hdr);
    auto it = rr_cache.find(req_token);
    if (it != rr_cache.end()) return it->second;
    P2pRpcRr *rr = consume_rr();
    set_conn_info(&rr->_client_conn_info, rpc_hdr);
    rr->req_token = req_token;
    rr_cache[req_token] = rr;
    return rr;
  }

  // (:111-119)
  inline void append_to_rr(p2p_rpc_hdr *rpc_hdr, uintptr_t transport_mbuf, uintptr_t hdr_buf,
                           uintptr_t payload_buf, size_t payload_item_size)
  {
    P2pRpcRr *rr = get_rr(rpc_hdr);
    rr->rr_emplace_mbuf(transport_mbuf, hdr_buf, payload_buf, payload_item_size,
                        rpc_frag_index(rpc_hdr, hdr_profile));
    // REF64: one server-wide request size decides (is_rr_ready).  BL58 headers
    // carry their request's fragment count, so requests may differ in size.
    const bool ready = hdr_profile == SG_HDR_REF64
                           ? rr->is_rr_ready()
                           : rr->payload_bufs->num_items == reinterpret_cast<bl58_rpc_hdr *>(rpc_hdr)->num_frags;
    if (ready) mark_rx_ready_rr(rr);
  }

  // (:121-135) an empty free ring grows the pool, as the reference does
  inline P2pRpcRr *consume_rr()
  {
    void *p = nullptr;
    if (free_rr_pool->dequeue(&p) == -ENOENT) {
      std::printf("Warning!, P2pRpcRRPool is empty, allocating new rr\n");
      p = rr_clone_alloc(proto_rr);
      rr_pool.push_back(static_cast<P2pRpcRr *>(p));
    }
    if (p == nullptr) {
      std::printf("Out of memory, exiting...");
      std::exit(1);
    }
    P2pRpcRr *rr = static_cast<P2pRpcRr *>(p);
    rr->rr_state = RR_PROCESS;
    return rr;
  }

  // (:137-147)  payload_size is reset by the sender before this (rr_send,
  // src/transport/dpdk_transport_ng.h:318-320); done here too so that a reaped
  // rr never starts its next request half full.
  inline void reap_rr(P2pRpcRr *rr)
  {
    rr->rr_state = RR_UNUSED;
    rr->transport_mbufs->num_items = 0;
    rr->hdr_bufs->num_items = 0;
    rr->payload_bufs->num_items = 0;
    rr->payload_size = 0;
    rr->req_token = 0;
    rr->pkt_base = frag_pkt_base;
    if (free_rr_pool->enqueue(rr) == -ENOBUFS) {
      std::printf("Warning!, P2pRpcRRPool is full, de-allocating rr: %p\n", (void *)rr);
      for (auto &q : rr_pool)
        if (q == rr) q = nullptr;
      delete rr;
    }
  }

  // (:149-155)
  inline void mark_rx_ready_rr(P2pRpcRr *rr)
  {
    rr_cache.erase(rr->req_token);
    rr->rr_state = RR_READY;
    while (rx_ready_rr_pool->enqueue(rr) != 0) {
    }
  }

  inline void mark_tx_ready_rr(P2pRpcRr *rr)
  {
    while (tx_ready_rr_pool->enqueue(rr) != 0) {
    }
  }

  inline P2pRpcRr *consume_rx_ready_rr()
  {
    void *p = nullptr;
    return rx_ready_rr_pool->dequeue(&p) == -ENOENT ? nullptr : static_cast<P2pRpcRr *>(p);
  }

  inline int get_next_rx_ready_rr(P2pRpcRr **next_rr)
  {
    *next_rr = consume_rx_ready_rr();
    return *next_rr != nullptr ? 1 : 0;
  }

  inline P2pRpcRr *consume_tx_ready_rr()
  {
    void *p = nullptr;
    return tx_ready_rr_pool->dequeue(&p) == -ENOENT ? nullptr : static_cast<P2pRpcRr *>(p);
  }
};
