// sg_engine.h -- the copy-engine interface of the reference
// (src/p2p_rpc_sg_engine.h) with a HIP engine for gfx950 behind it.
//
//   gather_skbs / scatter_skbs   host-side run-table builders (:19-73)
//   P2pRpcSgEngine               the abstract engine a server selects (:75-105)
//   P2pRpcSgZcEngine             zero-copy: hands out the first payload pointer (:109-134)
//   P2pRpcSgHipEngine            stands where P2pRpcSgGpuEngine stood (:185-308):
//                                the same four calls, synchronous, plus batched
//                                calls that move every ready request at once
//
// There is no CPU copy engine here: the reference's P2pRpcSgCpuEngine exists in
// this repository only as the test oracle.
#pragma once

#include <atomic>
#include <cstdio>
#include <cstring>
#include <vector>

#include <hip/hip_runtime.h>

#include "sg_hip.h"
#include "sg_rr.h"
#include "sg_stats.h"
#include "sg_tables.h"

// Fragment table (in seq order) -> run list into app_buf.  o_buf is the running
// sum of the fragment sizes; a fragment extends the current run exactly when
// it starts where the previous fragment ended.
static inline void gather_skbs(p2p_sk_buf *skb, p2p_bufs *buf_ptrs, uint8_t *app_buf)
{
  uintptr_t app_addr = (uintptr_t)app_buf;
  size_t run = 0;
  uintptr_t prev_end = 0;
  // entry 0 is written even for an empty table, as the reference does
  const int n = buf_ptrs->num_items;
  for (int i = 0; i < (n > 0 ? n : 1); i++) {
    const uintptr_t p = buf_ptrs->burst_items[i];
    const size_t sz = buf_ptrs->item_size[i];
    if (i > 0 && p == prev_end) {
      skb->len[run] += sz;
    } else {
      if (i > 0) run++;
      skb->i_buf[run] = p;
      skb->o_buf[run] = app_addr;
      skb->len[run] = sz;
    }
    prev_end = p + sz;
    app_addr += sz;
  }
  skb->num_items = run + 1;
}

// Mirror image: i_buf walks the app buffer, o_buf points at the packets.
static inline void scatter_skbs(p2p_sk_buf *skb, p2p_bufs *buf_ptrs, uint8_t *app_buf)
{
  uintptr_t app_addr = (uintptr_t)app_buf;
  size_t run = 0;
  uintptr_t prev_end = 0;
  const int n = buf_ptrs->num_items;
  for (int i = 0; i < (n > 0 ? n : 1); i++) {
    const uintptr_t p = buf_ptrs->burst_items[i];
    const size_t sz = buf_ptrs->item_size[i];
    if (i > 0 && p == prev_end) {
      skb->len[run] += sz;
    } else {
      if (i > 0) run++;
      skb->i_buf[run] = app_addr;
      skb->o_buf[run] = p;
      skb->len[run] = sz;
    }
    prev_end = p + sz;
    app_addr += sz;
  }
  skb->num_items = run + 1;
}

class P2pRpcSgEngine {
 public:
  int num_instances = 1;         // parallel instances of the copy engine
  int device_id = 0;
  uint16_t app_queue_length = 1; // queue length of each instance
#ifdef PROFILE_MODE
  // nanoseconds per gather / scatter call and runs per gather, printed when the engine goes
  // (src/p2p_rpc_sg_engine.h:83-92)
  uint64_t SStartNs = 0, GStartNs = 0;
  std::vector<uint64_t> SDelay, GDelay;
  std::vector<uint64_t> numSkbs;
#endif
  virtual ~P2pRpcSgEngine()
  {
    PROF_PRINT("Gather", GDelay);
    PROF_PRINT("Scatter", SDelay);
    PROF_PRINT("Gather-NumSKBS", numSkbs);
  }

  // API v0
  virtual void gather(P2pRpcRr *, uint8_t *) = 0;
  virtual void scatter(P2pRpcRr *, uint8_t *) = 0;
  // API v1
  virtual void gather(P2pRpcRr *, g_params *) = 0;
  virtual void scatter(P2pRpcRr *, g_params *) = 0;
};

class P2pRpcSgZcEngine : public P2pRpcSgEngine {
 public:
  inline void gather(P2pRpcRr *rpc_rr, g_params *app_stub) override
  {
    app_stub->req = (uint8_t *)rpc_rr->payload_bufs->burst_items[0];
    app_stub->resp = (uint8_t *)rpc_rr->payload_bufs->burst_items[0];
    std::atomic_thread_fence(std::memory_order_release);
  }
  inline void scatter(P2pRpcRr *, g_params *) override {}
  inline void gather(P2pRpcRr *, uint8_t *) override {}
  inline void scatter(P2pRpcRr *, uint8_t *) override {}
};

// Where the packet buffers of a transport live, for the batched calls: a
// P2pRpcRr holds payload POINTERS; the batched kernels want slot indices.
struct SgRingView {
  sg_ring_desc desc;
  uintptr_t base() const { return (uintptr_t)desc.base; }
  uint32_t hdr_len() const { return desc.hdr_profile == SG_HDR_REF64 ? 64u : 58u; }
  // slot index of a payload pointer, or -1 if it is not a payload start of this ring
  int64_t slot_of_payload(uintptr_t payload) const
  {
    const uintptr_t off = payload - base() - hdr_len();
    if (payload < base() + hdr_len() || off % desc.slot_size) return -1;
    const uintptr_t s = off / desc.slot_size;
    return s < desc.n_slots ? (int64_t)s : -1;
  }
  // The same for a walk over many pointers: the ring's constants taken once, and slots of a power
  // of two bytes (the usual mbuf sizes) found by a shift instead of a division per fragment.
  struct Walk {
    uintptr_t lo;
    uint32_t slot_size, n_slots, shift;  // shift == 0: divide
    int64_t operator()(uintptr_t payload) const
    {
      const uintptr_t off = payload - lo;
      if (payload < lo) return -1;
      uintptr_t s;
      if (shift) {
        if (off & (slot_size - 1u)) return -1;
        s = off >> shift;
      } else {
        if (off % slot_size) return -1;
        s = off / slot_size;
      }
      return s < n_slots ? (int64_t)s : -1;
    }
  };
  Walk walk() const
  {
    const uint32_t ss = desc.slot_size;
    const bool pow2 = ss > 1 && (ss & (ss - 1u)) == 0;
    return Walk{base() + hdr_len(), ss, desc.n_slots, pow2 ? (uint32_t)__builtin_ctz(ss) : 0u};
  }
};

class P2pRpcSgHipEngine : public P2pRpcSgEngine {
  // One context (and stream) per direction, as the reference keeps a gather_ctx and a scatter_ctx
  // (src/p2p_rpc_sg_engine.h:185-196): the two halves of the shunter's loop touch different
  // memory and run side by side.  Calls that take ready-made argument blocks (tables the caller
  // or the device reassembly left on the device) all go to the first, in stream order.
  sg_hip_ctx *ctx;
  sg_hip_ctx *ctx_tx;
  uint32_t max_reqs, max_frames;

  // Tables of a batched call reach the device through one of two stages per direction that take
  // turns, each with an event behind its last call, so a call waits only if the stage it is about
  // to overwrite is still being read -- the call before the previous one of its direction -- and
  // the tables of the next gather are on their way while the current one copies.  A stage is a block of pinned
  // host memory (what the host writes) and a block of device memory (what the kernels read).
  struct Stage {
    uint32_t *h = nullptr, *d = nullptr;
    size_t cap_h = 0, cap_d = 0;  // 32-bit words
    hipEvent_t ev = nullptr;      // behind the call that read the stage
    hipEvent_t packed = nullptr;  // behind the pull of the tables into the stage
    bool busy = false;
  };
  Stage stage[2][2];  // [direction: 0 gather, 1 scatter][turn]: a gather call never waits for a scatter's stage
  int turn[2] = {0, 0};
  // fragment tables the device reads in place (frag_tables()) and the stream their pull runs on,
  // beside the copy of the call before
  sg_frag_table *tables = nullptr;
  uint32_t n_tables = 0;
  hipStream_t pack_stream = nullptr;
  hipStream_t tx_stream = nullptr;  // the scatter context's stream (made here so that its hardware queue can be chosen)
  // no stream on a hardware queue of its own was to be had: the work then runs one after the other
  bool pack_queue_shared = false, tx_queue_shared = false;

  void fail(const char *what, int rc, const sg_hip_ctx *c = nullptr) const
  {
    // the reference's engines report and go on (src/p2p_rpc_sg_engine.h:283-298)
    std::printf("P2pRpcSgHipEngine: %s failed (%d): %s\n", what, rc, sg_hip_last_error(c ? c : ctx));
  }

  hipStream_t stream(int dir) const { return static_cast<hipStream_t>(sg_hip_stream(dir ? ctx_tx : ctx)); }

  struct OnDevice {
    int prev = -1;
    explicit OnDevice(int dev)
    {
      if (hipGetDevice(&prev) != hipSuccess || prev == dev) prev = -1;
      else (void)hipSetDevice(dev);
    }
    ~OnDevice()
    {
      if (prev >= 0) (void)hipSetDevice(prev);
    }
  };

  Stage *take_stage(int dir, size_t h_words, size_t d_words)
  {
    Stage &s = stage[dir][turn[dir]];
    turn[dir] ^= 1;
    if (s.busy) {
      (void)hipEventSynchronize(s.ev);
      s.busy = false;
    }
    if (h_words > s.cap_h) {
      if (s.h) (void)hipHostFree(s.h);
      s.h = nullptr;
      s.cap_h = 0;
      const size_t want = h_words + h_words / 2 + 64;
      if (hipHostMalloc((void **)&s.h, want * 4, hipHostMallocDefault) != hipSuccess) return nullptr;
      s.cap_h = want;
    }
    if (d_words > s.cap_d) {
      if (s.d) (void)hipFree(s.d);
      s.d = nullptr;
      s.cap_d = 0;
      const size_t want = d_words + d_words / 2 + 64;
      if (hipMalloc((void **)&s.d, want * 4) != hipSuccess) return nullptr;
      s.cap_d = want;
    }
    if (!s.ev && hipEventCreateWithFlags(&s.ev, hipEventDisableTiming) != hipSuccess) return nullptr;
    if (!s.packed && hipEventCreateWithFlags(&s.packed, hipEventDisableTiming) != hipSuccess) return nullptr;
    return &s;
  }

  // The host's image of a stage to the device, in the order of the direction's stream: a kernel
  // reads the pinned block across the bus.  (An asynchronous copy call for it made the calling
  // thread wait behind copies queued on the other direction's stream.)
  bool send_stage(Stage *s, size_t words, int dir)
  {
    sg_pack_args pa;
    std::memset(&pa, 0, sizeof pa);
    pa.blob_src = s->h;
    pa.blob_dst = s->d;
    pa.blob_words = (uint32_t)words;
    pa.stream = stream(dir);
    return sg_hip_pack_tables(dir ? ctx_tx : ctx, &pa) == SG_OK;
  }

  void stage_in_use(Stage *s, int dir)
  {
    if (hipEventRecord(s->ev, stream(dir)) == hipSuccess) s->busy = true;
    else (void)hipStreamSynchronize(stream(dir));
  }

  // A stream that dispatches to another hardware queue than those in `avoid` (streams that share a
  // queue run one after the other, and the runtime deals its few queues out in turns): streams are
  // made until one answers differently, the others given back.  Falls back to the first made;
  // *shared then says so.
  hipStream_t stream_apart(const uint64_t *avoid, int n_avoid, bool *shared)
  {
    hipStream_t tried[8], found = nullptr;
    int n_tried = 0;
    for (; n_tried < 8 && !found; n_tried++) {
      if (hipStreamCreateWithFlags(&tried[n_tried], hipStreamNonBlocking) != hipSuccess) break;
      uint64_t q = 0;
      bool apart = sg_hip_stream_queue(ctx, tried[n_tried], &q) == SG_OK && q != 0;
      for (int k = 0; k < n_avoid; k++) apart = apart && q != avoid[k];
      if (apart) found = tried[n_tried];
    }
    *shared = !found;
    if (!found && n_tried) found = tried[0];
    for (int i = 0; i < n_tried; i++)
      if (tried[i] != found) (void)hipStreamDestroy(tried[i]);
    return found;
  }

  // Every request of the batch keeps a table of this engine's, all counted from one base that
  // lies at or below `ring`: the device can pull them.
  bool can_pull(P2pRpcRr *const *rrs, uint32_t n, const SgRingView &ring) const
  {
    if (!tables || n == 0) return false;
    const uintptr_t base = rrs[0]->pkt_base;
    if (ring.base() < base) return false;
    for (uint32_t r = 0; r < n; r++) {
      const sg_frag_table *t = rrs[r]->frag_table;
      if (!t || t < tables || t >= tables + n_tables || rrs[r]->pkt_base != base) return false;
    }
    return true;
  }

  // The pull runs on a stream of its own, beside whatever the direction's stream is copying, and
  // the calling thread waits for it (tens of microseconds across the bus) before it queues the
  // copy: a wait queued on the copy's stream instead costs that stream some ten microseconds of
  // idling per call, while this thread has nothing else to do until the copy can be queued.
  // (The pull in front of the copy on the copy's own stream, nothing to wait for, was measured as
  // well: between the walk and this form it wins nowhere by more than a few per cent.)
  int pull(Stage *st, sg_pack_args *pa)
  {
    pa->tables = tables;
    pa->n_tables = n_tables;
    pa->stream = pack_stream;
    int rc = sg_hip_pack_tables(ctx, pa);
    if (rc != SG_OK) return rc;
    if (hipEventRecord(st->packed, pack_stream) != hipSuccess) return SG_E_HIP;
    // polled, not slept on: the runtime's blocking wait wakes this thread some twenty microseconds
    // after the event, which is as long as the pull itself takes
    for (;;) {
      const hipError_t e = hipEventQuery(st->packed);
      if (e == hipSuccess) return SG_OK;
      if (e != hipErrorNotReady) return SG_E_HIP;
      __builtin_ia32_pause();
    }
  }

 public:
  int last_rc = SG_OK;  // result of the most recent call (the virtuals return nothing)
  // How a batched call's tables reach the device, by the call's number of fragments (frames).
  // Below pull_min_items the calling thread walks them (0.65 ns per fragment), and a call of up to
  // in_place_max_bytes of tables leaves them in the pinned stage, where the kernels read them;
  // from pull_min_items on the device pulls them beside the copy of the call before (see pull():
  // some 30 us of launch, bus and wait however small the call, hidden behind a large copy).
  size_t pull_min_items = 49152;
  size_t in_place_max_bytes = 128 * 1024;
  // PROFILE_MODE: nanoseconds the calling thread spent inside each batched call (table building
  // and launches; the copy itself runs on after the call returns)
  std::vector<uint64_t> GBatchHostNs, SBatchHostNs;

  explicit P2pRpcSgHipEngine(int _device_id, uint32_t _max_reqs = 4096, uint32_t _max_frames = 65536,
                             void *stream = nullptr)
      : max_reqs(_max_reqs), max_frames(_max_frames)
  {
    device_id = _device_id;
    sg_hip_cfg cfg{sizeof(sg_hip_cfg), max_reqs, max_frames, 0, stream};
    ctx = sg_hip_create(device_id, &cfg);
    if (ctx) {
      // the scatter side on a stream of its own, on another hardware queue than the gather's
      OnDevice on(device_id);
      uint64_t q_g = 0;
      (void)sg_hip_stream_queue(ctx, nullptr, &q_g);
      tx_stream = stream_apart(&q_g, 1, &tx_queue_shared);
    }
    sg_hip_cfg cfg_tx{sizeof(sg_hip_cfg), max_reqs, max_frames, 0, tx_stream};
    ctx_tx = ctx ? sg_hip_create(device_id, &cfg_tx) : nullptr;
    if (!ctx || !ctx_tx) {
      // nothing can be moved without the device: say so and stop, as checkCudaErrors did
      std::printf("P2pRpcSgHipEngine: cannot start on device %d: %s\n", device_id, sg_hip_last_error(nullptr));
      std::exit(1);
    }
  }

  ~P2pRpcSgHipEngine() override
  {
    OnDevice on(device_id);
    (void)sg_hip_sync(ctx);
    (void)sg_hip_sync(ctx_tx);
    if (pack_stream) {
      (void)hipStreamSynchronize(pack_stream);
      (void)hipStreamDestroy(pack_stream);
    }
    for (auto &pair : stage)
      for (Stage &s : pair) {
        if (s.h) (void)hipHostFree(s.h);
        if (s.d) (void)hipFree(s.d);
        if (s.ev) (void)hipEventDestroy(s.ev);
        if (s.packed) (void)hipEventDestroy(s.packed);
      }
    if (tables) (void)hipHostFree(tables);
    sg_hip_destroy(ctx_tx);
    if (tx_stream) (void)hipStreamDestroy(tx_stream);
    sg_hip_destroy(ctx);
#ifdef PROFILE_MODE
    PROF_PRINT("GatherBatch-host", GBatchHostNs);
    PROF_PRINT("ScatterBatch-host", SBatchHostNs);
#endif
  }

  sg_hip_ctx *context() { return ctx; }        // gather side; calls with ready-made argument blocks
  sg_hip_ctx *tx_context() { return ctx_tx; }  // scatter side of the calls that take P2pRpcRr objects
  int sync()
  {
    const int a = sg_hip_sync(ctx), b = sg_hip_sync(ctx_tx);
    return last_rc = a != SG_OK ? a : b;
  }

  // `n` fragment tables in pinned host memory that this engine's device reads in place
  // (allocated once; a later call returns the same tables if they are enough, else nullptr).
  // Hand them to the request pool (P2pRpcRRPool::attach_frag_tables): the receive thread then
  // keeps them as it files fragments, and the batched calls below pull them from the device
  // instead of walking every fragment on the host.
  sg_frag_table *frag_tables(uint32_t n)
  {
    if (tables) return n <= n_tables ? tables : nullptr;
    OnDevice on(device_id);
    if (hipHostMalloc((void **)&tables, sizeof(sg_frag_table) * (size_t)n, hipHostMallocDefault) != hipSuccess) {
      tables = nullptr;
      return nullptr;
    }
    // the pull has to run BESIDE the copies: a stream on a hardware queue of its own
    uint64_t q[2] = {0, 0};
    (void)sg_hip_stream_queue(ctx, nullptr, &q[0]);
    (void)sg_hip_stream_queue(ctx_tx, nullptr, &q[1]);
    pack_stream = stream_apart(q, 2, &pack_queue_shared);
    if (!pack_stream) {
      (void)hipHostFree(tables);
      tables = nullptr;
      return nullptr;
    }
    std::memset(tables, 0xff, sizeof(sg_frag_table) * (size_t)n);
    n_tables = n;
    return tables;
  }

  // ---- the reference's four calls: one request, synchronous ----
  inline void gather(P2pRpcRr *rpc_rr, g_params *app_stub) override { gather(rpc_rr, app_stub->req); }
  inline void scatter(P2pRpcRr *rpc_rr, g_params *app_stub) override { scatter(rpc_rr, app_stub->resp); }

  inline void gather(P2pRpcRr *rpc_rr, uint8_t *payload) override
  {
#ifdef PROFILE_MODE
    GStartNs = getCurNs();
#endif
    gather_skbs(rpc_rr->payload_sk_bufs, rpc_rr->payload_bufs, payload);
    last_rc = sg_hip_gather(ctx, reinterpret_cast<const sg_sk_buf *>(rpc_rr->payload_sk_bufs));
#ifdef PROFILE_MODE
    GDelay.push_back(getCurNs() - GStartNs);
    numSkbs.push_back(rpc_rr->payload_sk_bufs->num_items);
#endif
    if (last_rc != SG_OK) fail("gather", last_rc);
  }

  inline void scatter(P2pRpcRr *rpc_rr, uint8_t *payload) override
  {
#ifdef PROFILE_MODE
    SStartNs = getCurNs();
#endif
    scatter_skbs(rpc_rr->payload_sk_bufs, rpc_rr->payload_bufs, payload);
    last_rc = sg_hip_scatter(ctx_tx, reinterpret_cast<const sg_sk_buf *>(rpc_rr->payload_sk_bufs));
#ifdef PROFILE_MODE
    SDelay.push_back(getCurNs() - SStartNs);
#endif
    if (last_rc != SG_OK) fail("scatter", last_rc, ctx_tx);
  }

  // Header rewrite of one response on the GPU (rr_swap_hdr with device memory,
  // src/transport/dpdk_transport_ng.h:157-159, left unimplemented there).
  inline void swap_hdrs(P2pRpcRr *rpc_rr, uint32_t hdr_profile, size_t payload_size, uint32_t mtu, uint32_t flags)
  {
    last_rc = sg_hip_swap_hdrs(ctx, reinterpret_cast<const sg_hbufs *>(rpc_rr->hdr_bufs), hdr_profile,
                               payload_size, mtu, flags);
    if (last_rc != SG_OK) fail("swap_hdrs", last_rc);
  }

  // Headers of a freshly allocated response from the connection template
  // (rr_set_hdr, src/transport/dpdk_transport_ng.h:113-141), written on the GPU.
  inline void set_hdrs(const p2p_rpc_conn_info *conn, P2pRpcRr *rpc_rr, uint32_t hdr_profile, size_t payload_size,
                       uint32_t mtu, uint32_t flags)
  {
    last_rc = sg_hip_set_hdrs(ctx, reinterpret_cast<const sg_hbufs *>(rpc_rr->hdr_bufs),
                              reinterpret_cast<const uint8_t *>(&conn->hdr_template), rpc_rr->req_token,
                              hdr_profile, payload_size, mtu, flags);
    if (last_rc != SG_OK) fail("set_hdrs", last_rc);
  }

  // ---- batched: every ready request in one call ----
  // With tables that are on the device already (what reassemble() leaves there).
  int gather_batch(const sg_gather_args *a)
  {
    last_rc = sg_hip_gather_batch(ctx, a);
    if (last_rc != SG_OK) fail("gather_batch", last_rc);
    return last_rc;
  }
  int scatter_batch(const sg_scatter_args *a)
  {
    last_rc = sg_hip_scatter_batch(ctx, a);
    if (last_rc != SG_OK) fail("scatter_batch", last_rc);
    return last_rc;
  }

  // The receive thread's per-packet work for one burst, on the device
  // (rr_recv_ng + get_rr + rr_emplace_mbuf + is_rr_ready,
  // src/transport/dpdk_transport_ng.h:176-218): requests that the burst
  // completes come out as tables gather_batch(const sg_gather_args *) takes;
  // the others stay on the device for later bursts.  counts (4 words or
  // nullptr): requests, fragments, arrivals dropped, requests in flight.
  int reassemble(const sg_reassemble_args *a, uint32_t *counts)
  {
    last_rc = sg_hip_reassemble(ctx, a, counts);
    if (last_rc != SG_OK) fail("reassemble", last_rc);
    return last_rc;
  }

  // Gathers n requests whose payload pointers lie in `ring` into `app`
  // (consecutive bump-ring positions or tensor-major buffers), in the order
  // given (src/splitrpc_server/p2p_rpc_dpdk_server.cc:117-150 for every ready
  // request at once).  fixed_req_size / rule_mtu as in sg_gather_args.  Returns
  // SG_OK or the error; `flags` may carry SG_F_ASYNC.  slot_state (or nullptr)
  // and n_slot_states as in sg_gather_args.
  // Where every request keeps a fragment table of this engine's (frag_tables())
  // the host names the tables -- two words per request -- and the device pulls
  // them on a stream of its own, beside the copy of the call before; otherwise the
  // host turns every payload pointer into its slot index and ships the result.
  int gather_batch(P2pRpcRr *const *rrs, uint32_t n, const SgRingView &ring, const sg_app_desc &app,
                   uint64_t *offsets_out_dev, uint64_t fixed_req_size, uint32_t rule_mtu, uint32_t flags,
                   uint32_t *slot_state = nullptr, uint32_t n_slot_states = 0)
  {
#ifdef PROFILE_MODE
    const uint64_t t0 = getCurNs();
#endif
    size_t n_frags = 0;
    for (uint32_t r = 0; r < n; r++) n_frags += rrs[r]->payload_bufs->num_items;
    if (n > max_reqs || n_frags > max_frames) return last_rc = SG_E_INVAL;
    if (n == 0) return last_rc = SG_OK;
    OnDevice on(device_id);
    const bool pulled = n_frags >= pull_min_items && can_pull(rrs, n, ring);
    const bool lens_from_headers = pulled && ring.desc.hdr_profile == SG_HDR_BL58;
    const size_t d_words = 2 * n_frags + n + 1;
    Stage *st = take_stage(0, pulled ? 2 * (size_t)n + 1 : d_words, d_words);
    if (!st) return last_rc = SG_E_NOMEM;
    const uint32_t *dv = st->d;  // where the kernels read the tables
    if (pulled) {
      uint32_t *idx = st->h, *first = st->h + n;
      uint32_t f = 0;
      for (uint32_t r = 0; r < n; r++) {
        idx[r] = (uint32_t)(rrs[r]->frag_table - tables);
        first[r] = f;
        f += rrs[r]->payload_bufs->num_items;
      }
      first[n] = f;
      sg_pack_args pa;
      std::memset(&pa, 0, sizeof pa);
      pa.n_req = n;
      pa.table_idx = idx;
      pa.req_first = first;
      pa.n_frags = (uint32_t)n_frags;
      pa.pkt_base = rrs[0]->pkt_base;
      pa.ring = ring.desc;
      pa.frag_slot = st->d;
      // the 58-byte header carries every fragment's length, which is where the receive path took
      // item_size from: the kernels read it there, and half the bytes stay off the bus
      pa.frag_len = lens_from_headers ? nullptr : st->d + n_frags;
      pa.req_first_out = st->d + 2 * n_frags;
      last_rc = pull(st, &pa);
      if (last_rc != SG_OK) {
        fail("pack_tables", last_rc);
        return last_rc;
      }
    } else {
      uint32_t *slot = st->h, *len = st->h + n_frags, *first = st->h + 2 * n_frags;
      size_t f = 0;
      const SgRingView::Walk slot_of = ring.walk();
      for (uint32_t r = 0; r < n; r++) {
        const p2p_bufs *b = rrs[r]->payload_bufs;
        first[r] = (uint32_t)f;
        for (int i = 0; i < b->num_items; i++, f++) {
          const int64_t s = slot_of(b->burst_items[i]);
          if (s < 0) return last_rc = SG_E_INVAL;
          slot[f] = (uint32_t)s;
          len[f] = (uint32_t)b->item_size[i];
        }
      }
      first[n] = (uint32_t)f;
      // a small call's tables stay where they are: the kernels read the pinned stage across the bus
      // (a few tens of KB), which saves the launch that would bring them over and the wait for it
      if (d_words * 4 <= in_place_max_bytes) dv = st->h;
      else if (!send_stage(st, d_words, 0)) return last_rc = SG_E_HIP;
    }
    sg_gather_args a;
    std::memset(&a, 0, sizeof a);
    a.ring = ring.desc;
    a.frag_slot = dv;
    a.frag_len = lens_from_headers ? nullptr : dv + n_frags;
    a.req_first = dv + 2 * n_frags;
    a.n_req = n;
    a.n_frags = (uint32_t)n_frags;
    a.app = app;
    a.offsets_out = offsets_out_dev;
    // (asking large calls to advance the cursor themselves, SG_F_SELF_ADVANCE, so that no kernel trails
    // the call, was measured here: 116 -> 119 us per step of 512 requests in 220672 fragments; more than
    // two stages per direction change nothing: the thread already waits for the device, not the reverse)
    a.flags = flags | (rule_mtu && fixed_req_size ? SG_F_RULE_FRAGS : 0u);
    a.mtu = rule_mtu;
    a.fixed_req_size = fixed_req_size;
    a.slot_state = slot_state;
    a.n_slot_states = n_slot_states;
    last_rc = sg_hip_gather_batch(ctx, &a);
    stage_in_use(st, 0);
#ifdef PROFILE_MODE
    GBatchHostNs.push_back(getCurNs() - t0);
#endif
    if (last_rc != SG_OK) fail("gather_batch", last_rc);
    return last_rc;
  }

  // The TX half for n requests at once (src/splitrpc_server/p2p_rpc_dpdk_server.cc:158-189 for
  // every WORK_COMPLETE slot): the response of rrs[k] is read from `app` (next bump-ring positions
  // or tensor-major buffers), cut at `mtu` into the response buffers rrs[k]->payload_bufs names
  // (rr_alloc_mbufs has put them there; they lie in `tx`), and every frame's header is written
  // from the request's connection template with its token, sequence number, lengths and the sums
  // `flags` asks for (rr_set_hdr, src/transport/dpdk_transport_ng.h:113-141) -- payload and
  // headers in one kernel.  The response size of a request is what its buffers add up to
  // (P2pRpcRr::payload_size, which rr_append_mbuf keeps).  Tables are pulled by the device where
  // the requests keep them, as in gather_batch; tokens, sizes and templates (80 bytes per request)
  // are written by the host either way.
  int scatter_batch(P2pRpcRr *const *rrs, uint32_t n, const SgRingView &tx, const sg_app_desc &app, uint32_t mtu,
                    uint32_t flags, uint32_t *slot_state = nullptr, uint32_t n_slot_states = 0)
  {
#ifdef PROFILE_MODE
    const uint64_t t0 = getCurNs();
#endif
    size_t n_frames = 0;
    for (uint32_t r = 0; r < n; r++) n_frames += rrs[r]->payload_bufs->num_items;
    if (n > max_reqs || n_frames > max_frames) return last_rc = SG_E_INVAL;
    if (n == 0) return last_rc = SG_OK;
    OnDevice on(device_id);
    const bool pulled = n_frames >= pull_min_items && can_pull(rrs, n, tx);
    // device: u32 tx_slot[n_frames], u32 first[n + 1], pad to 8 bytes, then the per-request words:
    // u64 token[n], u64 size[n], u8 template[64 n]
    const size_t w32 = (n_frames + n + 1 + 1) & ~(size_t)1;
    const size_t per_req_words = 2 * (size_t)n + 2 * n + 16 * n;
    const size_t d_words = w32 + per_req_words;
    // host, pulled: u32 idx[n], u32 first[n + 1], pad, the per-request words; else the device's image
    const size_t h32 = pulled ? ((2 * (size_t)n + 1 + 1) & ~(size_t)1) : w32;
    Stage *st = take_stage(1, h32 + per_req_words, d_words);
    if (!st) return last_rc = SG_E_NOMEM;
    uint64_t *token = reinterpret_cast<uint64_t *>(st->h + h32), *size = token + n;
    uint8_t *tmpl = reinterpret_cast<uint8_t *>(size + n);
    uint32_t *slot = st->h, *first = pulled ? st->h + n : st->h + n_frames;
    size_t f = 0;
    bool one_size = true;
    const SgRingView::Walk slot_of = tx.walk();
    for (uint32_t r = 0; r < n; r++) {
      const p2p_bufs *b = rrs[r]->payload_bufs;
      first[r] = (uint32_t)f;
      uint64_t total = 0;
      if (pulled) {
        slot[r] = (uint32_t)(rrs[r]->frag_table - tables);
        total = rrs[r]->payload_size;
        f += b->num_items;
      } else {
        for (int i = 0; i < b->num_items; i++, f++) {
          const int64_t s = slot_of(b->burst_items[i]);
          if (s < 0) return last_rc = SG_E_INVAL;
          slot[f] = (uint32_t)s;
          total += b->item_size[i];
        }
      }
      size[r] = total;
      one_size = one_size && total == size[0];
      token[r] = rrs[r]->req_token;
      std::memcpy(tmpl + 64 * (size_t)r, &rrs[r]->_client_conn_info.hdr_template, 64);
    }
    first[n] = (uint32_t)f;
    const uint32_t *dv = st->d;  // where the kernels read the tables
    if (pulled) {
      sg_pack_args pa;
      std::memset(&pa, 0, sizeof pa);
      pa.n_req = n;
      pa.table_idx = slot;
      pa.req_first = first;
      pa.n_frags = (uint32_t)n_frames;
      pa.pkt_base = rrs[0]->pkt_base;
      pa.ring = tx.desc;
      pa.frag_slot = st->d;
      pa.req_first_out = st->d + n_frames;
      pa.blob_src = st->h + h32;
      pa.blob_dst = st->d + w32;
      pa.blob_words = (uint32_t)per_req_words;
      last_rc = pull(st, &pa);
      if (last_rc != SG_OK) {
        fail("pack_tables", last_rc);
        return last_rc;
      }
    } else if (d_words * 4 <= in_place_max_bytes) {
      dv = st->h;  // a small call: read in place, as in gather_batch
    } else if (!send_stage(st, d_words, 1)) {
      return last_rc = SG_E_HIP;
    }
    sg_scatter_args a;
    std::memset(&a, 0, sizeof a);
    a.rx = tx.desc;  // headers come from templates: no request ring is read
    a.tx = tx.desc;
    a.tx_slot = dv;
    a.resp_first = dv + n_frames;
    const uint64_t *d64 = reinterpret_cast<const uint64_t *>(dv + w32);
    a.req_token = d64;
    a.resp_size = one_size ? nullptr : d64 + n;
    a.fixed_resp_size = one_size ? size[0] : 0;
    a.hdr_templates = reinterpret_cast<const uint8_t *>(d64 + 2 * n);
    a.n_req = n;
    a.n_frames = (uint32_t)n_frames;
    a.mtu = mtu;
    a.flags = flags;
    a.app = app;
    a.slot_state = slot_state;
    a.n_slot_states = n_slot_states;
    last_rc = sg_hip_scatter_batch(ctx_tx, &a);
    stage_in_use(st, 1);
#ifdef PROFILE_MODE
    SBatchHostNs.push_back(getCurNs() - t0);
#endif
    if (last_rc != SG_OK) fail("scatter_batch", last_rc, ctx_tx);
    return last_rc;
  }
};
