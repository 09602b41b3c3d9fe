/*
 * sg_hip.h -- C ABI of the MI355X (gfx950) scatter-gather engine.
 *
 * Drop-in boundary for SplitRPC's p2p_rpc_sg_engine path.  Plain C: pointers
 * and sizes only.  Every pointer named "device" must be addressable by the
 * GPU the context was created on (hipMalloc, VMM mapping, or pinned host
 * memory); the library never allocates or frees payload memory.
 *
 * Reads around a run.  The copy kernels load 16-byte chunks at 16-byte aligned
 * addresses whatever the address of a run (a fragment's payload, a piece of a
 * tensor): up to 15 bytes before the first and after the last byte of a run are
 * read, and discarded, when they share such a chunk with bytes of the run.  A
 * chunk never spans a page, so whatever memory holds the run holds every byte
 * that is read; nothing outside a run is ever written.
 *
 * Return convention: 0 on success, a negative SG_E_* code on failure (the
 * reference's sg_on_gpu returns 1/0, src/transport/g_copy_ng.cu:169-223; the
 * C++ engine above this ABI keeps that convention for its callers).
 * sg_hip_last_error() gives the text of the last failure on a context.
 * No exceptions cross the ABI.  A context is used by one thread at a time
 * (the reference constructs and uses its engine on the shunter thread,
 * src/splitrpc_server/p2p_rpc_dpdk_server.cc:79-87); different contexts may
 * be used from different threads at the same time (a shunter thread per
 * receive queue, each with a context of its own).
 */
#ifndef SG_HIP_H
#define SG_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SG_HIP_ABI_VERSION 3

/* Error codes. */
#define SG_OK 0
#define SG_E_INVAL (-22)   /* bad argument, size beyond what the context was sized for */
#define SG_E_NOMEM (-12)   /* context scratch could not be allocated */
#define SG_E_HIP (-5)      /* a HIP call failed; see sg_hip_last_error() */
#define SG_E_DATA (-74)    /* a kernel found tables or headers it refused to follow
                              (slot index out of range, length beyond the slot, ...) */

/* Wire-header profiles.  REF64 is the reference's p2p_rpc_hdr
 * (src/p2p_rpc.h:10-17): 42 B Eth/IPv4/UDP, u64 req_token @42,
 * i64 sock_perf_header @50, u16 seq_num @58, pad to 64; payload @64.
 * BL58: u64 req_id @42, u16 frag_idx @50, u16 num_frags @52,
 * u32 payload_len @54; payload @58. */
#define SG_HDR_BL58 0u
#define SG_HDR_REF64 1u

/* Flags. */
#define SG_F_IPV4_CSUM (1u << 0)       /* finished IPv4 header checksum (RFC 1071); the
                                          reference leaves it to the NIC,
                                          src/transport/dpdk_rx_tx.h:143 */
#define SG_F_UDP_CSUM_PSEUDO (1u << 1) /* raw pseudo-header sum in udp.check, as
                                          add_udp_cksum does, src/p2p_rpc.h:58-61 */
#define SG_F_UDP_CSUM_FULL (1u << 2)   /* finished UDP checksum over header + payload (RFC 768) */
#define SG_F_REF_QUIRKS (1u << 3)      /* pseudo sum takes UDP length as tot_len - version*4,
                                          src/eth_common.h:111-112 */
#define SG_F_RULE_FRAGS (1u << 4)       /* gather: the caller states that every request has
                                          fixed_req_size bytes cut by the fragmenting rule at mtu
                                          (all fragments mtu bytes, the last the remainder,
                                          src/transport/dpdk_rx_tx.h:137-139).  Offsets are then
                                          multiples and no descriptor pass runs; every fragment's
                                          real length is held against the rule and a batch that
                                          departs from it is refused with SG_E_DATA (its
                                          destination bytes are then undefined). */
#define SG_F_NO_FUSE (1u << 5)          /* scatter: run the descriptor pass even where the copy
                                          kernel could derive the descriptors (for experiments) */
#define SG_F_REUSE_DESC (1u << 6)       /* scatter: the frames of this call are the fragments the latest
                                          gather call with a descriptor pass on this context described --
                                          same slots (tx_slot == its frag_slot), same lengths, same
                                          requests in the same arena (an echo, answered in place or not):
                                          its descriptors and arena offsets are used as they stand and no
                                          descriptor pass runs.  Held against what that pass recorded: its
                                          counts, its arena (base and capacity) and the slot size its
                                          lengths were checked against -- a call with other counts, another
                                          arena or a TX ring of smaller slots moves nothing -- and every
                                          frame against this call's TX ring and mtu; either way the call
                                          reports SG_E_DATA.  resp_size is not read; the response cursor
                                          ends up where the request cursor did */
#define SG_F_ASYNC (1u << 16)          /* enqueue only; completion through sg_hip_sync() */
#define SG_F_NO_XCD_REMAP (1u << 17)   /* launch-order = item order (for experiments) */
#define SG_F_NO_SMALL (1u << 18)       /* one wavefront per frame even for short frames (for experiments) */
#define SG_F_FORCE_SMALL (1u << 19)    /* short remainder frames always go several to a wavefront, also where
                                          the call is too small for the extra launch to pay (for tests) */
#define SG_F_SELF_ADVANCE (1u << 20)   /* a call whose copy kernel derives its offsets from the bump-ring
                                          cursor has that kernel advance the cursor too, whatever the
                                          call's size, instead of a one-workgroup kernel behind it: one
                                          graph node fewer per call.  The library picks this by itself for
                                          calls of few wavefronts; a call that publishes slot states
                                          always has the kernel behind it. */
#define SG_F_TAIL_KERNEL (1u << 21)    /* the opposite: always the kernel behind the call (for experiments) */
#define SG_F_SMALL_GROUPS (1u << 22)   /* sg_hip_reassemble: the call is meant to run BESIDE a long copy
                                          kernel of another stream (another receive queue's gather, or
                                          this queue's previous burst): its kernels then come in
                                          workgroups of 256 threads, which find room on a chip that such a
                                          kernel keeps full, where the usual ones of 1024 wait until it
                                          ends.  Same results.  A call that runs alone is faster without. */

/* States of an application slot (APP_RR_STATUS, src/p2p_rpc_app_ctx.h:22). */
#define SG_SLOT_FREE 0u
#define SG_SLOT_RX_COMPLETE 1u
#define SG_SLOT_WORK_COMPLETE 2u
#define SG_SLOT_TX_COMPLETE 3u

#define SG_MAX_BI_SIZE 1024 /* src/p2p_bufs.h:10 */
#define SG_MAX_TENSORS 4    /* src/p2p_rpc_app_stub.h:10 */

/* Layout twins of the reference's fixed tables (src/p2p_bufs.h:15-40), so a
 * P2pRpcRr's tables can be handed over without conversion. */
#pragma pack(push, 1)
typedef struct sg_hbufs {
  uint64_t burst_items[SG_MAX_BI_SIZE];
  uint16_t num_items;
} sg_hbufs; /* == p2p_hbufs, 8194 B */

typedef struct sg_sk_buf {
  uint64_t i_buf[SG_MAX_BI_SIZE];
  uint64_t o_buf[SG_MAX_BI_SIZE];
  uint64_t len[SG_MAX_BI_SIZE - 1];
  uint64_t num_items;
} sg_sk_buf; /* == p2p_sk_buf == g_copy_params, 24576 B */
#pragma pack(pop)

typedef struct sg_hip_ctx sg_hip_ctx;

typedef struct sg_hip_cfg {
  uint32_t struct_size; /* sizeof(sg_hip_cfg), for ABI growth */
  uint32_t max_reqs;    /* largest n_req of one batch call (0: 4096) */
  uint32_t max_frames;  /* largest fragment / response-frame count of one batch call (0: 65536) */
  uint32_t flags;       /* reserved, 0 */
  void *stream;         /* hipStream_t to launch on; NULL: the context creates one */
} sg_hip_cfg;

/* A ring of packet-buffer slots in device memory. */
typedef struct sg_ring_desc {
  void *base;           /* device */
  uint32_t n_slots;
  uint32_t slot_size;   /* bytes, even */
  uint32_t hdr_profile; /* SG_HDR_* */
  uint32_t reserved;
} sg_ring_desc;

/* Where request bytes go and response bytes come from.
 * n_tensors == 0: one packed arena addressed through the device-resident
 * bump ring (P2pRpcTring::get_next, src/p2p_rpc_tring.h:27-33): request r
 * starts where request r-1 ended, modulo arena_cap.  arena_mirrored != 0
 * says the arena's pages are mapped twice back to back
 * (src/p2p_rpc_app_rr_mem_pool.h:302-306) so that [arena, arena + 2*cap) is
 * addressable and a request may run past the end; otherwise a run that
 * crosses the end is split.  The requests of one gather call must fit the
 * arena together (the reference's slot states guarantee as much,
 * src/p2p_rpc_app_rr.h:127-134): a larger batch would overwrite its own first
 * requests and is refused.
 * n_tensors >= 1: tensor-major buffers in the sense of g_params_v2
 * (src/p2p_rpc_app_stub.h:11-20): a request's byte stream is tensor 0's
 * bytes, then tensor 1's, ...; tensor t of request r lives at
 * tensor_base[t] + r * tensor_size[t]. */
typedef struct sg_app_desc {
  void *tensor_base[SG_MAX_TENSORS]; /* device */
  uint64_t tensor_size[SG_MAX_TENSORS];
  uint32_t n_tensors;
  uint32_t arena_mirrored;
  void *arena; /* device */
  uint64_t arena_cap;
} sg_app_desc;

/* One gather batch: the fragment tables of n_req reassembled requests in
 * compact CSR form (what P2pRpcRr::payload_bufs holds per request,
 * src/p2p_rpc_rr_ng.h:29-31, with pointers reduced to slot indices).
 * "device" below is memory the device can read: device memory, or -- for the
 * tables of a small call, a few tens of KB -- pinned host memory, which the
 * kernels then read across the bus (that saves the copy and the launch that
 * makes it; tables of large calls belong in device memory: bus reads in
 * flight beside a copy kernel slow it down).  The same holds for the tables of
 * sg_scatter_args. */
typedef struct sg_gather_args {
  sg_ring_desc ring;
  const uint32_t *frag_slot; /* device, n_frags: ring slot of each fragment; requests in
                                batch order, fragments in seq order inside a request */
  const uint32_t *frag_len;  /* device, n_frags payload bytes, or NULL: read payload_len
                                from each slot's header (BL58 only) */
  const uint32_t *req_first; /* device, n_req + 1: first fragment of each request */
  uint32_t n_req;
  uint32_t n_frags;
  sg_app_desc app;
  uint64_t *offsets_out; /* device, n_req + 1 arena offsets (packed mode), or NULL */
  uint32_t flags;
  uint32_t mtu;            /* payload bytes per full fragment; used with SG_F_RULE_FRAGS */
  uint64_t fixed_req_size; /* non-zero: every request must total exactly this many bytes (the
                              reference's server-wide request size, is_rr_ready,
                              src/p2p_rpc_rr_ng.h:107-110); a batch holding another size is
                              refused with SG_E_DATA.  0: sizes are whatever the fragments add
                              up to and offsets come from a prefix scan */
  /* Counts that stay on the device: [0] requests, [1] fragments, as
   * sg_hip_reassemble leaves them in sg_reassemble_args.counts_out.  n_req and
   * n_frags above are then upper bounds that size the launches (a count beyond
   * its bound is refused with SG_E_DATA); no host synchronization sits between
   * the reassembly and this call.  NULL: n_req and n_frags are the counts. */
  const uint32_t *counts; /* device, or NULL */
  /* Application slot ring (the h_state words of P2pRpcAppRrPool,
   * src/p2p_rpc_app_rr.h:15-46,127-134): request k of the batch fills slot
   * (producer index + k) mod n_slot_states; once the batch is in place a kernel
   * behind the copy kernel sets those words from SG_SLOT_FREE to
   * SG_SLOT_RX_COMPLETE (what the shunter does at
   * src/splitrpc_server/p2p_rpc_dpdk_server.cc:130) and advances the producer
   * index, which lives on the device (sg_hip_set_slot_index).  A slot found in
   * another state is still overwritten and the call reports SG_E_DATA: the
   * caller keeps at most n_slot_states requests between gather and scatter, as
   * the reference's flow control does (:117).  A call that refuses any part of
   * its input (SG_E_DATA) publishes no states and leaves the index where it
   * was.  The words may live in device memory or in pinned host memory the
   * worker's loop polls.  NULL: no ring. */
  uint32_t *slot_state; /* device-addressable, n_slot_states words, or NULL */
  uint32_t n_slot_states;
  uint32_t reserved2;
} sg_gather_args;

/* One scatter batch.  Response r has resp_size[r] bytes (fixed_resp_size when
 * resp_size is NULL), cut into frames of at most mtu bytes by the reference's
 * fragmenting rule (src/transport/dpdk_rx_tx.h:137-139).  Frame f of the
 * batch is written to TX slot tx_slot[f]; its header is the header found in
 * RX slot hdr_src_slot[f], rewritten (swap_eth_hdr + add_ip_udp_len +
 * add_udp_cksum, src/p2p_rpc.h:51-83, and the routing fields rr_set_hdr
 * writes, src/transport/dpdk_transport_ng.h:129-131).  tx may alias rx; then
 * hdr_src_slot[f] must equal tx_slot[f] or be a slot no frame of the batch
 * writes. */
typedef struct sg_scatter_args {
  sg_ring_desc rx;
  sg_ring_desc tx;
  const uint32_t *tx_slot;      /* device, n_frames */
  const uint32_t *hdr_src_slot; /* device, n_frames */
  const uint32_t *resp_first;   /* device, n_req + 1 */
  const uint64_t *resp_size;    /* device, n_req, or NULL */
  uint64_t fixed_resp_size;
  uint32_t n_req;
  uint32_t n_frames;
  uint32_t mtu;
  uint32_t flags; /* SG_F_* */
  sg_app_desc app;
  uint64_t *offsets_out; /* device, n_req + 1, or NULL */
  /* Headers from connection templates instead of from request headers: what
   * rr_set_hdr does for freshly allocated response buffers
   * (src/transport/dpdk_transport_ng.h:113-141).  hdr_templates holds one
   * 64-byte template per request (P2pRpcRr::_client_conn_info.hdr_template,
   * already pointing at the client: set_conn_info, src/p2p_rpc_conn_info.h:73-84);
   * frame i of request r gets a copy of template r with token req_token[r]
   * (the template's own when req_token is NULL), seq_num / frag_idx i,
   * lengths and sums.  Nothing is swapped and hdr_src_slot is not read. */
  const uint8_t *hdr_templates; /* device, n_req * 64 bytes at an even address, or NULL: swap request headers */
  const uint64_t *req_token;    /* device, n_req, or NULL */
  /* One header source per request instead of one per frame: every frame of
   * response r answers the header in RX slot hdr_src_req[r] (what
   * sg_hip_reassemble leaves in req_hdr_slot).  Used when hdr_src_slot is NULL. */
  const uint32_t *hdr_src_req; /* device, n_req, or NULL */
  /* Device-resident request count, as in sg_gather_args: counts[0] responses
   * are served, n_req and n_frames are upper bounds (frame tables must be
   * valid up to the bounds). */
  const uint32_t *counts;      /* device, or NULL */
  /* Application slot ring: the n_req slots from the consumer index on
   * (sg_hip_set_slot_index, which = 1) are expected in SG_SLOT_WORK_COMPLETE;
   * behind the copy kernel they are set to SG_SLOT_FREE
   * (src/splitrpc_server/p2p_rpc_dpdk_server.cc:158-175) and the index advances. */
  uint32_t *slot_state;        /* device-addressable, n_slot_states words, or NULL */
  uint32_t n_slot_states;
  uint32_t reserved2;
} sg_scatter_args;

/* One burst of arrivals to sort into requests on the device.  Replaces the
 * per-packet work of the receive thread: get_rr / rr_emplace_mbuf /
 * is_rr_ready / mark_rx_ready_rr (src/p2p_rpc_rr_pool_ng.h:97-119,149-155;
 * src/transport/dpdk_transport_ng.h:176-252, one NIC burst per call).  A
 * request is complete when num_frags fragments are in (BL58) or when its
 * payload bytes reach req_size (REF64, src/p2p_rpc_rr_ng.h:107-110).  Requests
 * that are still incomplete stay on the device, as rr_cache keeps them
 * (src/p2p_rpc_rr_pool_ng.h:97-119), and complete in whichever later call
 * brings their last fragment; up to max_reqs of the context may be in flight.
 * The requests completed by a call come out in completion order -- the order
 * in which their last fragment arrived, which is the order of the reference's
 * rx-ready ring -- as the CSR tables sg_hip_gather_batch takes, fragments of
 * earlier calls included, so the output tables need room for max_frames
 * fragments and max_reqs requests of the context.  Packets with token 0 are
 * dropped (:231).  As in the reference, duplicate fragments are not detected,
 * and a request holds at most SG_MAX_BI_SIZE fragments.  A token that comes
 * back within the burst that completes it is taken for the same request. */
typedef struct sg_reassemble_args {
  sg_ring_desc ring;
  const uint32_t *arrivals; /* device, n_arrivals: ring slots in arrival order */
  const uint32_t *len_nic;  /* device, n_slots: payload bytes of each slot as the NIC reports
                               them (required for REF64; NULL for BL58: read from the header) */
  uint32_t n_arrivals;      /* arrivals of this call; their upper bound with n_arrivals_dev */
  uint32_t flags;           /* SG_F_ASYNC: launch only, counts stay on the device */
  uint64_t req_size;        /* REF64: the server-wide request size */
  uint32_t *frag_slot;      /* device out, max_frames of the context */
  uint32_t *frag_len;       /* device out, max_frames of the context */
  uint32_t *req_first;      /* device out, max_reqs + 1 of the context */
  uint64_t *req_token;      /* device out, max_reqs, or NULL */
  uint32_t *req_hdr_slot;   /* device out, max_reqs, or NULL: the slot of each request's fragment 0,
                               whose header the responses answer (sg_scatter_args.hdr_src_req) */
  uint32_t *counts_out;     /* device out, 4 words, or NULL: requests completed, their fragments,
                               arrivals dropped, requests still in flight -- what
                               sg_gather_args.counts / sg_scatter_args.counts take */
  const uint32_t *n_arrivals_dev; /* device, or NULL: the arrival count when it is only known on
                                     the device (a burst whose length changes between graph replays) */
} sg_reassemble_args;

/* ---- lifetime -------------------------------------------------------------
 * Replaces P2pRpcSgGpuEngine's constructor/destructor work
 * (src/p2p_rpc_sg_engine.h:261-307: stubs, doorbells, streams, persistent
 * kernel start and stop).  No persistent kernel is started: work is launched
 * per call on the context's stream. */
sg_hip_ctx *sg_hip_create(int device_id, const sg_hip_cfg *cfg);
void sg_hip_destroy(sg_hip_ctx *ctx);
const char *sg_hip_last_error(const sg_hip_ctx *ctx); /* ctx may be NULL: creation errors */
int sg_hip_abi_version(void);
void *sg_hip_stream(sg_hip_ctx *ctx); /* the hipStream_t work is launched on */

/* The address of the hardware queue that `stream` (NULL: the context's own) dispatches to, as a
 * kernel launched on it sees it.  The runtime multiplexes streams over a handful of hardware
 * queues, and streams that share one run their kernels one after the other whatever the streams'
 * own order: a caller that wants two streams to run side by side (the pull of the next call's
 * tables beside the current call's copy) creates streams until two of them answer differently.
 * Launches a one-wavefront kernel on the stream and waits for it.  No counterpart in the reference. */
int sg_hip_stream_queue(sg_hip_ctx *ctx, void *stream, uint64_t *queue_out);

/* Waits for everything enqueued on the context and returns SG_E_DATA if any
 * kernel since the last sync refused part of its input. */
int sg_hip_sync(sg_hip_ctx *ctx);

/* ---- per-request entry points (API v0 / v1 parity) --------------------------
 * Replace sg_on_gpu(CopyCtx*, p2p_sk_buf*) + the doorbell wait
 * (src/transport/g_copy_ng.cu:186-223, src/p2p_rpc_sg_engine.h:198-239):
 * copy every run of a host-built run table; i_buf/o_buf hold device
 * addresses.  Synchronous: on return the bytes are in place. */
int sg_hip_gather(sg_hip_ctx *ctx, const sg_sk_buf *skb);
int sg_hip_scatter(sg_hip_ctx *ctx, const sg_sk_buf *skb);

/* Replaces do_g_pp(ctx, p2p_hbufs*) (src/transport/g_udp_handler.cuh:20-24,
 * g_udp_handler.cu:96-123,172-178) and swap_hdrs_on_cpu
 * (src/transport/dpdk_transport_ng.h:70-84): rewrite in place the headers a
 * table of device header pointers names; header i gets frag_idx i,
 * num_frags = num_items and payload_len = min(remaining, mtu) of
 * payload_size.  Synchronous. */
int sg_hip_swap_hdrs(sg_hip_ctx *ctx, const sg_hbufs *hdrs, uint32_t hdr_profile,
                     uint64_t payload_size, uint32_t mtu, uint32_t flags);

/* Replaces rr_set_hdr (src/transport/dpdk_transport_ng.h:113-141): fill the
 * headers of freshly allocated response buffers from a connection template.
 * hdr_template is a HOST pointer to the 64 bytes of
 * p2p_rpc_conn_info::hdr_template (src/p2p_rpc_conn_info.h:21-30); header i
 * becomes a copy of it with req_token, seq_num / frag_idx i, lengths and the
 * sums `flags` asks for.  Synchronous. */
int sg_hip_set_hdrs(sg_hip_ctx *ctx, const sg_hbufs *hdrs, const uint8_t *hdr_template,
                    uint64_t req_token, uint32_t hdr_profile, uint64_t payload_size, uint32_t mtu,
                    uint32_t flags);

/* ---- batched entry points ----------------------------------------------------
 * No counterpart call in the reference (which handles one request per
 * doorbell round trip, src/p2p_rpc_sg_engine.h:198-218); the per-request
 * semantics are those of P2pRpcSgCpuEngine::gather / scatter
 * (src/p2p_rpc_sg_engine.h:150-164) applied to every request of the batch,
 * with request offsets taken from the bump ring.  Synchronous unless
 * SG_F_ASYNC is set; an SG_F_ASYNC call does nothing on the stream but launch
 * kernels (no allocation, no copy, no memset).  The bump-ring cursor of an
 * arena lives on the device and only kernels advance it: the copy kernel where a
 * descriptor pass has read the cursor before it; where the copy kernel reads the
 * cursor itself (SG_F_RULE_FRAGS; scatter of one response size), that same
 * kernel for calls of up to 65536 wavefronts (it tells its own write from the
 * previous call's by the queue and dispatch id of its launch) and a
 * one-workgroup kernel behind it for larger calls and for calls that publish
 * slot states (SG_F_SELF_ADVANCE / SG_F_TAIL_KERNEL pick either).  Calls
 * recorded into a HIP graph -- any number of them, replayed from any stream --
 * therefore continue the ring on every replay.  Calls on one context must
 * not overlap in time (one stream, or streams ordered by events).
 * What a self-advancing launch knows itself by is its queue's address, its
 * dispatch id there and the context's own count of such calls; sg_hip_create
 * launches two probes and keeps to the kernel behind the call for good if the
 * runtime does not hand out distinct pairs.  A caller that brings its own
 * stream and destroys and re-creates it between calls needs nothing further:
 * the count goes on where the new queue's dispatch ids start over.
 *
 * The cursor after a refusal.  A call the host refuses (SG_E_INVAL) launches
 * nothing and leaves the cursor alone.  With a descriptor pass (no
 * SG_F_RULE_FRAGS; scatter with resp_size or SG_F_NO_FUSE) a batch the device
 * refuses (SG_E_DATA) moves nothing and does not advance the cursor.  Without
 * one (SG_F_RULE_FRAGS; scatter of one response size) the advance depends on
 * n_req and the size alone: the cursor moves by the whole batch, and
 * offsets_out is complete, even if a fragment was dropped for a bad slot index.
 * The refusal bits stay up until the next sg_hip_sync(): asynchronous
 * descriptor-pass calls queued behind a refused one move nothing either. */
int sg_hip_gather_batch(sg_hip_ctx *ctx, const sg_gather_args *args);
int sg_hip_scatter_batch(sg_hip_ctx *ctx, const sg_scatter_args *args);

/* One pass of the shunter's loop in one call: the gather of the requests that
 * became ready and the scatter of the responses that are done, which the
 * reference issues one after the other on every turn of shunter_loop
 * (src/splitrpc_server/p2p_rpc_dpdk_server.cc:117-150 and :158-189).  The
 * result is that of sg_hip_gather_batch(ctx, gather) followed by
 * sg_hip_scatter_batch(ctx, scatter).  Where both halves are single-kernel
 * calls on packed arenas whose kernels advance their cursors themselves
 * (SG_F_RULE_FRAGS gather of fragments of at most 2016 bytes, short last
 * fragments included; a scatter of one response size in frames of at most
 * 2016 bytes, or of frames of at most 128 bytes without the full UDP
 * checksum; no slot ring), the two together are no more wavefronts than the
 * chip holds at once (8192), and neither touches the other's memory (the TX
 * ring apart from the RX ring, the response buffers apart from the request
 * buffers), both travel in ONE launch: a call of a batch or two costs more
 * in launches than in bytes, and this halves them.  Any other pair of calls
 * is made as two calls, gather first (larger calls are faster that way, on a
 * stream each).  Synchronous unless both argument blocks carry SG_F_ASYNC. */
int sg_hip_shunt_batch(sg_hip_ctx *ctx, const sg_gather_args *gather, const sg_scatter_args *scatter);

/* Fragment tables the device reads where the receive thread writes them.
 * The reference's receive thread files every fragment in its request's table
 * as it arrives (P2pRpcRr::rr_emplace_mbuf, src/p2p_rpc_rr_ng.h:96-105) and the
 * shunter later walks those tables fragment by fragment on the host
 * (gather_skbs, src/p2p_rpc_sg_engine.h:19-45).  With one sg_frag_table per
 * request in memory the device can read (pinned host memory), written at the
 * same place in the same order, a batched call needs no per-fragment work on
 * the host: it names one table per request, and sg_hip_pack_tables pulls the
 * tables into the CSR arrays sg_hip_gather_batch / sg_hip_scatter_batch take.
 *   off[i]  (payload address of fragment i - pkt_base) / 2, pkt_base being any
 *           even address at or below the packet memory (8 GiB are in reach);
 *           0xffffffff: no such fragment
 *   len[i]  payload bytes of fragment i
 * An entry that is not the payload start of a slot of `ring` comes out as slot
 * 0xffffffff, which the batched calls refuse with SG_E_DATA. */
typedef struct sg_frag_table {
  uint32_t off[SG_MAX_BI_SIZE];
  uint32_t len[SG_MAX_BI_SIZE];
} sg_frag_table; /* 8 KiB */

typedef struct sg_pack_args {
  const sg_frag_table *tables; /* device-addressable, n_tables, 16-byte aligned */
  uint32_t n_tables;
  uint32_t n_req;
  const uint32_t *table_idx;   /* device-addressable, n_req: the table of each request */
  const uint32_t *req_first;   /* device-addressable, n_req + 1: running sum of the requests' fragment counts */
  uint32_t n_frags;            /* == req_first[n_req] */
  uint32_t reserved;
  uint64_t pkt_base;
  sg_ring_desc ring;           /* the ring the fragments lie in (its header profile gives the payload offset) */
  uint32_t *frag_slot;         /* device out, n_frags */
  uint32_t *frag_len;          /* device out, n_frags, or NULL */
  uint32_t *req_first_out;     /* device out, n_req + 1, or NULL */
  /* words copied along by the same launch (what else the call behind needs on the device:
   * tokens, response sizes, header templates), or NULL / 0 */
  const uint32_t *blob_src;    /* device-addressable */
  uint32_t *blob_dst;          /* device */
  uint32_t blob_words;
  uint32_t reserved2;
  void *stream;                /* hipStream_t to launch on; NULL: the context's.  On a stream of its own the
                                  pull of the next call's tables runs beside the current call's copy (the
                                  caller orders the two streams with an event) */
} sg_pack_args;

/* Launches only; nothing is waited for.  n_req == 0 with blob_words != 0 brings the words along
 * and nothing else.  No counterpart call in the reference. */
int sg_hip_pack_tables(sg_hip_ctx *ctx, const sg_pack_args *args);

/* The gather call for callers that cannot allocate.  No counterpart in the
 * reference: it is for code running under HIP graph capture, tight serving
 * loops and harnesses that forbid hipMalloc.  Same semantics and same kernels
 * as sg_hip_gather_batch, but without a context: the descriptor scratch lives
 * in a static device array of about 1.1 MiB that each GPU the library runs on
 * holds until the process ends, which is why one call takes at most
 * SG_STATIC_MAX_REQS requests in SG_STATIC_MAX_FRAMES fragments (a larger batch
 * is refused with SG_E_INVAL; split it or use a context).  The call launches
 * kernels on `stream` (NULL: the default stream) and returns; it allocates and
 * frees nothing, copies nothing, and never waits.  The first call on a device
 * looks up that device's copy of the array.
 *   cursor  device word holding the bump-ring position of the arena, read and
 *           advanced by the call; NULL: a word inside the array, which starts
 *           at zero and carries over from call to call
 *   status  device word that receives refusal bits (non-zero after the stream
 *           has drained: something was refused, as SG_E_DATA from
 *           sg_hip_sync).  The caller zeroes it: with a descriptor pass a
 *           non-zero status on entry means "refused" and nothing moves.  NULL:
 *           a word inside the array, cleared by each call, that nobody reads.
 * All calls on one GPU share that GPU's array: calls that overlap in time on
 * one GPU (two streams, two threads) race and must not be made.
 * sg_hip_last_error(NULL) gives the text of a refusal by the host. */
#define SG_STATIC_MAX_REQS 4096u
#define SG_STATIC_MAX_FRAMES 65536u
int sg_hip_gather_batch_static(int device_id, void *stream, const sg_gather_args *args, uint64_t *cursor,
                               uint32_t *status);

/* Sorts a burst of arrivals into requests (see sg_reassemble_args).
 * Synchronous unless SG_F_ASYNC is set; then counts_host_out is not written and
 * the counts are where counts_out says.  counts_host_out (4 words, or NULL):
 * requests completed, their fragments, arrivals dropped, requests still in
 * flight.  The first call on a context allocates the request table and the
 * record pool (8 KiB per request of max_reqs): make it, or
 * sg_hip_reassemble_reset, before recording calls into a graph. */
int sg_hip_reassemble(sg_hip_ctx *ctx, const sg_reassemble_args *args, uint32_t *counts_host_out);

/* Drops every request in flight (and allocates the state on first use). */
int sg_hip_reassemble_reset(sg_hip_ctx *ctx);

/* Drops the requests that no fragment has come in for during the last
 * max_age_calls calls of sg_hip_reassemble: a request that lost a fragment is
 * parked for good in the reference (src/p2p_rpc_rr_pool_ng.h:57-64 lists such
 * leftovers at shutdown); here the caller can clear them out.  Synchronous. */
int sg_hip_reassemble_evict(sg_hip_ctx *ctx, uint32_t max_age_calls, uint32_t *n_evicted_out);

/* Device-resident bump-ring cursors (P2pRpcTring::prev_offset,
 * src/p2p_rpc_tring.h:14-16), one for the request arena (which = 0) and one
 * for the response arena (which = 1).  Both calls synchronize. */
int sg_hip_set_cursor(sg_hip_ctx *ctx, int which, uint64_t value);
int sg_hip_get_cursor(sg_hip_ctx *ctx, int which, uint64_t *value);

/* Device-resident indices into the application slot ring, the shunter's
 * rr_pi_idx and rr_ci_idx (src/splitrpc_server/p2p_rpc_dpdk_server.cc:98,141,183):
 * which = 0 the next slot a gather fills, which = 1 the next slot a scatter
 * serves.  Both calls synchronize. */
int sg_hip_set_slot_index(sg_hip_ctx *ctx, int which, uint32_t value);
int sg_hip_get_slot_index(sg_hip_ctx *ctx, int which, uint32_t *value);

/* ---- measurement -------------------------------------------------------------
 * With profiling on, every kernel launch is bracketed by HIP events on the
 * context's stream (the PROFILE_MODE GDelay/SDelay vectors of the reference,
 * src/p2p_rpc_sg_engine.h:83-92, at kernel granularity).  which: 0 descriptor
 * build, 1 gather copy, 2 scatter copy + header rewrite, 3 per-request run
 * copy, 4 header-only rewrite, 5 reassembly (all of its kernels together).
 * sg_hip_kernel_time synchronizes, returns the accumulated milliseconds and launch count since profiling was switched on,
 * and leaves the accumulators running. */
int sg_hip_set_profiling(sg_hip_ctx *ctx, int on);
int sg_hip_kernel_time(sg_hip_ctx *ctx, int which, double *total_ms, uint64_t *launches);

#ifdef __cplusplus
}
#endif
#endif /* SG_HIP_H */
