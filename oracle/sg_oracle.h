/*
 * sg_oracle.h -- CPU restatement of SplitRPC's scatter-gather data path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing the library ships may include, link or
 * call this file; it exists so that the tests, the smoke check and the CPU
 * leg of the benchmark have an independent answer to compare the HIP path
 * with.  Every function names the reference source it restates
 * (paths relative to the reference tree).
 *
 * How each function is pinned (what a wrong sign / index / dropped term would
 * trip over) is listed next to it.  Functions marked PARITY UNPINNED have no
 * reference-held vector and no reference build here; they follow the cited
 * standard and are checked against that standard's invariants only.
 *
 *   sgo_ipv4_pseudo_csum  compiled reference eth_common.h (oracle/_ref) on
 *                         seeded headers + hand-computed vector
 *   sgo_tring_get_next    compiled reference p2p_rpc_tring.h (oracle/_ref)
 *   table layouts         sizeof/offsetof of compiled reference p2p_bufs.h,
 *                         p2p_rpc_app_stub.h (oracle/_ref)
 *   sgo_gather_skbs /     closed form out[off_i + k] = frag_i[k]; brute force;
 *   sgo_scatter_skbs      runs merge iff pointers abut; permutation invariance
 *   sgo_swap_eth_hdr      involution, untouched bytes unchanged, hand vector
 *   sgo_add_ip_udp_len    big-endian closed form (28 + L, 8 + L)
 *   sgo_ipv4_hdr_csum     RFC 1071 textbook header (-> b861), verify-to-ffff
 *                         PARITY UNPINNED vs the reference: the reference
 *                         leaves this to NIC offload (dpdk_rx_tx.h:143)
 *   sgo_udp_full_csum     RFC 768 verify-to-ffff, scalar byte loop, 0->ffff
 *                         PARITY UNPINNED vs the reference (NIC offload)
 *   sgo_gen_hdr_template  compiled reference eth_common.h templates (oracle/_ref)
 *   sgo_set_conn_info     every byte range against its source, untouched
 *                         bytes unchanged
 *   sgo_template_resp_hdr identity: template path == swap path when the
 *   sgo_rewrite_resp_hdr  template carries the identity the request was sent
 *                         to (two independent routes to one header)
 *   sgo_reassemble        arrival-order invariance, brute-force reassembly
 *   sgo_gather_batch /    pure-Python brute force (byte-wise arena wrap,
 *   sgo_scatter_batch     tensor-major split, big-endian header arithmetic)
 *   echo / vec_add bytes  lib_loadgen/echo_client.cc:11-32,
 *                         vec_add_client.cc:11-19 patterns
 */
#ifndef SG_ORACLE_H
#define SG_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- wire format ------------------------------------------------------- */

enum {
  SGO_ETH_LEN = 14,
  SGO_IP_OFF = 14,
  SGO_UDP_OFF = 34,
  SGO_L4_END = 42, /* UDP_HEADER_LEN, eth_common.h:48 */
};

/* Header profiles.  REF64 is the reference's own p2p_rpc_hdr (p2p_rpc.h:10-17):
 * u64 req_token @42, i64 sock_perf_header @50, u16 seq_num @58, pad to 64.
 * BL58 is the benchmark profile: u64 req_id @42, u16 frag_idx @50,
 * u16 num_frags @52, u32 payload_len @54, payload @58. */
enum { SGO_HDR_BL58 = 0, SGO_HDR_REF64 = 1 };

/* Flags of the response-header rewrite. */
enum {
  SGO_F_IPV4_CSUM = 1u << 0,       /* finished IPv4 header checksum (RFC 1071) */
  SGO_F_UDP_CSUM_PSEUDO = 1u << 1, /* reference style: raw pseudo-header sum */
  SGO_F_UDP_CSUM_FULL = 1u << 2,   /* finished UDP checksum (RFC 768) */
  SGO_F_REF_QUIRKS = 1u << 3,      /* UDP length = tot_len - version*4 */
};

static inline uint32_t sgo_hdr_len(uint32_t profile) { return profile == SGO_HDR_REF64 ? 64u : 58u; }

void sgo_swap_eth_hdr(uint8_t *hdr);
void sgo_add_ip_udp_len(uint8_t *hdr, uint16_t pkt_len);
uint16_t sgo_ipv4_pseudo_csum(const uint8_t *ip, int ref_quirk);
void sgo_add_udp_cksum(uint8_t *hdr, int ref_quirk);
void sgo_set_sockperf_header(uint8_t *hdr);
void sgo_set_conn_info(uint8_t *tmpl, const uint8_t *recv_hdr, uint32_t profile);
uint16_t sgo_ipv4_hdr_csum(const uint8_t *ip);
uint16_t sgo_udp_full_csum(const uint8_t *ip, const uint8_t *udp);
void sgo_gen_hdr_template(uint8_t *hdr, const uint8_t src_mac[6], const uint8_t dst_mac[6],
                          uint32_t src_ip, uint32_t dst_ip, int src_port, int dst_port);

/* One response frame: swap + routing fields + lengths + checksums.
 * `hdr` holds a copy of a request frame's header on entry. */
void sgo_rewrite_resp_hdr(uint8_t *hdr, uint32_t profile, uint32_t flags, uint16_t frag_idx,
                          uint16_t num_frags, uint32_t payload_len);
/* rr_set_hdr (transport/dpdk_transport_ng.h:113-141): header from a template. */
void sgo_template_resp_hdr(uint8_t *hdr, const uint8_t *tmpl, uint32_t profile, uint32_t flags,
                           uint64_t req_token, uint16_t frag_idx, uint16_t num_frags,
                           uint32_t payload_len);

/* ---- fixed-capacity tables (p2p_bufs.h:10-40) --------------------------- */

#define SGO_MAX_BI_SIZE 1024

#pragma pack(push, 1)
typedef struct {
  uint64_t burst_items[SGO_MAX_BI_SIZE];
  uint16_t num_items;
} sgo_hbufs;

typedef struct {
  uint64_t burst_items[SGO_MAX_BI_SIZE];
  uint64_t item_size[SGO_MAX_BI_SIZE];
  uint16_t num_items;
} sgo_bufs;

typedef struct {
  uint64_t i_buf[SGO_MAX_BI_SIZE];
  uint64_t o_buf[SGO_MAX_BI_SIZE];
  uint64_t len[SGO_MAX_BI_SIZE - 1];
  uint64_t num_items;
} sgo_sk_buf;
#pragma pack(pop)

void sgo_gather_skbs(sgo_sk_buf *skb, const sgo_bufs *bufs, uint64_t app_buf);
void sgo_scatter_skbs(sgo_sk_buf *skb, const sgo_bufs *bufs, uint64_t app_buf);
int sgo_sg_on_cpu(const sgo_sk_buf *skb);

/* ---- fragmenting rule, bump ring ---------------------------------------- */

uint32_t sgo_num_frames(uint64_t size, uint32_t mtu);
uint32_t sgo_frame_len(uint64_t size, uint32_t mtu, uint32_t i);

typedef struct {
  uint64_t base, capacity, prev_offset, prev_addr;
} sgo_tring;
void sgo_tring_init(sgo_tring *t, uint64_t base, uint64_t capacity);
uint64_t sgo_tring_get_next(sgo_tring *t, uint64_t size);

/* ---- request reassembly (p2p_rpc_rr_ng.h, p2p_rpc_rr_pool_ng.h) ---------- */

/* Replays `n_arrivals` ring slots in arrival order through the reference's
 * get_rr / rr_emplace_mbuf / is_rr_ready logic and emits the fragment tables
 * of the completed requests, in completion order (the order the rx-ready ring
 * would hand them to the shunter).  Returns the number of completed requests,
 * or -1 on table overflow.  `req_size` is the server-wide request size of the
 * REF64 profile; with BL58 a request is complete when num_frags fragments are
 * in.  frag_len_nic gives per-slot payload bytes for REF64 (the NIC's pkt_len
 * minus the header); may be NULL for BL58. */
typedef struct {
  uint8_t *base;
  uint32_t n_slots;
  uint32_t slot_size;
  uint32_t profile;
} sgo_ring;

int64_t sgo_reassemble(const sgo_ring *ring, const uint32_t *arrivals, uint32_t n_arrivals,
                       const uint32_t *frag_len_nic, uint64_t req_size, uint32_t *frag_slot_out,
                       uint32_t *frag_len_out, uint32_t *req_first_out, uint64_t *req_token_out,
                       uint32_t max_req, uint32_t max_frag);

/* ---- batch composites: what the HIP path is compared with ---------------- */

#define SGO_MAX_TENSORS 4 /* p2p_rpc_app_stub.h:10 */

typedef struct {
  uint8_t *base[SGO_MAX_TENSORS]; /* tensor-major destinations (g_params_v2) */
  uint64_t size[SGO_MAX_TENSORS]; /* bytes per request in each tensor */
  uint32_t n_tensors;             /* 0: packed arena addressed through the bump ring */
  uint8_t *arena;                 /* packed mode: arena base */
  uint64_t arena_cap;             /* packed mode: bump-ring capacity */
} sgo_app_bufs;

/* Gather n_req requests (CSR fragment tables) from the ring into the app
 * buffers: per request build the p2p_bufs table in seq order, gather_skbs,
 * memcpy per run (P2pRpcSgCpuEngine::gather, p2p_rpc_sg_engine.h:150-156).
 * Packed mode: request offsets come from the bump ring starting at *cursor
 * (P2pRpcAppRrPool::get_next, p2p_rpc_app_rr.h:127-134); offsets_out gets
 * n_req+1 entries (start of each request and the end of the last).  Returns
 * number of runs copied or -1. */
int64_t sgo_gather_batch(const sgo_ring *ring, const uint32_t *frag_slot, const uint32_t *frag_len,
                         const uint32_t *req_first, uint32_t n_req, const sgo_app_bufs *app,
                         uint64_t *cursor, uint64_t *offsets_out);

/* Scatter n_req responses into TX ring slots and rewrite their headers.
 * Response r has resp_size[r] bytes (or fixed_resp_size when resp_size is
 * NULL) cut by the fragmenting rule at `mtu`; frame f of the batch goes to
 * tx_slot[f]; its header is rewritten from the request header found in
 * rx ring slot hdr_src_slot[f].  Payload source: packed arena through the
 * bump ring, or tensor-major outputs.  With hdr_templates (n_req x 64 bytes)
 * the header of every frame of response r is built from template r and
 * req_token[r] instead (rr_set_hdr) and hdr_src_slot is not read.
 * Returns number of frames or -1. */
int64_t sgo_scatter_batch(const sgo_ring *rx, const sgo_ring *tx, const uint32_t *tx_slot,
                          const uint32_t *hdr_src_slot, const uint32_t *resp_first,
                          const uint64_t *resp_size, uint64_t fixed_resp_size, uint32_t n_req,
                          uint32_t mtu, uint32_t flags, const sgo_app_bufs *app, uint64_t *cursor,
                          uint64_t *offsets_out, const uint8_t *hdr_templates,
                          const uint64_t *req_token);

/* Single-threaded timing helpers used by the CPU-baseline leg of the
 * benchmark: run the composite `iters` times over `n_rings` rotated copies and
 * return elapsed seconds. */
double sgo_now_sec(void);

#ifdef __cplusplus
}
#endif
#endif
