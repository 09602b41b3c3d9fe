/*
 * sg_oracle.c -- CPU restatement of SplitRPC's scatter-gather data path.
 * TEST INFRASTRUCTURE ONLY: see sg_oracle.h for who may use it and for how
 * each function is pinned.  Plain C99, single-threaded, no dependencies.
 */
#include "sg_oracle.h"

#include <stdlib.h>
#include <string.h>
#include <time.h>

/* ---- little helpers ------------------------------------------------------ */

static inline uint16_t rd16(const uint8_t *p) { uint16_t v; memcpy(&v, p, 2); return v; }
static inline void wr16(uint8_t *p, uint16_t v) { memcpy(p, &v, 2); }
static inline uint32_t rd32(const uint8_t *p) { uint32_t v; memcpy(&v, p, 4); return v; }
static inline void wr32(uint8_t *p, uint32_t v) { memcpy(p, &v, 4); }
static inline uint64_t rd64(const uint8_t *p) { uint64_t v; memcpy(&v, p, 8); return v; }
static inline void wr64(uint8_t *p, uint64_t v) { memcpy(p, &v, 8); }
static inline uint16_t bswap16(uint16_t v) { return (uint16_t)((v >> 8) | (v << 8)); }
/* host is little-endian x86: htons == ntohs == bswap16 */
static inline uint16_t be16(uint16_t host) { return bswap16(host); }

/* ---- header rewrite ------------------------------------------------------- */

/* swap_eth_hdr, p2p_rpc.h:64-83: exchange dst/src MAC, src/dst IPv4, src/dst
 * UDP port; zero ip.check and udp.check. */
void sgo_swap_eth_hdr(uint8_t *h)
{
  uint8_t mac[6];
  memcpy(mac, h + 6, 6);     /* tmp = src */
  memcpy(h + 6, h + 0, 6);   /* src = dst */
  memcpy(h + 0, mac, 6);     /* dst = tmp */
  uint32_t ip = rd32(h + 26);
  wr32(h + 26, rd32(h + 30));
  wr32(h + 30, ip);
  wr16(h + 24, 0);
  uint16_t port = rd16(h + 34);
  wr16(h + 34, rd16(h + 36));
  wr16(h + 36, port);
  wr16(h + 40, 0);
}

/* add_ip_udp_len, p2p_rpc.h:51-56: tot_len = htons(20 + 8 + pkt_len),
 * udp.len = htons(8 + pkt_len); pkt_len counts RPC tail + payload. */
void sgo_add_ip_udp_len(uint8_t *h, uint16_t pkt_len)
{
  wr16(h + 16, be16((uint16_t)(20 + 8 + pkt_len)));
  wr16(h + 38, be16((uint16_t)(8 + pkt_len)));
}

/* ipv4_pseudo_csum, eth_common.h:92-130 (device twin
 * transport/g_udp_handler.cu:67-94).  Native-order 16-bit sum over
 * {src_ip, dst_ip, 0, proto, htons(udp_len)} followed by four bytes the
 * reference never writes (taken as zero here), folded twice, NOT complemented.
 * ref_quirk: the reference derives udp_len as tot_len - version*4 (= 16 for
 * IPv4) rather than tot_len - ihl*4. */
uint16_t sgo_ipv4_pseudo_csum(const uint8_t *ip, int ref_quirk)
{
  uint8_t psd[16];
  memset(psd, 0, sizeof psd);
  memcpy(psd + 0, ip + 12, 4);
  memcpy(psd + 4, ip + 16, 4);
  psd[8] = 0;
  psd[9] = ip[9];
  unsigned hdr_bytes = ref_quirk ? (unsigned)(ip[0] >> 4) * 4u : (unsigned)(ip[0] & 0x0f) * 4u;
  int len = (int)bswap16(rd16(ip + 2)) - (int)hdr_bytes;
  wr16(psd + 10, be16((uint16_t)len));
  uint32_t sum = 0;
  for (int i = 0; i < 8; i++) sum += rd16(psd + 2 * i);
  sum = (sum & 0xffffu) + (sum >> 16);
  sum = (sum & 0xffffu) + (sum >> 16);
  return (uint16_t)sum;
}

/* add_udp_cksum, p2p_rpc.h:58-61: raw pseudo sum stored in udp.check. */
void sgo_add_udp_cksum(uint8_t *h, int ref_quirk)
{
  wr16(h + 40, sgo_ipv4_pseudo_csum(h + SGO_IP_OFF, ref_quirk));
}

/* set_sockperf_header, p2p_rpc.h:47-49 (REF64 only): clear the low 32 bits. */
void sgo_set_sockperf_header(uint8_t *h)
{
  wr64(h + 50, rd64(h + 50) & 0xFFFFFFFF00000000ull);
}

/* set_conn_info, p2p_rpc_conn_info.h:73-84: copy the RPC tail of the first
 * received packet into the template and point the template at the sender. */
void sgo_set_conn_info(uint8_t *tmpl, const uint8_t *recv, uint32_t profile)
{
  uint32_t hl = sgo_hdr_len(profile);
  memcpy(tmpl + SGO_L4_END, recv + SGO_L4_END, hl - SGO_L4_END);
  memcpy(tmpl + 36, recv + 34, 2); /* dst_port <- src_port */
  memcpy(tmpl + 30, recv + 26, 4); /* dst_ip   <- src_ip   */
  memcpy(tmpl + 0, recv + 6, 6);   /* dst_mac  <- src_mac  */
}

/* gen_eth/ipv4/udp_header_template, eth_common.h:51-89 as composed by
 * init_conn_info, p2p_rpc_conn_info.h:32-48.  IPs and ports in host order.
 * (udp.len starts as htons(20+8) in the reference, eth_common.h:85.) */
void sgo_gen_hdr_template(uint8_t *h, const uint8_t src_mac[6], const uint8_t dst_mac[6],
                          uint32_t src_ip, uint32_t dst_ip, int src_port, int dst_port)
{
  memcpy(h + 6, src_mac, 6);
  memcpy(h + 0, dst_mac, 6);
  wr16(h + 12, be16(0x0800));
  h[14] = 0x45;        /* version 4, ihl 5 */
  h[15] = 0x01;        /* ecn = 1 in the low two bits, dscp 0 */
  wr16(h + 16, be16(28));
  wr16(h + 18, 0);
  wr16(h + 20, 0);
  h[22] = 128;
  h[23] = 17;
  wr16(h + 24, 0);
  wr32(h + 26, __builtin_bswap32(src_ip));
  wr32(h + 30, __builtin_bswap32(dst_ip));
  wr16(h + 34, be16((uint16_t)src_port));
  wr16(h + 36, be16((uint16_t)dst_port));
  wr16(h + 38, be16(28));
  wr16(h + 40, 0);
}

/* Finished IPv4 header checksum, RFC 1071 over ihl*4 bytes with the check
 * field taken as zero.  The reference leaves this to the NIC
 * (PKT_TX_IP_CKSUM, transport/dpdk_rx_tx.h:143).  Returned in the byte order
 * to store with a native 16-bit write. */
uint16_t sgo_ipv4_hdr_csum(const uint8_t *ip)
{
  unsigned n = (unsigned)(ip[0] & 0x0f) * 4u;
  uint32_t sum = 0;
  for (unsigned i = 0; i < n; i += 2) {
    if (i == 10) continue;
    sum += (uint32_t)ip[i] << 8 | ip[i + 1];
  }
  while (sum >> 16) sum = (sum & 0xffffu) + (sum >> 16);
  return be16((uint16_t)~sum);
}

/* Finished UDP checksum, RFC 768: pseudo header + UDP header (check = 0) +
 * data, odd byte padded with zero, complemented, 0 transmitted as 0xffff.
 * Length is udp.len.  The reference leaves this to the NIC
 * (PKT_TX_UDP_CKSUM). */
uint16_t sgo_udp_full_csum(const uint8_t *ip, const uint8_t *udp)
{
  unsigned ulen = (unsigned)udp[4] << 8 | udp[5];
  uint32_t sum = 0;
  for (int i = 12; i < 20; i += 2) sum += (uint32_t)ip[i] << 8 | ip[i + 1];
  sum += ip[9];
  sum += ulen;
  for (unsigned i = 0; i + 1 < ulen; i += 2) {
    if (i == 6) continue;
    sum += (uint32_t)udp[i] << 8 | udp[i + 1];
    if (sum >> 24) sum = (sum & 0xffffu) + (sum >> 16);
  }
  if (ulen & 1) sum += (uint32_t)udp[ulen - 1] << 8;
  while (sum >> 16) sum = (sum & 0xffffu) + (sum >> 16);
  uint16_t c = (uint16_t)~sum;
  if (c == 0) c = 0xffff;
  return be16(c);
}

static void finish_lengths_and_csums(uint8_t *h, uint32_t profile, uint32_t flags,
                                     uint32_t payload_len, const uint8_t *payload_for_csum)
{
  (void)payload_for_csum;
  uint32_t tail = sgo_hdr_len(profile) - SGO_L4_END;
  sgo_add_ip_udp_len(h, (uint16_t)(tail + payload_len));
  if (flags & SGO_F_UDP_CSUM_PSEUDO) sgo_add_udp_cksum(h, (flags & SGO_F_REF_QUIRKS) != 0);
  if (flags & SGO_F_IPV4_CSUM) wr16(h + 24, sgo_ipv4_hdr_csum(h + SGO_IP_OFF));
}

/* Response header by in-place swap: swap_hdrs_on_cpu,
 * transport/dpdk_transport_ng.h:70-84 (swap_eth_hdr, add_ip_udp_len with
 * tail + payload, add_udp_cksum) plus the routing fields rr_set_hdr writes
 * (:129-131: token kept, seq_num = i, set_sockperf_header).  BL58 also
 * carries num_frags and payload_len.  Checksums beyond the reference's raw
 * pseudo sum are opt-in flags.  The full UDP checksum needs the payload and
 * is finished by the caller (sgo_scatter_batch) once the payload is in place. */
void sgo_rewrite_resp_hdr(uint8_t *h, uint32_t profile, uint32_t flags, uint16_t frag_idx,
                          uint16_t num_frags, uint32_t payload_len)
{
  sgo_swap_eth_hdr(h);
  if (profile == SGO_HDR_REF64) {
    wr16(h + 58, frag_idx);
    sgo_set_sockperf_header(h);
  } else {
    wr16(h + 50, frag_idx);
    wr16(h + 52, num_frags);
    wr32(h + 54, payload_len);
  }
  finish_lengths_and_csums(h, profile, flags, payload_len, NULL);
}

/* rr_set_hdr, transport/dpdk_transport_ng.h:113-141: copy the connection
 * template, then token, seq_num, sockperf, lengths, pseudo sum. */
void sgo_template_resp_hdr(uint8_t *h, const uint8_t *tmpl, uint32_t profile, uint32_t flags,
                           uint64_t req_token, uint16_t frag_idx, uint16_t num_frags,
                           uint32_t payload_len)
{
  memcpy(h, tmpl, sgo_hdr_len(profile));
  wr64(h + 42, req_token);
  if (profile == SGO_HDR_REF64) {
    wr16(h + 58, frag_idx);
    sgo_set_sockperf_header(h);
  } else {
    wr16(h + 50, frag_idx);
    wr16(h + 52, num_frags);
    wr32(h + 54, payload_len);
  }
  finish_lengths_and_csums(h, profile, flags, payload_len, NULL);
}

/* ---- run descriptors ------------------------------------------------------ */

/* gather_skbs, p2p_rpc_sg_engine.h:19-45.  o_buf is the running sum of the
 * fragment sizes in table order; fragment i joins the previous run iff its
 * pointer equals the previous fragment's end.  Entry 0 is always emitted,
 * even when num_items == 0 (as the reference does). */
void sgo_gather_skbs(sgo_sk_buf *skb, const sgo_bufs *b, uint64_t app_buf)
{
  uint64_t app = app_buf;
  uint64_t k = 0;
  skb->i_buf[0] = b->burst_items[0];
  skb->o_buf[0] = app;
  skb->len[0] = b->item_size[0];
  app += b->item_size[0];
  uint64_t end = b->burst_items[0] + b->item_size[0];
  for (int i = 1; i < (int)b->num_items; i++) {
    if (b->burst_items[i] == end) {
      skb->len[k] += b->item_size[i];
    } else {
      k++;
      skb->i_buf[k] = b->burst_items[i];
      skb->o_buf[k] = app;
      skb->len[k] = b->item_size[i];
    }
    end = b->burst_items[i] + b->item_size[i];
    app += b->item_size[i];
  }
  skb->num_items = k + 1;
}

/* scatter_skbs, p2p_rpc_sg_engine.h:49-73: mirror image, i_buf walks the app
 * buffer and o_buf points at the packet payloads. */
void sgo_scatter_skbs(sgo_sk_buf *skb, const sgo_bufs *b, uint64_t app_buf)
{
  uint64_t app = app_buf;
  uint64_t k = 0;
  skb->i_buf[0] = app;
  skb->o_buf[0] = b->burst_items[0];
  skb->len[0] = b->item_size[0];
  app += b->item_size[0];
  uint64_t end = b->burst_items[0] + b->item_size[0];
  for (int i = 1; i < (int)b->num_items; i++) {
    if (b->burst_items[i] == end) {
      skb->len[k] += b->item_size[i];
    } else {
      k++;
      skb->i_buf[k] = app;
      skb->o_buf[k] = b->burst_items[i];
      skb->len[k] = b->item_size[i];
    }
    end = b->burst_items[i] + b->item_size[i];
    app += b->item_size[i];
  }
  skb->num_items = k + 1;
}

/* P2pRpcSgCpuEngine::sg_on_cpu, p2p_rpc_sg_engine.h:139-145. */
int sgo_sg_on_cpu(const sgo_sk_buf *skb)
{
  for (uint64_t i = 0; i < skb->num_items; i++)
    memcpy((void *)(uintptr_t)skb->o_buf[i], (const void *)(uintptr_t)skb->i_buf[i], skb->len[i]);
  return 1;
}

/* ---- fragmenting rule, bump ring ------------------------------------------ */

/* rr_alloc_mbufs, transport/dpdk_transport_ng.h:332: ceil(size / MTU). */
uint32_t sgo_num_frames(uint64_t size, uint32_t mtu)
{
  return (uint32_t)((size + mtu - 1) / mtu);
}

/* alloc_dpdk_mbufs, transport/dpdk_rx_tx.h:137-139: frame i carries
 * min(remaining, MTU). */
uint32_t sgo_frame_len(uint64_t size, uint32_t mtu, uint32_t i)
{
  /* after i full-or-final frames the remainder is size - i*mtu, floored at 0 */
  uint64_t taken = (uint64_t)i * mtu;
  uint64_t rem = taken < size ? size - taken : 0;
  return (uint32_t)(rem <= mtu ? rem : mtu);
}

/* P2pRpcTring, p2p_rpc_tring.h:19-33. */
void sgo_tring_init(sgo_tring *t, uint64_t base, uint64_t capacity)
{
  t->base = base;
  t->capacity = capacity;
  t->prev_offset = 0;
  t->prev_addr = base;
}

uint64_t sgo_tring_get_next(sgo_tring *t, uint64_t size)
{
  uint64_t ret = t->prev_addr;
  t->prev_offset = (t->prev_offset + size) % t->capacity;
  t->prev_addr = t->base + t->prev_offset;
  return ret;
}

/* ---- request reassembly --------------------------------------------------- */

/* One in-flight request: the state P2pRpcRr keeps (p2p_rpc_rr_ng.h:13-35)
 * reduced to what the data path reads. */
typedef struct {
  uint64_t token;
  uint64_t payload_size;
  uint32_t num_items;
  uint32_t want_frags;
  int used;
  uint32_t slot[SGO_MAX_BI_SIZE];
  uint32_t len[SGO_MAX_BI_SIZE];
} rr_state;

/* get_rr (p2p_rpc_rr_pool_ng.h:97-109): find the request by token or take a
 * fresh one.  rr_emplace_mbuf (p2p_rpc_rr_ng.h:96-105): table entry at index
 * seq_num, num_items++, payload_size += item_size.  is_rr_ready (:107-110):
 * payload_size == max_payload_size; BL58 requests carry their own num_frags
 * and are ready when that many fragments are in.  Completed requests leave in
 * completion order (mark_rx_ready_rr, p2p_rpc_rr_pool_ng.h:149-155).
 * Packets with token 0 are dropped (transport/dpdk_transport_ng.h:196). */
int64_t sgo_reassemble(const sgo_ring *ring, const uint32_t *arrivals, uint32_t n_arrivals,
                       const uint32_t *frag_len_nic, uint64_t req_size, uint32_t *frag_slot_out,
                       uint32_t *frag_len_out, uint32_t *req_first_out, uint64_t *req_token_out,
                       uint32_t max_req, uint32_t max_frag)
{
  uint32_t cap = 64, n_live = 0;
  rr_state **live = (rr_state **)calloc(cap, sizeof *live);
  uint32_t n_done = 0, n_out = 0;
  int64_t rc = 0;
  if (!live) return -1;
  req_first_out[0] = 0;
  for (uint32_t a = 0; a < n_arrivals; a++) {
    uint32_t s = arrivals[a];
    const uint8_t *h = ring->base + (uint64_t)s * ring->slot_size;
    uint64_t token = rd64(h + 42);
    if (token == 0) continue;
    uint32_t seq, len, want;
    if (ring->profile == SGO_HDR_REF64) {
      seq = rd16(h + 58);
      len = frag_len_nic[s];
      want = 0;
    } else {
      seq = rd16(h + 50);
      want = rd16(h + 52);
      len = frag_len_nic ? frag_len_nic[s] : rd32(h + 54);
    }
    if (seq >= SGO_MAX_BI_SIZE) { rc = -1; break; }
    rr_state *rr = NULL;
    for (uint32_t i = 0; i < n_live; i++)
      if (live[i]->token == token) { rr = live[i]; break; }
    if (!rr) {
      if (n_live == cap) {
        cap *= 2;
        rr_state **nl = (rr_state **)realloc(live, cap * sizeof *live);
        if (!nl) { rc = -1; break; }
        live = nl;
      }
      rr = (rr_state *)calloc(1, sizeof *rr);
      if (!rr) { rc = -1; break; }
      rr->token = token;
      rr->want_frags = want;
      live[n_live++] = rr;
    }
    rr->slot[seq] = s;
    rr->len[seq] = len;
    rr->num_items++;
    rr->payload_size += len;
    int ready = ring->profile == SGO_HDR_REF64 ? rr->payload_size == req_size
                                               : rr->num_items == rr->want_frags;
    if (ready) {
      if (n_done >= max_req || n_out + rr->num_items > max_frag) { rc = -1; break; }
      for (uint32_t i = 0; i < rr->num_items; i++) {
        frag_slot_out[n_out] = rr->slot[i];
        frag_len_out[n_out] = rr->len[i];
        n_out++;
      }
      req_token_out[n_done] = token;
      n_done++;
      req_first_out[n_done] = n_out;
      for (uint32_t i = 0; i < n_live; i++)
        if (live[i] == rr) { live[i] = live[--n_live]; break; }
      free(rr);
    }
  }
  for (uint32_t i = 0; i < n_live; i++) free(live[i]);
  free(live);
  return rc < 0 ? rc : (int64_t)n_done;
}

/* ---- batch composites ------------------------------------------------------ */

/* Copy through a bump-ring arena whose physical pages are mapped twice
 * back-to-back (p2p_rpc_app_rr_mem_pool.h:302-306): offset o and o + capacity
 * alias, so a run that crosses the end lands at the start. */
static void copy_into_arena(uint8_t *arena, uint64_t cap, uint64_t off, const uint8_t *src,
                            uint64_t len)
{
  while (len) {
    uint64_t o = off % cap;
    uint64_t n = cap - o < len ? cap - o : len;
    memcpy(arena + o, src, n);
    src += n; off += n; len -= n;
  }
}

static void copy_from_arena(const uint8_t *arena, uint64_t cap, uint64_t off, uint8_t *dst,
                            uint64_t len)
{
  while (len) {
    uint64_t o = off % cap;
    uint64_t n = cap - o < len ? cap - o : len;
    memcpy(dst, arena + o, n);
    dst += n; off += n; len -= n;
  }
}

/* Split [off, off+len) of request r's byte stream over the tensor-major
 * buffers of g_params_v2 (p2p_rpc_app_stub.h:11-20): the stream is tensor 0's
 * bytes, then tensor 1's, ...; tensor t of request r lives at
 * base[t] + r * size[t]. */
static void copy_tensor_major(const sgo_app_bufs *app, uint32_t r, uint64_t off, uint8_t *pkt,
                              uint64_t len, int to_app)
{
  uint64_t t0 = 0;
  for (uint32_t t = 0; t < app->n_tensors && len; t++) {
    uint64_t t1 = t0 + app->size[t];
    if (off < t1) {
      uint64_t n = t1 - off < len ? t1 - off : len;
      uint8_t *p = app->base[t] + (uint64_t)r * app->size[t] + (off - t0);
      if (to_app) memcpy(p, pkt, n); else memcpy(pkt, p, n);
      pkt += n; off += n; len -= n;
    }
    t0 = t1;
  }
}

int64_t sgo_gather_batch(const sgo_ring *ring, const uint32_t *frag_slot, const uint32_t *frag_len,
                         const uint32_t *req_first, uint32_t n_req, const sgo_app_bufs *app,
                         uint64_t *cursor, uint64_t *offsets_out)
{
  const uint32_t hl = sgo_hdr_len(ring->profile);
  sgo_bufs *bufs = (sgo_bufs *)malloc(sizeof *bufs);
  sgo_sk_buf *skb = (sgo_sk_buf *)malloc(sizeof *skb);
  int64_t runs = 0;
  if (!bufs || !skb) { free(bufs); free(skb); return -1; }
  sgo_tring tr;
  if (app->n_tensors == 0) {
    sgo_tring_init(&tr, 0, app->arena_cap);
    tr.prev_offset = *cursor % app->arena_cap;
    tr.prev_addr = tr.prev_offset;
  }
  for (uint32_t r = 0; r < n_req; r++) {
    uint32_t f0 = req_first[r], f1 = req_first[r + 1];
    /* the run table has room for 1023 lengths (p2p_bufs.h:37): a 1024th run
     * would overwrite num_items in the reference.  Refused here. */
    if (f1 - f0 > SGO_MAX_BI_SIZE - 1) { runs = -1; break; }
    uint64_t total = 0;
    bufs->num_items = (uint16_t)(f1 - f0);
    for (uint32_t f = f0; f < f1; f++) {
      const uint8_t *slot = ring->base + (uint64_t)frag_slot[f] * ring->slot_size;
      uint32_t len = frag_len ? frag_len[f] : rd32(slot + 54);
      bufs->burst_items[f - f0] = (uint64_t)(uintptr_t)(slot + hl);
      bufs->item_size[f - f0] = len;
      total += len;
    }
    if (f1 == f0) { /* a request with no fragments moves nothing */
      if (app->n_tensors == 0 && offsets_out) offsets_out[r] = tr.prev_offset;
      continue;
    }
    /* run list relative to app address 0; the copy below resolves it */
    sgo_gather_skbs(skb, bufs, 0);
    uint64_t base_off = 0;
    if (app->n_tensors == 0) {
      base_off = sgo_tring_get_next(&tr, total);
      if (offsets_out) offsets_out[r] = base_off;
    }
    for (uint64_t k = 0; k < skb->num_items; k++) {
      const uint8_t *src = (const uint8_t *)(uintptr_t)skb->i_buf[k];
      if (app->n_tensors == 0)
        copy_into_arena(app->arena, app->arena_cap, base_off + skb->o_buf[k], src, skb->len[k]);
      else
        copy_tensor_major(app, r, skb->o_buf[k], (uint8_t *)(uintptr_t)src, skb->len[k], 1);
      runs++;
    }
  }
  if (runs >= 0 && app->n_tensors == 0) {
    if (offsets_out) offsets_out[n_req] = tr.prev_offset;
    *cursor = tr.prev_offset;
  }
  free(bufs);
  free(skb);
  return runs;
}

int64_t sgo_scatter_batch(const sgo_ring *rx, const sgo_ring *tx, const uint32_t *tx_slot,
                          const uint32_t *hdr_src_slot, const uint32_t *resp_first,
                          const uint64_t *resp_size, uint64_t fixed_resp_size, uint32_t n_req,
                          uint32_t mtu, uint32_t flags, const sgo_app_bufs *app, uint64_t *cursor,
                          uint64_t *offsets_out, const uint8_t *hdr_templates,
                          const uint64_t *req_token)
{
  const uint32_t hl = sgo_hdr_len(tx->profile);
  sgo_bufs *bufs = (sgo_bufs *)malloc(sizeof *bufs);
  sgo_sk_buf *skb = (sgo_sk_buf *)malloc(sizeof *skb);
  int64_t frames = 0;
  if (!bufs || !skb) { free(bufs); free(skb); return -1; }
  sgo_tring tr;
  if (app->n_tensors == 0) {
    sgo_tring_init(&tr, 0, app->arena_cap);
    tr.prev_offset = *cursor % app->arena_cap;
    tr.prev_addr = tr.prev_offset;
  }
  for (uint32_t r = 0; r < n_req; r++) {
    uint64_t size = resp_size ? resp_size[r] : fixed_resp_size;
    uint32_t f0 = resp_first[r], f1 = resp_first[r + 1];
    uint32_t nf = f1 - f0;
    if (nf > SGO_MAX_BI_SIZE - 1 || nf != sgo_num_frames(size, mtu)) { frames = -1; break; }
    uint64_t base_off = 0;
    if (app->n_tensors == 0) {
      base_off = nf ? sgo_tring_get_next(&tr, size) : tr.prev_offset;
      if (offsets_out) offsets_out[r] = base_off;
    }
    if (nf == 0) continue;
    /* headers first: the frames take the request header found in the rx ring
     * (rr_set_hdr runs before the payload copy, p2p_rpc_dpdk_server.cc:132-136) */
    bufs->num_items = (uint16_t)nf;
    for (uint32_t i = 0; i < nf; i++) {
      uint8_t *slot = tx->base + (uint64_t)tx_slot[f0 + i] * tx->slot_size;
      uint32_t len = sgo_frame_len(size, mtu, i);
      uint8_t h[64];
      if (hdr_templates) {
        /* fresh response buffers: rr_set_hdr, transport/dpdk_transport_ng.h:113-141 */
        const uint8_t *t = hdr_templates + (uint64_t)r * 64;
        uint64_t tok = req_token ? req_token[r] : rd64(t + 42);
        sgo_template_resp_hdr(h, t, tx->profile, flags, tok, (uint16_t)i, (uint16_t)nf, len);
      } else {
        const uint8_t *hsrc = rx->base + (uint64_t)hdr_src_slot[f0 + i] * rx->slot_size;
        memcpy(h, hsrc, hl);
        sgo_rewrite_resp_hdr(h, tx->profile, flags, (uint16_t)i, (uint16_t)nf, len);
      }
      memcpy(slot, h, hl);
      bufs->burst_items[i] = (uint64_t)(uintptr_t)(slot + hl);
      bufs->item_size[i] = len;
    }
    sgo_scatter_skbs(skb, bufs, 0);
    for (uint64_t k = 0; k < skb->num_items; k++) {
      uint8_t *dst = (uint8_t *)(uintptr_t)skb->o_buf[k];
      if (app->n_tensors == 0)
        copy_from_arena(app->arena, app->arena_cap, base_off + skb->i_buf[k], dst, skb->len[k]);
      else
        copy_tensor_major(app, r, skb->i_buf[k], dst, skb->len[k], 0);
    }
    if (flags & SGO_F_UDP_CSUM_FULL) {
      for (uint32_t i = 0; i < nf; i++) {
        uint8_t *slot = tx->base + (uint64_t)tx_slot[f0 + i] * tx->slot_size;
        wr16(slot + 40, 0);
        wr16(slot + 40, sgo_udp_full_csum(slot + SGO_IP_OFF, slot + SGO_UDP_OFF));
      }
    }
    frames += nf;
  }
  if (frames >= 0 && app->n_tensors == 0) {
    if (offsets_out) offsets_out[n_req] = tr.prev_offset;
    *cursor = tr.prev_offset;
  }
  free(bufs);
  free(skb);
  return frames;
}

double sgo_now_sec(void)
{
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}
