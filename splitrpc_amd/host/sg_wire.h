// sg_wire.h -- wire structs and the per-connection header template of the
// reference (src/eth_common.h:13-46, src/p2p_rpc.h:10-45,
// src/p2p_rpc_conn_info.h), host side.  Only what the receive path needs to
// file a packet under its request lives here; rewriting response headers is
// the GPU's work (sg_hip_scatter_batch / sg_hip_swap_hdrs).
#pragma once

#include <arpa/inet.h>

#include <cstdint>
#include <cstring>
#include <sstream>
#include <string>

#include "sg_hip.h"

#pragma pack(push, 1)
struct mac_addr {
  uint8_t addr[6];
};

struct eth_hdr {
  mac_addr dst_mac_;
  mac_addr src_mac_;
  uint16_t eth_type_;
};

// Network byte order.  Byte 0 is version (high nibble) and ihl (low nibble).
struct ipv4_hdr {
  uint8_t ihl : 4;
  uint8_t version : 4;
  uint8_t ecn : 2;
  uint8_t dscp : 6;
  uint16_t tot_len;
  uint16_t id;
  uint16_t frag_off;
  uint8_t ttl;
  uint8_t protocol;
  uint16_t check;
  uint32_t src_ip;
  uint32_t dst_ip;
};

struct udp_hdr {
  uint16_t src_port;
  uint16_t dst_port;
  uint16_t len;
  uint16_t check;
};

static constexpr int UDP_HEADER_LEN = sizeof(eth_hdr) + sizeof(ipv4_hdr) + sizeof(udp_hdr);
static constexpr uint16_t ETHER_TYPE_IPV4 = 0x0800;

// The reference's RPC header (src/p2p_rpc.h:10-17): 64 bytes.
struct p2p_rpc_hdr {
  uint8_t pkt_hdr_t[UDP_HEADER_LEN];
  uint64_t req_token;
  int64_t sock_perf_header;
  uint16_t seq_num;
  uint8_t _pad[64 - (UDP_HEADER_LEN + sizeof(uint64_t) + sizeof(int64_t) + sizeof(uint16_t))];
};

// The 58-byte benchmark profile: request id, fragment index, fragment count
// and payload bytes travel in the header.
struct bl58_rpc_hdr {
  uint8_t pkt_hdr_t[UDP_HEADER_LEN];
  uint64_t req_id;
  uint16_t frag_idx;
  uint16_t num_frags;
  uint32_t payload_len;
};
#pragma pack(pop)

static_assert(UDP_HEADER_LEN == 42, "L2-L4 header");
static_assert(sizeof(p2p_rpc_hdr) == 64 && offsetof(p2p_rpc_hdr, seq_num) == 58, "REF64 header");
static_assert(sizeof(bl58_rpc_hdr) == 58 && offsetof(bl58_rpc_hdr, payload_len) == 54, "BL58 header");

static const size_t RPC_HEADER_LEN = sizeof(p2p_rpc_hdr);
static const size_t RPC_HEADER_TAIL_LEN = RPC_HEADER_LEN - UDP_HEADER_LEN;

static inline uint32_t rpc_header_len(uint32_t profile) { return profile == SG_HDR_REF64 ? 64u : 58u; }

static inline eth_hdr *get_eth_header(p2p_rpc_hdr *h) { return reinterpret_cast<eth_hdr *>(h->pkt_hdr_t); }
static inline ipv4_hdr *get_ip_header(p2p_rpc_hdr *h) { return reinterpret_cast<ipv4_hdr *>(h->pkt_hdr_t + sizeof(eth_hdr)); }
static inline udp_hdr *get_udp_header(p2p_rpc_hdr *h)
{
  return reinterpret_cast<udp_hdr *>(h->pkt_hdr_t + sizeof(eth_hdr) + sizeof(ipv4_hdr));
}
// Both profiles keep the 64-bit request token at byte 42.
static inline uintptr_t get_req_token(const p2p_rpc_hdr *h) { return static_cast<uintptr_t>(h->req_token); }
static inline uint16_t get_seq_num(const p2p_rpc_hdr *h) { return h->seq_num; }
static inline void *get_req_tail(p2p_rpc_hdr *h) { return reinterpret_cast<uint8_t *>(h) + UDP_HEADER_LEN; }

// Fragment index of a received header under either profile.
static inline uint16_t rpc_frag_index(const void *hdr, uint32_t profile)
{
  return profile == SG_HDR_REF64 ? static_cast<const p2p_rpc_hdr *>(hdr)->seq_num
                                 : static_cast<const bl58_rpc_hdr *>(hdr)->frag_idx;
}

// src/eth_common.h:132-169
static inline uint32_t ipv4_from_str(const char *ip)
{
  uint32_t addr = 0;
  if (inet_pton(AF_INET, ip, &addr) != 1) std::printf("inet_pton() failed for %s\n", ip);
  return ntohl(addr);
}

static inline mac_addr mac_from_string(const std::string &mac_str)
{
  std::stringstream ss(mac_str);
  mac_addr ret{};
  for (int i = 0; i < 6; i++) {
    std::string tok;
    std::getline(ss, tok, ':');
    ret.addr[i] = static_cast<uint8_t>(std::stoi(tok, nullptr, 16));
  }
  return ret;
}

// Pre-built header of a connection (src/p2p_rpc_conn_info.h:8-16).
struct p2p_rpc_conn_info {
  p2p_rpc_hdr hdr_template;
};

static inline p2p_rpc_conn_info *alloc_conn_info()
{
  p2p_rpc_conn_info *c = new p2p_rpc_conn_info;
  std::memset(c, 0, sizeof *c);
  return c;
}

static inline void release_conn_info(p2p_rpc_conn_info *c) { delete c; }

// src/eth_common.h:51-89 composed as in src/p2p_rpc_conn_info.h:32-48.
static inline p2p_rpc_conn_info *init_conn_info(int src_port, int dst_port, const char *src_ip_str,
                                                const char *dst_ip_str, mac_addr src_mac, mac_addr dst_mac)
{
  p2p_rpc_conn_info *c = alloc_conn_info();
  eth_hdr *e = get_eth_header(&c->hdr_template);
  e->src_mac_ = src_mac;
  e->dst_mac_ = dst_mac;
  e->eth_type_ = htons(ETHER_TYPE_IPV4);
  ipv4_hdr *ip = get_ip_header(&c->hdr_template);
  ip->version = 4;
  ip->ihl = 5;
  ip->ecn = 1;
  ip->dscp = 0;
  ip->tot_len = htons(sizeof(ipv4_hdr) + sizeof(udp_hdr));
  ip->id = 0;
  ip->frag_off = 0;
  ip->ttl = 128;
  ip->protocol = IPPROTO_UDP;
  ip->src_ip = htonl(ipv4_from_str(src_ip_str));
  ip->dst_ip = htonl(ipv4_from_str(dst_ip_str));
  ip->check = 0;
  udp_hdr *u = get_udp_header(&c->hdr_template);
  u->len = htons(sizeof(ipv4_hdr) + sizeof(udp_hdr));
  u->src_port = htons(src_port);
  u->dst_port = htons(dst_port);
  u->check = 0;
  return c;
}

// "mac,ip,port" of the server (src/p2p_rpc_conn_info.h:50-70)
static inline p2p_rpc_conn_info *initialize_src_conn_info(const std::string &src_uri)
{
  std::stringstream ss(src_uri);
  std::string mac, ip, port;
  std::getline(ss, mac, ',');
  std::getline(ss, ip, ',');
  std::getline(ss, port, ',');
  mac_addr m = mac_from_string(mac);
  return init_conn_info(std::stoi(port), 0, ip.c_str(), "0.0.0.0", m, m);
}

// First packet of a request: remember its RPC tail and where to answer
// (src/p2p_rpc_conn_info.h:73-84).
static inline void set_conn_info(p2p_rpc_conn_info *existing, p2p_rpc_hdr *recv)
{
  std::memcpy(get_req_tail(&existing->hdr_template), get_req_tail(recv), RPC_HEADER_TAIL_LEN);
  get_udp_header(&existing->hdr_template)->dst_port = get_udp_header(recv)->src_port;
  get_ip_header(&existing->hdr_template)->dst_ip = get_ip_header(recv)->src_ip;
  get_eth_header(&existing->hdr_template)->dst_mac_ = get_eth_header(recv)->src_mac_;
}
