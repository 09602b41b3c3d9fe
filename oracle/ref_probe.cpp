// ref_probe.cpp -- thin C entry points over the reference's OWN headers, built
// only where the reference tree is present (see Makefile, target _ref).
// TEST INFRASTRUCTURE ONLY.  The reference headers are included from where
// they lie; nothing of them is copied.  Only headers that compile from the
// reference's own files are used: eth_common.h, p2p_bufs.h,
// p2p_rpc_app_stub.h, p2p_rpc_tring.h.  Everything that includes
// utils/config_utils.h (p2p_rpc.h, p2p_rpc_sg_engine.h, p2p_rpc_rr_ng.h, ...)
// needs spdlog, which neither the reference tree nor this image holds, and
// everything under transport/ needs DPDK or CUDA: those stay unbuilt.
#include <cstdio>
#include <cstdint>
#include <cstddef>
#include <cstring>

#include "eth_common.h"
#include "p2p_bufs.h"
#include "p2p_rpc_app_stub.h"
#include "p2p_rpc_tring.h"

extern "C" {

// Layout facts of the kept tables and wire structs.
uint64_t ref_layout(int what)
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
    default: return ~0ull;
  }
}

// ipv4_pseudo_csum sums 16 bytes of a 16-byte stack buffer of which it writes
// 12.  To make the call repeatable the probe first paints the stack below the
// caller with `fill`, then calls the reference function from the same depth.
// Built at -O0 so that the buffer really lives on the stack.
__attribute__((noinline)) static void paint_stack(uint8_t fill)
{
  volatile uint8_t pad[4096];
  for (size_t i = 0; i < sizeof pad; i++) pad[i] = fill;
}

__attribute__((noinline)) static uint16_t call_csum(struct ipv4_hdr *ip)
{
  return ipv4_pseudo_csum(ip);
}

uint16_t ref_ipv4_pseudo_csum(const uint8_t *ip20, uint8_t stack_fill)
{
  struct ipv4_hdr ip;
  memcpy(&ip, ip20, sizeof ip);
  paint_stack(stack_fill);
  return call_csum(&ip);
}

// Bit-field view of byte 0 (ihl low nibble, version high nibble).
void ref_ip_nibbles(const uint8_t *ip20, int *ihl, int *version)
{
  struct ipv4_hdr ip;
  memcpy(&ip, ip20, sizeof ip);
  *ihl = ip.ihl;
  *version = ip.version;
}

// Header templates (eth_common.h:51-89), written at 0/14/34 of a 42-byte buffer.
void ref_gen_hdr_template(uint8_t *h, const uint8_t *src_mac, const uint8_t *dst_mac,
                          uint32_t src_ip, uint32_t dst_ip, int src_port, int dst_port)
{
  mac_addr s, d;
  memcpy(s.addr, src_mac, 6);
  memcpy(d.addr, dst_mac, 6);
  gen_eth_header_template((eth_hdr *)h, &s, &d);
  gen_ipv4_header_template((ipv4_hdr *)(h + sizeof(eth_hdr)), src_ip, dst_ip);
  gen_udp_header_template((udp_hdr *)(h + sizeof(eth_hdr) + sizeof(ipv4_hdr)), src_port, dst_port);
}

// P2pRpcTring (p2p_rpc_tring.h): replay a list of sizes, return each address.
void ref_tring_replay(uint64_t base, uint64_t capacity, const uint64_t *sizes, uint32_t n,
                      uint64_t *out)
{
  P2pRpcTring t((void *)base, capacity);
  for (uint32_t i = 0; i < n; i++) out[i] = (uint64_t)(uintptr_t)t.get_next(sizes[i]);
}

}  // extern "C"
