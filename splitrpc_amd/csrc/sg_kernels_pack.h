// sg_kernels_pack.h -- fragment tables kept where the device can read them
// (pinned host memory the receive thread writes as fragments arrive) pulled
// into the CSR tables the batched calls take: one table per request, payload
// addresses turned into slot indices of the call's ring.  The host names a
// table per request and touches no fragment.  A part of sg_hip.hip's
// translation unit, included there and nowhere else.
#pragma once

#include "sg_device.h"

namespace {

struct PackArgs {
  const sg_frag_table *tables;
  const uint32_t *table_idx;
  const uint32_t *req_first;
  uint32_t n_req;
  uint32_t n_frags;
  uint32_t n_tables;
  uint64_t delta;       // (ring base + header length) - pkt_base: what lies between an entry and its slot's payload
  uint64_t ring_bytes;  // n_slots * slot_size
  uint32_t slot_size;
  uint32_t n_slots;
  uint32_t *frag_slot;
  uint32_t *frag_len;
  uint32_t *req_first_out;
  const uint32_t *blob_src;
  uint32_t *blob_dst;
  uint32_t blob_words;
  uint32_t req_blocks;  // workgroups that pull tables; the ones behind them copy the blob
};

// L lanes per request, each taking four entries per step (the host launches L = 16 whatever the
// tables' length: what a pull costs the copy kernel beside it grows with the bus reads in flight).
// An entry that is no payload start of the ring becomes slot 0xffffffff, which
// the gather and scatter kernels refuse.
template <int L>
__global__ __launch_bounds__(kBlock) void k_pack_tables(PackArgs a)
{
  constexpr uint32_t G = kBlock / L;  // requests per workgroup
  if (blockIdx.x >= a.req_blocks) {
    // the words that travel along (per-request data such as tokens and header templates)
    const uint32_t n_copy = gridDim.x - a.req_blocks;
    for (uint32_t i = (blockIdx.x - a.req_blocks) * kBlock + threadIdx.x; i < a.blob_words; i += n_copy * kBlock)
      a.blob_dst[i] = a.blob_src[i];
    return;
  }
  const uint32_t r = blockIdx.x * G + threadIdx.x / L, gl = threadIdx.x & (L - 1);
  if (r >= a.n_req) return;
  const uint32_t f0 = a.req_first[r], f1 = a.req_first[r + 1], t = a.table_idx[r];
  if (gl == 0 && a.req_first_out) {
    a.req_first_out[r] = f0;
    if (r == a.n_req - 1) a.req_first_out[a.n_req] = f1;
  }
  if (f1 < f0 || f1 - f0 > SG_MAX_BI_SIZE || f1 > a.n_frags) return;  // no such table: the call's own checks refuse the CSR
  const sg_frag_table *tab = a.tables + t;
  const uint32_t n = f1 - f0;
  // Four entries per lane and load (16 bytes): the tables lie across the bus, where few large reads
  // fare better than many small ones.  Tables are 8 KiB apart, so off[] and len[] are 16-byte aligned.
  for (uint32_t i = gl * 4; i < n; i += L * 4) {
    u32x4 off = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu}, len = {0u, 0u, 0u, 0u};
    if (t < a.n_tables) {
      off = *reinterpret_cast<const u32x4 *>(tab->off + i);
      if (a.frag_len) len = *reinterpret_cast<const u32x4 *>(tab->len + i);
    }
#pragma unroll
    for (uint32_t k = 0; k < 4; k++) {
      if (i + k >= n) break;
      uint32_t slot = 0xffffffffu;
      // payload address - ring base - header length, which must be a whole number of slots
      const uint64_t at = (uint64_t)off[k] << 1, rel = at - a.delta;
      if (off[k] != 0xffffffffu && at >= a.delta && rel < a.ring_bytes) {
        const uint64_t s = rel / a.slot_size;
        if (s * a.slot_size == rel) slot = (uint32_t)s;
      }
      a.frag_slot[f0 + i + k] = slot;
      if (a.frag_len) a.frag_len[f0 + i + k] = len[k];
    }
  }
}

}  // namespace
