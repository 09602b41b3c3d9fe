// sg_tables.h -- the reference's fixed-capacity tables and application stubs,
// kept name for name and byte for byte so that code written against
// src/p2p_bufs.h and src/p2p_rpc_app_stub.h compiles and links unchanged.
#pragma once

#include <cstddef>
#include <cstdint>
#include <cstdio>

#include "sg_hip.h"

// src/p2p_bufs.h:10-11 -- has to stay below 2^16
const uint16_t MAX_BI_SIZE = SG_MAX_BI_SIZE;
const uint16_t MAX_WI_SIZE = 1024;

#pragma pack(push, 1)
// src/p2p_bufs.h:15-18: pointers to RPC headers or to transport buffers
struct p2p_hbufs {
  uintptr_t burst_items[MAX_BI_SIZE];
  uint16_t num_items;
};

// src/p2p_bufs.h:23-27: <pointer to payload, payload bytes> per fragment
struct p2p_bufs {
  uintptr_t burst_items[MAX_BI_SIZE];
  size_t item_size[MAX_BI_SIZE];
  uint16_t num_items;
};

// src/p2p_bufs.h:33-40: run list.  RX: i_buf -> packet, o_buf -> app buffer;
// TX the other way round.  len has MAX_BI_SIZE - 1 entries: a table can
// describe at most 1023 runs.
class p2p_sk_buf {
 public:
  uintptr_t i_buf[MAX_BI_SIZE];
  uintptr_t o_buf[MAX_BI_SIZE];
  size_t len[MAX_BI_SIZE - 1];
  size_t num_items;
};

// src/p2p_rpc_app_stub.h:10-29
#define MAX_NUM_TENSORS SG_MAX_TENSORS
class g_params_v2 {
 public:
  uintptr_t inputs[MAX_NUM_TENSORS];
  uintptr_t outputs[MAX_NUM_TENSORS];
  size_t input_tensor_size[MAX_NUM_TENSORS];
  size_t output_tensor_size[MAX_NUM_TENSORS];
};

class g_params {
 public:
  uint8_t *req;   // request payload
  uint8_t *resp;  // response payload
};
#pragma pack(pop)

static_assert(sizeof(p2p_hbufs) == 8194 && sizeof(p2p_hbufs) == sizeof(sg_hbufs), "p2p_hbufs layout");
static_assert(sizeof(p2p_bufs) == 16386, "p2p_bufs layout");
static_assert(sizeof(p2p_sk_buf) == 24576 && sizeof(p2p_sk_buf) == sizeof(sg_sk_buf), "p2p_sk_buf layout");
static_assert(offsetof(p2p_sk_buf, num_items) == offsetof(sg_sk_buf, num_items), "p2p_sk_buf layout");
static_assert(sizeof(g_params) == 16 && sizeof(g_params_v2) == 128, "app stub layout");

// src/p2p_bufs.h:42-62: eyeball dumps
static inline void print_bufs(const p2p_bufs *bufs)
{
  std::printf("BUF: %p, num_items: %d\n", (const void *)bufs, bufs->num_items);
  for (size_t i = 0; i < bufs->num_items; i++)
    std::printf("i: %zu, bi_ptr: %p, bi_size: %zu\n", i, (void *)bufs->burst_items[i], (size_t)bufs->item_size[i]);
}

static inline void print_skb(const p2p_sk_buf *skb)
{
  std::printf("SKB: %p, num_items: %zu\n", (const void *)skb, (size_t)skb->num_items);
  for (size_t i = 0; i < skb->num_items; i++)
    std::printf("i: %zu, i_buf: %p, o_buf: %p, len: %zu\n", i, (void *)skb->i_buf[i], (void *)skb->o_buf[i],
                (size_t)skb->len[i]);
}
