// sg_hip.hip -- C ABI and host side of the gfx950 scatter-gather engine; the
// kernels it launches are in sg_kernels_prep.h, sg_kernels_copy.h and
// sg_kernels_reassemble.h, one translation unit with this file.
//
// Three kernels carry a batch:
//   k_prep_*   one workgroup (or, for short requests, one wavefront) per
//              request: exclusive scan of the fragment lengths (-> offset of
//              every fragment inside its request, the running sum gather_skbs
//              keeps, src/p2p_rpc_sg_engine.h:22-43) and the request total.
//              Emits 16-byte run descriptors.  k_req_scan then scans the
//              request totals through the device-resident bump-ring cursor
//              (src/p2p_rpc_tring.h:27-33); with one size for all requests the
//              offsets are multiples and k_prep_* writes them itself.
//   k_gather   one wavefront per fragment run: ring slot payload -> tensor.
//   k_scatter  one wavefront per response frame: tensor -> TX slot payload,
//              header rewrite, checksums.
// When the caller declares one request size and the fragmenting rule, the
// descriptor pass is skipped: k_gather_rule and the FUSED form of k_scatter
// derive every offset themselves and hold the tables against the rule.
// Plus k_copy_runs / k_swap_hdrs for the per-request entry points and k_ra_*
// for sorting a burst of arrivals into requests (sg_hip_reassemble).
#include <hip/hip_runtime.h>

#include <errno.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <mutex>
#include <new>
#include <vector>

#include "../../include/sg_hip.h"
#include "sg_device.h"

using namespace sg;

#include "sg_kernels_prep.h"
#include "sg_kernels_copy.h"
#include "sg_kernels_reassemble.h"
#include "sg_kernels_pack.h"

// ---------------------------------------------------------------------------
// scratch of the allocation-free entry point
// ---------------------------------------------------------------------------
// One array per GPU the library runs on, held until the process ends.  Host
// code never uses the array's name as an address: the address on each device
// comes from hipGetSymbolAddress (static_scratch_of below).
namespace {
constexpr size_t kStaticDesc = sizeof(u32x4) * (size_t)SG_STATIC_MAX_FRAMES;
constexpr size_t kStaticReq = sizeof(uint64_t) * (size_t)SG_STATIC_MAX_REQS;
constexpr size_t kStaticTile = sizeof(uint64_t) * (SG_STATIC_MAX_REQS / kPartMin + 2);
constexpr size_t kStaticWords = 256;  // cursors, staged cursors, status, refusal flag
// 64-bit words a context keeps beside its scratch: two cursors of kCurWords each, their staged
// successors, the two slot indices (one word), the descriptor tag (four words)
constexpr size_t kCtxWords = 2 * kCurWords + 8;
static_assert(2 + 1 + kTagWords / 2 <= 8, "the words behind the cursors");
constexpr size_t kStaticBytes = kStaticDesc + 2 * kStaticReq + kStaticTile + kStaticWords;
}  // namespace
static __device__ __align__(256) uint8_t scratch[kStaticBytes];

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------

struct EvPair {
  hipEvent_t a, b;
  int which;
};

// Device memory a batched call works in, beyond its inputs and outputs.  A
// context owns one set (allocated at creation); the allocation-free entry
// point uses a set carved out of a static device array.
struct Scratch {
  uint32_t max_reqs = 0, max_frames = 0;
  u32x4 *desc = nullptr;         // run descriptors, max_frames
  uint64_t *req_size = nullptr;  // max_reqs
  uint64_t *req_off = nullptr;   // max_reqs
  uint64_t *tile_tot = nullptr;  // one total per kScanTile requests, for the tiled request scan
  // bump-ring cursors (request arena, response arena) and the values a
  // descriptor pass stages for the copy kernel to commit
  uint64_t *cursor[2] = {nullptr, nullptr};
  uint64_t *next_cursor[2] = {nullptr, nullptr};
  // the cursors are pairs of cells (a context: the single-kernel calls advance them themselves) or
  // plain words (the allocation-free entry point, whose caller may bring the word)
  bool cursor_cells = false;
  uint32_t *slot_idx[2] = {nullptr, nullptr};  // next slot of the application ring to fill / to serve
  uint32_t *desc_tag = nullptr;    // kTag* words: what the descriptors in `desc` were made of and held against
  uint32_t *desc_gen = nullptr;    // host counter behind the generation (one per scratch)
  uint32_t *call_seq = nullptr;    // host count of self-advancing launches (a context's; part of their stamps)
  bool stamps_ok = false;          // launches on this device tell themselves apart by queue and dispatch id
  uint32_t *csum_part = nullptr;   // kPartStride words per frame (two-phase UDP checksum of long frames)
  uint32_t *csum_valid = nullptr;  // one mark per frame, zero between calls
  uint32_t *status = nullptr;
  volatile uint32_t *flag = nullptr;  // raised with every refusal (pinned host memory in a context)
};

struct sg_hip_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  bool own_stream = false;
  uint32_t max_reqs = 0, max_frames = 0;
  // device scratch
  u32x4 *desc = nullptr;
  uint64_t *req_size = nullptr;
  uint64_t *req_off = nullptr;
  uint64_t *tile_tot = nullptr;  // one total per 4096 requests, for the tiled request scan
  // kCurWords words each: request-arena cursor, response-arena cursor; then their staged
  // successors, the two slot indices, the descriptor tag
  uint64_t *cursors = nullptr;
  uint32_t *csum_scratch = nullptr;  // csum_part and csum_valid
  uint32_t desc_gen = 0;
  uint32_t call_seq = 0;
  uint32_t *status = nullptr;
  Scratch sc;
  // pinned staging for the per-request entry points (device reads it in place)
  Run *h_runs = nullptr;
  uint32_t h_runs_cap = 0;
  uint64_t *h_ptrs = nullptr;
  uint64_t *h_probe = nullptr;   // pinned: what a probe launch saw of itself (queue address, dispatch id), twice
  uint32_t *h_status = nullptr;  // pinned: [0] copy of status (read back only after a refusal), [1] the refusal flag
  volatile uint32_t *h_flag = nullptr;
  // profiling
  bool profiling = false;
  std::vector<EvPair> ev_used, ev_free;
  double prof_ms[6] = {0, 0, 0, 0, 0, 0};
  uint64_t prof_n[6] = {0, 0, 0, 0, 0, 0};
  // reassembly scratch, allocated by the first sg_hip_reassemble call
  void *ra_mem = nullptr;
  uint32_t ra_cells = 0;    // cells of the request table (power of two >= 4 * max_reqs)
  uint32_t ra_records = 0;  // records of the pool (power of two >= max_reqs)
  uint32_t *h_counts = nullptr;  // pinned: requests, fragments, dropped, in flight (written by k_ra_scan itself)
  char err[512] = {0};
};

static char g_create_err[512];

static int fail(sg_hip_ctx *c, int code, const char *fmt, ...)
{
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(c ? c->err : g_create_err, 512, fmt, ap);
  va_end(ap);
  return code;
}

#define HIP_TRY(c, call)                                                                      \
  do {                                                                                        \
    hipError_t e_ = (call);                                                                   \
    if (e_ != hipSuccess)                                                                     \
      return fail((c), SG_E_HIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e_),       \
                  __FILE__, __LINE__);                                                        \
  } while (0)

namespace {

struct DeviceGuard {
  int prev = -1;
  bool ok = false;
  explicit DeviceGuard(int dev)
  {
    if (hipGetDevice(&prev) == hipSuccess) {
      if (prev == dev) ok = true;
      else ok = hipSetDevice(dev) == hipSuccess;
    }
  }
  ~DeviceGuard()
  {
    if (ok && prev >= 0) (void)hipSetDevice(prev);
  }
};

uint32_t hdr_len_of(uint32_t profile) { return profile == SG_HDR_REF64 ? 64u : 58u; }

int check_ring(sg_hip_ctx *c, const sg_ring_desc &r, const char *what)
{
  if (!r.base || r.n_slots == 0) return fail(c, SG_E_INVAL, "%s ring: null base or no slots", what);
  if (r.hdr_profile > SG_HDR_REF64) return fail(c, SG_E_INVAL, "%s ring: unknown header profile %u", what, r.hdr_profile);
  if (r.slot_size < hdr_len_of(r.hdr_profile) || (r.slot_size & 1u))
    return fail(c, SG_E_INVAL, "%s ring: slot size %u must be even and hold a header", what, r.slot_size);
  if ((uintptr_t)r.base & 1u) return fail(c, SG_E_INVAL, "%s ring: base address must be even", what);
  return SG_OK;
}

int check_app(sg_hip_ctx *c, const sg_app_desc &a, AppDev *out, uint64_t *max_req_bytes)
{
  if (a.n_tensors > SG_MAX_TENSORS) return fail(c, SG_E_INVAL, "n_tensors %u > %d", a.n_tensors, SG_MAX_TENSORS);
  memset(out, 0, sizeof *out);
  out->n_tensors = a.n_tensors;
  *max_req_bytes = 0;
  if (a.n_tensors == 0) {
    if (!a.arena || a.arena_cap == 0) return fail(c, SG_E_INVAL, "packed mode needs an arena and a capacity");
    out->arena = static_cast<uint8_t *>(a.arena);
    out->cap = a.arena_cap;
    out->mirrored = a.arena_mirrored ? 1u : 0u;
    return SG_OK;
  }
  for (uint32_t t = 0; t < a.n_tensors; t++) {
    if (!a.tensor_base[t] || a.tensor_size[t] == 0)
      return fail(c, SG_E_INVAL, "tensor %u: null base or zero size", t);
    out->tensor_base[t] = static_cast<uint8_t *>(a.tensor_base[t]);
    out->tensor_size[t] = a.tensor_size[t];
    *max_req_bytes += a.tensor_size[t];
  }
  return SG_OK;
}

// Launch geometry for one wavefront per item; with the XCD-aware order the
// grid is padded to whole rounds of kXcds * kXcdRun workgroups.
void geometry(uint64_t n_waves, bool want_remap, uint32_t *grid, uint32_t *remap)
{
  const uint32_t groups = (uint32_t)((n_waves + kWavesPerBlock - 1) / kWavesPerBlock);
  const uint32_t round = kXcds * kXcdRun;
  if (want_remap && groups >= 2 * round) {
    *grid = (groups + round - 1) / round * round;
    *remap = 1;
  } else {
    *grid = groups;
    *remap = 0;
  }
}

int prof_begin(sg_hip_ctx *c, int which)
{
  if (!c || !c->profiling) return SG_OK;
  EvPair p;
  if (!c->ev_free.empty()) {
    p = c->ev_free.back();
    c->ev_free.pop_back();
  } else {
    HIP_TRY(c, hipEventCreate(&p.a));
    HIP_TRY(c, hipEventCreate(&p.b));
  }
  p.which = which;
  HIP_TRY(c, hipEventRecord(p.a, c->stream));
  c->ev_used.push_back(p);
  return SG_OK;
}

int prof_end(sg_hip_ctx *c)
{
  if (!c || !c->profiling) return SG_OK;
  HIP_TRY(c, hipEventRecord(c->ev_used.back().b, c->stream));
  return SG_OK;
}

int prof_drain(sg_hip_ctx *c)
{
  for (EvPair &p : c->ev_used) {
    float ms = 0.f;
    HIP_TRY(c, hipEventElapsedTime(&ms, p.a, p.b));
    c->prof_ms[p.which] += ms;
    c->prof_n[p.which] += 1;
    c->ev_free.push_back(p);
  }
  c->ev_used.clear();
  return SG_OK;
}

// The word a kernel reads the cursor from when nothing advances it beside that kernel.
const uint64_t *plain_cursor(const Scratch &sc, int which)
{
  return sc.cursor_cells ? sc.cursor[which] + kCurPlain : sc.cursor[which];
}

// A context's single-kernel call advances its cursor itself when it is small: finding the live
// cell costs every wavefront some twenty scalar instructions, the one-workgroup kernel behind the
// call 2 to 4 us of stream time whatever the call's size.  Measured per step (gather and scatter
// call on a stream each): 16 requests of 602112 bytes 13.0 -> 8.9 us, eight such batches in one
// call 31.6 -> 30.7 us, 32 batches 105.9 -> 105.3 us; 8192 requests of 3136 bytes 18.1 -> 16.0 us,
// 65536 of them 89.8 -> 90.4 us; 256 requests of 1.5 MB in 8800-byte fragments 233.5 -> 235.6 us.
// A call that publishes slot states has the kernel behind it anyway.
constexpr uint64_t kSelfAdvanceMaxWaves = 65536;
bool self_advancing(const Scratch &sc, bool packed, const void *slot_state, uint64_t waves, uint32_t flags)
{
  if ((flags & SG_F_TAIL_KERNEL) || !sc.stamps_ok) return false;
  return packed && sc.cursor_cells && !slot_state && (waves <= kSelfAdvanceMaxWaves || (flags & SG_F_SELF_ADVANCE));
}


// Descriptor build: kernel shape by the average request, then the bump-ring
// scan of the request totals where offsets are not plain multiples.
int launch_prep(sg_hip_ctx *c, const Scratch &sc, hipStream_t st, const PrepArgs &args)
{
  int rc = prof_begin(c, 0);
  if (rc != SG_OK) return rc;
  PrepArgs p = args;
  const uint32_t avg = p.n_items / p.n_req;
  const bool tiled = p.packed && !p.fixed_offsets && !(p.n_req <= 2 * kScanTile || p.counts);
  // requests per entry of the workgroup sums k_prep_group leaves for the tiled scan
  const uint32_t per_part = avg <= 8 ? 4 * kWavesPerBlock : avg <= 16 ? 2 * kWavesPerBlock : 0;
  if (tiled && per_part) p.part = sc.tile_tot;
  if (avg <= 8) {
    k_prep_group<16><<<(p.n_req + 4 * kWavesPerBlock - 1) / (4 * kWavesPerBlock), kBlock, 0, st>>>(p);
  } else if (avg <= 16) {
    k_prep_group<32><<<(p.n_req + 2 * kWavesPerBlock - 1) / (2 * kWavesPerBlock), kBlock, 0, st>>>(p);
  } else if (avg <= 32) {
    k_prep_wave<<<(p.n_req + kWavesPerBlock - 1) / kWavesPerBlock, kBlock, 0, st>>>(p);
  } else if (avg <= 256) {
    k_prep_block<256><<<p.n_req, 256, 0, st>>>(p);
  } else {
    k_prep_block<1024><<<p.n_req, 1024, 0, st>>>(p);
  }
  if (p.packed && !p.fixed_offsets) {
    if (p.n_req <= 2 * kScanTile || p.counts) {  // counts on the device: one workgroup walks whatever is there
      k_req_scan<<<1, kScanBlock, 0, st>>>(p);
    } else {
      const uint32_t n_tiles = (p.n_req + kScanTile - 1) / kScanTile;
      if (p.part) {
        k_req_scan_parts<<<n_tiles, kScanBlock, 0, st>>>(p, per_part, n_tiles);
      } else {
        // (one launch in which every workgroup adds up the REQUEST sizes before its tile by itself
        // was measured at 32768 requests: 30.6 us for the descriptor pass against 26.9 us with these)
        k_req_scan_local<<<n_tiles, kScanBlock, 0, st>>>(p, sc.tile_tot);
        k_req_scan_add<<<n_tiles, kScanBlock, 0, st>>>(p, sc.tile_tot, n_tiles);
      }
    }
  }
  return prof_end(c);
}

// Behind the copy kernel: advance the cursor (single-kernel calls on a packed
// arena) and publish slot states (where the caller keeps a slot ring).
void launch_finish(const Scratch &sc, hipStream_t st, uint64_t *cursor, uint64_t size, uint64_t cap, uint32_t n_req,
                   const uint32_t *counts, uint32_t *state, uint32_t n_states, int which, bool all_or_nothing)
{
  if (!cursor && !state) return;
  FinishArgs f;
  memset(&f, 0, sizeof f);
  f.cursor = cursor;
  f.cursor_cells = sc.cursor_cells ? 1u : 0u;
  f.size = size;
  f.cap = cap;
  f.n_req = n_req;
  f.counts = counts;
  f.state = state;
  f.n_states = n_states;
  f.slot_idx = sc.slot_idx[which];
  // gather fills FREE slots and publishes RX_COMPLETE; scatter serves WORK_COMPLETE slots and
  // frees them (src/splitrpc_server/p2p_rpc_dpdk_server.cc:130,175; states src/p2p_rpc_app_ctx.h:22)
  f.expect = which == 0 ? SG_SLOT_FREE : SG_SLOT_WORK_COMPLETE;
  f.publish = which == 0 ? SG_SLOT_RX_COMPLETE : SG_SLOT_FREE;
  f.all_or_nothing = all_or_nothing ? 1u : 0u;
  f.status = sc.status;
  f.status_flag = sc.flag;
  k_finish<<<1, kBlock, 0, st>>>(f);
}

int finish(sg_hip_ctx *c, uint32_t flags)
{
  HIP_TRY(c, hipGetLastError());
  if (!c) return SG_OK;  // allocation-free entry point: launches only
  if (flags & SG_F_ASYNC) {
    // keep the event list bounded on long asynchronous runs
    if (c->profiling && c->ev_used.size() > 4096) return sg_hip_sync(c);
    return SG_OK;
  }
  return sg_hip_sync(c);
}

}  // namespace

// Walks the tensor-major buffers once per fragment index (all requests of the call have `size`
// bytes cut at `mtu`): where fragment i lands, for every i.  Returns the number of entries, or 0
// when there is no plan (more fragments per request than entries, a tensor of 4 GiB or more per
// request).
static uint32_t fill_plan(const AppDev &app, uint64_t size, uint32_t mtu, uint64_t per, FragPlan *plan)
{
  if (per > kPlanMax) return 0;
  for (uint32_t t = 0; t < app.n_tensors; t++)
    if (app.tensor_size[t] > 0xffffffffull) return 0;
  for (uint32_t i = 0; i < per; i++) {
    const uint64_t off = (uint64_t)i * mtu;
    const uint64_t len = size - off < mtu ? size - off : mtu;
    FragPlan &fp = plan[i];
    memset(&fp, 0, sizeof fp);
    fp.kind = 2;
    uint64_t t0 = 0;
    for (uint32_t t = 0; t < app.n_tensors; t++) {
      const uint64_t t1 = t0 + app.tensor_size[t];
      if (off < t1) {
        fp.base_a = (uint64_t)(uintptr_t)app.tensor_base[t] + (off - t0);
        fp.stride_a = (uint32_t)app.tensor_size[t];
        if (off + len <= t1) {
          fp.kind = 0;
          fp.len_a = (uint32_t)len;
        } else if (t + 1 < app.n_tensors && off + len <= t1 + app.tensor_size[t + 1]) {
          fp.kind = 1;
          fp.len_a = (uint32_t)(t1 - off);
          fp.base_b = (uint64_t)(uintptr_t)app.tensor_base[t + 1];
          fp.stride_b = (uint32_t)app.tensor_size[t + 1];
        }
        break;
      }
      t0 = t1;
    }
  }
  return (uint32_t)per;
}

// floor(n / d) == (n * M) >> (27 + l) for every n < 2^27, with l = ceil(log2 d), M = ceil(2^(27 + l) / d)
static void magic_div(uint64_t d, uint32_t *mul, uint32_t *shift)
{
  uint32_t l = 0;
  while ((1ull << l) < d) l++;
  *shift = 27 + l;
  *mul = (uint32_t)(((1ull << *shift) + d - 1) / d);
}

// Lanes a short frame of at most `bytes` payload bytes is given (two steps of L - 1
// chunks without looping), or 0 where a whole wavefront per frame is the better deal.
// Groups of 8 lanes pay up to 128 bytes (131072 single-fragment requests and their responses,
// 4 -> 8 to a wavefront: gather 18.4 -> 13.3 us at 40 bytes, 20.5 -> 18.6 us at 128, 24.6 -> 24.9 us
// at 200; scatter 26.2 -> 21.7 us at 40, 25.6 -> 23.9 us at 128, 29.2 -> 32.0 us at 224); `eight`:
// the caller has kernels for such groups.
static uint32_t small_lanes(uint64_t bytes, bool eight = true)
{
  if (eight && bytes <= 128) return 8;
  if (bytes <= 2 * 15 * 16) return 16;
  if (bytes <= 2 * 31 * 16) return 32;
  return 0;
}

// Remainder fragments get wavefronts of their own kind when they are a good share of the
// call's wavefronts -- and, where that takes a launch of its own (scatter), when the call is
// large enough to hide one more launch.
static bool small_last_pays(uint64_t per_req, uint32_t n_req, uint32_t flags, bool own_launch)
{
  if (per_req < 2) return false;
  return (flags & SG_F_FORCE_SMALL) || (per_req <= 8 && (!own_launch || n_req >= 1024));
}

// adv: the kernel takes the cursor from the context's cells and advances it (self-advancing call)
template <bool ADV>
static void launch_scatter_small_as(hipStream_t st, const ScatterArgs &sa, uint32_t lanes, uint32_t n_frames, bool full_csum)
{
  const uint32_t per_wave = kWave / lanes;
  const uint32_t grid = (n_frames + per_wave * kWavesPerBlock - 1) / (per_wave * kWavesPerBlock);
  if (lanes == 8 && full_csum) k_scatter_small<8, true, ADV><<<grid, kBlock, 0, st>>>(sa);
  else if (lanes == 8) k_scatter_small<8, false, ADV><<<grid, kBlock, 0, st>>>(sa);
  else if (lanes == 16 && full_csum) k_scatter_small<16, true, ADV><<<grid, kBlock, 0, st>>>(sa);
  else if (lanes == 16) k_scatter_small<16, false, ADV><<<grid, kBlock, 0, st>>>(sa);
  else if (full_csum) k_scatter_small<32, true, ADV><<<grid, kBlock, 0, st>>>(sa);
  else k_scatter_small<32, false, ADV><<<grid, kBlock, 0, st>>>(sa);
}
static void launch_scatter_small(hipStream_t st, const ScatterArgs &sa, uint32_t lanes, uint32_t n_frames, bool full_csum,
                                 bool adv)
{
  if (adv) launch_scatter_small_as<true>(st, sa, lanes, n_frames, full_csum);
  else launch_scatter_small_as<false>(st, sa, lanes, n_frames, full_csum);
}

// Long frames with the full UDP checksum go to several wavefronts per frame when the
// scratch has room for their sums (k_scatter<.., DEFER> + k_udp_finish).
static bool csum_in_two_phases(const Scratch &sc, uint32_t pieces, bool full_csum)
{
  return full_csum && pieces > 1 && pieces + 1 <= kPartStride && sc.csum_part != nullptr;
}

template <bool FUSED, bool ADV = false>
static void launch_scatter(hipStream_t st, const ScatterArgs &sa, uint32_t grid, bool full_csum, bool defer = false)
{
  const bool lng = sa.pieces > 1;
  if (defer) {
    k_scatter<true, FUSED, true, true, ADV><<<grid, kBlock, 0, st>>>(sa);
    k_udp_finish<FUSED><<<(sa.n_items + kBlock - 1) / kBlock, kBlock, 0, st>>>(sa);
  } else if (full_csum && lng) k_scatter<true, FUSED, true, false, ADV><<<grid, kBlock, 0, st>>>(sa);
  else if (full_csum) k_scatter<true, FUSED, false, false, ADV><<<grid, kBlock, 0, st>>>(sa);
  else if (lng) k_scatter<false, FUSED, true, false, ADV><<<grid, kBlock, 0, st>>>(sa);
  else k_scatter<false, FUSED, false, false, ADV><<<grid, kBlock, 0, st>>>(sa);
}

// The declared-rule gather in its shapes: all fragments short / a short last fragment per request
// dealt in turns with the others / long fragments on several wavefronts.
template <bool ADV>
static void launch_gather_rule(hipStream_t st, const GatherRuleArgs &ga, uint32_t grid, uint32_t small_all,
                               uint32_t small_last, uint32_t n_items)
{
  if (small_all) {
    const uint32_t per_wave = kWave / small_all;
    const uint32_t sgrid = (n_items + per_wave * kWavesPerBlock - 1) / (per_wave * kWavesPerBlock);
    if (small_all == 8) k_gather_small<8, ADV><<<sgrid, kBlock, 0, st>>>(ga);
    else if (small_all == 16) k_gather_small<16, ADV><<<sgrid, kBlock, 0, st>>>(ga);
    else k_gather_small<32, ADV><<<sgrid, kBlock, 0, st>>>(ga);
  } else if (small_last == 16) {
    if (ga.pieces > 1) k_gather_rule<true, 16, ADV><<<grid, kBlock, 0, st>>>(ga);
    else k_gather_rule<false, 16, ADV><<<grid, kBlock, 0, st>>>(ga);
  } else if (small_last == 32) {
    if (ga.pieces > 1) k_gather_rule<true, 32, ADV><<<grid, kBlock, 0, st>>>(ga);
    else k_gather_rule<false, 32, ADV><<<grid, kBlock, 0, st>>>(ga);
  } else {
    if (ga.pieces > 1) k_gather_rule<true, 0, ADV><<<grid, kBlock, 0, st>>>(ga);
    else k_gather_rule<false, 0, ADV><<<grid, kBlock, 0, st>>>(ga);
  }
}

// One direction's share of a launch that carries both (sg_hip_shunt_batch).
struct ShuntHalf {
  GatherRuleArgs g;
  ScatterArgs s;
  uint32_t g_grid = 0, s_grid = 0;
  uint32_t g_small = 0;  // lanes of the gather's short last fragments (0: none)
  uint32_t s_small = 0;  // lanes of the scatter's frames when all are short (0: a wavefront each)
  bool full_csum = false;
};
constexpr int kNoShare = 1;  // the call needs kernels of its own

// What a self-advancing launch tells itself from every other launch by, as one wavefront sees it.
__global__ void k_stamp_probe(uint64_t *out)
{
  if (threadIdx.x == 0) {
    out[0] = launch_queue(0);
    out[1] = launch_stamp();
  }
}

extern "C" {

int sg_hip_abi_version(void) { return SG_HIP_ABI_VERSION; }

const char *sg_hip_last_error(const sg_hip_ctx *ctx) { return ctx ? ctx->err : g_create_err; }

void *sg_hip_stream(sg_hip_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

static int create_impl(sg_hip_ctx *c, int device_id, const sg_hip_cfg *cfg)
{
  int n_dev = 0;
  HIP_TRY(nullptr, hipGetDeviceCount(&n_dev));
  if (device_id < 0 || device_id >= n_dev)
    return fail(nullptr, SG_E_INVAL, "device %d not present (%d devices)", device_id, n_dev);
  c->device = device_id;
  DeviceGuard g(device_id);
  if (!g.ok) return fail(nullptr, SG_E_HIP, "cannot select device %d", device_id);
  hipDeviceProp_t prop;
  HIP_TRY(nullptr, hipGetDeviceProperties(&prop, device_id));
  if (prop.warpSize != (int)kWave)
    return fail(nullptr, SG_E_INVAL, "device %d has %d-wide wavefronts; this library is built for 64", device_id, prop.warpSize);
  c->max_reqs = cfg && cfg->max_reqs ? cfg->max_reqs : 4096u;
  c->max_frames = cfg && cfg->max_frames ? cfg->max_frames : 65536u;
  if (cfg && cfg->stream) {
    c->stream = static_cast<hipStream_t>(cfg->stream);
  } else {
    HIP_TRY(nullptr, hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking));
    c->own_stream = true;
  }
  HIP_TRY(nullptr, hipMalloc(&c->desc, sizeof(u32x4) * (size_t)c->max_frames));
  HIP_TRY(nullptr, hipMalloc(&c->req_size, sizeof(uint64_t) * (size_t)c->max_reqs));
  HIP_TRY(nullptr, hipMalloc(&c->req_off, sizeof(uint64_t) * (size_t)c->max_reqs));
  HIP_TRY(nullptr, hipMalloc(&c->tile_tot, sizeof(uint64_t) * ((size_t)c->max_reqs / kPartMin + 2)));
  HIP_TRY(nullptr, hipMalloc(&c->cursors, kCtxWords * sizeof(uint64_t)));
  HIP_TRY(nullptr, hipMalloc(&c->status, sizeof(uint32_t)));
  HIP_TRY(nullptr, hipMalloc(&c->csum_scratch, sizeof(uint32_t) * (size_t)c->max_frames * (kPartStride + 1)));
  HIP_TRY(nullptr, hipMemsetAsync(c->csum_scratch, 0, sizeof(uint32_t) * (size_t)c->max_frames * (kPartStride + 1), c->stream));
  {
    // both cursors at 0: cell 0 of the pair is the live one (version 1 against the other cell's 0)
    uint64_t init[kCtxWords] = {0};
    init[kCurStamp] = init[kCurWords + kCurStamp] = 1;
    HIP_TRY(nullptr, hipMemcpy(c->cursors, init, sizeof init, hipMemcpyHostToDevice));
  }
  HIP_TRY(nullptr, hipMemsetAsync(c->status, 0, sizeof(uint32_t), c->stream));
  c->h_runs_cap = 8192;
  HIP_TRY(nullptr, hipHostMalloc(&c->h_runs, sizeof(Run) * c->h_runs_cap, hipHostMallocDefault));
  HIP_TRY(nullptr, hipHostMalloc(&c->h_ptrs, sizeof(uint64_t) * (SG_MAX_BI_SIZE + 8), hipHostMallocDefault));
  HIP_TRY(nullptr, hipHostMalloc(&c->h_status, 2 * sizeof(uint32_t), hipHostMallocDefault));
  c->h_status[0] = c->h_status[1] = 0;
  c->h_flag = c->h_status + 1;
  HIP_TRY(nullptr, hipStreamSynchronize(c->stream));
  // The self-advancing cursor rests on every launch seeing a queue address and a dispatch id of
  // its own.  Two probe launches show whether this runtime hands them out: if their pairs agree,
  // or come back empty, calls on this context keep to the kernel behind the call.
  {
    HIP_TRY(nullptr, hipHostMalloc(&c->h_probe, 4 * sizeof(uint64_t), hipHostMallocDefault));
    volatile uint64_t *probe = c->h_probe;
    probe[0] = probe[1] = probe[2] = probe[3] = 0;
    k_stamp_probe<<<1, kWave, 0, c->stream>>>(c->h_probe);
    k_stamp_probe<<<1, kWave, 0, c->stream>>>(c->h_probe + 2);
    HIP_TRY(nullptr, hipGetLastError());
    HIP_TRY(nullptr, hipStreamSynchronize(c->stream));
    c->sc.stamps_ok = probe[0] != 0 && probe[2] != 0 && !(probe[0] == probe[2] && probe[1] == probe[3]);
  }
  Scratch &sc = c->sc;
  sc.max_reqs = c->max_reqs;
  sc.max_frames = c->max_frames;
  sc.desc = c->desc;
  sc.req_size = c->req_size;
  sc.req_off = c->req_off;
  sc.tile_tot = c->tile_tot;
  sc.cursor[0] = c->cursors + 0;
  sc.cursor[1] = c->cursors + kCurWords;
  sc.cursor_cells = true;
  sc.next_cursor[0] = c->cursors + 2 * kCurWords;
  sc.next_cursor[1] = c->cursors + 2 * kCurWords + 1;
  sc.slot_idx[0] = reinterpret_cast<uint32_t *>(c->cursors + 2 * kCurWords + 2);
  sc.slot_idx[1] = sc.slot_idx[0] + 1;
  sc.desc_tag = reinterpret_cast<uint32_t *>(c->cursors + 2 * kCurWords + 3);
  sc.desc_gen = &c->desc_gen;
  sc.call_seq = &c->call_seq;
  sc.csum_part = c->csum_scratch;
  sc.csum_valid = c->csum_scratch + (size_t)c->max_frames * kPartStride;
  sc.status = c->status;
  sc.flag = c->h_flag;
  return SG_OK;
}

sg_hip_ctx *sg_hip_create(int device_id, const sg_hip_cfg *cfg)
{
  g_create_err[0] = 0;
  if (cfg && cfg->struct_size != sizeof(sg_hip_cfg)) {
    fail(nullptr, SG_E_INVAL, "sg_hip_cfg.struct_size %u != %zu", cfg->struct_size, sizeof(sg_hip_cfg));
    return nullptr;
  }
  sg_hip_ctx *c = new (std::nothrow) sg_hip_ctx();
  if (!c) {
    fail(nullptr, SG_E_NOMEM, "out of host memory");
    return nullptr;
  }
  if (create_impl(c, device_id, cfg) != SG_OK) {
    sg_hip_destroy(c);
    return nullptr;
  }
  return c;
}

void sg_hip_destroy(sg_hip_ctx *c)
{
  if (!c) return;
  DeviceGuard g(c->device);
  if (c->stream) (void)hipStreamSynchronize(c->stream);
  for (EvPair &p : c->ev_used) { (void)hipEventDestroy(p.a); (void)hipEventDestroy(p.b); }
  for (EvPair &p : c->ev_free) { (void)hipEventDestroy(p.a); (void)hipEventDestroy(p.b); }
  (void)hipFree(c->desc);
  (void)hipFree(c->req_size);
  (void)hipFree(c->req_off);
  (void)hipFree(c->tile_tot);
  (void)hipFree(c->cursors);
  (void)hipFree(c->csum_scratch);
  (void)hipFree(c->status);
  if (c->h_runs) (void)hipHostFree(c->h_runs);
  if (c->h_ptrs) (void)hipHostFree(c->h_ptrs);
  if (c->h_status) (void)hipHostFree(c->h_status);
  if (c->h_probe) (void)hipHostFree(c->h_probe);
  if (c->h_counts) (void)hipHostFree(c->h_counts);
  (void)hipFree(c->ra_mem);
  if (c->own_stream && c->stream) (void)hipStreamDestroy(c->stream);
  delete c;
}

int sg_hip_stream_queue(sg_hip_ctx *c, void *stream, uint64_t *queue_out)
{
  if (!c || !queue_out) return fail(c, SG_E_INVAL, "null argument");
  DeviceGuard g(c->device);
  hipStream_t st = stream ? static_cast<hipStream_t>(stream) : c->stream;
  volatile uint64_t *probe = c->h_probe;
  probe[0] = 0;
  k_stamp_probe<<<1, kWave, 0, st>>>(c->h_probe);
  HIP_TRY(c, hipGetLastError());
  HIP_TRY(c, hipStreamSynchronize(st));
  *queue_out = probe[0];
  return SG_OK;
}

int sg_hip_sync(sg_hip_ctx *c)
{
  if (!c) return SG_E_INVAL;
  DeviceGuard g(c->device);
  HIP_TRY(c, hipStreamSynchronize(c->stream));
  int rc = prof_drain(c);
  if (rc != SG_OK) return rc;
  if (*c->h_flag) {
    // the rare path: fetch the bits, then clear both words
    HIP_TRY(c, hipMemcpyAsync(c->h_status, c->status, sizeof(uint32_t), hipMemcpyDeviceToHost, c->stream));
    HIP_TRY(c, hipMemsetAsync(c->status, 0, sizeof(uint32_t), c->stream));
    HIP_TRY(c, hipStreamSynchronize(c->stream));
    *c->h_flag = 0;
    const uint32_t st = c->h_status[0];
    return fail(c, SG_E_DATA, "kernel refused input:%s%s%s%s%s%s%s%s",
                (st & kStBadSlot) ? " slot index beyond ring;" : "",
                (st & kStBadLen) ? " fragment longer than a slot holds;" : "",
                (st & kStBadSize) ? " request larger than its destination;" : "",
                (st & kStBadFrames) ? " frame count disagrees with size/mtu;" : "",
                (st & kStBadTable) ? " CSR table does not tile the items;" : "",
                (st & kStNotRule) ? " a fragment's length departs from the fragmenting rule;" : "",
                (st & kStSlotState) ? " an application slot was not in the state the call expects;" : "",
                (st & kStPoolFull) ? " more requests in flight than the reassembly pool holds;" : "");
  }
  return SG_OK;
}

int sg_hip_set_cursor(sg_hip_ctx *c, int which, uint64_t value)
{
  if (!c || which < 0 || which > 1) return fail(c, SG_E_INVAL, "cursor index %d", which);
  DeviceGuard g(c->device);
  HIP_TRY(c, hipStreamSynchronize(c->stream));
  uint64_t cells[kCurWords] = {0};  // the value in cell 0, one version ahead of cell 1, and in the plain word
  cells[kCurValue] = cells[kCurPlain] = value;
  cells[kCurStamp] = 1;
  HIP_TRY(c, hipMemcpy(c->sc.cursor[which], cells, sizeof cells, hipMemcpyHostToDevice));
  return SG_OK;
}

int sg_hip_get_cursor(sg_hip_ctx *c, int which, uint64_t *value)
{
  if (!c || !value || which < 0 || which > 1) return fail(c, SG_E_INVAL, "cursor index %d", which);
  DeviceGuard g(c->device);
  HIP_TRY(c, hipStreamSynchronize(c->stream));
  // between kernels the plain word and the live cell agree
  HIP_TRY(c, hipMemcpy(value, c->sc.cursor[which] + kCurPlain, sizeof *value, hipMemcpyDeviceToHost));
  return SG_OK;
}

int sg_hip_set_slot_index(sg_hip_ctx *c, int which, uint32_t value)
{
  if (!c || which < 0 || which > 1) return fail(c, SG_E_INVAL, "slot index %d", which);
  DeviceGuard g(c->device);
  HIP_TRY(c, hipStreamSynchronize(c->stream));
  HIP_TRY(c, hipMemcpy(c->sc.slot_idx[which], &value, sizeof value, hipMemcpyHostToDevice));
  return SG_OK;
}

int sg_hip_get_slot_index(sg_hip_ctx *c, int which, uint32_t *value)
{
  if (!c || !value || which < 0 || which > 1) return fail(c, SG_E_INVAL, "slot index %d", which);
  DeviceGuard g(c->device);
  HIP_TRY(c, hipStreamSynchronize(c->stream));
  HIP_TRY(c, hipMemcpy(value, c->sc.slot_idx[which], sizeof *value, hipMemcpyDeviceToHost));
  return SG_OK;
}

int sg_hip_set_profiling(sg_hip_ctx *c, int on)
{
  if (!c) return SG_E_INVAL;
  int rc = sg_hip_sync(c);
  c->profiling = on != 0;
  for (int i = 0; i < 6; i++) { c->prof_ms[i] = 0; c->prof_n[i] = 0; }
  return rc;
}

int sg_hip_kernel_time(sg_hip_ctx *c, int which, double *total_ms, uint64_t *launches)
{
  if (!c || which < 0 || which > 5) return fail(c, SG_E_INVAL, "kernel index %d", which);
  int rc = sg_hip_sync(c);
  if (total_ms) *total_ms = c->prof_ms[which];
  if (launches) *launches = c->prof_n[which];
  return rc;
}

// ---- per-request ------------------------------------------------------------

// Runs longer than this are cut so that no single wavefront walks megabytes.
static const uint64_t kRunChunk = 16384;

static int copy_skb(sg_hip_ctx *c, const sg_sk_buf *skb)
{
  if (!c || !skb) return fail(c, SG_E_INVAL, "null argument");
  if (skb->num_items > SG_MAX_BI_SIZE - 1)
    return fail(c, SG_E_INVAL, "run table holds %llu runs; len[] has room for %d",
                (unsigned long long)skb->num_items, SG_MAX_BI_SIZE - 1);
  DeviceGuard g(c->device);
  // the pinned staging buffer is reused: the previous launch must have read it
  HIP_TRY(c, hipStreamSynchronize(c->stream));
  uint32_t n = 0;
  for (uint64_t i = 0; i < skb->num_items; i++) {
    uint64_t src = skb->i_buf[i], dst = skb->o_buf[i], len = skb->len[i];
    if (len && (!src || !dst)) return fail(c, SG_E_INVAL, "run %llu has a null address", (unsigned long long)i);
    while (len) {
      uint64_t piece = len;
      if (piece > kRunChunk) {
        // cut where the destination is 16-byte aligned so later pieces need no head bytes
        piece = kRunChunk - (dst & 15u);
      }
      if (n == c->h_runs_cap) {
        // flush what is staged and start over
        int rc = prof_begin(c, 3);
        if (rc != SG_OK) return rc;
        k_copy_runs<<<(n + kWavesPerBlock - 1) / kWavesPerBlock, kBlock, 0, c->stream>>>(c->h_runs, n);
        rc = prof_end(c);
        if (rc != SG_OK) return rc;
        HIP_TRY(c, hipStreamSynchronize(c->stream));
        n = 0;
      }
      c->h_runs[n++] = Run{src, dst, piece};
      src += piece; dst += piece; len -= piece;
    }
  }
  if (n) {
    int rc = prof_begin(c, 3);
    if (rc != SG_OK) return rc;
    k_copy_runs<<<(n + kWavesPerBlock - 1) / kWavesPerBlock, kBlock, 0, c->stream>>>(c->h_runs, n);
    rc = prof_end(c);
    if (rc != SG_OK) return rc;
  }
  return finish(c, 0);
}

int sg_hip_gather(sg_hip_ctx *c, const sg_sk_buf *skb) { return copy_skb(c, skb); }
int sg_hip_scatter(sg_hip_ctx *c, const sg_sk_buf *skb) { return copy_skb(c, skb); }

static int fill_hdrs(sg_hip_ctx *c, const sg_hbufs *hdrs, const uint8_t *tmpl, uint64_t token,
                     uint32_t profile, uint64_t payload_size, uint32_t mtu, uint32_t flags)
{
  if (!c || !hdrs) return fail(c, SG_E_INVAL, "null argument");
  if (profile > SG_HDR_REF64) return fail(c, SG_E_INVAL, "unknown header profile %u", profile);
  if (hdrs->num_items > SG_MAX_BI_SIZE) return fail(c, SG_E_INVAL, "header table holds %u entries", hdrs->num_items);
  if (mtu == 0) return fail(c, SG_E_INVAL, "mtu is zero");
  if (flags & SG_F_UDP_CSUM_FULL) return fail(c, SG_E_INVAL, "a header-only rewrite cannot finish the UDP checksum");
  const uint32_t n = hdrs->num_items;
  if (n == 0) return SG_OK;
  DeviceGuard g(c->device);
  HIP_TRY(c, hipStreamSynchronize(c->stream));
  for (uint32_t i = 0; i < n; i++) {
    if (!hdrs->burst_items[i]) return fail(c, SG_E_INVAL, "header %u is null", i);
    c->h_ptrs[i] = hdrs->burst_items[i];
  }
  // the template rides behind the pointer table in the same pinned block
  const uint8_t *d_tmpl = nullptr;
  if (tmpl) {
    memcpy(c->h_ptrs + SG_MAX_BI_SIZE, tmpl, 64);
    d_tmpl = reinterpret_cast<const uint8_t *>(c->h_ptrs + SG_MAX_BI_SIZE);
  }
  int rc = prof_begin(c, 4);
  if (rc != SG_OK) return rc;
  k_swap_hdrs<<<(n + kWavesPerBlock - 1) / kWavesPerBlock, kBlock, 0, c->stream>>>(
      c->h_ptrs, n, hdr_len_of(profile), profile == SG_HDR_REF64, flags & 0xfu, payload_size, mtu,
      d_tmpl, token);
  rc = prof_end(c);
  if (rc != SG_OK) return rc;
  return finish(c, 0);
}

int sg_hip_swap_hdrs(sg_hip_ctx *c, const sg_hbufs *hdrs, uint32_t profile, uint64_t payload_size,
                     uint32_t mtu, uint32_t flags)
{
  return fill_hdrs(c, hdrs, nullptr, 0, profile, payload_size, mtu, flags);
}

int sg_hip_set_hdrs(sg_hip_ctx *c, const sg_hbufs *hdrs, const uint8_t *hdr_template, uint64_t req_token,
                    uint32_t profile, uint64_t payload_size, uint32_t mtu, uint32_t flags)
{
  if (!hdr_template) return fail(c, SG_E_INVAL, "null header template");
  return fill_hdrs(c, hdrs, hdr_template, req_token, profile, payload_size, mtu, flags);
}

// ---- batched ------------------------------------------------------------------

// The gather call proper.  `c` may be null (allocation-free entry point): then
// errors go to the creation-error text, nothing is profiled and nothing waits.
// `half` (sg_hip_shunt_batch): nothing is launched; a call that can share a launch with the other
// direction leaves its kernel arguments there and returns SG_OK, any other returns kNoShare.
// `zero_words` (allocation-free entry point): two status words to clear ahead of the first kernel,
// once the host has found nothing to refuse.
static int gather_impl(sg_hip_ctx *c, const Scratch &sc, hipStream_t st, const sg_gather_args *a,
                       ShuntHalf *half = nullptr, uint32_t *zero_words = nullptr)
{
  int rc = check_ring(c, a->ring, "rx");
  if (rc != SG_OK) return rc;
  if (a->n_req == 0) return half ? kNoShare : SG_OK;
  if (a->n_req > sc.max_reqs) return fail(c, SG_E_INVAL, "n_req %u > max_reqs %u", a->n_req, sc.max_reqs);
  if (a->n_frags > sc.max_frames) return fail(c, SG_E_INVAL, "n_frags %u > max_frames %u", a->n_frags, sc.max_frames);
  if ((!a->frag_slot && a->n_frags) || !a->req_first) return fail(c, SG_E_INVAL, "null fragment tables");
  if (!a->frag_len && a->n_frags && a->ring.hdr_profile != SG_HDR_BL58)
    return fail(c, SG_E_INVAL, "REF64 headers carry no payload length: frag_len is required");
  AppDev app;
  uint64_t max_req_bytes;
  rc = check_app(c, a->app, &app, &max_req_bytes);
  if (rc != SG_OK) return rc;
  const bool packed = app.n_tensors == 0;
  if (a->slot_state && a->n_slot_states == 0) return fail(c, SG_E_INVAL, "a slot ring of no slots");
  if (a->slot_state && a->n_req > a->n_slot_states)
    return fail(c, SG_E_INVAL, "%u requests do not fit a ring of %u application slots", a->n_req, a->n_slot_states);
  // a batch larger than the arena would lap itself and its wavefronts would race for the same bytes
  if (packed && a->fixed_req_size && (uint64_t)a->n_req * a->fixed_req_size > app.cap)
    return fail(c, SG_E_INVAL, "%u requests of %llu bytes do not fit an arena of %llu bytes", a->n_req,
                (unsigned long long)a->fixed_req_size, (unsigned long long)app.cap);

  const uint32_t hl0 = hdr_len_of(a->ring.hdr_profile);
  if (a->flags & SG_F_RULE_FRAGS) {
    // one size, cut by the rule: no descriptor pass, the copy kernel derives everything
    if (!a->fixed_req_size || !a->mtu) return fail(c, SG_E_INVAL, "SG_F_RULE_FRAGS needs fixed_req_size and mtu");
    if ((uint64_t)a->mtu + hl0 > a->ring.slot_size) return fail(c, SG_E_INVAL, "mtu %u + %u header bytes does not fit a %u-byte slot", a->mtu, hl0, a->ring.slot_size);
    const uint64_t per = (a->fixed_req_size + a->mtu - 1) / a->mtu;
    // with the counts on the device n_req and n_frags are bounds: the launch covers per * n_req fragments
    if (a->counts ? per * a->n_req > sc.max_frames : per * a->n_req != a->n_frags)
      return fail(c, SG_E_INVAL, "%u requests of %llu bytes at mtu %u are %llu fragments, not %u", a->n_req, (unsigned long long)a->fixed_req_size, a->mtu, (unsigned long long)(per * a->n_req), a->n_frags);
    const uint32_t n_items = (uint32_t)(per * a->n_req);
    if (n_items >= (1u << 27)) return fail(c, SG_E_INVAL, "%u fragments in one call: the limit is 2^27 - 1", n_items);
    if (a->fixed_req_size > 0xffffffffull || (packed ? a->fixed_req_size > app.cap : a->fixed_req_size > max_req_bytes))
      return fail(c, SG_E_INVAL, "request size %llu does not fit its destination", (unsigned long long)a->fixed_req_size);
    GatherRuleArgs ga;
    memset(&ga, 0, sizeof ga);
    ga.ring = static_cast<const uint8_t *>(a->ring.base);
    ga.frag_slot = a->frag_slot;
    ga.dst = packed ? app.arena : app.tensor_base[0];
    ga.cursor = sc.cursor[0];
    ga.size = a->fixed_req_size;
    ga.cap = packed ? app.cap : 0;
    ga.n_items = n_items;
    ga.counts = a->counts;
    ga.per_req = (uint32_t)per;
    magic_div(per, &ga.div_mul, &ga.div_shift);
    // short fragments go several to a wavefront: all of them where a full fragment is short, else
    // the remainder fragment that ends every request
    const uint64_t full_frag = a->fixed_req_size < a->mtu ? a->fixed_req_size : a->mtu;
    const uint64_t last_frag = a->fixed_req_size - (per - 1) * a->mtu;
    uint32_t small_all = 0, small_last = 0;
    if (!(a->flags & SG_F_NO_SMALL)) {
      small_all = small_lanes(full_frag);
      // (a short last fragment rides in k_gather_rule, which has no groups of 8)
      if (!small_all && last_frag < a->mtu && small_last_pays(per, a->n_req, a->flags, false)) small_last = small_lanes(last_frag, false);
    }
    ga.per_launch = small_last ? (uint32_t)per - 1 : (uint32_t)per;
    magic_div(ga.per_launch, &ga.lmul, &ga.lshift);
    ga.mtu = a->mtu;
    ga.slot_size = a->ring.slot_size;
    ga.hl = hl0;
    ga.n_slots = a->ring.n_slots;
    ga.n_req = a->n_req;
    ga.frag_len = a->frag_len;
    ga.first = a->req_first;
    ga.offsets_out = packed ? a->offsets_out : nullptr;
    ga.status = sc.status;
    ga.status_flag = sc.flag;
    ga.app = app;
    ga.pieces = pieces_for(a->mtu);
    if (app.n_tensors > 1) ga.n_plan = fill_plan(app, a->fixed_req_size, a->mtu, per, ga.plan);
    uint32_t grid, remap;
    uint64_t waves = (uint64_t)a->n_req * ga.per_launch * ga.pieces;
    if (small_last) {
      // turns of `period` wavefronts: the full fragments of 64 / small_last requests, then their remainders
      const uint32_t per_turn = kWave / small_last;
      ga.period = ga.per_launch * ga.pieces * per_turn + 1;
      magic_div(ga.period, &ga.pmul, &ga.pshift);
      waves = (uint64_t)((a->n_req + per_turn - 1) / per_turn) * ga.period;
      if (waves >= (1u << 27)) return fail(c, SG_E_INVAL, "%llu wavefronts in one call: the limit is 2^27 - 1", (unsigned long long)waves);
    }
    geometry(waves, !(a->flags & SG_F_NO_XCD_REMAP), &grid, &remap);
    const bool self_advance = self_advancing(sc, packed, a->slot_state, waves, a->flags);
    ga.cursor = const_cast<uint64_t *>(plain_cursor(sc, 0));
    ga.opts = (remap ? kOptRemap : 0u) | (app.mirrored ? kOptMirrored : 0u) |
              (app.n_tensors > 1 ? kOptMultiTensor : 0u) | (small_last ? kOptSmallLast : 0u) |
              ((((uintptr_t)a->ring.base | a->ring.slot_size) & 15u) ? 0u : kOptHdrChunk);
    if (half) {
      // one wavefront per fragment (short last fragments may ride along), the cursor advanced by the
      // kernel itself: the shapes k_shunt carries
      if (!self_advance || small_all || ga.pieces != 1) return kNoShare;
      ga.call_seq = ++*sc.call_seq;
      half->g = ga;
      half->g_grid = grid;
      half->g_small = small_last;
      return SG_OK;
    }
    if (self_advance) ga.call_seq = ++*sc.call_seq;
    if (zero_words) k_zero_words<<<1, kBlock, 0, st>>>(zero_words, 2);
    rc = prof_begin(c, 1);
    if (rc != SG_OK) return rc;
    if (self_advance) launch_gather_rule<true>(st, ga, grid, small_all, small_last, n_items);
    else launch_gather_rule<false>(st, ga, grid, small_all, small_last, n_items);
    rc = prof_end(c);
    if (rc != SG_OK) return rc;
    launch_finish(sc, st, packed && !self_advance ? sc.cursor[0] : nullptr, a->fixed_req_size, app.cap, a->n_req,
                  a->counts, a->slot_state, a->n_slot_states, 0, false);
    return finish(c, a->flags);
  }

  if (half) return kNoShare;  // a descriptor pass: kernels of its own
  PrepArgs p;
  memset(&p, 0, sizeof p);
  p.mode = 0;
  p.n_req = a->n_req;
  p.arena_base = (uint64_t)(uintptr_t)app.arena;
  p.ring = static_cast<const uint8_t *>(a->ring.base);
  p.n_slots = a->ring.n_slots;
  p.slot_size = a->ring.slot_size;
  p.hl = hdr_len_of(a->ring.hdr_profile);
  p.item_slot = a->frag_slot;
  p.item_len = a->frag_len;
  p.first = a->req_first;
  p.n_items = a->n_frags;
  p.packed = packed;
  p.cap = app.cap;
  p.max_req_bytes = max_req_bytes;
  p.desc = sc.desc;
  p.req_size = sc.req_size;
  p.req_off = sc.req_off;
  p.fixed_size = a->fixed_req_size;
  p.fixed_offsets = p.packed && a->fixed_req_size != 0;
  p.cursor = plain_cursor(sc, 0);
  p.next_cursor = sc.next_cursor[0];
  p.offsets_out = packed ? a->offsets_out : nullptr;
  p.counts = a->counts;
  if (sc.desc_gen) {
    p.desc_tag = sc.desc_tag;
    p.gen = ++*sc.desc_gen ? *sc.desc_gen : ++*sc.desc_gen;  // never zero
  }
  p.status = sc.status;
  p.status_flag = sc.flag;
  if (zero_words) k_zero_words<<<1, kBlock, 0, st>>>(zero_words, 2);
  rc = launch_prep(c, sc, st, p);
  if (rc != SG_OK) return rc;

  // the copy kernel also commits the advanced cursor, so a batch of empty requests still launches it
  if (a->n_frags || packed) {
    GatherArgs ga;
    memset(&ga, 0, sizeof ga);
    ga.desc = sc.desc;
    ga.req_off = sc.req_off;
    ga.ring = p.ring;
    ga.slot_size = p.slot_size;
    ga.hl = p.hl;
    ga.n_items = a->n_frags;
    ga.status = sc.status;
    ga.status_flag = sc.flag;
    if (packed) {
      ga.cursor = sc.cursor[0];
      ga.next_cursor = sc.next_cursor[0];
      ga.cursor_cells = sc.cursor_cells ? 1u : 0u;
    }
    ga.counts = a->counts;
    ga.app = app;
    ga.pieces = pieces_for(p.slot_size - p.hl);
    uint32_t grid;
    geometry((uint64_t)(a->n_frags ? a->n_frags : 1u) * ga.pieces, !(a->flags & SG_F_NO_XCD_REMAP), &grid, &ga.remap);
    rc = prof_begin(c, 1);
    if (rc != SG_OK) return rc;
    if (ga.pieces > 1) k_gather<true><<<grid, kBlock, 0, st>>>(ga);
    else k_gather<false><<<grid, kBlock, 0, st>>>(ga);
    rc = prof_end(c);
    if (rc != SG_OK) return rc;
  }
  launch_finish(sc, st, nullptr, 0, 0, a->n_req, a->counts, a->slot_state, a->n_slot_states, 0, true);
  return finish(c, a->flags);
}

int sg_hip_gather_batch(sg_hip_ctx *c, const sg_gather_args *a)
{
  if (!c || !a) return fail(c, SG_E_INVAL, "null argument");
  DeviceGuard g(c->device);
  return gather_impl(c, c->sc, c->stream, a);
}

static int scatter_impl(sg_hip_ctx *c, const Scratch &sc, hipStream_t st, const sg_scatter_args *a,
                        ShuntHalf *half = nullptr)
{
  int rc = check_ring(c, a->rx, "rx");
  if (rc != SG_OK) return rc;
  rc = check_ring(c, a->tx, "tx");
  if (rc != SG_OK) return rc;
  if (a->rx.hdr_profile != a->tx.hdr_profile) return fail(c, SG_E_INVAL, "rx and tx rings differ in header profile");
  if (a->n_req == 0) return half ? kNoShare : SG_OK;
  if (a->n_req > sc.max_reqs) return fail(c, SG_E_INVAL, "n_req %u > max_reqs %u", a->n_req, sc.max_reqs);
  if (a->n_frames > sc.max_frames) return fail(c, SG_E_INVAL, "n_frames %u > max_frames %u", a->n_frames, sc.max_frames);
  if (!a->resp_first || (a->n_frames && (!a->tx_slot || (!a->hdr_src_slot && !a->hdr_src_req && !a->hdr_templates))))
    return fail(c, SG_E_INVAL, "null frame tables");
  if ((uintptr_t)a->hdr_templates & 1u) return fail(c, SG_E_INVAL, "hdr_templates must start at an even address");
  const uint32_t hl = hdr_len_of(a->tx.hdr_profile);
  if (a->mtu == 0 || (uint64_t)a->mtu + hl > a->tx.slot_size)
    return fail(c, SG_E_INVAL, "mtu %u + %u header bytes does not fit a %u-byte slot", a->mtu, hl, a->tx.slot_size);
  if ((uint64_t)a->mtu + (hl - 42u) + 28u > 0xffffu) return fail(c, SG_E_INVAL, "mtu %u overflows the IPv4 length field", a->mtu);
  AppDev app;
  uint64_t max_req_bytes;
  rc = check_app(c, a->app, &app, &max_req_bytes);
  if (rc != SG_OK) return rc;
  const bool packed = app.n_tensors == 0;
  if (a->slot_state && a->n_slot_states == 0) return fail(c, SG_E_INVAL, "a slot ring of no slots");
  if (a->slot_state && a->n_req > a->n_slot_states)
    return fail(c, SG_E_INVAL, "%u responses do not fit a ring of %u application slots", a->n_req, a->n_slot_states);

  const bool reuse = (a->flags & SG_F_REUSE_DESC) != 0;
  if (reuse && (!packed || !sc.desc_gen || !*sc.desc_gen))
    return fail(c, SG_E_INVAL, "SG_F_REUSE_DESC needs a packed arena and a descriptor pass of an earlier call on this context");
  const bool fused = a->resp_size == nullptr && !(a->flags & (SG_F_NO_FUSE | SG_F_REUSE_DESC));
  if (fused) {
    if (a->fixed_resp_size == 0 || a->fixed_resp_size > 0xffffffffull)
      return fail(c, SG_E_INVAL, "fixed response size %llu out of range", (unsigned long long)a->fixed_resp_size);
    const uint64_t per = (a->fixed_resp_size + a->mtu - 1) / a->mtu;
    if (a->counts ? per * a->n_req > a->n_frames : per * a->n_req != a->n_frames)
      return fail(c, SG_E_INVAL, "%u responses of %llu bytes at mtu %u are %llu frames, not %u", a->n_req, (unsigned long long)a->fixed_resp_size, a->mtu, (unsigned long long)(per * a->n_req), a->n_frames);
    const uint32_t n_items = (uint32_t)(per * a->n_req);
    if (app.n_tensors == 0 ? a->fixed_resp_size > app.cap : a->fixed_resp_size > max_req_bytes)
      return fail(c, SG_E_INVAL, "response size %llu does not fit its source", (unsigned long long)a->fixed_resp_size);
    ScatterArgs sa;
    memset(&sa, 0, sizeof sa);
    sa.hdr_src_slot = a->hdr_src_slot;
    sa.hdr_templates = a->hdr_templates;
    sa.req_token = a->req_token;
    sa.rx = static_cast<const uint8_t *>(a->rx.base);
    sa.rx_slot_size = a->rx.slot_size;
    sa.rx_n_slots = a->rx.n_slots;
    sa.tx = static_cast<uint8_t *>(a->tx.base);
    sa.tx_slot_size = a->tx.slot_size;
    sa.hl = hl;
    sa.ref64 = a->tx.hdr_profile == SG_HDR_REF64;
    sa.flags = a->flags & 0xfu;
    sa.n_items = n_items;
    sa.n_req = a->n_req;
    sa.counts = a->counts;
    sa.hdr_src_req = a->hdr_templates ? nullptr : a->hdr_src_req;
    sa.status = sc.status;
    sa.status_flag = sc.flag;
    sa.app = app;
    sa.rule.item_slot = a->tx_slot;
    sa.rule.first = a->resp_first;
    sa.rule.size = a->fixed_resp_size;
    sa.rule.mtu = a->mtu;
    sa.rule.per_req = (uint32_t)per;
    sa.rule.per_launch = (uint32_t)per;
    magic_div(per, &sa.rule.div_mul, &sa.rule.div_shift);
    if (n_items >= (1u << 27)) return fail(c, SG_E_INVAL, "%u frames in one call: the limit is 2^27 - 1", n_items);
    sa.rule.n_req = a->n_req;
    sa.rule.n_slots = a->tx.n_slots;
    sa.rule.single_wrap = app.n_tensors == 0 && (uint64_t)a->n_req * a->fixed_resp_size <= app.cap;
    sa.rule.offsets_out = packed ? a->offsets_out : nullptr;
    if (app.n_tensors > 0) sa.n_plan = fill_plan(app, a->fixed_resp_size, a->mtu, per, sa.plan);
    sa.pieces = pieces_for(a->mtu);
    uint32_t grid;
    // short frames go several to a wavefront: all of them where a full frame is short, else the
    // remainder frame that ends every response
    const bool full_csum = (a->flags & SG_F_UDP_CSUM_FULL) != 0;
    const uint64_t full_frame = a->fixed_resp_size < a->mtu ? a->fixed_resp_size : a->mtu;
    const uint64_t last_frame = a->fixed_resp_size - (per - 1) * a->mtu;
    uint32_t small_all = 0, small_last = 0;
    if (!(a->flags & SG_F_NO_SMALL)) {
      small_all = small_lanes(full_frame);
      if (!small_all && last_frame < a->mtu && small_last_pays(per, a->n_req, a->flags, true)) small_last = small_lanes(last_frame);
    }
    // the call's last kernel that reads the cursor advances it where the call is self-advancing;
    // a kernel before that one has no writer beside it and reads the plain word
    const bool self_advance = self_advancing(sc, packed, a->slot_state, (uint64_t)n_items * sa.pieces, a->flags);
    sa.rule.cursor = const_cast<uint64_t *>(plain_cursor(sc, 1));
    if (half) {
      // one kernel that advances the cursor itself: a wavefront per frame, or eight short frames to a wavefront
      const bool own_small_launch = !small_all && small_last;
      if (!self_advance || own_small_launch || sa.pieces != 1 || (small_all && (small_all != 8 || full_csum)))
        return kNoShare;
      sa.rule.call_seq = ++*sc.call_seq;
      magic_div(sa.rule.per_launch, &sa.rule.lmul, &sa.rule.lshift);
      if (small_all) grid = (n_items + 8 * kWavesPerBlock - 1) / (8 * kWavesPerBlock);
      else geometry((uint64_t)n_items, !(a->flags & SG_F_NO_XCD_REMAP), &grid, &sa.remap);
      half->s = sa;
      half->s_grid = grid;
      half->s_small = small_all;
      half->full_csum = full_csum;
      return SG_OK;
    }
    if (self_advance) sa.rule.call_seq = ++*sc.call_seq;
    rc = prof_begin(c, 2);
    if (rc != SG_OK) return rc;
    if (small_all) {
      launch_scatter_small(st, sa, small_all, n_items, full_csum, self_advance);
    } else {
      if (small_last) sa.rule.per_launch = (uint32_t)per - 1;
      magic_div(sa.rule.per_launch, &sa.rule.lmul, &sa.rule.lshift);
      const bool defer = csum_in_two_phases(sc, sa.pieces, full_csum);
      sa.csum_part = sc.csum_part;
      sa.csum_valid = sc.csum_valid;
      geometry((uint64_t)a->n_req * sa.rule.per_launch * ((full_csum && !defer) ? 1u : sa.pieces),
               !(a->flags & SG_F_NO_XCD_REMAP), &grid, &sa.remap);
      // (the remainder frames' kernel on a second stream beside this one, forked and joined with
      // events, was measured as well: both kinds of wavefront at once cost the full frames more
      // than the overlap gains, 180 against 172 us on 131072 responses of 1400 + 1400 + 272 bytes)
      if (small_last) {
        launch_scatter<true>(st, sa, grid, full_csum, defer);
        launch_scatter_small(st, sa, small_last, a->n_req, full_csum, self_advance);
      } else if (self_advance) {
        launch_scatter<true, true>(st, sa, grid, full_csum, defer);
      } else {
        launch_scatter<true>(st, sa, grid, full_csum, defer);
      }
    }
    rc = prof_end(c);
    if (rc != SG_OK) return rc;
    launch_finish(sc, st, packed && !self_advance ? sc.cursor[1] : nullptr, a->fixed_resp_size, app.cap, a->n_req,
                  a->counts, a->slot_state, a->n_slot_states, 1, false);
    return finish(c, a->flags);
  }

  if (half) return kNoShare;  // a descriptor pass: kernels of its own
  PrepArgs p;
  memset(&p, 0, sizeof p);
  p.mode = 1;
  p.n_req = a->n_req;
  p.arena_base = (uint64_t)(uintptr_t)app.arena;
  p.n_slots = a->tx.n_slots;
  p.slot_size = a->tx.slot_size;
  p.hl = hl;
  p.mtu = a->mtu;
  p.item_slot = a->tx_slot;
  p.first = a->resp_first;
  p.sizes = a->resp_size;
  p.fixed_size = a->fixed_resp_size;
  p.n_items = a->n_frames;
  p.packed = app.n_tensors == 0;
  p.cap = app.cap;
  p.max_req_bytes = max_req_bytes;
  p.desc = sc.desc;
  p.req_size = sc.req_size;
  p.req_off = sc.req_off;
  p.fixed_offsets = p.packed && a->resp_size == nullptr;
  p.cursor = plain_cursor(sc, 1);
  p.next_cursor = sc.next_cursor[1];
  p.offsets_out = packed ? a->offsets_out : nullptr;
  if (!a->hdr_templates) {
    if (a->hdr_src_req) p.hdr_src_req = a->hdr_src_req;
    else p.hdr_src_slot = a->hdr_src_slot;
    p.rx_n_slots = a->rx.n_slots;
  }
  p.counts = a->counts;
  if (sc.desc_gen && !reuse) {
    p.desc_tag = sc.desc_tag;
    p.gen = ++*sc.desc_gen ? *sc.desc_gen : ++*sc.desc_gen;
  }
  p.status = sc.status;
  p.status_flag = sc.flag;
  if (!reuse) {
    rc = launch_prep(c, sc, st, p);
    if (rc != SG_OK) return rc;
  }

  if (a->n_frames || packed) {
    ScatterArgs sa;
    memset(&sa, 0, sizeof sa);
    sa.desc = sc.desc;
    sa.req_off = sc.req_off;
    sa.first = a->resp_first;
    sa.hdr_src_slot = a->hdr_src_slot;
    sa.hdr_templates = a->hdr_templates;
    sa.req_token = a->req_token;
    sa.rx = static_cast<const uint8_t *>(a->rx.base);
    sa.rx_slot_size = a->rx.slot_size;
    sa.rx_n_slots = a->rx.n_slots;
    sa.tx = static_cast<uint8_t *>(a->tx.base);
    sa.tx_slot_size = a->tx.slot_size;
    sa.hl = hl;
    sa.ref64 = a->tx.hdr_profile == SG_HDR_REF64;
    sa.flags = a->flags & 0xfu;
    sa.n_items = a->n_frames;
    sa.n_req = a->n_req;
    sa.counts = a->counts;
    sa.hdr_src_req = a->hdr_templates ? nullptr : a->hdr_src_req;
    sa.status = sc.status;
    sa.status_flag = sc.flag;
    if (packed) {
      sa.cursor = sc.cursor[1];
      sa.next_cursor = sc.next_cursor[1];
      sa.cursor_cells = sc.cursor_cells ? 1u : 0u;
    }
    if (reuse) {
      // the response cursor ends up where the reused descriptors end
      sa.next_cursor = sc.next_cursor[0];
      sa.desc_tag = sc.desc_tag;
      sa.reuse_gen = *sc.desc_gen;
      sa.tx_n_slots = a->tx.n_slots;
      sa.offsets_out = a->offsets_out;
    }
    sa.app = app;
    sa.rule.mtu = a->mtu;  // reused descriptors are held against it
    sa.pieces = pieces_for(a->mtu);
    uint32_t grid;
    const bool full_csum = (a->flags & SG_F_UDP_CSUM_FULL) != 0;
    const bool defer = csum_in_two_phases(sc, sa.pieces, full_csum);
    sa.csum_part = sc.csum_part;
    sa.csum_valid = sc.csum_valid;
    geometry((uint64_t)(a->n_frames ? a->n_frames : 1u) * ((full_csum && !defer) ? 1u : sa.pieces),
             !(a->flags & SG_F_NO_XCD_REMAP), &grid, &sa.remap);
    rc = prof_begin(c, 2);
    if (rc != SG_OK) return rc;
    launch_scatter<false>(st, sa, grid, full_csum, defer);
    rc = prof_end(c);
    if (rc != SG_OK) return rc;
  }
  launch_finish(sc, st, nullptr, 0, 0, a->n_req, a->counts, a->slot_state, a->n_slot_states, 1, true);
  return finish(c, a->flags);
}

int sg_hip_scatter_batch(sg_hip_ctx *c, const sg_scatter_args *a)
{
  if (!c || !a) return fail(c, SG_E_INVAL, "null argument");
  DeviceGuard g(c->device);
  return scatter_impl(c, c->sc, c->stream, a);
}

// ---- both directions in one launch ---------------------------------------------

static bool ranges_overlap(const void *a, uint64_t an, const void *b, uint64_t bn)
{
  const uintptr_t a0 = (uintptr_t)a, b0 = (uintptr_t)b;
  return a0 < b0 + bn && b0 < a0 + an;
}

int sg_hip_shunt_batch(sg_hip_ctx *c, const sg_gather_args *g, const sg_scatter_args *s)
{
  if (!c || !g || !s) return fail(c, SG_E_INVAL, "null argument");
  DeviceGuard guard(c->device);
  const uint32_t async = g->flags & s->flags & SG_F_ASYNC;
  // What the gather writes (requests) against everything the scatter touches (responses, the ring
  // its headers come from, TX slots), and what the scatter writes (TX slots) against what the gather
  // reads (RX slots): halves that touch each other's memory run one after the other.  Application
  // memory is an arena or, tensor-major, n_req rows per tensor.
  struct Range { const void *p; uint64_t n; };
  auto app_ranges = [](const sg_app_desc &app, uint32_t n_req, Range *out) {
    uint32_t k = 0;
    if (app.n_tensors == 0) out[k++] = Range{app.arena, app.arena_cap * (app.arena_mirrored ? 2u : 1u)};
    else
      for (uint32_t t = 0; t < app.n_tensors && t < SG_MAX_TENSORS; t++)
        out[k++] = Range{app.tensor_base[t], app.tensor_size[t] * n_req};
    return k;
  };
  Range gw[SG_MAX_TENSORS + 1], st[SG_MAX_TENSORS + 3];
  const uint32_t n_gw = app_ranges(g->app, g->n_req, gw);
  uint32_t n_st = app_ranges(s->app, s->n_req, st);
  const Range s_tx{s->tx.base, (uint64_t)s->tx.n_slots * s->tx.slot_size};
  st[n_st++] = s_tx;
  st[n_st++] = Range{s->rx.base, (uint64_t)s->rx.n_slots * s->rx.slot_size};
  bool apart = !ranges_overlap(s_tx.p, s_tx.n, g->ring.base, (uint64_t)g->ring.n_slots * g->ring.slot_size);
  for (uint32_t i = 0; i < n_gw; i++)
    for (uint32_t j = 0; j < n_st; j++) apart = apart && !ranges_overlap(gw[i].p, gw[i].n, st[j].p, st[j].n);
  // Both halves are looked at before either is launched: a call the host refuses launches nothing.
  // A half that cannot share a launch leaves no trace; both are then made as calls of their own.
  ShuntHalf h;
  const uint32_t seq0 = c->call_seq;
  const int rg = gather_impl(c, c->sc, c->stream, g, &h);
  if (rg < 0) return rg;
  const int rs = scatter_impl(c, c->sc, c->stream, s, &h);
  if (rs < 0) return rs;
  // a shared launch pays while the chip holds the whole call at once (one resnet50-sized batch 8.9 ->
  // 7.8 us per step, two batches 10.9 -> 11.5 us)
  constexpr uint32_t kAtOnce = 2048;  // workgroups of 256 threads resident on 256 CUs
  if (apart && rg == SG_OK && rs == SG_OK && h.g_grid + h.s_grid <= kAtOnce) {
    ShuntArgs sh;
    sh.g = h.g;
    sh.s = h.s;
    sh.s_blocks = h.s_grid;
    const uint32_t total = h.g_grid + h.s_grid;
    int rc = prof_begin(c, 1);
    if (rc != SG_OK) return rc;
    const hipStream_t st = c->stream;
#define SG_SHUNT(G, S, C) k_shunt<G, S, C><<<total, kBlock, 0, st>>>(sh)
    if (h.s_small) {
      if (h.g_small == 16) SG_SHUNT(16, 8, false);
      else if (h.g_small == 32) SG_SHUNT(32, 8, false);
      else SG_SHUNT(0, 8, false);
    } else if (h.full_csum) {
      if (h.g_small == 16) SG_SHUNT(16, 0, true);
      else if (h.g_small == 32) SG_SHUNT(32, 0, true);
      else SG_SHUNT(0, 0, true);
    } else {
      if (h.g_small == 16) SG_SHUNT(16, 0, false);
      else if (h.g_small == 32) SG_SHUNT(32, 0, false);
      else SG_SHUNT(0, 0, false);
    }
#undef SG_SHUNT
    rc = prof_end(c);
    if (rc != SG_OK) return rc;
    return finish(c, async);
  }
  c->call_seq = seq0;
  int rc = gather_impl(c, c->sc, c->stream, g);
  if (rc != SG_OK) return rc;
  return scatter_impl(c, c->sc, c->stream, s);
}

// ---- fragment tables pulled from where the receive thread keeps them -----------

int sg_hip_pack_tables(sg_hip_ctx *c, const sg_pack_args *a)
{
  if (!c || !a) return fail(c, SG_E_INVAL, "null argument");
  if (a->blob_words && (!a->blob_src || !a->blob_dst)) return fail(c, SG_E_INVAL, "null blob");
  if (a->n_req == 0 && a->blob_words) {
    // no tables, only words to bring along
    DeviceGuard g(c->device);
    PackArgs p;
    memset(&p, 0, sizeof p);
    p.blob_src = a->blob_src;
    p.blob_dst = a->blob_dst;
    p.blob_words = a->blob_words;
    const uint32_t blocks = (a->blob_words + 4 * kBlock - 1) / (4 * kBlock);
    k_pack_tables<16><<<blocks > 256 ? 256u : blocks, kBlock, 0, a->stream ? static_cast<hipStream_t>(a->stream) : c->stream>>>(p);
    HIP_TRY(c, hipGetLastError());
    return SG_OK;
  }
  int rc = check_ring(c, a->ring, "packet");
  if (rc != SG_OK) return rc;
  if (a->n_req == 0) return SG_OK;
  if (!a->tables || !a->table_idx || !a->req_first || (a->n_frags && !a->frag_slot)) return fail(c, SG_E_INVAL, "null tables");
  const uint32_t hl = hdr_len_of(a->ring.hdr_profile);
  if ((a->pkt_base & 1u) || (uint64_t)(uintptr_t)a->ring.base < a->pkt_base)
    return fail(c, SG_E_INVAL, "pkt_base must be even and at or below the ring");
  if ((uintptr_t)a->tables & 15u) return fail(c, SG_E_INVAL, "fragment tables must start at a 16-byte aligned address");
  DeviceGuard g(c->device);
  PackArgs p;
  memset(&p, 0, sizeof p);
  p.tables = a->tables;
  p.table_idx = a->table_idx;
  p.req_first = a->req_first;
  p.n_req = a->n_req;
  p.n_frags = a->n_frags;
  p.n_tables = a->n_tables;
  p.delta = (uint64_t)(uintptr_t)a->ring.base + hl - a->pkt_base;
  p.ring_bytes = (uint64_t)a->ring.n_slots * a->ring.slot_size;
  p.slot_size = a->ring.slot_size;
  p.n_slots = a->ring.n_slots;
  p.frag_slot = a->frag_slot;
  p.frag_len = a->frag_len;
  p.req_first_out = a->req_first_out;
  p.blob_src = a->blob_src;
  p.blob_dst = a->blob_dst;
  p.blob_words = a->blob_words;
  hipStream_t st = a->stream ? static_cast<hipStream_t>(a->stream) : c->stream;
  // Sixteen lanes per request, whatever the tables' length: the pull is bound by the bus either way
  // (512 tables of 431 entries: 21 us with 16 or with 64 lanes each), but reads across the bus that
  // are in flight hold up the memory traffic of a copy kernel running beside them -- a gather of
  // 104 us took 114 us beside a pull with 64 lanes per request and 106 us beside one with 16.
  constexpr uint32_t lanes = 16;
  p.req_blocks = (a->n_req + kBlock / lanes - 1) / (kBlock / lanes);
  const uint32_t copy_blocks = a->blob_words ? (a->blob_words + 4 * kBlock - 1) / (4 * kBlock) : 0u;
  const uint32_t grid = p.req_blocks + (copy_blocks > 64 ? 64u : copy_blocks);
  k_pack_tables<lanes><<<grid, kBlock, 0, st>>>(p);
  HIP_TRY(c, hipGetLastError());
  return SG_OK;
}

// ---- allocation-free gather ---------------------------------------------------

namespace {
constexpr int kStaticMaxDevices = 64;
std::mutex g_static_mu;
uint8_t *g_static_ptr[kStaticMaxDevices];  // device address of `scratch` on each GPU, once asked for

// The device address of this GPU's copy of the static array (every GPU holds
// its own copy at its own address).  The device must be current.
int static_scratch_of(int device, uint8_t **out)
{
  if (device < 0 || device >= kStaticMaxDevices) return fail(nullptr, SG_E_INVAL, "device %d out of range", device);
  std::lock_guard<std::mutex> lock(g_static_mu);
  if (!g_static_ptr[device]) {
    uint8_t *p = nullptr;
    HIP_TRY(nullptr, hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch)));
    if (!p) return fail(nullptr, SG_E_HIP, "hipGetSymbolAddress returned a null address on device %d", device);
    g_static_ptr[device] = p;
  }
  *out = g_static_ptr[device];
  return SG_OK;
}
}  // namespace

int sg_hip_gather_batch_static(int device_id, void *stream, const sg_gather_args *a, uint64_t *cursor,
                               uint32_t *status)
{
  if (!a) return fail(nullptr, SG_E_INVAL, "null argument");
  DeviceGuard g(device_id);
  if (!g.ok) return fail(nullptr, SG_E_HIP, "cannot select device %d", device_id);
  uint8_t *base = nullptr;
  int rc = static_scratch_of(device_id, &base);
  if (rc != SG_OK) return rc;
  if (a->n_req > SG_STATIC_MAX_REQS || a->n_frags > SG_STATIC_MAX_FRAMES)
    return fail(nullptr, SG_E_INVAL,
                "%u requests in %u fragments: the allocation-free gather takes at most %u requests in %u fragments",
                a->n_req, a->n_frags, (unsigned)SG_STATIC_MAX_REQS, (unsigned)SG_STATIC_MAX_FRAMES);
  hipStream_t st = static_cast<hipStream_t>(stream);
  Scratch sc;
  sc.max_reqs = SG_STATIC_MAX_REQS;
  sc.max_frames = SG_STATIC_MAX_FRAMES;
  uint8_t *m = base;
  sc.desc = reinterpret_cast<u32x4 *>(m); m += kStaticDesc;
  sc.req_size = reinterpret_cast<uint64_t *>(m); m += kStaticReq;
  sc.req_off = reinterpret_cast<uint64_t *>(m); m += kStaticReq;
  sc.tile_tot = reinterpret_cast<uint64_t *>(m); m += kStaticTile;
  uint64_t *w64 = reinterpret_cast<uint64_t *>(m);      // [0] the array's own cursor, [1] unused, [2] staged cursor
  uint32_t *w32 = reinterpret_cast<uint32_t *>(m + 64);  // [0] the array's own status word, [1] refusal flag
  sc.cursor[0] = cursor ? cursor : w64;
  sc.cursor[1] = nullptr;
  sc.next_cursor[0] = w64 + 2;
  sc.next_cursor[1] = nullptr;
  sc.status = status ? status : w32;
  sc.flag = w32 + 1;
  sc.slot_idx[0] = w32 + 2;  // the array's own producer index, for callers that pass a slot ring
  sc.slot_idx[1] = w32 + 3;
  // descriptors, request totals, offsets and the staged cursor are written by this call's own
  // kernels before they are read; the array's own status word would carry the last call's
  // refusals: it is cleared ahead of the call's first kernel, once the host has nothing to refuse
  return gather_impl(nullptr, sc, st, a, nullptr, status ? nullptr : w32);
}

// ---- reassembly ----------------------------------------------------------------

namespace {

uint32_t pow2_at_least(uint64_t v)
{
  uint32_t p = 1;
  while (p < v) p <<= 1;
  return p;
}

// Carves the reassembly state out of c->ra_mem (allocating it first where needed).
int ra_state(sg_hip_ctx *c, RaArgs *r, bool *fresh)
{
  const uint32_t n_max = c->max_frames;
  const uint32_t cells = pow2_at_least(4ull * c->max_reqs < 2 * kRaBucket ? 2 * kRaBucket : 4ull * c->max_reqs);
  const uint32_t records = pow2_at_least(c->max_reqs);
  const size_t n_blk = (n_max + kRaSmallBlock - 1) / kRaSmallBlock + 1;  // a total per workgroup of k_ra_flag, the small ones
  const size_t bytes = (size_t)cells * (8 + 8 + 4 * 4) + (size_t)records * SG_MAX_BI_SIZE * 8 + (size_t)records * 4 +
                       kRaWords * 4 + (size_t)n_max * (3 * 4 + 8) + n_blk * 8 + 256;
  *fresh = false;
  if (!c->ra_mem) {
    // the small allocation first: a context never holds the state without its pinned counts
    if (!c->h_counts) {
      HIP_TRY(c, hipHostMalloc((void **)&c->h_counts, 4 * sizeof(uint32_t), hipHostMallocDefault));
      memset(c->h_counts, 0, 4 * sizeof(uint32_t));
    }
    HIP_TRY(c, hipMalloc(&c->ra_mem, bytes));
    c->ra_cells = cells;
    c->ra_records = records;
    *fresh = true;
  }
  memset(r, 0, sizeof *r);
  uint8_t *m = static_cast<uint8_t *>(c->ra_mem);
  r->keys = reinterpret_cast<unsigned long long *>(m); m += (size_t)cells * 8;
  r->acc = reinterpret_cast<unsigned long long *>(m); m += (size_t)cells * 8;
  r->tab = reinterpret_cast<unsigned long long *>(m); m += (size_t)records * SG_MAX_BI_SIZE * 8;
  r->arr_pack = reinterpret_cast<unsigned long long *>(m); m += (size_t)n_max * 8;
  r->blk = reinterpret_cast<unsigned long long *>(m); m += n_blk * 8;
  r->want = reinterpret_cast<uint32_t *>(m); m += (size_t)cells * 4;
  r->last = reinterpret_cast<uint32_t *>(m); m += (size_t)cells * 4;
  r->rec = reinterpret_cast<uint32_t *>(m); m += (size_t)cells * 4;
  r->seen = reinterpret_cast<uint32_t *>(m); m += (size_t)cells * 4;
  r->free_ring = reinterpret_cast<uint32_t *>(m); m += (size_t)records * 4;
  r->words = reinterpret_cast<uint32_t *>(m); m += kRaWords * 4;
  r->arr_cell = reinterpret_cast<uint32_t *>(m); m += (size_t)n_max * 4;
  r->arr_len = reinterpret_cast<uint32_t *>(m); m += (size_t)n_max * 4;
  r->arr_fidx = reinterpret_cast<uint32_t *>(m);
  r->bmask = cells / kRaBucket - 1;
  r->rmask = records - 1;
  r->counts_host = c->h_counts;
  r->status = c->status;
  r->status_flag = c->h_flag;
  return SG_OK;
}

void ra_launch_reset(sg_hip_ctx *c, const RaArgs &r)
{
  const size_t items = (size_t)c->ra_records * SG_MAX_BI_SIZE > c->ra_cells ? (size_t)c->ra_records * SG_MAX_BI_SIZE
                                                                            : c->ra_cells;
  k_ra_reset<<<(uint32_t)((items + 255) / 256), 256, 0, c->stream>>>(r, c->ra_cells, c->ra_records);
}

}  // namespace

int sg_hip_reassemble_reset(sg_hip_ctx *c)
{
  if (!c) return SG_E_INVAL;
  DeviceGuard g(c->device);
  RaArgs r;
  bool fresh;
  int rc = ra_state(c, &r, &fresh);
  if (rc != SG_OK) return rc;
  ra_launch_reset(c, r);
  return finish(c, 0);
}

int sg_hip_reassemble_evict(sg_hip_ctx *c, uint32_t max_age_calls, uint32_t *n_evicted_out)
{
  if (!c) return SG_E_INVAL;
  if (n_evicted_out) *n_evicted_out = 0;
  if (!c->ra_mem) return SG_OK;  // nothing has come in yet
  DeviceGuard g(c->device);
  RaArgs r;
  bool fresh;
  int rc = ra_state(c, &r, &fresh);
  if (rc != SG_OK) return rc;
  k_zero_words<<<1, kBlock, 0, c->stream>>>(r.words + kRaEvicted, 1);
  k_ra_evict<<<(c->ra_cells + kWavesPerBlock - 1) / kWavesPerBlock, kBlock, 0, c->stream>>>(r, c->ra_cells, max_age_calls);
  rc = finish(c, 0);
  if (rc != SG_OK) return rc;
  uint32_t n = 0;
  HIP_TRY(c, hipMemcpy(&n, r.words + kRaEvicted, sizeof n, hipMemcpyDeviceToHost));
  if (n_evicted_out) *n_evicted_out = n;
  return SG_OK;
}

int sg_hip_reassemble(sg_hip_ctx *c, const sg_reassemble_args *a, uint32_t *counts_host_out)
{
  if (!c || !a) return fail(c, SG_E_INVAL, "null argument");
  int rc = check_ring(c, a->ring, "rx");
  if (rc != SG_OK) return rc;
  if (counts_host_out) memset(counts_host_out, 0, 4 * sizeof(uint32_t));
  if (a->n_arrivals > c->max_frames) return fail(c, SG_E_INVAL, "n_arrivals %u > max_frames %u of this context", a->n_arrivals, c->max_frames);
  if ((a->n_arrivals && !a->arrivals) || !a->frag_slot || !a->frag_len || !a->req_first) return fail(c, SG_E_INVAL, "null tables");
  const bool ref64 = a->ring.hdr_profile == SG_HDR_REF64;
  if (ref64 && (!a->len_nic || !a->req_size)) return fail(c, SG_E_INVAL, "REF64 headers need len_nic and the server-wide request size");
  DeviceGuard g(c->device);

  RaArgs r;
  bool fresh;
  rc = ra_state(c, &r, &fresh);
  if (rc != SG_OK) return rc;
  if (fresh) ra_launch_reset(c, r);
  r.ring = static_cast<const uint8_t *>(a->ring.base);
  r.n_slots = a->ring.n_slots;
  r.slot_size = a->ring.slot_size;
  r.ref64 = ref64;
  r.n = a->n_arrivals;
  r.n_dev = a->n_arrivals_dev;
  r.arrivals = a->arrivals;
  r.len_nic = a->len_nic;
  r.req_size = a->req_size;
  r.max_req = c->max_reqs;
  r.max_frag = c->max_frames;
  // workgroups of 256 threads where the caller says the call runs beside a long kernel
  const bool small_groups = (a->flags & SG_F_SMALL_GROUPS) != 0;
  r.blk_size = small_groups ? kRaSmallBlock : kRaBlock;
  r.n_blocks = (a->n_arrivals + r.blk_size - 1) / r.blk_size;
  r.frag_slot = a->frag_slot;
  r.frag_len = a->frag_len;
  r.req_first = a->req_first;
  r.req_token = a->req_token;
  r.req_hdr_slot = a->req_hdr_slot;
  r.counts_out = a->counts_out;

  const uint32_t g_take = (a->n_arrivals + kRaTakeBlock - 1) / kRaTakeBlock;
  rc = prof_begin(c, 5);
  if (rc != SG_OK) return rc;
  if (a->n_arrivals <= (uint32_t)kRaTakeBlock) {
    // a NIC burst (an empty one still leaves its counts): one workgroup, one launch
    k_ra_burst<<<1, kRaTakeBlock, 0, c->stream>>>(r);
  } else {
    if (small_groups) {
      k_ra_insert<kRaSmallBlock><<<r.n_blocks, kRaSmallBlock, 0, c->stream>>>(r);
      k_ra_flag<kRaSmallBlock><<<r.n_blocks, kRaSmallBlock, 0, c->stream>>>(r);
      k_ra_scan<kRaSmallBlock><<<1, kRaSmallBlock, 0, c->stream>>>(r);
      k_ra_emit<kRaSmallBlock><<<r.n_blocks, kRaSmallBlock, 0, c->stream>>>(r);
    } else {
      k_ra_insert<kRaTakeBlock><<<g_take, kRaTakeBlock, 0, c->stream>>>(r);
      k_ra_flag<kRaBlock><<<r.n_blocks, kRaBlock, 0, c->stream>>>(r);
      k_ra_scan<kRaBlock><<<1, kRaBlock, 0, c->stream>>>(r);
      k_ra_emit<kRaTakeBlock><<<g_take, kRaTakeBlock, 0, c->stream>>>(r);
    }
  }
  rc = prof_end(c);
  if (rc != SG_OK) return rc;
  rc = finish(c, a->flags);
  if (rc != SG_OK || (a->flags & SG_F_ASYNC)) return rc;
  if (counts_host_out) memcpy(counts_host_out, c->h_counts, 4 * sizeof(uint32_t));
  return SG_OK;
}

}  // extern "C"
