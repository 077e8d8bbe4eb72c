// Host side of libflashMoe.so: workspace layout, validation, launch, the C ABI
// of include/flash_moe.h and the C++ interface of include/iMoeKernelLauncher.h.
//
// Differences from the reference's host launcher
// (src/hip/launcher/moeKernelLauncher.hip:58-212) that matter to callers:
//  * shape, dtype and top-k are run-time fields, not compile-time constants
//  * all per-launcher state travels in the kernel argument, so any number of
//    launchers can live on one device (the reference keeps its state in
//    process-global __constant__ symbols)
//  * a launch issues exactly one kernel and no memset/memcpy: the kernel
//    returns its counters to zero itself, which also makes a launch capturable
//    in a HIP graph
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>

#include "../../include/iMoeKernelLauncher.h"
#include "moe_params.h"

namespace fmoe {
hipError_t launch_stream_kernel(const Params& p, int dtype, int grid, hipStream_t stream);
hipError_t prepare_stream_kernel();
hipError_t pack_weights(const void* src, void* dst, int dtype, int E, int H, int I, int which,
                        hipStream_t stream);
hipError_t launch_tiled_kernel(const Params& p, int grid, hipStream_t stream);
hipError_t prepare_tiled_kernel();
hipError_t stream_kernel_occupancy(int dtype, int* per_cu);
hipError_t tiled_kernel_occupancy(int* per_cu);
int tiled_max_tokens();
hipError_t launch_rmsnorm(const void* x, const void* gamma, void* xn, int dtype, int T, int H, double eps,
                          hipStream_t stream);
size_t tiled_y_bytes(size_t rows, size_t hidden);
}

#define FMOE_FILENAME (strrchr(__FILE__, '/') ? strrchr(__FILE__, '/') + 1 : __FILE__)

// Same convention as the reference (src/hip/hipHostCommon.h:11-19): print to
// stdout, return the first failing code.
#define FMOE_HIP_CHECK(expr)                                               \
  do {                                                                     \
    const hipError_t fmoe_err_ = (expr);                                   \
    if (fmoe_err_ != hipSuccess) {                                         \
      printf("[MOE HIP ERROR: %s:%i]: %s\n", FMOE_FILENAME, __LINE__,      \
             hipGetErrorString(fmoe_err_));                                \
      fflush(stdout);                                                      \
      return fmoe_err_;                                                    \
    }                                                                      \
  } while (0)

#define FMOE_FAIL(code, fmt, ...)                                                      \
  do {                                                                                 \
    printf("[MOE ERROR: %s:%i]: " fmt "\n", FMOE_FILENAME, __LINE__, ##__VA_ARGS__);   \
    fflush(stdout);                                                                    \
    return (code);                                                                     \
  } while (0)

namespace {

constexpr long long kMaxRows = 1ll << 21;  // max_tokens * top_k a launcher may be sized for

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

struct Layout {
  size_t ctl, wgflags, g1_done, tok_arrive, cand, topk_idx, topk_w, masks, word_prefix,
      expert_count, expert_offset, perm, row_w, mtiles, h, y, xn, pack1, pack2, total;
  size_t zero_bytes;  // leading region that must be zero before a launch
  int W, max_mtiles;
};

constexpr int kMaxGroups = 1024;  // workgroups a launch may use (one per CU)

// AUTO hands a batch to the tiled variant from this many rows an expert on (on average):
// packed weights / the caller's row-major weights. Below it the streaming variant runs, which
// is what its share of `y` is sized for.
constexpr int kAutoTiledRowsPacked = 26;
constexpr int kAutoTiledRowsRowMajor = 14;

// need_tiled: the tiled variant may run on this workspace.
Layout make_layout(const FlashMoeLayerDesc& d, bool need_tiled) {
  Layout L{};
  const size_t rows = static_cast<size_t>(d.max_tokens) * d.top_k;
  const size_t esz = d.dtype == FLASH_MOE_BF16 ? 2 : 4;
  L.W = (d.max_tokens + 63) / 64;
  L.max_mtiles = static_cast<int>((rows + fmoe::SKINNY_MT - 1) / fmoe::SKINNY_MT) + d.experts;
  size_t off = 0;
  auto take = [&](size_t bytes) {
    const size_t at = off;
    off = align_up(off + bytes, 256);
    return at;
  };
  // zero-initialised region first: control block, per-tile counters, masks
  L.ctl = take(sizeof(fmoe::Control));
  L.wgflags = take(sizeof(fmoe::WgFlags) * kMaxGroups);
  L.g1_done = take(sizeof(fmoe::ControlLine) * L.max_mtiles);
  L.masks = take(sizeof(unsigned long long) * d.experts * L.W);
  L.tok_arrive = take(sizeof(unsigned) * d.max_tokens);
  L.zero_bytes = off;
  L.cand = take(sizeof(unsigned long long) * d.max_tokens * d.experts);
  L.word_prefix = take(sizeof(int) * d.experts * L.W);
  L.topk_idx = take(sizeof(int) * rows);
  L.topk_w = take(sizeof(float) * rows);
  L.expert_count = take(sizeof(int) * d.experts);
  L.expert_offset = take(sizeof(int) * (d.experts + 1));
  L.perm = take(sizeof(int) * rows);
  L.row_w = take(sizeof(float) * rows);
  L.mtiles = take(sizeof(fmoe::TileDesc) * L.max_mtiles);
  (void)need_tiled;  // both variants keep h as [rows, I], rows in permuted order
  const size_t h_rows = rows;
  L.h = take(esz * h_rows * d.intermediate);
  // y: the streaming variant keeps every (token, slot) row in float, the tiled variant in
  // bf16. When every batch that asks for the tiled variant gets it (tiled_all) and AUTO hands
  // it the large batches, the streaming one only ever sees batches below the switch-over.
  const bool tiled_all = need_tiled && static_cast<long long>(d.max_tokens) * d.hidden * 2 < (1ll << 32);
  const size_t stream_rows =
      tiled_all && d.sched == FLASH_MOE_SCHED_TILED ? 0
      : tiled_all && d.sched == FLASH_MOE_SCHED_AUTO ? std::min<size_t>(rows, kAutoTiledRowsPacked * static_cast<size_t>(d.experts))
                                                     : rows;
  L.y = take(std::max(sizeof(float) * stream_rows * d.hidden,
                      need_tiled ? fmoe::tiled_y_bytes(rows, d.hidden) : 0));
  L.xn = take((d.flags & FLASH_MOE_FLAG_RMSNORM) ? esz * static_cast<size_t>(d.max_tokens) * d.hidden : 0);
  const bool pack = (d.flags & FLASH_MOE_FLAG_PACK_WEIGHTS) != 0;
  L.pack1 = take(pack ? esz * d.experts * 2 * d.intermediate * d.hidden : 0);
  L.pack2 = take(pack ? esz * d.experts * d.hidden * d.intermediate : 0);
  L.total = off;
  return L;
}

hipError_t validate(const FlashMoeLayerDesc* d) {
  if (d == nullptr) FMOE_FAIL(hipErrorInvalidValue, "null layer description");
  if (d->dtype != FLASH_MOE_F32 && d->dtype != FLASH_MOE_BF16)
    FMOE_FAIL(hipErrorInvalidValue, "dtype %i is neither float32 (0) nor bfloat16 (1)", d->dtype);
  if (d->experts < 1 || d->experts > fmoe::MAX_EXPERTS)
    FMOE_FAIL(hipErrorInvalidValue, "experts = %i, supported 1..%i", d->experts,
              fmoe::MAX_EXPERTS);
  if (d->top_k < 1 || d->top_k > d->experts || d->top_k > fmoe::MAX_TOPK)
    FMOE_FAIL(hipErrorInvalidValue, "top_k = %i, supported 1..min(experts, %i)", d->top_k,
              fmoe::MAX_TOPK);
  if (d->hidden < 64 || d->hidden % 64 != 0)
    FMOE_FAIL(hipErrorInvalidValue, "hidden = %i must be a positive multiple of 64", d->hidden);
  if (d->intermediate < 32 || d->intermediate % 32 != 0)
    FMOE_FAIL(hipErrorInvalidValue, "intermediate = %i must be a positive multiple of 32",
              d->intermediate);
  if (d->max_tokens < 1) FMOE_FAIL(hipErrorInvalidValue, "max_tokens = %i", d->max_tokens);
  // Capacity comes before any pointer is looked at, as in the reference
  // (src/hip/launcher/moeKernelLauncher.hip:117-135; pinned there by
  // test/singleGPU/cpp/moe/moeApiTest.cpp:5-12 with null weights).
  if (static_cast<long long>(d->max_tokens) * d->top_k > kMaxRows)
    FMOE_FAIL(hipErrorUnknown,
              "max_tokens = %i is beyond capacity: this configuration handles %lli tokens",
              d->max_tokens, kMaxRows / d->top_k);
  if (d->sched < FLASH_MOE_SCHED_AUTO || d->sched > FLASH_MOE_SCHED_TILED)
    FMOE_FAIL(hipErrorInvalidValue, "sched = %i", d->sched);
  if ((d->flags & ~(FLASH_MOE_FLAG_PACK_WEIGHTS | FLASH_MOE_FLAG_WEIGHTS_PREPACKED |
                    FLASH_MOE_FLAG_RMSNORM | FLASH_MOE_FLAG_RESIDUAL)) != 0)
    FMOE_FAIL(hipErrorInvalidValue, "unknown flag bits 0x%x", d->flags);
  if ((d->flags & FLASH_MOE_FLAG_PACK_WEIGHTS) && (d->flags & FLASH_MOE_FLAG_WEIGHTS_PREPACKED))
    FMOE_FAIL(hipErrorInvalidValue, "weights that are already packed need no packed copy");
  return hipSuccess;
}

// The tiled variant needs bf16, tile-aligned shapes and token rows it can
// address with 32-bit byte offsets. AUTO takes it once an expert sees about 26
// rows on average when the weights are packed (30B shape, us, streaming / tiled:
// T=320 284 / 301, T=384 293 / 301, T=448 314 / 299, T=512 339 / 304; 235B shape:
// T=320 905 / 960, T=384 934 / 969, T=512 1054 / 976), and from about 14 rows on
// the caller's row-major weights, which the streaming variant reads half a
// cache line at a time (30B: T=192 309 / 318, T=256 318 / 318, T=320 346 / 320;
// 235B: T=192 1030 / 1001, T=256 1055 / 1007, T=384 1142 / 1015).
bool tiled_eligible(const FlashMoeLayerDesc& d, int tokens_num) {
  return d.dtype == FLASH_MOE_BF16 && d.hidden % 256 == 0 && d.intermediate % 128 == 0 &&
         tokens_num <= fmoe::tiled_max_tokens() &&
         static_cast<long long>(tokens_num) * d.hidden * 2 < (1ll << 32);
}

int sched_for(const FlashMoeLayerDesc& d, int tokens_num) {
  if (d.sched == FLASH_MOE_SCHED_STREAM) return FLASH_MOE_SCHED_STREAM;
  if (!tiled_eligible(d, tokens_num)) return FLASH_MOE_SCHED_STREAM;
  if (d.sched == FLASH_MOE_SCHED_TILED) return FLASH_MOE_SCHED_TILED;
  const long long rows = static_cast<long long>(tokens_num) * d.top_k;
  const bool packed = (d.flags & (FLASH_MOE_FLAG_PACK_WEIGHTS | FLASH_MOE_FLAG_WEIGHTS_PREPACKED)) != 0;
  return rows >= static_cast<long long>(packed ? kAutoTiledRowsPacked : kAutoTiledRowsRowMajor) * d.experts
             ? FLASH_MOE_SCHED_TILED
             : FLASH_MOE_SCHED_STREAM;
}

// Whether any batch size up to max_tokens may run the tiled variant.
bool may_run_tiled(const FlashMoeLayerDesc& d) {
  return d.sched != FLASH_MOE_SCHED_STREAM && tiled_eligible(d, 1);
}

}  // namespace

struct FlashMoeLauncher {
  FlashMoeLayerDesc desc;
  Layout layout;
  char* ws = nullptr;
  int device = 0;
  int num_cus = 0;
  long long ticks_per_ms = 100000;
  long long spin_limit = 0;
  int last_tokens = 0;
  fmoe::TraceRec* trace = nullptr;
  unsigned trace_cap = 0;
  // One word of pinned host memory that a failing launch's last worker adds its error
  // bits to (null for the launcher-less entry point, which may not allocate).
  unsigned reported_error = 0;         // bits Launch has reported since the last flashMoeStatus
  unsigned* host_error = nullptr;      // host address
  unsigned* host_error_dev = nullptr;  // the same word as the device addresses it
};

namespace {

fmoe::Params make_params(const FlashMoeLauncher* l, const void* tokens, void* output, int T) {
  const FlashMoeLayerDesc& d = l->desc;
  const Layout& L = l->layout;
  fmoe::Params p{};
  p.T = T;
  p.E = d.experts;
  p.H = d.hidden;
  p.K = d.top_k;
  p.I = d.intermediate;
  p.W = L.W;
  p.n_groups = l->num_cus < kMaxGroups ? l->num_cus : kMaxGroups;
  p.n_workers = p.n_groups * 8;
  p.fuse_scatter = (static_cast<long long>(T) * d.top_k <= 2048) ? 1 : 0;
  // Early gate/up tasks wait inside the kernel for the routing, so every routing
  // task must be among the tickets the workers start with: they go to the first
  // workgroups, four dot tasks and four select/scan tasks each (half of the
  // workgroups at most, to leave workers for the weights).
  const int dot_tasks = ((T + fmoe::ROUTER_TOK - 1) / fmoe::ROUTER_TOK) *
                        ((d.experts + fmoe::ROUTER_EXP - 1) / fmoe::ROUTER_EXP);
  // bf16 layers run the logit chains on the matrix core, 16 tokens x 16 experts
  // per workgroup, while every such task finds a workgroup of its own
  const int dot16_tasks = ((T + 15) / 16) * ((d.experts + 15) / 16);
  p.dot16 = (d.dtype == FLASH_MOE_BF16 && d.hidden % fmoe::DOT16_KC == 0 &&
             dot16_tasks <= p.n_groups)
                ? 1
                : 0;
  const int routing_groups =
      std::max(p.dot16 ? dot16_tasks : (dot_tasks + 3) / 4, (T + 4) / 4);
  // Early mode hands out the tasks of every expert, used or not (an unused one
  // costs a ticket and a wasted first round of loads), so it needs a batch that
  // reaches most experts: T*k >= E (measured on the 30B shape, with it / without:
  // T=8 167 / 145 us, T=16 199 / 200, T=24 227 / 242, T=64 263 / 278).
  const bool reaches_experts =
      static_cast<long long>(T) * d.top_k >= static_cast<long long>(d.experts);
  // An early task serves one block of 16 rows, or two; a tile with more starts
  // over from the tile table once the scan is done. So: one block up to 9 rows
  // per expert on average, two up to 24 (30B shape, us, none / one / two: T=64
  // 239 / 222 / 226, T=128 257 / 241 / 242, T=160 265 / 259 / 252, T=192 273 / 263 /
  // 259, T=256 284 / 289 / 272; 235B shape: T=128 821 / 792 / 805, T=192 865 / 850 /
  // 833, T=256 894 / 942 / 856).
  const long long slots = static_cast<long long>(T) * d.top_k;
  const int early_blocks = slots <= 9ll * d.experts ? 1 : slots <= 24ll * d.experts ? 2 : 0;
  p.early = (reaches_experts && early_blocks != 0 && p.fuse_scatter &&
             T <= fmoe::EARLY_MAX_TOKENS &&
             d.experts * ((T + 63) / 64) <= fmoe::SCAN_LDS_WORDS && d.experts <= L.max_mtiles &&
             routing_groups <= p.n_groups / 2)
                ? early_blocks
                : 0;
  p.max_mtiles = L.max_mtiles;
  p.spin_limit = l->spin_limit;
  p.tokens = (d.flags & FLASH_MOE_FLAG_RMSNORM) ? static_cast<const void*>(l->ws + L.xn) : tokens;
  p.residual = (d.flags & FLASH_MOE_FLAG_RESIDUAL) ? tokens : nullptr;
  p.gate = d.gate_weights;
  p.ffn1 = d.ffn1_weights;
  p.ffn2 = d.ffn2_weights;
  p.bias = d.router_bias;
  const bool pack = (d.flags & FLASH_MOE_FLAG_PACK_WEIGHTS) != 0;
  const bool prepacked = (d.flags & FLASH_MOE_FLAG_WEIGHTS_PREPACKED) != 0;
  // A launcher with its own packed copy has both forms and picks per launch. float32 batches
  // with 16 or more rows an expert run faster on the row-major tensors (30B shape, us,
  // row-major / packed: T=128 538 / 473, T=192 615 / 565, T=256 592 / 627, T=512 845 / 1088,
  // T=8192 6770 / 10930: the streaming variant's row tiles of one expert each fetch its
  // weights again, and the row-major rows stream at the higher rate then); bf16 batches are
  // faster on the packed copy at every size.
  const bool use_packed = pack && !(d.dtype == FLASH_MOE_F32 &&
                                    static_cast<long long>(T) * d.top_k >= 16ll * d.experts);
  p.ffn1_packed = use_packed ? l->ws + L.pack1 : prepacked ? d.ffn1_weights : nullptr;
  p.ffn2_packed = use_packed ? l->ws + L.pack2 : prepacked ? d.ffn2_weights : nullptr;
  if (prepacked) p.ffn1 = p.ffn2 = nullptr;  // no row-major form exists
  p.out = output;
  char* w = l->ws;
  p.ctl = reinterpret_cast<fmoe::Control*>(w + L.ctl);
  p.wgflags = reinterpret_cast<fmoe::WgFlags*>(w + L.wgflags);
  p.g1_done = reinterpret_cast<fmoe::ControlLine*>(w + L.g1_done);
  p.tok_arrive = reinterpret_cast<unsigned*>(w + L.tok_arrive);
  p.cand = reinterpret_cast<unsigned long long*>(w + L.cand);
  p.masks = reinterpret_cast<unsigned long long*>(w + L.masks);
  p.word_prefix = reinterpret_cast<int*>(w + L.word_prefix);
  p.topk_idx = reinterpret_cast<int*>(w + L.topk_idx);
  p.topk_w = reinterpret_cast<float*>(w + L.topk_w);
  p.expert_count = reinterpret_cast<int*>(w + L.expert_count);
  p.expert_offset = reinterpret_cast<int*>(w + L.expert_offset);
  p.perm = reinterpret_cast<int*>(w + L.perm);
  p.row_w = reinterpret_cast<float*>(w + L.row_w);
  p.mtiles = reinterpret_cast<fmoe::TileDesc*>(w + L.mtiles);
  p.h = w + L.h;
  p.y = reinterpret_cast<float*>(w + L.y);
  p.host_error = l->host_error_dev;
  p.zero_words = static_cast<unsigned>(L.zero_bytes / 4);
  p.elem_bytes = d.dtype == FLASH_MOE_BF16 ? 2 : 4;
  p.trace = l->trace;
  p.trace_cap = l->trace_cap;
  return p;
}

}  // namespace

extern "C" {

const char* flashMoeVersion(void) { return "flashMoe-mi355x 0.3 (gfx950)"; }

int flashMoeAbi(int* version, size_t* desc_bytes) {
  if (version == nullptr) FMOE_FAIL(hipErrorInvalidValue, "null result pointer");
  *version = FLASH_MOE_ABI_VERSION;
  if (desc_bytes != nullptr) *desc_bytes = sizeof(FlashMoeLayerDesc);
  return hipSuccess;
}

int flashMoeSetDenseSmallBatch(FlashMoeLauncher* l, int enable) {
  (void)l;
  (void)enable;
  return hipSuccess;
}

int flashMoeWorkspaceBytes(const FlashMoeLayerDesc* desc, size_t* bytes) {
  const hipError_t v = validate(desc);
  if (v != hipSuccess) return v;
  if (bytes == nullptr) FMOE_FAIL(hipErrorInvalidValue, "null result pointer");
  *bytes = make_layout(*desc, may_run_tiled(*desc)).total;
  return hipSuccess;
}

namespace {
hipError_t check_pack_args(int dtype, int experts, int hidden, int intermediate, int which,
                           const void* a, const void* b) {
  if (dtype != FLASH_MOE_F32 && dtype != FLASH_MOE_BF16)
    FMOE_FAIL(hipErrorInvalidValue, "dtype %i is neither float32 (0) nor bfloat16 (1)", dtype);
  if (experts < 1 || hidden < 64 || hidden % 64 != 0 || intermediate < 32 || intermediate % 32 != 0)
    FMOE_FAIL(hipErrorInvalidValue, "shape E=%i H=%i I=%i", experts, hidden, intermediate);
  if (which != 0 && which != 1) FMOE_FAIL(hipErrorInvalidValue, "which = %i (0: ffn1, 1: ffn2)", which);
  if (a == nullptr || b == nullptr) FMOE_FAIL(hipErrorInvalidValue, "null weight pointer");
  return hipSuccess;
}
}  // namespace

int flashMoePackWeights(int dtype, int experts, int hidden, int intermediate, int which,
                        const void* src, void* dst, void* stream_) {
  const hipError_t v = check_pack_args(dtype, experts, hidden, intermediate, which, src, dst);
  if (v != hipSuccess) return v;
  if (src == dst) FMOE_FAIL(hipErrorInvalidValue, "src and dst must not overlap (see flashMoePackWeightsInPlace)");
  FMOE_HIP_CHECK(fmoe::pack_weights(src, dst, dtype, experts, hidden, intermediate, which,
                                    static_cast<hipStream_t>(stream_)));
  return hipSuccess;
}

int flashMoePackWeightsInPlace(int dtype, int experts, int hidden, int intermediate, int which,
                               void* weights, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const hipError_t v = check_pack_args(dtype, experts, hidden, intermediate, which, weights, weights);
  if (v != hipSuccess) return v;
  const size_t esz = dtype == FLASH_MOE_BF16 ? 2 : 4;
  const size_t per_expert = esz * (which == 0 ? 2 : 1) * static_cast<size_t>(intermediate) * hidden;
  void* staging = nullptr;
  FMOE_HIP_CHECK(hipMalloc(&staging, per_expert));
  hipError_t e = hipSuccess;
  for (int x = 0; x < experts && e == hipSuccess; ++x) {
    char* w = static_cast<char*>(weights) + per_expert * x;
    e = hipMemcpyAsync(staging, w, per_expert, hipMemcpyDeviceToDevice, stream);
    if (e == hipSuccess) e = fmoe::pack_weights(staging, w, dtype, 1, hidden, intermediate, which, stream);
  }
  const hipError_t s = hipStreamSynchronize(stream);
  (void)hipFree(staging);
  FMOE_HIP_CHECK(e);
  FMOE_HIP_CHECK(s);
  return hipSuccess;
}

int flashMoeRefreshWeights(FlashMoeLauncher* l, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (l == nullptr) FMOE_FAIL(hipErrorInvalidValue, "null launcher");
  const FlashMoeLayerDesc& d = l->desc;
  if ((d.flags & FLASH_MOE_FLAG_PACK_WEIGHTS) == 0) return hipSuccess;  // nothing is copied
  FMOE_HIP_CHECK(fmoe::pack_weights(d.ffn1_weights, l->ws + l->layout.pack1, d.dtype, d.experts,
                                    d.hidden, d.intermediate, 0, stream));
  FMOE_HIP_CHECK(fmoe::pack_weights(d.ffn2_weights, l->ws + l->layout.pack2, d.dtype, d.experts,
                                    d.hidden, d.intermediate, 1, stream));
  return hipSuccess;
}

int flashMoeCreate(FlashMoeLauncher** out, const FlashMoeLayerDesc* desc, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const hipError_t v = validate(desc);
  if (v != hipSuccess) return v;
  if (out == nullptr) FMOE_FAIL(hipErrorInvalidValue, "null launcher result pointer");
  if (desc->gate_weights == nullptr || desc->ffn1_weights == nullptr ||
      desc->ffn2_weights == nullptr)
    FMOE_FAIL(hipErrorInvalidValue, "null weight pointer");
  if ((desc->flags & FLASH_MOE_FLAG_RMSNORM) && (desc->norm_weight == nullptr || !(desc->norm_eps >= 0.0)))
    FMOE_FAIL(hipErrorInvalidValue, "FLASH_MOE_FLAG_RMSNORM needs norm_weight and norm_eps >= 0");

  FlashMoeLauncher* l = new (std::nothrow) FlashMoeLauncher();
  if (l == nullptr) FMOE_FAIL(hipErrorOutOfMemory, "host allocation failed");
  l->desc = *desc;
  l->layout = make_layout(*desc, may_run_tiled(*desc));

  auto fail = [&](hipError_t e) {
    if (l->ws) (void)hipFree(l->ws);
    if (l->host_error) (void)hipHostFree(l->host_error);
    delete l;
    printf("[MOE HIP ERROR: %s]: create failed: %s\n", FMOE_FILENAME, hipGetErrorString(e));
    return static_cast<int>(e);
  };
  hipError_t e;
  if ((e = hipGetDevice(&l->device)) != hipSuccess) return fail(e);
  if ((e = hipDeviceGetAttribute(&l->num_cus, hipDeviceAttributeMultiprocessorCount,
                                 l->device)) != hipSuccess)
    return fail(e);
  int khz = 0;
  if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, l->device) == hipSuccess &&
      khz > 0)
    l->ticks_per_ms = khz;
  l->spin_limit = 2000 * l->ticks_per_ms;
  if ((e = fmoe::prepare_stream_kernel()) != hipSuccess) return fail(e);
  if ((e = fmoe::prepare_tiled_kernel()) != hipSuccess) return fail(e);
  // Waits happen inside the kernels, so every workgroup of a launch must be resident at
  // once: one per CU, which both kernels' resources allow only if nothing else is asked of them.
  int per_cu = 0;
  if ((e = fmoe::stream_kernel_occupancy(desc->dtype, &per_cu)) != hipSuccess) return fail(e);
  if (per_cu < 1) return fail(hipErrorLaunchOutOfResources);
  if ((e = fmoe::tiled_kernel_occupancy(&per_cu)) != hipSuccess) return fail(e);
  if (per_cu < 1) return fail(hipErrorLaunchOutOfResources);
  if ((e = hipMalloc(reinterpret_cast<void**>(&l->ws), l->layout.total)) != hipSuccess)
    return fail(e);
  if ((e = hipHostMalloc(reinterpret_cast<void**>(&l->host_error), 64, hipHostMallocDefault)) !=
      hipSuccess)
    return fail(e);
  *l->host_error = 0u;
  if ((e = hipHostGetDevicePointer(reinterpret_cast<void**>(&l->host_error_dev), l->host_error,
                                   0)) != hipSuccess)
    return fail(e);
  if ((e = hipMemsetAsync(l->ws, 0, l->layout.zero_bytes, stream)) != hipSuccess) return fail(e);
  if (desc->flags & FLASH_MOE_FLAG_PACK_WEIGHTS) {
    static bool announced = false;  // once per process: the cost must not go unseen
    if (!announced) {
      announced = true;
      const double mib = static_cast<double>(l->layout.pack2 - l->layout.pack1 +
                                             (l->layout.total - l->layout.pack2)) / (1024.0 * 1024.0);
      // (a notice, not an error: to stderr, so that a program's own stdout stays its own)
      fprintf(stderr,
              "[MOE] launcher keeps a packed copy of the expert weights: +%.0f MiB of device memory per "
              "launcher (FLASH_MOE_FLAG_PACK_WEIGHTS; without the flag the row-major tensors are read in "
              "place, and flashMoePackWeightsInPlace needs no copy at all)\n", mib);
    }
    if ((e = static_cast<hipError_t>(flashMoeRefreshWeights(l, stream))) != hipSuccess)
      return fail(e);
  }
  if ((e = hipStreamSynchronize(stream)) != hipSuccess) return fail(e);
  *out = l;
  return hipSuccess;
}

int flashMoeSchedFor(FlashMoeLauncher* l, int tokens_num) {
  if (l == nullptr) return -1;
  return sched_for(l->desc, tokens_num);
}

int flashMoeLaunch(FlashMoeLauncher* l, const void* tokens, void* output, int tokens_num,
                   void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (l == nullptr) FMOE_FAIL(hipErrorInvalidValue, "null launcher");
  if (tokens_num < 0) FMOE_FAIL(hipErrorInvalidValue, "tokens_num = %i", tokens_num);
  if (tokens_num > l->desc.max_tokens)
    FMOE_FAIL(hipErrorUnknown, "tokens_num = %i exceeds max_tokens = %i", tokens_num,
              l->desc.max_tokens);
  // A launch that failed on the device (see flashMoeStatus for the bits) has left NaN in its
  // output and the launcher ready for use; the first Launch after it has finished reports it.
  if (l->host_error != nullptr) {
    const unsigned bits = *static_cast<volatile unsigned*>(l->host_error);
    if (bits != 0u) {
      *static_cast<volatile unsigned*>(l->host_error) = 0u;
      l->reported_error |= bits;
      FMOE_FAIL(hipErrorUnknown,
                "an earlier launch failed on the device (error bits 0x%x: 1 = a dependency wait "
                "ran out, 2 = row-tile table overflow); its output is NaN; nothing was launched now",
                bits);
    }
  }
  if (tokens_num == 0) return hipSuccess;
  if (tokens == nullptr || output == nullptr)
    FMOE_FAIL(hipErrorInvalidValue, "null tokens/output pointer");
  const fmoe::Params p = make_params(l, tokens, output, tokens_num);
  l->last_tokens = tokens_num;
  if (l->desc.flags & FLASH_MOE_FLAG_RMSNORM)
    FMOE_HIP_CHECK(fmoe::launch_rmsnorm(tokens, l->desc.norm_weight, l->ws + l->layout.xn, l->desc.dtype,
                                        tokens_num, l->desc.hidden, l->desc.norm_eps, stream));
  if (flashMoeSchedFor(l, tokens_num) == FLASH_MOE_SCHED_TILED) {
    FMOE_HIP_CHECK(fmoe::launch_tiled_kernel(p, p.n_groups, stream));
  } else {
    FMOE_HIP_CHECK(fmoe::launch_stream_kernel(p, l->desc.dtype, p.n_groups, stream));
  }
  return hipSuccess;
}

}  // extern "C"

// ------------------------------------------------ the entry point that allocates nothing
// Workspace of flashMoeLaunchNoAlloc: one array per device, loaded with the
// code object and held until the process ends. In host code the array's name is
// only a handle for hipGetSymbolAddress; the device address it yields, kept per
// device in g_static, is what kernels, fills and copies are given.
// Behind the workspace proper: one line whose first word collects the error bits of failed
// launches (the clearing kernel leaves it alone; flashMoeNoAllocStatus reads and clears it).
constexpr size_t kScratchErrorOffset = FLASH_MOE_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[FLASH_MOE_NOALLOC_SCRATCH_BYTES + 256];

namespace {

constexpr int kMaxDevices = 64;
struct StaticDevice {
  bool ready = false;
  unsigned char* ptr = nullptr;  // device address of `scratch` on this device
  int num_cus = 0;
  long long ticks_per_ms = 100000;
};
StaticDevice g_static[kMaxDevices];
std::mutex g_static_mutex;

// 16 bytes per thread; n16 = number of 16-byte words to clear
__global__ void zero_fill_kernel(uint4* dst, size_t n16) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n16) dst[i] = make_uint4(0u, 0u, 0u, 0u);
}

// Once per device, with that device current.
hipError_t static_device(int device, const StaticDevice** out) {
  std::lock_guard<std::mutex> lock(g_static_mutex);
  StaticDevice& sd = g_static[device];
  if (!sd.ready) {
    void* ptr = nullptr;
    FMOE_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (ptr == nullptr) FMOE_FAIL(hipErrorInvalidSymbol, "no device address for the static workspace");
    FMOE_HIP_CHECK(hipDeviceGetAttribute(&sd.num_cus, hipDeviceAttributeMultiprocessorCount, device));
    int khz = 0;
    if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, device) == hipSuccess && khz > 0)
      sd.ticks_per_ms = khz;
    FMOE_HIP_CHECK(fmoe::prepare_stream_kernel());
    FMOE_HIP_CHECK(fmoe::prepare_tiled_kernel());
    // as in flashMoeCreate: every workgroup of a launch must be resident at once
    int per_cu = 0;
    FMOE_HIP_CHECK(fmoe::stream_kernel_occupancy(FLASH_MOE_BF16, &per_cu));
    if (per_cu < 1) FMOE_FAIL(hipErrorLaunchOutOfResources, "the streaming kernel does not fit a CU");
    FMOE_HIP_CHECK(fmoe::stream_kernel_occupancy(FLASH_MOE_F32, &per_cu));
    if (per_cu < 1) FMOE_FAIL(hipErrorLaunchOutOfResources, "the streaming kernel does not fit a CU");
    FMOE_HIP_CHECK(fmoe::tiled_kernel_occupancy(&per_cu));
    if (per_cu < 1) FMOE_FAIL(hipErrorLaunchOutOfResources, "the tiled kernel does not fit a CU");
    // the error word starts at zero (the array is zero-initialised with the code object,
    // but a process may have failed launches behind it)
    FMOE_HIP_CHECK(hipMemset(static_cast<unsigned char*>(ptr) + kScratchErrorOffset, 0, 256));
    sd.ptr = static_cast<unsigned char*>(ptr);
    sd.ready = true;
  }
  *out = &sd;
  return hipSuccess;
}

}  // namespace

extern "C" {

int flashMoeLaunchNoAlloc(const FlashMoeLayerDesc* desc, const void* tokens, void* output,
                          int tokens_num, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const hipError_t v = validate(desc);
  if (v != hipSuccess) return v;
  if ((desc->flags & FLASH_MOE_FLAG_PACK_WEIGHTS) != 0)
    FMOE_FAIL(hipErrorInvalidValue,
              "the packed weight copy is weight-sized device memory; flashMoeLaunchNoAlloc has none");
  if (desc->gate_weights == nullptr || desc->ffn1_weights == nullptr ||
      desc->ffn2_weights == nullptr)
    FMOE_FAIL(hipErrorInvalidValue, "null weight pointer");
  if ((desc->flags & FLASH_MOE_FLAG_RMSNORM) && (desc->norm_weight == nullptr || !(desc->norm_eps >= 0.0)))
    FMOE_FAIL(hipErrorInvalidValue, "FLASH_MOE_FLAG_RMSNORM needs norm_weight and norm_eps >= 0");
  if (tokens_num < 0) FMOE_FAIL(hipErrorInvalidValue, "tokens_num = %i", tokens_num);
  if (tokens_num > desc->max_tokens)
    FMOE_FAIL(hipErrorUnknown, "tokens_num = %i exceeds max_tokens = %i", tokens_num,
              desc->max_tokens);
  if (tokens_num == 0) return hipSuccess;
  if (tokens == nullptr || output == nullptr)
    FMOE_FAIL(hipErrorInvalidValue, "null tokens/output pointer");

  // The workspace is laid out for this call alone: its batch, its variant.
  FlashMoeLauncher l;
  l.desc = *desc;
  l.desc.max_tokens = tokens_num;
  int sched = sched_for(l.desc, tokens_num);
  l.layout = make_layout(l.desc, sched == FLASH_MOE_SCHED_TILED);
  if (sched == FLASH_MOE_SCHED_TILED && desc->sched == FLASH_MOE_SCHED_AUTO &&
      l.layout.total > static_cast<size_t>(FLASH_MOE_NOALLOC_SCRATCH_BYTES)) {
    // AUTO: the streaming variant's workspace is smaller, and it serves any batch
    sched = FLASH_MOE_SCHED_STREAM;
    l.desc.sched = FLASH_MOE_SCHED_STREAM;
    l.layout = make_layout(l.desc, false);
  }
  if (l.layout.total > static_cast<size_t>(FLASH_MOE_NOALLOC_SCRATCH_BYTES))
    FMOE_FAIL(hipErrorUnknown,
              "%i tokens of this layer need %zu bytes of workspace; the static one holds %zu "
              "(use flashMoeCreate / flashMoeLaunch for this size)",
              tokens_num, l.layout.total, static_cast<size_t>(FLASH_MOE_NOALLOC_SCRATCH_BYTES));
  int device = 0;
  FMOE_HIP_CHECK(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices) FMOE_FAIL(hipErrorInvalidDevice, "device %i", device);
  const StaticDevice* sd = nullptr;
  const hipError_t se = static_device(device, &sd);
  if (se != hipSuccess) return se;
  l.ws = reinterpret_cast<char*>(sd->ptr);
  l.device = device;
  l.num_cus = sd->num_cus;
  l.ticks_per_ms = sd->ticks_per_ms;
  l.spin_limit = 2000 * sd->ticks_per_ms;
  // where a failing launch's last worker leaves its error bits: device memory here, no
  // pinned host word (that would be an allocation)
  l.host_error_dev = reinterpret_cast<unsigned*>(sd->ptr + kScratchErrorOffset);

  // The array keeps what the last call (of any shape) left in it: counters, flags
  // and masks of this call's layout must start at zero. A kernel, not a memset,
  // so that the call can be recorded into a HIP graph.
  const size_t n16 = (l.layout.zero_bytes + 15) / 16;
  hipLaunchKernelGGL(zero_fill_kernel, dim3(static_cast<unsigned>((n16 + 255) / 256)), dim3(256), 0,
                     stream, reinterpret_cast<uint4*>(sd->ptr), n16);
  FMOE_HIP_CHECK(hipGetLastError());
  const fmoe::Params p = make_params(&l, tokens, output, tokens_num);
  if (desc->flags & FLASH_MOE_FLAG_RMSNORM)
    FMOE_HIP_CHECK(fmoe::launch_rmsnorm(tokens, desc->norm_weight, l.ws + l.layout.xn, desc->dtype, tokens_num,
                                        desc->hidden, desc->norm_eps, stream));
  if (sched == FLASH_MOE_SCHED_TILED) {
    FMOE_HIP_CHECK(fmoe::launch_tiled_kernel(p, p.n_groups, stream));
  } else {
    FMOE_HIP_CHECK(fmoe::launch_stream_kernel(p, desc->dtype, p.n_groups, stream));
  }
  return hipSuccess;
}

int flashMoeNoAllocStatus(unsigned* error_bits, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (error_bits == nullptr) FMOE_FAIL(hipErrorInvalidValue, "null result pointer");
  int device = 0;
  FMOE_HIP_CHECK(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices) FMOE_FAIL(hipErrorInvalidDevice, "device %i", device);
  const StaticDevice* sd = nullptr;
  const hipError_t se = static_device(device, &sd);
  if (se != hipSuccess) return se;
  FMOE_HIP_CHECK(hipStreamSynchronize(stream));
  unsigned bits = 0;
  FMOE_HIP_CHECK(hipMemcpy(&bits, sd->ptr + kScratchErrorOffset, sizeof(bits), hipMemcpyDeviceToHost));
  if (bits != 0u) FMOE_HIP_CHECK(hipMemset(sd->ptr + kScratchErrorOffset, 0, sizeof(bits)));
  *error_bits = bits;
  return hipSuccess;
}

int flashMoeDestroy(FlashMoeLauncher* l, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (l == nullptr) return hipSuccess;
  FMOE_HIP_CHECK(hipStreamSynchronize(stream));
  FMOE_HIP_CHECK(hipFree(l->ws));
  if (l->host_error) FMOE_HIP_CHECK(hipHostFree(l->host_error));
  if (l->trace) FMOE_HIP_CHECK(hipFree(l->trace));
  delete l;
  return hipSuccess;
}

int flashMoeReadRouting(FlashMoeLauncher* l, int tokens_num, int* topk_idx, float* topk_w,
                        int* expert_counts, int* expert_offsets, int* perm, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (l == nullptr) FMOE_FAIL(hipErrorInvalidValue, "null launcher");
  if (tokens_num < 0 || tokens_num > l->desc.max_tokens)
    FMOE_FAIL(hipErrorInvalidValue, "tokens_num = %i", tokens_num);
  FMOE_HIP_CHECK(hipStreamSynchronize(stream));
  const size_t rows = static_cast<size_t>(tokens_num) * l->desc.top_k;
  const Layout& L = l->layout;
  if (topk_idx)
    FMOE_HIP_CHECK(hipMemcpy(topk_idx, l->ws + L.topk_idx, sizeof(int) * rows,
                             hipMemcpyDeviceToHost));
  if (topk_w)
    FMOE_HIP_CHECK(hipMemcpy(topk_w, l->ws + L.topk_w, sizeof(float) * rows,
                             hipMemcpyDeviceToHost));
  if (expert_counts)
    FMOE_HIP_CHECK(hipMemcpy(expert_counts, l->ws + L.expert_count, sizeof(int) * l->desc.experts,
                             hipMemcpyDeviceToHost));
  if (expert_offsets)
    FMOE_HIP_CHECK(hipMemcpy(expert_offsets, l->ws + L.expert_offset,
                             sizeof(int) * (l->desc.experts + 1), hipMemcpyDeviceToHost));
  if (perm)
    FMOE_HIP_CHECK(hipMemcpy(perm, l->ws + L.perm, sizeof(int) * rows, hipMemcpyDeviceToHost));
  return hipSuccess;
}

int flashMoeReadIntermediate(FlashMoeLauncher* l, int tokens_num, void* h, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (l == nullptr || h == nullptr) FMOE_FAIL(hipErrorInvalidValue, "null argument");
  if (tokens_num < 0 || tokens_num > l->desc.max_tokens)
    FMOE_FAIL(hipErrorInvalidValue, "tokens_num = %i", tokens_num);
  FMOE_HIP_CHECK(hipStreamSynchronize(stream));
  const size_t esz = l->desc.dtype == FLASH_MOE_BF16 ? 2 : 4;
  const size_t bytes = esz * static_cast<size_t>(tokens_num) * l->desc.top_k * l->desc.intermediate;
  FMOE_HIP_CHECK(hipMemcpy(h, l->ws + l->layout.h, bytes, hipMemcpyDeviceToHost));
  return hipSuccess;
}

int flashMoeReadDownRows(FlashMoeLauncher* l, int tokens_num, void* y, int* elem_dtype, int* weighted,
                         void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (l == nullptr || y == nullptr || elem_dtype == nullptr || weighted == nullptr)
    FMOE_FAIL(hipErrorInvalidValue, "null argument");
  if (tokens_num < 0 || tokens_num > l->desc.max_tokens)
    FMOE_FAIL(hipErrorInvalidValue, "tokens_num = %i", tokens_num);
  FMOE_HIP_CHECK(hipStreamSynchronize(stream));
  const bool tiled = sched_for(l->desc, tokens_num) == FLASH_MOE_SCHED_TILED;
  const size_t rows = static_cast<size_t>(tokens_num) * l->desc.top_k;
  const size_t bytes = rows * l->desc.hidden * (tiled ? 2 : 4);
  const size_t kept = (l->layout.xn - l->layout.y);  // the region's size up to the next one
  if (bytes > kept) FMOE_FAIL(hipErrorInvalidValue, "the workspace keeps fewer down-projection rows than %zu", rows);
  *elem_dtype = tiled ? FLASH_MOE_BF16 : FLASH_MOE_F32;
  *weighted = tiled ? 0 : 1;
  FMOE_HIP_CHECK(hipMemcpy(y, l->ws + l->layout.y, bytes, hipMemcpyDeviceToHost));
  return hipSuccess;
}

int flashMoeStatus(FlashMoeLauncher* l, unsigned* error_bits, unsigned* launches, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (l == nullptr) FMOE_FAIL(hipErrorInvalidValue, "null launcher");
  FMOE_HIP_CHECK(hipStreamSynchronize(stream));
  fmoe::Control c;
  FMOE_HIP_CHECK(hipMemcpy(&c, l->ws + l->layout.ctl, sizeof(c), hipMemcpyDeviceToHost));
  unsigned bits = c.error.v | l->reported_error;
  l->reported_error = 0u;
  if (l->host_error != nullptr) {
    bits |= *static_cast<volatile unsigned*>(l->host_error);
    *static_cast<volatile unsigned*>(l->host_error) = 0u;
  }
  if (error_bits) *error_bits = bits;
  if (launches) *launches = c.launches.v;
  if (c.error.v != 0u) {
    // an aborted launch leaves counters and masks in an arbitrary state
    FMOE_HIP_CHECK(hipMemset(l->ws, 0, l->layout.zero_bytes));
  }
  return hipSuccess;
}

int flashMoeTraceEnable(FlashMoeLauncher* l, unsigned capacity) {
  if (l == nullptr) FMOE_FAIL(hipErrorInvalidValue, "null launcher");
  FMOE_HIP_CHECK(hipDeviceSynchronize());
  if (l->trace) {
    FMOE_HIP_CHECK(hipFree(l->trace));
    l->trace = nullptr;
    l->trace_cap = 0;
  }
  if (capacity == 0) return hipSuccess;
  FMOE_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&l->trace),
                           sizeof(fmoe::TraceRec) * static_cast<size_t>(capacity)));
  FMOE_HIP_CHECK(hipMemset(l->trace, 0xFF, sizeof(fmoe::TraceRec) * static_cast<size_t>(capacity)));
  l->trace_cap = capacity;
  return hipSuccess;
}

int flashMoeTraceRead(FlashMoeLauncher* l, void* records, unsigned max_records, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (l == nullptr || records == nullptr) FMOE_FAIL(hipErrorInvalidValue, "null argument");
  if (l->trace == nullptr) FMOE_FAIL(hipErrorInvalidValue, "tracing is not enabled");
  FMOE_HIP_CHECK(hipStreamSynchronize(stream));
  const unsigned n = max_records < l->trace_cap ? max_records : l->trace_cap;
  FMOE_HIP_CHECK(hipMemcpy(records, l->trace, sizeof(fmoe::TraceRec) * static_cast<size_t>(n),
                           hipMemcpyDeviceToHost));
  FMOE_HIP_CHECK(hipMemset(l->trace, 0xFF, sizeof(fmoe::TraceRec) * static_cast<size_t>(l->trace_cap)));
  return hipSuccess;
}

int flashMoeSetWaitLimitMs(FlashMoeLauncher* l, double ms) {
  if (l == nullptr || !(ms > 0.0)) FMOE_FAIL(hipErrorInvalidValue, "bad wait limit");
  l->spin_limit = static_cast<long long>(ms * static_cast<double>(l->ticks_per_ms));
  if (l->spin_limit < 1) l->spin_limit = 1;
  return hipSuccess;
}

}  // extern "C"

// ------------------------------------------------- C++ interface (drop-in)
namespace moe {

IMoeKernelLauncher::~IMoeKernelLauncher() {}

namespace {
class FusedMoeLauncher final : public IMoeKernelLauncher {
 public:
  explicit FusedMoeLauncher(FlashMoeLauncher* h) : handle_(h) {}
  hipError_t Launch(const void* tokens, void* output, int tokensNum,
                    hipStream_t stream) override {
    return static_cast<hipError_t>(flashMoeLaunch(handle_, tokens, output, tokensNum, stream));
  }
  FlashMoeLauncher* handle() const { return handle_; }
  void release() { handle_ = nullptr; }

 private:
  FlashMoeLauncher* handle_;
};
}  // namespace
}  // namespace moe

extern "C" {

moe::DistributedUniqueId GetDistributedUniqueId(bool empty) {
  // The reference asks rocSHMEM for an id unless `empty`
  // (src/moeKernelLauncher.cpp:15-30). There is no inter-GPU transport here,
  // so both cases give the all-zero id.
  (void)empty;
  moe::DistributedUniqueId id;
  memset(id.data, 0, sizeof(id.data));
  return id;
}

hipError_t CreateLauncherEx(moe::IMoeKernelLauncher** launcher, const FlashMoeLayerDesc* desc,
                            hipStream_t stream) {
  if (launcher == nullptr) FMOE_FAIL(hipErrorInvalidValue, "null launcher result pointer");
  FlashMoeLauncher* h = nullptr;
  const int e = flashMoeCreate(&h, desc, stream);
  if (e != hipSuccess) return static_cast<hipError_t>(e);
  moe::FusedMoeLauncher* obj = new (std::nothrow) moe::FusedMoeLauncher(h);
  if (obj == nullptr) {
    (void)flashMoeDestroy(h, stream);
    FMOE_FAIL(hipErrorOutOfMemory, "host allocation failed");
  }
  *launcher = obj;
  return hipSuccess;
}

hipError_t CreateLauncher(moe::IMoeKernelLauncher** launcher, const void* gateWeights,
                          const void* ffn1ExpertWeights, const void* ffn2ExpertWeights,
                          int maxTokens, hipStream_t stream, const moe::DistributedUniqueId& uid,
                          int rank, int worldSize) {
  (void)uid;
  // shape of src/hip/common/metadata.h:7-13
  FlashMoeLayerDesc d{};
  d.experts = 128;
  d.hidden = 2048;
  d.intermediate = 768;
  d.top_k = 8;
  d.dtype = FLASH_MOE_F32;
  d.max_tokens = maxTokens;
  d.sched = FLASH_MOE_SCHED_AUTO;
  // A caller of this entry point cannot say how its weights are to be read, so it gets the
  // fast way: a packed copy in the workspace (announced by flashMoeCreate). CreateLauncherEx
  // with flags = 0 reads the row-major tensors in place.
  d.flags = FLASH_MOE_FLAG_PACK_WEIGHTS;
  d.gate_weights = gateWeights;
  d.ffn1_weights = ffn1ExpertWeights;
  d.ffn2_weights = ffn2ExpertWeights;
  d.router_bias = nullptr;
  if (worldSize != 1 || rank != 0)
    FMOE_FAIL(hipErrorInvalidValue,
              "rank %i of %i: only rank 0 of a world of 1 is supported (no inter-GPU transport)",
              rank, worldSize);
  return CreateLauncherEx(launcher, &d, stream);
}

hipError_t DestroyLauncher(moe::IMoeKernelLauncher* launcher, hipStream_t stream) {
  if (launcher == nullptr) return hipSuccess;
  moe::FusedMoeLauncher* obj = static_cast<moe::FusedMoeLauncher*>(launcher);
  const int e = flashMoeDestroy(obj->handle(), stream);
  if (e != hipSuccess) return static_cast<hipError_t>(e);
  delete obj;
  return hipSuccess;
}

FlashMoeLauncher* LauncherHandle(moe::IMoeKernelLauncher* launcher) {
  if (launcher == nullptr) return nullptr;
  return static_cast<moe::FusedMoeLauncher*>(launcher)->handle();
}

}  // extern "C"
