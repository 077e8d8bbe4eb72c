// Shared host/device description of one launch of the fused MoE layer.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fmoe {

enum : int { DT_F32 = 0, DT_BF16 = 1 };

// Error bits a kernel may raise in Control::error (sticky until the host
// clears it).
enum : unsigned {
  ERR_TIMEOUT = 1u,   // a bounded dependency wait ran out
  ERR_CAPACITY = 2u,  // more row tiles than the tables were sized for
};

// Rows of one expert handled by one tile task of the streaming ("skinny") path.
constexpr int SKINNY_MT = 64;
// Widths of one wave task: gate/up task = 32 gate + 32 up weight rows,
// down task = 64 weight rows.
constexpr int G1_NB = 2;  // 16-wide column blocks per gate/up wave task
constexpr int G2_NB = 4;  // 16-wide column blocks per down wave task
// Output columns summed by one combine task.
constexpr int COMBINE_COLS = 256;
constexpr int ROUTER_TOK = 8;    // streaming variant: tokens per router dot task
constexpr int ROUTER_EXP = 8;    // streaming variant: experts per router dot task
constexpr int DOT16_KC = 256;    // streaming variant, matrix-core router: k per LDS stage
constexpr int SCAN_LDS_WORDS = 1024;  // mask words (experts x 64-token words) the small-batch scan keeps in LDS
constexpr int EARLY_MAX_TOKENS = 384;  // batches up to this size may take their gate/up weights before the routing is known
constexpr int MAX_EXPERTS = 256;  // experts are spread 64 per wave register slot
constexpr int MAX_TOPK = 32;

// Dependency counters and the ticket dispenser, one 128-byte line each so that
// pollers of one counter do not queue behind atomics on another. Everything
// except `error` and `launches` is zero before a launch and is returned to zero
// by the last worker to leave.
struct alignas(128) ControlLine {
  unsigned v;
  unsigned pad[31];
};
struct Control {
  ControlLine ticket;       // next task number
  ControlLine router_done;  // tokens whose routing is final
  ControlLine perm_done;    // scatter tasks finished
  ControlLine g2_done;      // down-projection tasks finished
  ControlLine exit_count;   // workers that have left the loop
  ControlLine n_mtiles;     // row tiles produced by the scan
  ControlLine error;        // sticky error bits
  ControlLine launches;     // completed launches (diagnostic)
  ControlLine xq[8];        // tiled variant: per-XCD ticket counters of the GEMM tasks
  ControlLine cticket;      // tiled variant: combine tickets
  ControlLine scan_done;    // tiled variant: per-expert scan tasks finished
};

// Phase flags, one line per workgroup: the worker that completes a phase
// writes every workgroup's copy, so waiting workers poll a line nobody else
// touches instead of queueing on one address.
// FLAG_ROUTED (streaming variant, early mode): every token's top-k entries are final.
enum : int { FLAG_SCAN = 0, FLAG_PERM = 1, FLAG_G2 = 2, FLAG_ROUTED = 3 };
struct alignas(128) WgFlags {
  unsigned f[32];
};

struct TileDesc {  // one row tile: `rows` consecutive permuted rows of one expert
  int expert;
  int row0;
  int rows;
  int shared;  // streaming variant: the expert has other row tiles, which read the same weights
};

// One record per executed task when tracing is on (times: 100 MHz wall clock).
struct TraceRec {
  unsigned ticket;
  unsigned kind;    // 0 router dot, 1 scan, 2 scatter, 3 gate/up, 4 down, 5 combine, 6 select
  unsigned worker;  // workgroup * waves_per_group + wave
  unsigned aux;     // task-specific (row tile, token ...)
  long long t_fetch;  // before the ticket was drawn
  long long t_ready;  // dependencies satisfied, work starts
  long long t_end;    // work finished and signalled
  long long pad;
};

struct Params {
  int T, E, H, K, I;
  int W;          // 64-bit mask words per expert (row stride of `masks`)
  int n_workers;  // waves (skinny kernel) taking tickets
  int max_mtiles;
  long long spin_limit;  // bound on one dependency wait, 100 MHz ticks

  const void* tokens;  // [T,H]: what the router and the gate/up projection read (the caller's rows, or their RMSNorm)
  const void* residual;  // [T,H] rows added to the output (the caller's rows), or null
  const void* gate;    // [E,H]
  const void* ffn1;    // [E,2I,H]  rows 0..I-1 gate proj, I..2I-1 up proj
  const void* ffn2;    // [E,H,I]
  const float* bias;   // [E] or null
  // Optional re-laid-out copies of the expert weights for the streaming variant
  // (null: read the caller's layout). One gate/up or down wave task reads its
  // slice front to back: [expert][column block][k-step][weight block][lane][16 B].
  const void* ffn1_packed;
  const void* ffn2_packed;
  void* out;           // [T,H], may alias tokens

  int* topk_idx;              // [T,K]
  float* topk_w;              // [T,K]
  unsigned long long* masks;  // [E,W] bit t of word t/64: token t selected the expert
  int* word_prefix;           // [E,W] rows of the expert before word w
  int* expert_count;          // [E]
  int* expert_offset;         // [E+1]
  int* perm;                  // [T*K] permuted row -> t*K+slot
  float* row_w;               // [T*K] gate weight of the permuted row
  TileDesc* mtiles;           // [max_mtiles]
  void* h;                    // [T*K, I] SwiGLU output, layer dtype
  float* y;                   // [T*K, H] weighted down-projection rows, by t*K+slot
  Control* ctl;
  WgFlags* wgflags;                // [n_groups]
  ControlLine* g1_done;            // [max_mtiles] gate/up tasks finished per row tile
  unsigned long long* cand;        // [T,E] router candidate keys
  unsigned* tok_arrive;            // [T] expert groups of the token whose keys are in
  int n_groups;                    // workgroups in the grid
  int fuse_scatter;                // 1: the scan task also writes the permutation
  int early;                       // 1, 2: row tile e belongs to expert e (empty or not), so gate/up tasks are
                                   //    handed out at launch and fetch their first weights under the routing
  int dot16;                       // 1 (streaming variant, bf16): the logit chains run on the matrix core, 16 tokens x
                                   //    16 experts per workgroup, on the first workgroups before they take tickets
  // What the last worker out needs when a launch has raised an error bit: it fills `out`
  // with NaN, returns the workspace's leading zero_words 32-bit words (counters, flags,
  // masks; `ctl` is the workspace's first byte) to zero, and adds the bits to *host_error
  // (pinned host memory the host reads without waiting for the stream; may be null).
  unsigned* host_error;
  unsigned zero_words;
  int elem_bytes;     // of tokens / out: 2 or 4
  TraceRec* trace;    // null unless tracing; indexed by ticket
  unsigned trace_cap;
};

// How device code reaches the launch parameters. A kernel parameter whose address
// is passed to a function is copied to the wave's private memory first, and every
// field read in a task then goes through the vector memory pipeline, behind the
// weight loads. A kernel that defines FMOE_PARAMS_IN_KERNARG before including
// this header reads them in place in the kernel-argument segment instead
// (constant address space): a field costs a scalar load that the scalar cache
// serves. Both kernels do.
#if defined(__HIP_DEVICE_COMPILE__) && defined(FMOE_PARAMS_IN_KERNARG)
typedef const __attribute__((address_space(4))) Params& ParamsRef;
#else
typedef const Params& ParamsRef;
#endif

}  // namespace fmoe
