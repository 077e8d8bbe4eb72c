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
constexpr int MAX_EXPERTS = 256;  // experts are spread 64 per wave register slot
constexpr int MAX_TOPK = 32;

// Dependency counters and the ticket dispenser. Everything up to `error` is
// zero before a launch and is returned to zero by the last worker to leave.
struct Control {
  unsigned ticket;       // next task number
  unsigned router_done;  // router tasks finished
  unsigned scan_done;    // 1 once expert offsets and the tile table exist
  unsigned perm_done;    // scatter tasks finished
  unsigned g2_done;      // down-projection tasks finished
  unsigned exit_count;   // workers that have left the loop
  unsigned n_mtiles;     // row tiles produced by the scan
  unsigned reserved0;
  unsigned error;        // sticky error bits
  unsigned launches;     // completed launches (diagnostic)
  unsigned reserved1[6];
};

struct TileDesc {  // one row tile: `rows` consecutive permuted rows of one expert
  int expert;
  int row0;
  int rows;
  int pad;
};

struct Params {
  int T, E, H, K, I;
  int W;          // 64-bit mask words per expert (row stride of `masks`)
  int n_workers;  // waves (skinny kernel) taking tickets
  int max_mtiles;
  long long spin_limit;  // bound on one dependency wait, 100 MHz ticks

  const void* tokens;  // [T,H]
  const void* gate;    // [E,H]
  const void* ffn1;    // [E,2I,H]  rows 0..I-1 gate proj, I..2I-1 up proj
  const void* ffn2;    // [E,H,I]
  const float* bias;   // [E] or null
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
  unsigned* g1_done;  // [max_mtiles] gate/up tasks finished per row tile
};

}  // namespace fmoe
