// Persistent MoE kernel, tiled ("fat") variant for gfx950: the shape for
// batches where an expert sees hundreds of rows (prefill) and the layer is
// bound by MFMA throughput, bf16 only.
//
// One workgroup of 8 waves per CU (two per SIMD) draws workgroup-wide task
// tickets from the same kind of counter as the streaming variant; tasks depend
// only on tasks with smaller tickets. Stages (ticket order):
//   router   32 tokens x all experts: logits in the oracle's summation order
//            as a chain of f32 matrix instructions (four waves multiply, four
//            waves load through LDS), then top-k / softmax
//   scan     one wave per expert: counts and running prefixes of its mask
//            words; then one short task: offsets and the 256-row tile table
//   scatter  32 tokens: permuted row of every (token, slot)
//   gate/up  (row tile, 128 h columns): 256x256 MFMA tile, gate and up
//            columns side by side so that SiLU(gate)*up happens in registers
//   down     (row tile, 256 output columns): same tile, weighted bf16 rows to y
//   combine  8 tokens: out = sum over slots of y
// GEMM tile: 256 token rows x 256 weight rows, K stepped by 32 through four LDS
// stages that are filled straight from global memory; each wave owns 128
// weight rows x 64 token rows of it as 4x2 MFMA 32x32x16 blocks, 128
// accumulator registers. Weight rows are the MFMA "A" operand so that a lane
// ends up with runs of 4 consecutive output columns of one token row.
//
// Replaces, for this regime, the reference's moeKernel
// (src/hip/kernel/moeKernel.h:37-107) and its TILE_M=1 GEMV tiles
// (src/hip/kernel/tasks/internal/gemmImpl/basicGemmTileImpl.h:14-94).
#include <type_traits>

#define FMOE_PARAMS_IN_KERNARG 1
#include "moe_device.h"

namespace fmoe {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int TM = 256;            // token rows per tile
constexpr int TN = 256;            // weight rows per tile
constexpr int TK = 32;             // k per LDS stage (one 64-byte row slice)
constexpr int STAGES = 4;          // LDS stages in flight
constexpr int STAGE_BYTES = (TM + TN) * TK * 2;  // 32 KiB: weight rows, then token rows
constexpr int T_THREADS = 512;
constexpr int WAVES = T_THREADS / 64;  // two per SIMD: one wave's loads and LDS reads hide behind the other's MFMAs
constexpr int WJ = 16 / WAVES;         // 32-row token blocks per wave (each wave: 128 weight rows x 32*WJ token rows)
constexpr int LQ = 16 / WAVES;         // 16-row loads per operand, stage and wave
constexpr int G1_COLS = TN / 2;    // h columns per gate/up task
constexpr int RT_TOK = 32;         // tokens per router / scatter task
constexpr int CMB_TOK = 8;         // tokens per combine task

constexpr int TILE_LDS_BYTES = STAGES * STAGE_BYTES;  // 131072
constexpr int ROUTER_LDS_BYTES = 4 * 24576 + RT_TOK * MAX_EXPERTS * 4 + WAVES * MAX_TOPK * 8;
// Tall row tiles: an expert's last 1..TALL_EXTRA rows join its last full tile instead of
// costing a pass of their own over the expert's weights.
constexpr int TALL_EXTRA = 64;
constexpr int TALL_TM = TM + TALL_EXTRA;                       // 320 token rows
constexpr int TALL_STAGE_BYTES = (TN + TALL_TM) * TK * 2;      // 36 KiB: weight rows, then token rows
constexpr int TALL_LDS_BYTES = STAGES * TALL_STAGE_BYTES;      // 147456
constexpr int HT_ROWS = TALL_TM;                               // rows a row tile owns in h
constexpr int TILED_LDS_BYTES_0 = TILE_LDS_BYTES > ROUTER_LDS_BYTES ? TILE_LDS_BYTES : ROUTER_LDS_BYTES;
constexpr int TILED_LDS_BYTES = TILED_LDS_BYTES_0 > TALL_LDS_BYTES ? TILED_LDS_BYTES_0 : TALL_LDS_BYTES;

extern __shared__ __align__(16) unsigned char lds_raw[];

// ---------------------------------------------------------- workgroup helpers
// Values that are the same in every lane but that the compiler cannot prove so
// (they come through a struct reference): pin them to scalar registers, so
// loops and branches on them stay scalar.
__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
template <typename T>
__device__ __forceinline__ T* uni(T* ptr) {
  const unsigned long long v = reinterpret_cast<unsigned long long>(ptr);
  const unsigned lo = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(v));
  const unsigned hi = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(v >> 32));
  return reinterpret_cast<T*>((static_cast<unsigned long long>(hi) << 32) | lo);
}

struct WgShared {  // small static LDS block
  unsigned ticket;
  unsigned next;
  unsigned ok;
  unsigned flag[4];
};

// Thread 0 waits (bounded) for *p >= target; every thread learns the outcome.
__device__ __forceinline__ bool wg_wait_ge(ParamsRef p, const unsigned* ptr, unsigned target,
                                           WgShared* sh) {
  if (threadIdx.x == 0) {
    unsigned ok = 1u;
    if (ld_relaxed(ptr) < target) {
      const long long t0 = wall_clock64();
      unsigned spins = 0;
      while (ld_relaxed(ptr) < target) {
        if ((++spins & 31u) == 0u && ld_relaxed(&p.ctl->error.v) != 0u) {
          ok = 0u;
          break;
        }
        if (wall_clock64() - t0 > p.spin_limit) {
          or_relaxed(&p.ctl->error.v, ERR_TIMEOUT);
          ok = 0u;
          break;
        }
        __builtin_amdgcn_s_sleep(16);
      }
    }
    sh->ok = ok;
  }
  __syncthreads();
  const bool ok = sh->ok != 0u;
  __syncthreads();
  fence_acquire();
  return ok;
}

__device__ __forceinline__ bool wg_wait_flag(ParamsRef p, int which, WgShared* sh) {
  if (sh->flag[which] != 0u) return true;  // seen before by this workgroup
  const bool ok = wg_wait_ge(p, &p.wgflags[blockIdx.x].f[which], 1u, sh);
  if (ok && threadIdx.x == 0) sh->flag[which] = 1u;
  __syncthreads();
  return ok;
}

// All threads' stores have completed, then one thread bumps the counter. Tile
// data (h, y) is written through to device-coherent memory, so completion is
// all a reader on another XCD needs (WRITEBACK adds an agent-scope release for
// data written with ordinary cached stores; no task does that at present).
// Readers of h and y use ordinary loads: every cache line of them has a single
// writer and is not read before it is final, so no reader can hold a stale copy.
template <bool WRITEBACK>
__device__ __forceinline__ unsigned wg_arrive(unsigned* counter, WgShared* sh) {
  fence_release();
  __syncthreads();
  if (threadIdx.x == 0) {
    if (WRITEBACK) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    sh->ticket = add_relaxed(counter, 1u);
  }
  __syncthreads();
  const unsigned old = sh->ticket;
  __syncthreads();
  return old;
}

// The same, and the workgroup's next ticket from `queue` in the same trip to
// memory: thread 0 sends both atomics before it looks at either result.
__device__ __forceinline__ unsigned wg_arrive_and_draw(unsigned* counter, unsigned* queue,
                                                       unsigned& next, WgShared* sh) {
  fence_release();
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned old = add_relaxed(counter, 1u);
    const unsigned nxt = add_relaxed(queue, 1u);
    sh->ticket = old;
    sh->next = nxt;
  }
  __syncthreads();
  const unsigned old = sh->ticket;
  next = sh->next;
  __syncthreads();
  return old;
}

__device__ __forceinline__ void wg_broadcast_flag(ParamsRef p, int which) {
  const int n = p.n_groups;
  WgFlags* flags = p.wgflags;
  for (int g = threadIdx.x; g < n; g += blockDim.x) st_relaxed(&flags[g].f[which], 1u);
}

// ------------------------------------------------- direct-to-LDS load helpers
#define FMOE_G1 __attribute__((address_space(1)))
#define FMOE_L3 __attribute__((address_space(3)))

__device__ __forceinline__ f32x16 mma32(const uint4& a, const uint4& b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                 __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// wait until at most N of this wave's vector-memory operations are outstanding
// (they complete in order); nothing else is waited for
template <int N>
__device__ __forceinline__ void wait_vm() {
  __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// One wave-wide 16-byte-per-lane load from global memory straight into LDS:
// lane l's 16 bytes from base + off land at LDS byte address lds_addr + 16*l.
// Written as assembly so that the compiler does not order LDS reads of other
// stages behind it; completion is tracked by hand with wait_vm.
__device__ __forceinline__ void load_to_lds(unsigned off, const unsigned char* base, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(off), "s"(base), "s"(lds_addr)
               : "memory");
}


// --------------------------------------------------------------------- router
// Logits as in test/singleGPU/cpp/moe/reference/refGemm.h:21-24: one chain per
// output, k ascending, one rounding per step. The chain runs on the matrix
// core: V_MFMA_F32_32X32X2_F32 adds its two products to the accumulator one
// after the other in k order (checked bit for bit against a CPU fmaf chain; so
// do 16X16X1 and 16X16X4), and a product of two bf16 values is exact in float,
// so every step is the oracle's acc = fmaf(x, w, acc). A dependent chain of
// these instructions runs at the matrix core's full rate (64 cycles each).
// Waves 0..3 carry 32 tokens x 32 experts each, one wave per SIMD; waves 4..7
// are the loaders: they bring the 32 token rows and
// 128 expert rows in, 64 k at a time, with coalesced direct-to-LDS loads, four
// stages deep. Stage rows are 144 bytes (128 of data, 16 of padding), so the
// 16-byte reads of 16 rows at one k fall into different banks and every read
// address is a per-lane base plus an immediate. (One LDS read costs a wave
// about 22 cycles of issue whatever its width, hence 16-byte reads.)
// Then selection as in refTopk.h:36-58 / refMoeGate.h:27-30.
constexpr int RT_ROW_BYTES = 144;
constexpr int RT_LOADS = 6;                       // loads per loader wave and stage
constexpr int RT_STAGE_BYTES = 4 * RT_LOADS * 1024;  // 24 KiB
constexpr int RT_TOK_LOADS = (RT_TOK * 9 + 63) / 64; // loads that hold token rows
constexpr int RT_EXP_BASE = RT_TOK_LOADS * 1024;     // byte offset of the expert rows in a stage
constexpr int RT_STAGES = 4;
static_assert(RT_EXP_BASE + 128 * RT_ROW_BYTES <= RT_STAGE_BYTES, "router stage too small");

__device__ __noinline__ void tiled_router_task(ParamsRef pv, int blk) {
  ParamsRef p = uniform_params(pv);
  const int T = uni(p.T), E = uni(p.E), H = uni(p.H);
  const unsigned char* tokens = uni(reinterpret_cast<const unsigned char*>(p.tokens));
  const unsigned char* gate = uni(reinterpret_cast<const unsigned char*>(p.gate));
  const float* bias = uni(p.bias);
  unsigned* keys = reinterpret_cast<unsigned*>(lds_raw + RT_STAGES * RT_STAGE_BYTES);  // [RT_TOK][MAX_EXPERTS] ordered logits
  double* sel = reinterpret_cast<double*>(keys + RT_TOK * MAX_EXPERTS);  // WAVES x MAX_TOPK
  const unsigned lds_addr = uni(static_cast<unsigned>(
      reinterpret_cast<size_t>((FMOE_L3 unsigned char*)lds_raw)));
  const int tid = threadIdx.x;
  const int wave = uni(tid >> 6), lane = tid & 63;
  const bool loader = wave >= 4;
  const int t0 = uni(blk) * RT_TOK;
  const int nsteps = H >> 6;

  for (int e0 = 0; e0 < E; e0 += 128) {
    // loader: load ld = 6*w + i fills the 64 16-byte slots from slot 64*ld on. Loads
    // 0..4 hold the token rows, loads 5..23 the expert rows (from byte RT_EXP_BASE);
    // within a region slot g is position g % 9 of row g / 9 (position 8 is padding,
    // slots past the last row repeat it).
    unsigned goff[RT_LOADS];
#pragma unroll
    for (int i = 0; i < RT_LOADS; ++i) {
      const int ld = (wave & 3) * RT_LOADS + i;  // uniform
      const bool tok = ld < RT_TOK_LOADS;
      const int g = (tok ? ld : ld - RT_TOK_LOADS) * 64 + lane;
      const int row = min(g / 9, (tok ? RT_TOK : 128) - 1);
      const int pos = min(g % 9, 7);
      const int grow = tok ? min(t0 + row, T - 1) : min(e0 + row, E - 1);
      goff[i] = static_cast<unsigned>(grow) * static_cast<unsigned>(H * 2) + pos * 16;
    }
    auto issue = [&](int step) {
      const int src = min(step, nsteps - 1);  // past the end: refill with the last step (never read)
      const unsigned st = lds_addr + (step & (RT_STAGES - 1)) * RT_STAGE_BYTES +
                          ((wave & 3) * RT_LOADS) * 1024;
#pragma unroll
      for (int i = 0; i < RT_LOADS; ++i) {
        const bool tok = (wave & 3) * RT_LOADS + i < RT_TOK_LOADS;
        load_to_lds(goff[i], (tok ? tokens : gate) + static_cast<size_t>(src) * 128, st + i * 1024);
      }
    };
    // consumer: wave w multiplies the 32 token rows with expert rows 32*w .. 32*w+31.
    // Lane l: row l % 32 of both; V_MFMA_F32_32X32X2_F32 takes k = 2*s + l/32 from it,
    // i.e. the low or the high half of 32-bit word s of the row: the byte permute
    // moves that half into the upper 16 bits of a zero word, which makes the float.
    const int r32 = lane & 31, kh = lane >> 5;
    const unsigned pick = kh ? 0x07060C0Cu : 0x05040C0Cu;
    const unsigned char* xptr = lds_raw + r32 * RT_ROW_BYTES;
    const unsigned char* wptr = lds_raw + RT_EXP_BASE + ((wave & 3) * 32 + r32) * RT_ROW_BYTES;
    f32x16 acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.0f;

    // Operands of half a stage: four 16-byte chunks (8 k each) of both rows.
    struct Half {
      uint4 a[4], w[4];
    };
    auto read_half = [&](Half& h, int stage, int hf) {
      const int so = (stage & (RT_STAGES - 1)) * RT_STAGE_BYTES + hf * 64;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        h.a[c] = *reinterpret_cast<const uint4*>(xptr + so + c * 16);
        h.w[c] = *reinterpret_cast<const uint4*>(wptr + so + c * 16);
      }
    };
    // The 16 MFMAs of one half, and between them the reads of another half: one pair
    // of reads after every fourth MFMA. A read costs the wave about 20 cycles of
    // issue, which fits in the 64 cycles the next (dependent) MFMA has to wait anyway;
    // the scheduling barriers keep the compiler from moving the reads to the end.
    auto chain_and_read = [&](const Half& h, Half& nx, int stage, int hf) {
      const int so = (stage & (RT_STAGES - 1)) * RT_STAGE_BYTES + hf * 64;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const unsigned xw[4] = {h.a[c].x, h.a[c].y, h.a[c].z, h.a[c].w};
        const unsigned ww[4] = {h.w[c].x, h.w[c].y, h.w[c].z, h.w[c].w};
#pragma unroll
        for (int m = 0; m < 4; ++m)
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(
              __uint_as_float(__builtin_amdgcn_perm(xw[m], 0u, pick)),
              __uint_as_float(__builtin_amdgcn_perm(ww[m], 0u, pick)), acc, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        nx.a[c] = *reinterpret_cast<const uint4*>(xptr + so + c * 16);
        nx.w[c] = *reinterpret_cast<const uint4*>(wptr + so + c * 16);
        __builtin_amdgcn_sched_barrier(0);
      }
    };

    // Loaders and consumers run separate loops with the same number of barriers:
    // barrier s (in the middle of step s) means "stage s+1 is in, nobody reads
    // stage s any more".
    if (loader) {
      issue(0);
      issue(1);
      issue(2);
      issue(3);
      wait_vm<3 * RT_LOADS>();
      __builtin_amdgcn_s_barrier();  // stage 0 is in
      for (int s = 0; s < nsteps; ++s) {
        wait_vm<2 * RT_LOADS>();  // stage s+1 is in; s+2 and s+3 may be in flight
        __builtin_amdgcn_s_barrier();
        issue(s + RT_STAGES);     // into the stage every consumer has just left
      }
    } else {
      Half h0, h1;
      __builtin_amdgcn_s_barrier();  // stage 0 is in
      asm volatile("" ::: "memory");
      read_half(h0, 0, 0);
      for (int s = 0; s < nsteps; ++s) {
        chain_and_read(h0, h1, s, 1);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // this wave no longer reads stage s
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // past the last stage this reads the stage the loaders refilled with the last
        // step's data again; the values are never used
        chain_and_read(h1, h0, s + 1, 0);
      }
    }
    if (loader) wait_vm<0>();       // nothing may land in a stage after this slab
    __builtin_amdgcn_s_barrier();   // the stages may be refilled for the next slab
    asm volatile("" ::: "memory");
    if (!loader) {
      // acc[r] of lane l: token 8*(r/4) + 4*(l/32) + r%4, expert e0 + 32*w + l%32
      const int e = e0 + (wave & 3) * 32 + r32;
      const float bv = (bias != nullptr && e < E) ? as_global(bias)[e] : 0.0f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float v = acc[r];
        if (bias != nullptr) v = __fadd_rn(v, bv);
        if (e < MAX_EXPERTS)
          keys[(8 * (r >> 2) + 4 * kh + (r & 3)) * MAX_EXPERTS + e] = ordered_bits(v, e < E);
      }
    }
  }
  __syncthreads();
  // selection: the tokens are dealt out over all waves
  double* lex = sel + wave * MAX_TOPK;
  for (int i = 0; i < RT_TOK / WAVES; ++i) {
    const int tl = wave * (RT_TOK / WAVES) + i;
    const int t = t0 + tl;
    if (t < T) {
      unsigned val[MAX_EXPERTS / 64];
#pragma unroll
      for (int j = 0; j < MAX_EXPERTS / 64; ++j) {
        const int e = lane + 64 * j;
        val[j] = e < E ? keys[tl * MAX_EXPERTS + e] : 0u;
      }
      router_select_max(p, t, val, lex);
    }
  }
}

// The same for 16 tokens, used while that still gives every workgroup at most one
// router task (T <= 16 x workgroups): with 32-token tasks half of the CUs or more
// would sit through the router idle. The chains run on V_MFMA_F32_16X16X4_F32
// (which also adds its products in k order, one rounding each): wave w carries
// the 16 tokens x experts 16w..16w+15 of the slab. All eight waves load: 64 k of
// the 16 token rows and the 128 expert rows per stage, rows 144 bytes apart as
// above. Lane l multiplies row l % 16 of both operands at k = 4*s + l/16: of the
// eight bf16 a 16-byte read brings, elements l/16 and 4 + l/16, each moved into
// the upper half of a zero word by one byte permute.
constexpr int RT16_TOK = 16;
__device__ __forceinline__ void load_to_lds_addr(const unsigned char* addr, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :
               : "v"(addr), "s"(lds_addr)
               : "memory");
}

__device__ __noinline__ void tiled_router16_task(ParamsRef pv, int blk) {
  ParamsRef p = uniform_params(pv);
  const int T = uni(p.T), E = uni(p.E), H = uni(p.H);
  const unsigned char* tokens = uni(reinterpret_cast<const unsigned char*>(p.tokens));
  const unsigned char* gate = uni(reinterpret_cast<const unsigned char*>(p.gate));
  const float* bias = uni(p.bias);
  unsigned* keys = reinterpret_cast<unsigned*>(lds_raw + RT_STAGES * RT_STAGE_BYTES);  // [RT16_TOK][MAX_EXPERTS]
  double* sel = reinterpret_cast<double*>(keys + RT_TOK * MAX_EXPERTS);                // WAVES x MAX_TOPK
  const unsigned lds_addr = uni(static_cast<unsigned>(
      reinterpret_cast<size_t>((FMOE_L3 unsigned char*)lds_raw)));
  const int tid = threadIdx.x;
  const int wave = uni(tid >> 6), lane = tid & 63;
  const int t0 = uni(blk) * RT16_TOK;
  const int nsteps = H >> 6;
  // slot g of a stage (16 bytes): position g % 9 of row g / 9 (position 8 is padding);
  // rows 0..15 are the tokens, 16..143 the experts of the slab; slots past the last row repeat it
  constexpr int NL = 3;  // loads per wave and stage: 1536 slots >= 144 rows x 9
  constexpr int NROWS = RT16_TOK + 128;
  static_assert(NROWS * 9 <= WAVES * NL * 64 && WAVES * NL * 1024 == RT_STAGE_BYTES, "router stage");
  const int r16 = lane & 15, kq = lane >> 4;
  const unsigned pick = kq == 0 ? 0x01000C0Cu : kq == 1 ? 0x03020C0Cu : kq == 2 ? 0x05040C0Cu : 0x07060C0Cu;
  const int xoff = r16 * RT_ROW_BYTES;
  const int woff = (RT16_TOK + 16 * wave + r16) * RT_ROW_BYTES;
  for (int e0 = 0; e0 < E; e0 += 128) {
    const unsigned char* src[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int g = (wave * NL + i) * 64 + lane;
      const int row = min(g / 9, NROWS - 1);
      const int pos = min(g % 9, 7);
      const unsigned char* base =
          row < RT16_TOK ? tokens + static_cast<size_t>(min(t0 + row, T - 1)) * H * 2
                         : gate + static_cast<size_t>(min(e0 + row - RT16_TOK, E - 1)) * H * 2;
      src[i] = base + pos * 16;
    }
    auto issue = [&](int step) {  // past the last step: the last one again, into a stage nobody reads
      const size_t koff = static_cast<size_t>(min(step, nsteps - 1)) * 128;
      const unsigned st = lds_addr + (step & (RT_STAGES - 1)) * RT_STAGE_BYTES + wave * (NL * 1024);
#pragma unroll
      for (int i = 0; i < NL; ++i) load_to_lds_addr(src[i] + koff, st + i * 1024);
    };
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
    // Operands of half a stage (32 k): four 16-byte chunks of both rows. While the 8
    // matrix instructions of one half run, the next half is read, one chunk of both
    // rows after each pair; the scheduling barriers keep the reads from being
    // gathered in front of their first use, where their latency would be exposed.
    struct Half {
      uint4 a[4], w[4];
    };
    auto read_chunk = [&](Half& h, const unsigned char* hb, int c4) {
      h.a[c4] = *reinterpret_cast<const uint4*>(hb + xoff + 16 * c4);
      h.w[c4] = *reinterpret_cast<const uint4*>(hb + woff + 16 * c4);
    };
    auto chain_and_read = [&](const Half& h, Half& nx, const unsigned char* nb) {
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) {
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(
            __uint_as_float(__builtin_amdgcn_perm(h.a[c4].y, h.a[c4].x, pick)),
            __uint_as_float(__builtin_amdgcn_perm(h.w[c4].y, h.w[c4].x, pick)), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(
            __uint_as_float(__builtin_amdgcn_perm(h.a[c4].w, h.a[c4].z, pick)),
            __uint_as_float(__builtin_amdgcn_perm(h.w[c4].w, h.w[c4].z, pick)), acc, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        read_chunk(nx, nb, c4);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
#pragma unroll
    for (int st = 0; st < RT_STAGES; ++st) issue(st);
    wait_vm<(RT_STAGES - 1) * NL>();
    __builtin_amdgcn_s_barrier();  // stage 0 is in
    asm volatile("" ::: "memory");
    Half h0, h1;
#pragma unroll
    for (int c4 = 0; c4 < 4; ++c4) read_chunk(h0, lds_raw, c4);
    for (int st = 0; st < nsteps; ++st) {
      chain_and_read(h0, h1, lds_raw + (st & (RT_STAGES - 1)) * RT_STAGE_BYTES + 64);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // this wave no longer reads stage st
      wait_vm<(RT_STAGES - 2) * NL>();                    // its loads of stage st+1 are in
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      issue(st + RT_STAGES);
      // after the last step this reads a stage that is being refilled; the values are never used
      chain_and_read(h1, h0, lds_raw + ((st + 1) & (RT_STAGES - 1)) * RT_STAGE_BYTES);
    }
    wait_vm<0>();                  // nothing may land in a stage after this slab
    __builtin_amdgcn_s_barrier();  // the stages may be refilled for the next slab
    asm volatile("" ::: "memory");
    // acc[v] of lane l: token 4*(l/16) + v, expert e0 + 16*wave + l%16
    const int e = e0 + 16 * wave + r16;
    const float bv = (bias != nullptr && e < E) ? as_global(bias)[e] : 0.0f;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      float x = acc[v];
      if (bias != nullptr) x = __fadd_rn(x, bv);
      if (e < MAX_EXPERTS) keys[(4 * kq + v) * MAX_EXPERTS + e] = ordered_bits(x, e < E);
    }
  }
  __syncthreads();
  // selection: two tokens per wave
  double* lex = sel + wave * MAX_TOPK;
  for (int i = 0; i < RT16_TOK / WAVES; ++i) {
    const int tl = wave * (RT16_TOK / WAVES) + i;
    const int t = t0 + tl;
    if (t < T) {
      unsigned val[MAX_EXPERTS / 64];
#pragma unroll
      for (int j = 0; j < MAX_EXPERTS / 64; ++j) {
        const int e = lane + 64 * j;
        val[j] = e < E ? keys[tl * MAX_EXPERTS + e] : 0u;
      }
      router_select_max(p, t, val, lex);
    }
  }
}

// ----------------------------------------------------------------------- scan
// Same tables as the streaming variant's scan, in two steps. Expert scan: one
// wave per expert walks the expert's mask words 64 at a time and writes the
// running count in front of every word (word_prefix) and the expert's total.
// Final scan: one wave turns the totals into row offsets and the row-tile table.
constexpr int SCAN_EXPERTS = T_THREADS / 64;  // experts per expert-scan task

__device__ __noinline__ void tiled_expert_scan_task(ParamsRef pv, int blk) {
  ParamsRef p = uniform_params(pv);
  const int E = uni(p.E), W = uni(p.W), T = uni(p.T);
  const unsigned long long* masks = uni(p.masks);
  int* word_prefix = uni(p.word_prefix);
  int* expert_count = uni(p.expert_count);
  const int lane = threadIdx.x & 63;
  const int e = uni(blk) * SCAN_EXPERTS + uni(threadIdx.x >> 6);
  if (e >= E) return;
  const int wact = (T + 63) >> 6;
  int base = 0;
  for (int w0 = 0; w0 < wact; w0 += 64) {
    const int w = w0 + lane;
    const int c = w < wact ? __popcll(ldc(&masks[static_cast<size_t>(e) * W + w])) : 0;
    const int incl = wave_inclusive_scan(c);
    if (w < wact) stc(&word_prefix[static_cast<size_t>(e) * W + w], base + incl - c);
    base += __shfl(incl, 63, 64);
  }
  if (lane == 0) stc(&expert_count[e], base);
}

__device__ __noinline__ void tiled_scan_task(ParamsRef pv) {
  ParamsRef p = uniform_params(pv);
  const RouteTables r = route_tables(p);
  const int tid = threadIdx.x;
  if (tid < 64) {
    const int lane = tid;
    const int epl = (r.E + 63) >> 6;
    int base = 0, tile_base = 0;
    for (int j = 0; j < epl; ++j) {
      const int e = lane + 64 * j;
      const int c = e < r.E ? ldc(&r.expert_count[e]) : 0;
      const int incl = wave_inclusive_scan(c);
      const int off = base + incl - c;
      // Tiles of up to TALL_TM rows where that saves passes over the expert's weights
      // (a tall tile costs about an eighth more than one of TM rows): tiles keep TM
      // rows as long as the rest still fits the remaining tiles at TALL_TM each.
      const int nt_norm = (c + TM - 1) / TM, nt_tall = (c + TALL_TM - 1) / TALL_TM;
      const int nt = nt_tall * 9 < nt_norm * 8 ? nt_tall : nt_norm;
      const int tincl = wave_inclusive_scan(nt);
      const int toff = tile_base + tincl - nt;
      if (e < r.E) {
        stc(&r.expert_offset[e], off);
        int done = 0;
        for (int i = 0; i < nt; ++i) {
          const int left = c - done;
          const int tr = max(min(TM, left), left - TALL_TM * (nt - 1 - i));
          if (toff + i < r.max_mtiles) {
            stc16(&r.mtiles[toff + i],
                  make_uint4(static_cast<unsigned>(e), static_cast<unsigned>(off + done),
                             static_cast<unsigned>(tr), 0u));
          }
          done += tr;
        }
      }
      base += __shfl(incl, 63, 64);
      tile_base += __shfl(tincl, 63, 64);
    }
    if (lane == 0) {
      stc(&r.expert_offset[r.E], base);
      if (tile_base > r.max_mtiles) {
        or_relaxed(&p.ctl->error.v, ERR_CAPACITY);
        tile_base = 0;
      }
      stc(&p.ctl->n_mtiles.v, static_cast<unsigned>(tile_base));
    }
  }
  fence_release();
  __syncthreads();
  wg_broadcast_flag(p, FLAG_SCAN);
}

__device__ void tiled_scatter_task(ParamsRef p, int blk) {
  const RouteTables r = route_tables(p);
  const int i0 = blk * RT_TOK * r.K;
  const int n = min(RT_TOK * r.K, r.T * r.K - i0);
  for (int i = threadIdx.x; i < n; i += T_THREADS) scatter_entry(r, i0 + i);
}

// -------------------------------------------------------------- the GEMM tile
// Operands go HBM/L2 -> LDS directly (global_load_lds_dwordx4: lane l's 16
// bytes land at LDS base + 16*l, from any global address), four stages of 32
// k deep, so no register staging, no LDS write instructions and almost no VALU
// work in the loop. A wave issues in order: every LDS read (about 20 cycles)
// and every direct-to-LDS load it issues delays its own next MFMA, which is
// why two waves share a SIMD here: one multiplies while the other issues.
//
// LDS stage layout: rows of 64 bytes (32 bf16), unpadded, weight rows 0..255
// then token rows 0..255. Row R keeps its four 16-byte chunks permuted: chunk C
// sits at position C ^ ((R >> 2) & 3), so the 16 rows a quarter-wave reads
// together (256 bytes, all 64 banks) fall in 16 different 16-byte bank groups.
// One wave-wide load fills 16 rows; lane l loads the chunk that belongs at
// position l & 3 of row l >> 2.
// Weights come either from the caller's row-major matrices (64 bytes of each of
// 16 rows per load) or, when the launcher keeps the packed copy, from that: the
// streaming variant's layout holds every 16-row block of a k-step as one
// contiguous 1 KiB run [chunk 0..3][row 0..15][16 B], which a load fetches as
// eight whole cache lines. Measured with these loads on all CUs and four
// workgroups per XCD sharing a tile: 40 us per 2 MiB tile from 1 KiB runs, 50 us
// from 64-byte row segments 4096 bytes apart (all hits: 20 against 35 us). The
// block keeps that order in LDS; the fragment reads below allow for it.
struct TileRows {
  const unsigned char* wbase[LQ];  // uniform: where this wave's weight load q starts at k-step 0
  const unsigned char* tbase;      // uniform: tokens, or this tile's h rows
  unsigned wkstride;               // uniform: bytes from one k-step's weights to the next
  unsigned tkstride;               // uniform: the same for the token rows
  bool wpacked;                    // uniform: weight blocks are 1 KiB runs
  bool tpacked;                    // uniform: so are the token blocks (the down projection's h rows)
  unsigned woff[LQ];               // byte offset of this lane's 16 bytes of weight load q
  unsigned toff[LQ];               // token stage: this lane's chunk of stage row wave*16*LQ+q*16+(lane>>2)
};
static_assert(G1_NB == 2 && G2_NB == 4, "the tiled variant reads the packed copy as 32+32-row and 64-row tasks");


struct Frags {
  uint4 a[4];   // weight blocks
  uint4 b[WJ];  // token blocks
};

// Interleave hint for one half k-step: the 4 + WJ LDS reads spread evenly
// between the 4 * WJ matrix instructions.
__device__ __forceinline__ void interleave_reads_and_mfma() {
  constexpr int PER = (4 * WJ) / (4 + WJ);
#pragma unroll
  for (int n = 0; n < 4 + WJ; ++n) {
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);    // DS read
    __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);  // MFMA
  }
}

// acc[i][j] (+)= W-block i (32 weight rows) x token-block j (32 token rows).
// wblk[i]: first weight row of block i inside the weight stage; tokens of this
// wave start at tok0. JMAX: token blocks of this wave that are computed.
// Every wave loads its share of the weight rows of each stage whatever its
// JMAX; TOKL: it also loads its 32 token rows (false when they all lie past the
// tile's end: those stage rows then keep whatever they held, and feed only
// output rows that the epilogue drops).
template <int JMAX, bool TOKL>
__device__ __forceinline__ void tile_gemm_j(const TileRows& rows, int ksteps, const int (&wblk)[4],
                                            int tok0, f32x16 (&acc)[4][WJ]) {
  constexpr int NLQ = TOKL ? 2 * LQ : LQ;  // this wave's loads per stage
  const int lane = threadIdx.x & 63, wave = uni(threadIdx.x >> 6);
  const int r32 = lane & 31, kq = lane >> 5;
  const unsigned char* lds = lds_raw;
  const unsigned lds_addr = uni(static_cast<unsigned>(
      reinterpret_cast<size_t>((FMOE_L3 unsigned char*)lds_raw)));

  // load q (0..LQ-1: weight rows, LQ..2*LQ-1: token rows) of this wave's loads
  // of k-step ks into stage ks % STAGES
  auto issue_one = [&](int ks, int q) {
    const int src = ks;
    const unsigned st = lds_addr + (ks & (STAGES - 1)) * STAGE_BYTES + wave * (LQ * 1024);
    if (q < LQ) {
      load_to_lds(rows.woff[q], rows.wbase[q] + static_cast<size_t>(src) * rows.wkstride, st + q * 1024);
    } else {
      load_to_lds(rows.toff[q - LQ], rows.tbase + static_cast<size_t>(src) * rows.tkstride,
                  st + TN * TK * 2 + (q - LQ) * 1024);
    }
  };
  auto issue = [&](int ks) {
#pragma unroll
    for (int q = 0; q < NLQ; ++q) issue_one(ks, q);
  };

  // per-lane read offsets: row r32 of a block, chunk kk*2+kq at its permuted position
  const int swz = (r32 >> 2) & 3;
  const int rd0 = r32 * 64 + ((kq ^ swz) << 4);        // kk = 0
  const int rd1 = r32 * 64 + (((kq ^ swz) ^ 2) << 4);  // kk = 1

  // packed weight blocks: row r32 of a 32-row block is row r32 % 16 of its 16-row
  // block r32 / 16, chunk C of it at ((C * 16) + row) * 16
  const int ra0 = rows.wpacked ? (r32 >> 4) * 1024 + ((kq * 16 + (r32 & 15)) << 4) : rd0;
  const int ra1 = rows.wpacked ? (r32 >> 4) * 1024 + (((2 + kq) * 16 + (r32 & 15)) << 4) : rd1;
  auto read_a = [&](Frags& f, int ks, int kk, int i) {
    const unsigned char* st = lds + (ks & (STAGES - 1)) * STAGE_BYTES + (kk == 0 ? ra0 : ra1);
    if (JMAX > 0) f.a[i] = *reinterpret_cast<const uint4*>(st + wblk[i] * 64);
  };
  const int pk0 = (r32 >> 4) * 1024 + ((kq * 16 + (r32 & 15)) << 4);
  const int pk1 = (r32 >> 4) * 1024 + (((2 + kq) * 16 + (r32 & 15)) << 4);
  const int rb0 = rows.tpacked ? pk0 : rd0;
  const int rb1 = rows.tpacked ? pk1 : rd1;
  auto read_b = [&](Frags& f, int ks, int kk, int j) {
    const unsigned char* st = lds + (ks & (STAGES - 1)) * STAGE_BYTES + (kk == 0 ? rb0 : rb1);
    if (j < JMAX) f.b[j] = *reinterpret_cast<const uint4*>(st + TN * TK * 2 + (tok0 + j * 32) * 64);
  };
  auto read = [&](Frags& f, int ks, int kk) {
#pragma unroll
    for (int i = 0; i < 4; ++i) read_a(f, ks, kk, i);
#pragma unroll
    for (int j = 0; j < WJ; ++j) read_b(f, ks, kk, j);
  };
  auto mfma_block = [&](const Frags& f, int j) {
    if (j < JMAX) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[i][j] = mma32(f.a[i], f.b[j], acc[i][j]);
      }
    }
  };

  // k-step ks: fragments of its first half are in f0 on entry. While the first
  // half multiplies, the second half is read; while the second half multiplies,
  // the next stage is confirmed, the stage just finished is refilled, and the
  // next step's first half is read — loads and reads spread between the matrix
  // instructions. PENDING: loads of later stages that may still be in flight
  // when stage ks+1 has to be complete (2 * LQ per stage).
  Frags f0, f1;
  auto step = [&](int ks, auto pending_tag, auto refill_tag, auto last_tag) {
    constexpr int PENDING = decltype(pending_tag)::value;
    constexpr int REFILL = decltype(refill_tag)::value;  // 1: refill with stage ks+STAGES
    constexpr bool LAST = decltype(last_tag)::value;
    read(f1, ks, 1);
#pragma unroll
    for (int j = 0; j < WJ; ++j) mfma_block(f0, j);
    interleave_reads_and_mfma();
    __builtin_amdgcn_sched_barrier(0);
    if (!LAST) {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // nobody still reads stage ks after the barrier
      wait_vm<PENDING>();
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
#pragma unroll
      for (int g = 0; g < WJ; ++g) {
        mfma_block(f1, g);
        __builtin_amdgcn_sched_barrier(0);
        if (REFILL == 1) {
          if (2 * g < NLQ) issue_one(ks + STAGES, 2 * g);
          if (2 * g + 1 < NLQ) issue_one(ks + STAGES, 2 * g + 1);
        }

#pragma unroll
        for (int i = g * (4 / WJ); i < (g + 1) * (4 / WJ); ++i) read_a(f0, ks + 1, 0, i);
        read_b(f0, ks + 1, 0, g);
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
#pragma unroll
      for (int j = 0; j < WJ; ++j) mfma_block(f1, j);
    }
  };
  using I0 = std::integral_constant<int, 0>;
  using I8 = std::integral_constant<int, NLQ>;       // one later stage in flight
  using I16 = std::integral_constant<int, 2 * NLQ>;  // two later stages in flight

  using R0 = std::integral_constant<int, 0>;
  using R1 = std::integral_constant<int, 1>;
#pragma unroll
  for (int s = 0; s < STAGES; ++s) issue(s);  // ksteps >= STAGES for every admitted shape
  wait_vm<3 * NLQ>();
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  read(f0, 0, 0);
  int ks = 0;
  for (; ks + STAGES < ksteps; ++ks) step(ks, I16{}, R1{}, std::false_type{});
  step(ks++, I16{}, R0{}, std::false_type{});
  step(ks++, I8{}, R0{}, std::false_type{});
  step(ks++, I0{}, R0{}, std::false_type{});
  step(ks, I0{}, R0{}, std::true_type{});
  __syncthreads();  // the stages are free for the epilogue
}

// jmax is the same for the whole wave: one straight-line loop body per value.
// Rounding it up is safe: rows past the tile's end are clamped copies whose
// results the epilogue drops.
__device__ __forceinline__ void tile_gemm(const TileRows& rows, int ksteps, const int (&wblk)[4],
                                          int tok0, int jmax, bool tokl, f32x16 (&acc)[4][WJ]) {
  if (tokl) {
    if (jmax > WJ / 2) {
      tile_gemm_j<WJ, true>(rows, ksteps, wblk, tok0, acc);
    } else if (jmax > 0) {
      tile_gemm_j<WJ / 2, true>(rows, ksteps, wblk, tok0, acc);
    } else {
      tile_gemm_j<0, true>(rows, ksteps, wblk, tok0, acc);
    }
  } else {
    if (jmax > WJ / 2) {
      tile_gemm_j<WJ, false>(rows, ksteps, wblk, tok0, acc);
    } else if (jmax > 0) {
      tile_gemm_j<WJ / 2, false>(rows, ksteps, wblk, tok0, acc);
    } else {
      tile_gemm_j<0, false>(rows, ksteps, wblk, tok0, acc);
    }
  }
}

// The chunk lane `lane` of wave `wave` loads for stage row wave*16*LQ + q*16 + (lane >> 2):
// position lane & 3 of that row holds chunk (lane & 3) ^ ((row >> 2) & 3).
__device__ __forceinline__ int stage_row(int q) {
  return (threadIdx.x >> 6) * (16 * LQ) + q * 16 + ((threadIdx.x & 63) >> 2);
}
__device__ __forceinline__ unsigned stage_chunk_bytes(int row) {
  return static_cast<unsigned>(((threadIdx.x & 3) ^ ((row >> 2) & 3)) << 4);
}

// h of the tiled variant: row tile m owns HT_ROWS rows x I, stored the way the down
// projection's loads want them: [k-step of 32 columns][16-row block][chunk 0..3][row 0..15][16 B],
// so a block of a k-step is one 1 KiB run.
__device__ __forceinline__ size_t tiled_h_tile_bytes(int I) { return static_cast<size_t>(HT_ROWS) * I * 2; }

// gate/up: h[row, n0 .. n0+128) for one row tile
// (test/singleGPU/cpp/moe/reference/refExpertFFN1.h:51-65).
__device__ __noinline__ void tiled_gateup_task(ParamsRef pv, const TileDesc& tile_in, int m, int nblk) {
  ParamsRef p = uniform_params(pv);
  const int H = uni(p.H), I = uni(p.I), K = uni(p.K);
  TileDesc tile;
  tile.expert = uni(tile_in.expert);
  tile.row0 = uni(tile_in.row0);
  tile.rows = uni(tile_in.rows);
  const int n0 = uni(nblk) * G1_COLS;
  const unsigned short* w13 = uni(reinterpret_cast<const unsigned short*>(p.ffn1)) +
                              static_cast<size_t>(tile.expert) * 2 * I * H;
  TileRows rows;
  rows.wpacked = uni(p.ffn1_packed != nullptr ? 1 : 0) != 0;
  rows.wkstride = rows.wpacked ? 4096u : static_cast<unsigned>(TK * 2);
  rows.tkstride = static_cast<unsigned>(TK * 2);
  rows.tpacked = false;
  rows.tbase = uni(reinterpret_cast<const unsigned char*>(p.tokens));
#pragma unroll
  for (int q = 0; q < LQ; ++q) {
    const int row = stage_row(q);
    if (rows.wpacked) {
      // stage block B (16 rows): gate blocks 0..7, up blocks 8..15; the packed task
      // of 32 h columns holds gate blocks 0,1 and up blocks 2,3 of every k-step
      const int B = uni(static_cast<int>(threadIdx.x >> 6)) * LQ + q;
      const int half = B >> 3, b8 = B & 7;
      const size_t task = static_cast<size_t>(tile.expert) * (I / 32) + (n0 / 32 + (b8 >> 1));
      rows.wbase[q] = uni(reinterpret_cast<const unsigned char*>(p.ffn1_packed)) +
                      task * (static_cast<size_t>(H / 32) * 4096) + (2 * half + (b8 & 1)) * 1024;
      rows.woff[q] = (threadIdx.x & 63) * 16;
    } else {
      // weight stage rows 0..127: gate rows n0+row, 128..255: up rows I+n0+(row-128)
      const int wrow = row < G1_COLS ? n0 + row : I + n0 + (row - G1_COLS);
      rows.wbase[q] = reinterpret_cast<const unsigned char*>(w13);
      rows.woff[q] = static_cast<unsigned>(wrow) * static_cast<unsigned>(H * 2) + stage_chunk_bytes(row);
    }
    const int tok = ldc(&p.perm[tile.row0 + min(row, tile.rows - 1)]) / K;
    rows.toff[q] = static_cast<unsigned>(tok) * static_cast<unsigned>(H * 2) + stage_chunk_bytes(row);
  }
  const int wave = uni(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int wn = wave & 1, wm = wave >> 1;
  const int wblk[4] = {wn * 64, wn * 64 + 32, G1_COLS + wn * 64, G1_COLS + wn * 64 + 32};
  const int tok0 = wm * (32 * WJ);
  const int jmax = uni(min(WJ, max(0, (tile.rows - tok0 + 31) / 32)));
  const bool tokl = wave * (16 * LQ) < tile.rows;  // some of the token rows this wave loads exist
  // this wave's 64 columns are k-steps (n0 + 64*wn)/32 and the next of the tile's h
  unsigned char* h = uni(reinterpret_cast<unsigned char*>(p.h)) + static_cast<size_t>(uni(m)) * tiled_h_tile_bytes(I) +
                     static_cast<size_t>((n0 + wn * 64) / 32) * (HT_ROWS * 64);
  f32x16 acc[4][WJ];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < WJ; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  tile_gemm(rows, H / TK, wblk, tok0, jmax, tokl, acc);

  // Epilogue through LDS (the stage buffers are free now): each wave turns its
  // 32-token x 64-column blocks into full 128-byte row segments of h. Nothing
  // here waits for a store.
  const int r32 = lane & 31, kq = lane >> 5;
  constexpr int SLD = 64 + 8;  // slab row stride, bf16 elements
  unsigned short* slab = reinterpret_cast<unsigned short*>(lds_raw) + wave * 32 * SLD;
#pragma unroll
  for (int j = 0; j < WJ; ++j) {
    if (j < jmax) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          float hv[4];
#pragma unroll
          for (int v = 0; v < 4; ++v)
            hv[v] = silu_mul_fast(acc[i][j][g4 * 4 + v], acc[i + 2][j][g4 * 4 + v]);
          uint2 pk;
          pk.x = pack_bf16(hv[0], hv[1]);
          pk.y = pack_bf16(hv[2], hv[3]);
          *reinterpret_cast<uint2*>(slab + r32 * SLD + i * 32 + g4 * 8 + kq * 4) = pk;
        }
      lds_wave_sync();
#pragma unroll
      for (int it = 0; it < 4; ++it) {
        // one 1 KiB run: k-step it / 2 of this wave's two, 16-row block it % 2 of this token block
        const int ksl = it >> 1, b16 = it & 1;
        const int rr = b16 * 16 + (lane & 15), cc = ksl * 32 + (lane >> 4) * 8;
        const int trow = tok0 + j * 32 + rr;
        const uint4 v = *reinterpret_cast<const uint4*>(slab + rr * SLD + cc);
        if (trow < tile.rows)
          st16_through(h + static_cast<size_t>(ksl) * (HT_ROWS * 64) + ((tok0 + j * 32) / 16 + b16) * 1024 + lane * 16, v);
      }
      lds_wave_sync();
    }
  }
}

// down: y[t*K+slot, n0 .. n0+256) = w * (h[row] . W2[e]^T)
// (refFullMoe.h:58-65, src/hip/kernel/tasks/ffn2Task.h:37-40).
__device__ __noinline__ void tiled_down_task(ParamsRef pv, const TileDesc& tile_in, int m, int nblk) {
  ParamsRef p = uniform_params(pv);
  const int H = uni(p.H), I = uni(p.I);
  TileDesc tile;
  tile.expert = uni(tile_in.expert);
  tile.row0 = uni(tile_in.row0);
  tile.rows = uni(tile_in.rows);
  const int n0 = uni(nblk) * TN;
  const unsigned short* w2 = uni(reinterpret_cast<const unsigned short*>(p.ffn2)) +
                             static_cast<size_t>(tile.expert) * H * I;
  TileRows rows;
  rows.tbase = uni(reinterpret_cast<const unsigned char*>(p.h)) + static_cast<size_t>(uni(m)) * tiled_h_tile_bytes(I);
  rows.tkstride = static_cast<unsigned>(HT_ROWS * 64);
  rows.tpacked = true;
  rows.wpacked = uni(p.ffn2_packed != nullptr ? 1 : 0) != 0;
  rows.wkstride = rows.wpacked ? 4096u : static_cast<unsigned>(TK * 2);
#pragma unroll
  for (int q = 0; q < LQ; ++q) {
    const int row = stage_row(q);
    if (rows.wpacked) {
      // stage block B (16 rows of W2): the packed task of 64 output columns holds its blocks 0..3
      const int B = uni(static_cast<int>(threadIdx.x >> 6)) * LQ + q;
      const size_t task = static_cast<size_t>(tile.expert) * (H / 64) + (n0 / 64 + (B >> 2));
      rows.wbase[q] = uni(reinterpret_cast<const unsigned char*>(p.ffn2_packed)) +
                      task * (static_cast<size_t>(I / 32) * 4096) + (B & 3) * 1024;
      rows.woff[q] = (threadIdx.x & 63) * 16;
    } else {
      rows.wbase[q] = reinterpret_cast<const unsigned char*>(w2);
      rows.woff[q] = static_cast<unsigned>(n0 + row) * static_cast<unsigned>(I * 2) + stage_chunk_bytes(row);
    }
    // token stage block wave*LQ + q is one run of the tile's h (rows past the tile's
    // end were never written; their products are dropped)
    rows.toff[q] = static_cast<unsigned>((uni(static_cast<int>(threadIdx.x >> 6)) * LQ + q) * 1024 + (threadIdx.x & 63) * 16);
  }
  const int wave = uni(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int wn = wave & 1, wm = wave >> 1;
  const int wblk[4] = {wn * 128, wn * 128 + 32, wn * 128 + 64, wn * 128 + 96};
  const int tok0 = wm * (32 * WJ);
  const int jmax = uni(min(WJ, max(0, (tile.rows - tok0 + 31) / 32)));
  const bool tokl = wave * (16 * LQ) < tile.rows;  // some of the token rows this wave loads exist
  const int r32 = lane & 31, kq = lane >> 5;
  // y rows are bf16 here: H values per (token, slot)
  unsigned short* y = uni(reinterpret_cast<unsigned short*>(p.y)) + n0 + wn * 128 + (lane & 15) * 8;
  // gate weight and destination row (token*K + slot) of this lane's row in each token block
  float roww[WJ];
  int dstrow[WJ];
  {
    const float* row_w = uni(p.row_w) + tile.row0;
    const int* perm = uni(p.perm) + tile.row0;
#pragma unroll
    for (int j = 0; j < WJ; ++j) {
      const int myrow = tok0 + j * 32 + r32;
      const bool valid = myrow < tile.rows;
      roww[j] = valid ? ldc(&row_w[myrow]) : 0.0f;
      dstrow[j] = valid ? ldc(&perm[myrow]) : -1;
    }
  }
  f32x16 acc[4][WJ];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < WJ; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  tile_gemm(rows, I / TK, wblk, tok0, jmax, tokl, acc);

  // Epilogue through LDS: 32-token x 128-column blocks become 256-byte row
  // segments of y (bf16), scaled by the row's gate weight, at the row's
  // (token, slot). Nothing here waits for a store.
  constexpr int SLD = 128 + 8;  // slab row stride, bf16 elements
  unsigned short* slab = reinterpret_cast<unsigned short*>(lds_raw) + wave * (32 * SLD);
#pragma unroll
  for (int j = 0; j < WJ; ++j) {
    if (j < jmax) {
      const float w = roww[j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          uint2 pk;
          pk.x = pack_bf16(acc[i][j][g4 * 4 + 0] * w, acc[i][j][g4 * 4 + 1] * w);
          pk.y = pack_bf16(acc[i][j][g4 * 4 + 2] * w, acc[i][j][g4 * 4 + 3] * w);
          *reinterpret_cast<uint2*>(slab + r32 * SLD + i * 32 + g4 * 8 + kq * 4) = pk;
        }
      lds_wave_sync();
#pragma unroll
      for (int it = 0; it < 8; ++it) {
        // each quarter-wave stores one row: rows 4*it .. 4*it+3
        const int q = lane >> 4;
        const int d0 = __builtin_amdgcn_readlane(dstrow[j], it * 4);
        const int d1 = __builtin_amdgcn_readlane(dstrow[j], it * 4 + 1);
        const int d2 = __builtin_amdgcn_readlane(dstrow[j], it * 4 + 2);
        const int d3 = __builtin_amdgcn_readlane(dstrow[j], it * 4 + 3);
        const int dst = q == 0 ? d0 : q == 1 ? d1 : q == 2 ? d2 : d3;
        const uint4 v = *reinterpret_cast<const uint4*>(slab + (it * 4 + q) * SLD + (lane & 15) * 8);
        if (dst >= 0) st16_through(y + static_cast<size_t>(dst) * H, v);
      }
      lds_wave_sync();
    }
  }
}

// ------------------------------------------------------------ tall row tiles
// A row tile of 257..320 rows (an expert's last full tile plus its short tail):
// one pass over the expert's weights instead of two. Waves are laid out 4 (64
// weight rows, two blocks) x 2 (160 token rows, five blocks): 160 accumulator
// registers per lane. A stage holds 256 weight rows and 320 token rows (36 KiB);
// every wave loads two weight blocks, and token blocks wave, wave + 8 and (waves
// 0..3) wave + 16 of the twenty 16-row blocks. Otherwise as tile_gemm_j.
struct TallRows {
  const unsigned char* wbase[LQ];
  const unsigned char* tbase;
  unsigned wkstride, tkstride;
  bool wpacked, tpacked;
  unsigned woff[LQ];
  unsigned toff[3];
};
struct TallFrags {
  uint4 a[2];  // weight blocks
  uint4 b[5];  // token blocks
};

// NTB: token blocks of this wave that are computed (4 or 5); NTL: its token loads per stage (2 or 3)
template <int NTB, int NTL>
__device__ __forceinline__ void tall_gemm(const TallRows& rows, int ksteps, const int (&wblk)[2], int tok0,
                                          f32x16 (&acc)[2][5]) {
  constexpr int NLD = LQ + NTL;  // this wave's loads per stage
  static_assert(LQ == 2 && NLD <= 5, "tall tiles are written for eight waves");
  const int lane = threadIdx.x & 63, wave = uni(threadIdx.x >> 6);
  const int r32 = lane & 31, kq = lane >> 5;
  const unsigned char* lds = lds_raw;
  const unsigned lds_addr = uni(static_cast<unsigned>(
      reinterpret_cast<size_t>((FMOE_L3 unsigned char*)lds_raw)));

  auto issue_one = [&](int ks, int q) {
    const unsigned st = lds_addr + (ks & (STAGES - 1)) * TALL_STAGE_BYTES;
    if (q < LQ) {
      load_to_lds(rows.woff[q], rows.wbase[q] + static_cast<size_t>(ks) * rows.wkstride,
                  st + (wave * LQ + q) * 1024);
    } else {
      load_to_lds(rows.toff[q - LQ], rows.tbase + static_cast<size_t>(ks) * rows.tkstride,
                  st + TN * TK * 2 + (wave + 8 * (q - LQ)) * 1024);
    }
  };
  auto issue = [&](int ks) {
#pragma unroll
    for (int q = 0; q < NLD; ++q) issue_one(ks, q);
  };

  const int swz = (r32 >> 2) & 3;
  const int rd0 = r32 * 64 + ((kq ^ swz) << 4);
  const int rd1 = r32 * 64 + (((kq ^ swz) ^ 2) << 4);
  const int pk0 = (r32 >> 4) * 1024 + ((kq * 16 + (r32 & 15)) << 4);
  const int pk1 = (r32 >> 4) * 1024 + (((2 + kq) * 16 + (r32 & 15)) << 4);
  const int ra0 = rows.wpacked ? pk0 : rd0, ra1 = rows.wpacked ? pk1 : rd1;
  const int rb0 = rows.tpacked ? pk0 : rd0, rb1 = rows.tpacked ? pk1 : rd1;
  auto read_a = [&](TallFrags& f, int ks, int kk, int i) {
    const unsigned char* st = lds + (ks & (STAGES - 1)) * TALL_STAGE_BYTES + (kk == 0 ? ra0 : ra1);
    f.a[i] = *reinterpret_cast<const uint4*>(st + wblk[i] * 64);
  };
  auto read_b = [&](TallFrags& f, int ks, int kk, int j) {
    const unsigned char* st = lds + (ks & (STAGES - 1)) * TALL_STAGE_BYTES + (kk == 0 ? rb0 : rb1);
    if (j < NTB) f.b[j] = *reinterpret_cast<const uint4*>(st + TN * TK * 2 + (tok0 + j * 32) * 64);
  };
  auto read = [&](TallFrags& f, int ks, int kk) {
#pragma unroll
    for (int i = 0; i < 2; ++i) read_a(f, ks, kk, i);
#pragma unroll
    for (int j = 0; j < 5; ++j) read_b(f, ks, kk, j);
  };
  auto mfma_block = [&](const TallFrags& f, int j) {
    if (j < NTB) {
#pragma unroll
      for (int i = 0; i < 2; ++i) acc[i][j] = mma32(f.a[i], f.b[j], acc[i][j]);
    }
  };

  TallFrags f0, f1;
  auto step = [&](int ks, auto pending_tag, auto refill_tag, auto last_tag) {
    constexpr int PENDING = decltype(pending_tag)::value;
    constexpr int REFILL = decltype(refill_tag)::value;
    constexpr bool LAST = decltype(last_tag)::value;
    read(f1, ks, 1);
#pragma unroll
    for (int j = 0; j < 5; ++j) mfma_block(f0, j);
#pragma unroll
    for (int n = 0; n < 2 + NTB; ++n) {  // the reads spread between the matrix instructions
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (!LAST) {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // nobody still reads stage ks after the barrier
      wait_vm<PENDING>();
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
#pragma unroll
      for (int g = 0; g < 5; ++g) {
        mfma_block(f1, g);
        __builtin_amdgcn_sched_barrier(0);
        if (REFILL == 1 && g < NLD) issue_one(ks + STAGES, g);
        if (g < 2) read_a(f0, ks + 1, 0, g);
        read_b(f0, ks + 1, 0, g);
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 5; ++j) mfma_block(f1, j);
    }
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, NLD>;
  using I2 = std::integral_constant<int, 2 * NLD>;
  using R0 = std::integral_constant<int, 0>;
  using R1 = std::integral_constant<int, 1>;
#pragma unroll
  for (int st = 0; st < STAGES; ++st) issue(st);
  wait_vm<3 * NLD>();
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  read(f0, 0, 0);
  int ks = 0;
  for (; ks + STAGES < ksteps; ++ks) step(ks, I2{}, R1{}, std::false_type{});
  step(ks++, I2{}, R0{}, std::false_type{});
  step(ks++, I1{}, R0{}, std::false_type{});
  step(ks++, I0{}, R0{}, std::false_type{});
  step(ks, I0{}, R0{}, std::true_type{});
  __syncthreads();  // the stages are free for the epilogue
}

// dispatch on the wave's position: waves 0..3 own token rows 0..159 (all five blocks live, three
// token loads), waves 4..7 rows 160..319 (four or five blocks, two loads)
__device__ __forceinline__ void tall_gemm_dispatch(const TallRows& rows, int ksteps, const int (&wblk)[2],
                                                   int tok0, int ntb, f32x16 (&acc)[2][5]) {
  if (uni(static_cast<int>(threadIdx.x >> 6)) < 4) {
    tall_gemm<5, 3>(rows, ksteps, wblk, tok0, acc);
  } else if (ntb > 4) {
    tall_gemm<5, 2>(rows, ksteps, wblk, tok0, acc);
  } else {
    tall_gemm<4, 2>(rows, ksteps, wblk, tok0, acc);
  }
}

// the 16-row token block L (0..19) this wave loads as its q-th token load, or -1
__device__ __forceinline__ int tall_token_block(int q) {
  const int L = static_cast<int>(threadIdx.x >> 6) + 8 * q;
  return L < TALL_TM / 16 ? L : -1;
}

__device__ __noinline__ void tall_gateup_task(ParamsRef pv, const TileDesc& tile_in, int m, int nblk) {
  ParamsRef p = uniform_params(pv);
  const int H = uni(p.H), I = uni(p.I), K = uni(p.K);
  TileDesc tile;
  tile.expert = uni(tile_in.expert);
  tile.row0 = uni(tile_in.row0);
  tile.rows = uni(tile_in.rows);
  const int n0 = uni(nblk) * G1_COLS;
  const int wave = uni(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const unsigned short* w13 = uni(reinterpret_cast<const unsigned short*>(p.ffn1)) +
                              static_cast<size_t>(tile.expert) * 2 * I * H;
  TallRows rows;
  rows.wpacked = uni(p.ffn1_packed != nullptr ? 1 : 0) != 0;
  rows.wkstride = rows.wpacked ? 4096u : static_cast<unsigned>(TK * 2);
  rows.tkstride = static_cast<unsigned>(TK * 2);
  rows.tpacked = false;
  rows.tbase = uni(reinterpret_cast<const unsigned char*>(p.tokens));
#pragma unroll
  for (int q = 0; q < LQ; ++q) {
    const int row = stage_row(q);
    if (rows.wpacked) {
      const int B = wave * LQ + q;
      const int half = B >> 3, b8 = B & 7;
      const size_t task = static_cast<size_t>(tile.expert) * (I / 32) + (n0 / 32 + (b8 >> 1));
      rows.wbase[q] = uni(reinterpret_cast<const unsigned char*>(p.ffn1_packed)) +
                      task * (static_cast<size_t>(H / 32) * 4096) + (2 * half + (b8 & 1)) * 1024;
      rows.woff[q] = lane * 16;
    } else {
      const int wrow = row < G1_COLS ? n0 + row : I + n0 + (row - G1_COLS);
      rows.wbase[q] = reinterpret_cast<const unsigned char*>(w13);
      rows.woff[q] = static_cast<unsigned>(wrow) * static_cast<unsigned>(H * 2) + stage_chunk_bytes(row);
    }
  }
#pragma unroll
  for (int q = 0; q < 3; ++q) {
    const int L = max(tall_token_block(q), 0);
    const int row = L * 16 + (lane >> 2);
    const int tok = ldc(&p.perm[tile.row0 + min(row, tile.rows - 1)]) / K;
    rows.toff[q] = static_cast<unsigned>(tok) * static_cast<unsigned>(H * 2) + stage_chunk_bytes(row);
  }
  const int wn = wave & 3, wm = wave >> 2;
  const int wblk[2] = {wn * 32, G1_COLS + wn * 32};  // 32 gate rows and the matching 32 up rows
  const int tok0 = wm * 160;
  const int ntb = uni(min(5, (tile.rows - tok0 + 31) / 32));
  // this wave's 32 columns are k-step (n0 + 32*wn)/32 of the tile's h
  unsigned char* h = uni(reinterpret_cast<unsigned char*>(p.h)) + static_cast<size_t>(uni(m)) * tiled_h_tile_bytes(I) +
                     static_cast<size_t>((n0 + wn * 32) / 32) * (HT_ROWS * 64);
  f32x16 acc[2][5];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 5; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  tall_gemm_dispatch(rows, H / TK, wblk, tok0, ntb, acc);

  const int r32 = lane & 31, kq = lane >> 5;
  constexpr int SLD = 32 + 8;  // slab row stride, bf16 elements
  unsigned short* slab = reinterpret_cast<unsigned short*>(lds_raw) + wave * 32 * SLD;
#pragma unroll
  for (int j = 0; j < 5; ++j) {
    if (j < ntb) {
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        float hv[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) hv[v] = silu_mul_fast(acc[0][j][g4 * 4 + v], acc[1][j][g4 * 4 + v]);
        uint2 pk;
        pk.x = pack_bf16(hv[0], hv[1]);
        pk.y = pack_bf16(hv[2], hv[3]);
        *reinterpret_cast<uint2*>(slab + r32 * SLD + g4 * 8 + kq * 4) = pk;
      }
      lds_wave_sync();
#pragma unroll
      for (int b16 = 0; b16 < 2; ++b16) {
        // one 1 KiB run: 16-row block b16 of this token block, chunk lane / 16 of row lane % 16
        const int rr = b16 * 16 + (lane & 15), cc = (lane >> 4) * 8;
        const int trow = tok0 + j * 32 + rr;
        const uint4 v = *reinterpret_cast<const uint4*>(slab + rr * SLD + cc);
        if (trow < tile.rows) st16_through(h + ((tok0 + j * 32) / 16 + b16) * 1024 + lane * 16, v);
      }
      lds_wave_sync();
    }
  }
}

__device__ __noinline__ void tall_down_task(ParamsRef pv, const TileDesc& tile_in, int m, int nblk) {
  ParamsRef p = uniform_params(pv);
  const int H = uni(p.H), I = uni(p.I);
  TileDesc tile;
  tile.expert = uni(tile_in.expert);
  tile.row0 = uni(tile_in.row0);
  tile.rows = uni(tile_in.rows);
  const int n0 = uni(nblk) * TN;
  const int wave = uni(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const unsigned short* w2 = uni(reinterpret_cast<const unsigned short*>(p.ffn2)) +
                             static_cast<size_t>(tile.expert) * H * I;
  TallRows rows;
  rows.tbase = uni(reinterpret_cast<const unsigned char*>(p.h)) + static_cast<size_t>(uni(m)) * tiled_h_tile_bytes(I);
  rows.tkstride = static_cast<unsigned>(HT_ROWS * 64);
  rows.tpacked = true;
  rows.wpacked = uni(p.ffn2_packed != nullptr ? 1 : 0) != 0;
  rows.wkstride = rows.wpacked ? 4096u : static_cast<unsigned>(TK * 2);
#pragma unroll
  for (int q = 0; q < LQ; ++q) {
    const int row = stage_row(q);
    if (rows.wpacked) {
      const int B = wave * LQ + q;
      const size_t task = static_cast<size_t>(tile.expert) * (H / 64) + (n0 / 64 + (B >> 2));
      rows.wbase[q] = uni(reinterpret_cast<const unsigned char*>(p.ffn2_packed)) +
                      task * (static_cast<size_t>(I / 32) * 4096) + (B & 3) * 1024;
      rows.woff[q] = lane * 16;
    } else {
      rows.wbase[q] = reinterpret_cast<const unsigned char*>(w2);
      rows.woff[q] = static_cast<unsigned>(n0 + row) * static_cast<unsigned>(I * 2) + stage_chunk_bytes(row);
    }
  }
#pragma unroll
  for (int q = 0; q < 3; ++q) rows.toff[q] = static_cast<unsigned>(max(tall_token_block(q), 0) * 1024 + lane * 16);
  const int wn = wave & 3, wm = wave >> 2;
  const int wblk[2] = {wn * 64, wn * 64 + 32};
  const int tok0 = wm * 160;
  const int ntb = uni(min(5, (tile.rows - tok0 + 31) / 32));
  const int r32 = lane & 31, kq = lane >> 5;
  unsigned short* y = uni(reinterpret_cast<unsigned short*>(p.y)) + n0 + wn * 64 + (lane & 7) * 8;
  float roww[5];
  int dstrow[5];
  {
    const float* row_w = uni(p.row_w) + tile.row0;
    const int* perm = uni(p.perm) + tile.row0;
#pragma unroll
    for (int j = 0; j < 5; ++j) {
      const int myrow = tok0 + j * 32 + r32;
      const bool valid = myrow < tile.rows;
      roww[j] = valid ? ldc(&row_w[myrow]) : 0.0f;
      dstrow[j] = valid ? ldc(&perm[myrow]) : -1;
    }
  }
  f32x16 acc[2][5];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 5; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  tall_gemm_dispatch(rows, I / TK, wblk, tok0, ntb, acc);

  constexpr int SLD = 64 + 8;  // slab row stride, bf16 elements
  unsigned short* slab = reinterpret_cast<unsigned short*>(lds_raw) + wave * (32 * SLD);
#pragma unroll
  for (int j = 0; j < 5; ++j) {
    if (j < ntb) {
      const float w = roww[j];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          uint2 pk;
          pk.x = pack_bf16(acc[i][j][g4 * 4 + 0] * w, acc[i][j][g4 * 4 + 1] * w);
          pk.y = pack_bf16(acc[i][j][g4 * 4 + 2] * w, acc[i][j][g4 * 4 + 3] * w);
          *reinterpret_cast<uint2*>(slab + r32 * SLD + i * 32 + g4 * 8 + kq * 4) = pk;
        }
      lds_wave_sync();
#pragma unroll
      for (int it = 0; it < 4; ++it) {
        // eight lanes store one row's 128 bytes: rows 8*it .. 8*it+7
        const int q = lane >> 3;
        int dst = -1;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
          const int d = __builtin_amdgcn_readlane(dstrow[j], it * 8 + r);
          dst = q == r ? d : dst;
        }
        const uint4 v = *reinterpret_cast<const uint4*>(slab + (it * 8 + q) * SLD + (lane & 7) * 8);
        if (dst >= 0) st16_through(y + static_cast<size_t>(dst) * H, v);
      }
      lds_wave_sync();
    }
  }
}


// combine: out[t] = sum over slots, in slot order, of y[t*K+slot]
// (refFullMoe.h:35,62-65).
__device__ __noinline__ void tiled_combine_task(ParamsRef pv, int blk) {
  ParamsRef p = uniform_params(pv);
  const int H = uni(p.H), K = uni(p.K), T = uni(p.T), E = uni(p.E), W = uni(p.W);
  unsigned short* out = uni(reinterpret_cast<unsigned short*>(p.out));
  const unsigned short* y = uni(reinterpret_cast<const unsigned short*>(p.y));
  const int* topk_idx = uni(p.topk_idx);
  unsigned long long* masks = uni(p.masks);
  const int tid = threadIdx.x;
  const int t0 = uni(blk) * CMB_TOK;
  const int ntok = min(CMB_TOK, T - t0);
  // which (token, slot) pairs of this task hold an expert: one load each
  unsigned char* flag = lds_raw;  // [CMB_TOK * MAX_TOPK]
  if (tid < ntok * K) flag[tid] = ldc(&topk_idx[static_cast<size_t>(t0) * K + tid]) >= 0 ? 1 : 0;
  __syncthreads();
  // one item = 8 columns of one token; the K row loads of an item are in flight together
  const int cpr = H >> 3;  // items per token
  for (int it = tid; it < ntok * cpr; it += T_THREADS) {
    const int tl = it / cpr, c = (it - tl * cpr) << 3;
    const int t = t0 + tl;
    unsigned valid = 0u;
    for (int k = 0; k < K; ++k) valid |= static_cast<unsigned>(flag[tl * K + k]) << k;
    const unsigned short* yrow = y + static_cast<size_t>(t) * K * H + c;
    float s[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) s[i] = 0.0f;
    for (int k0 = 0; k0 < K; k0 += 8) {
      uint4 v[8];
#pragma unroll
      for (int k = 0; k < 8; ++k)
        if (k0 + k < K) v[k] = ld16_once(yrow + static_cast<size_t>(k0 + k) * H);
#pragma unroll
      for (int k = 0; k < 8; ++k)
        if (k0 + k < K && ((valid >> (k0 + k)) & 1u)) {
          float f[8];
          unpack<BF16>(v[k], f);
#pragma unroll
          for (int i = 0; i < 8; ++i) s[i] += f[i];
        }
    }
    st16(out + static_cast<size_t>(t) * H + c,
         u32x4{pack_bf16(s[0], s[1]), pack_bf16(s[2], s[3]), pack_bf16(s[4], s[5]),
               pack_bf16(s[6], s[7])});
  }
  for (int tl = 0; tl < ntok; ++tl) {
    const int t = t0 + tl;
    if ((t & 63) == 0) {
      for (int e = tid; e < E; e += T_THREADS) stc(&masks[static_cast<size_t>(e) * W + (t >> 6)], 0ull);
    }
  }
  __syncthreads();  // flag[] is reused by the next task
}

// ---------------------------------------------------------------- worker loop
// Ticket layout. The prologue (router, scan, scatter) uses one global counter.
// The GEMM tasks are split into eight queues, one per XCD: queue x owns a
// contiguous eighth of the row-tile table (which is sorted by expert), first all
// its gate/up tasks (tile-major), then all its down tasks. A workgroup serves
// the queue of the XCD it runs on, so tasks that share a token tile or a weight
// tile run on CUs behind the same L2 at about the same time, and a tile's h
// rows are consumed where they were produced. A workgroup whose queue is empty
// steals from the next queue. Dependencies stay inside one queue and point to
// smaller tickets, so whoever holds them is already running. Combine tasks
// come from a last global counter once every queue is empty.
__device__ __forceinline__ int xcc_id() {
  // HW_REG_XCC_ID (20), bits 0..3
  return __builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & 7;
}

// The launch parameters are read in place and the task calls keep the local
// calling convention, as in the streaming variant (see its worker loop).
__global__ __launch_bounds__(T_THREADS) __attribute__((disable_tail_calls)) void moe_tiled_kernel(
    const Params params) {
  ParamsRef p = kernel_params();
  __shared__ WgShared sh;
  if (threadIdx.x == 0) {
    sh.ticket = 0u;
    sh.ok = 1u;
    sh.flag[0] = sh.flag[1] = sh.flag[2] = sh.flag[3] = 0u;
  }
  __syncthreads();
  Control* ctl = p.ctl;
  const unsigned T = static_cast<unsigned>(p.T);
  const unsigned n_sc = (T + RT_TOK - 1u) / RT_TOK;  // scatter tasks
  // router tasks: of 16 tokens while every workgroup still gets at most one
  const bool router16 = (T + RT16_TOK - 1u) / RT16_TOK <= gridDim.x;
  const unsigned n_rt = router16 ? (T + RT16_TOK - 1u) / RT16_TOK : n_sc;
  const unsigned n_es = (static_cast<unsigned>(p.E) + SCAN_EXPERTS - 1u) / SCAN_EXPERTS;
  const unsigned t_escan0 = n_rt;
  const unsigned t_scan = n_rt + n_es;
  const unsigned t_scatter0 = t_scan + 1u;
  const unsigned t_dyn0 = t_scatter0 + n_sc;
  const unsigned nt1 = static_cast<unsigned>(p.I / G1_COLS);
  const unsigned nt2 = static_cast<unsigned>(p.H / TN);
  const unsigned ncmb = (T + CMB_TOK - 1u) / CMB_TOK;
  const unsigned n_groups = gridDim.x;
  const int home = xcc_id();
  bool first = true, ok = true;

  auto trace = [&](unsigned id, unsigned kind, unsigned aux, long long t_fetch, long long t_ready) {
    if (p.trace && threadIdx.x == 0 && id < p.trace_cap) {
      const long long t_end = wall_clock64();
      TraceRec* r = p.trace + id;
      st16(r, u32x4{id, kind, blockIdx.x, aux});
      st16(reinterpret_cast<char*>(r) + 16,
           u32x4{static_cast<unsigned>(t_fetch), static_cast<unsigned>(t_fetch >> 32),
                 static_cast<unsigned>(t_ready), static_cast<unsigned>(t_ready >> 32)});
      const unsigned x0 = 0u, x1 = 0u;
      st16(reinterpret_cast<char*>(r) + 32,
           u32x4{static_cast<unsigned>(t_end), static_cast<unsigned>(t_end >> 32), x0, x1});
    }
  };

  // ---- prologue: router, scan, scatter from the global counter
  while (ok) {
    const long long t_fetch = p.trace ? wall_clock64() : 0;
    if (threadIdx.x == 0) sh.ticket = first ? blockIdx.x : n_groups + add_relaxed(&ctl->ticket.v, 1u);
    first = false;
    __syncthreads();
    const unsigned tk = sh.ticket;
    __syncthreads();
    if (tk >= t_dyn0) break;
    long long t_ready = 0;
    if (tk < n_rt) {
      if (p.trace) t_ready = wall_clock64();
      if (router16) {
        tiled_router16_task(p, static_cast<int>(tk));
      } else {
        tiled_router_task(p, static_cast<int>(tk));
      }
      wg_arrive<false>(&ctl->router_done.v, &sh);
      trace(tk, 0, tk, t_fetch, t_ready);
    } else if (tk < t_scan) {
      ok = wg_wait_ge(p, &ctl->router_done.v, n_rt, &sh);
      if (ok) {
        if (p.trace) t_ready = wall_clock64();
        tiled_expert_scan_task(p, static_cast<int>(tk - t_escan0));
        wg_arrive<false>(&ctl->scan_done.v, &sh);
        trace(tk, 6, tk - t_escan0, t_fetch, t_ready);
      }
    } else if (tk == t_scan) {
      ok = wg_wait_ge(p, &ctl->scan_done.v, n_es, &sh);
      if (ok) {
        if (p.trace) t_ready = wall_clock64();
        tiled_scan_task(p);
        trace(tk, 1, 0, t_fetch, t_ready);
      }
    } else {
      ok = wg_wait_flag(p, FLAG_SCAN, &sh);
      if (ok) {
        if (p.trace) t_ready = wall_clock64();
        tiled_scatter_task(p, static_cast<int>(tk - t_scatter0));
        if (wg_arrive<false>(&ctl->perm_done.v, &sh) == n_sc - 1u) wg_broadcast_flag(p, FLAG_PERM);
        trace(tk, 2, tk - t_scatter0, t_fetch, t_ready);
      }
    }
  }

  // ---- GEMM tasks from the per-XCD queues
  unsigned nm = 0, n2_total = 0;
  if (ok) ok = wg_wait_flag(p, FLAG_SCAN, &sh);
  if (ok) {
    nm = ldc(&ctl->n_mtiles.v);
    n2_total = nm * nt2;
    ok = wg_wait_flag(p, FLAG_PERM, &sh);
  }
  for (int hop = 0; ok && hop < 8; ++hop) {
    const unsigned q = static_cast<unsigned>((home + hop) & 7);
    const unsigned lo = nm * q / 8u, hi = nm * (q + 1u) / 8u;
    const unsigned tiles = hi - lo;
    const unsigned q1 = tiles * nt1, q2 = tiles * nt2;
    // the first ticket of a queue is drawn on its own, the others together with the
    // arrival of the task before
    if (threadIdx.x == 0) sh.ticket = add_relaxed(&ctl->xq[q].v, 1u);
    __syncthreads();
    unsigned j = sh.ticket;
    __syncthreads();
    while (ok) {
      const long long t_fetch = p.trace ? wall_clock64() : 0;
      if (j >= q1 + q2) break;
      long long t_ready = 0;
      if (j < q1) {
        const unsigned m = lo + j / nt1;
        if (p.trace) t_ready = wall_clock64();
        const TileDesc tile = ld_tile(&p.mtiles[m]);
        if (tile.rows > TM) {
          tall_gateup_task(p, tile, static_cast<int>(m), static_cast<int>(j % nt1));
        } else {
          tiled_gateup_task(p, tile, static_cast<int>(m), static_cast<int>(j % nt1));
        }
        const unsigned done = j;
        wg_arrive_and_draw(&p.g1_done[m].v, &ctl->xq[q].v, j, &sh);
        trace(t_dyn0 + lo * nt1 + done, 3, m, t_fetch, t_ready);
      } else {
        const unsigned jj = j - q1;
        const unsigned m = lo + jj / nt2;
        const TileDesc tile = ld_tile(&p.mtiles[m]);  // in flight while thread 0 looks at the counter
        ok = wg_wait_ge(p, &p.g1_done[m].v, nt1, &sh);
        if (ok) {
          if (p.trace) t_ready = wall_clock64();
          if (tile.rows > TM) {
            tall_down_task(p, tile, static_cast<int>(m), static_cast<int>(jj % nt2));
          } else {
            tiled_down_task(p, tile, static_cast<int>(m), static_cast<int>(jj % nt2));
          }
          if (wg_arrive_and_draw(&ctl->g2_done.v, &ctl->xq[q].v, j, &sh) == n2_total - 1u)
            wg_broadcast_flag(p, FLAG_G2);
          trace(t_dyn0 + nm * nt1 + lo * nt2 + jj, 4, m, t_fetch, t_ready);
        }
      }
    }
  }

  // ---- combine tasks from the last global counter
  if (ok && n2_total != 0u) ok = wg_wait_flag(p, FLAG_G2, &sh);
  while (ok) {
    const long long t_fetch = p.trace ? wall_clock64() : 0;
    if (threadIdx.x == 0) sh.ticket = add_relaxed(&ctl->cticket.v, 1u);
    __syncthreads();
    const unsigned c = sh.ticket;
    __syncthreads();
    if (c >= ncmb) break;
    const long long t_ready = p.trace ? wall_clock64() : 0;
    tiled_combine_task(p, static_cast<int>(c));
    trace(t_dyn0 + nm * (nt1 + nt2) + c, 5, c, t_fetch, t_ready);
  }

  // The last workgroup out returns every counter to zero for the next launch.
  __syncthreads();
  if (threadIdx.x == 0) sh.ok = (add_relaxed(&ctl->exit_count.v, 1u) == n_groups - 1u) ? 1u : 0u;
  __syncthreads();
  if (sh.ok) {
    const unsigned nmr = min(ldc(&ctl->n_mtiles.v), static_cast<unsigned>(p.max_mtiles));
    for (unsigned i = threadIdx.x; i < nmr; i += T_THREADS) stc(&p.g1_done[i].v, 0u);
    for (unsigned g = threadIdx.x; g < n_groups; g += T_THREADS) {
      stc(&p.wgflags[g].f[FLAG_SCAN], 0u);
      stc(&p.wgflags[g].f[FLAG_PERM], 0u);
      stc(&p.wgflags[g].f[FLAG_G2], 0u);
    }
    if (threadIdx.x < 8) stc(&ctl->xq[threadIdx.x].v, 0u);
    if (threadIdx.x == 0) {
      stc(&ctl->launches.v, ldc(&ctl->launches.v) + 1u);
      stc(&ctl->router_done.v, 0u);
      stc(&ctl->perm_done.v, 0u);
      stc(&ctl->g2_done.v, 0u);
      stc(&ctl->n_mtiles.v, 0u);
      stc(&ctl->exit_count.v, 0u);
      stc(&ctl->cticket.v, 0u);
      stc(&ctl->scan_done.v, 0u);
      stc(&ctl->ticket.v, 0u);
    }
  }
}

// Largest token count of the tiled variant: the launcher's capacity at top-1.
int tiled_max_tokens() { return 1 << 21; }

hipError_t launch_tiled_kernel(const Params& p, int grid, hipStream_t stream) {
  hipLaunchKernelGGL(moe_tiled_kernel, dim3(grid), dim3(T_THREADS), TILED_LDS_BYTES, stream, p);
  return hipGetLastError();
}

hipError_t prepare_tiled_kernel() {
  return hipFuncSetAttribute(reinterpret_cast<const void*>(moe_tiled_kernel),
                             hipFuncAttributeMaxDynamicSharedMemorySize, TILED_LDS_BYTES);
}

}  // namespace fmoe
