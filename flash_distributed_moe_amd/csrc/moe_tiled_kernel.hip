// Persistent MoE kernel, tiled variant for gfx950: the shape for batches where an
// expert sees many rows (prefill) and the layer is bound by matrix throughput,
// bf16 only.
//
// One workgroup of 4 waves per CU (one per SIMD, each with the SIMD's whole
// register file) draws workgroup-wide task tickets from the same kind of counter
// as the streaming variant; tasks depend only on tasks with smaller tickets.
// Stages (ticket order):
//   router   16 tokens x all experts: logits in the oracle's summation order as
//            chains of f32 matrix instructions, then top-k / softmax
//   scan     one wave per expert: counts and running prefixes of its mask
//            words; then one short task: offsets and the row-tile table
//   scatter  32 tokens: permuted row of every (token, slot)
//   gate/up  (row tile, 128 h columns): 256 token rows x 256 weight rows, gate
//            and up rows side by side so that SiLU(gate)*up happens in registers
//   down     (row tile, 256 output columns): same tile, weighted bf16 rows to y
//   combine  8 tokens: out = sum over slots of y
// GEMM tile: up to 256 token rows x 256 weight rows, K stepped by 64 through two
// LDS stages that are filled straight from global memory in whole 128-byte
// lines; each wave owns 64 weight rows x all token rows of it as 2x8 MFMA
// 32x32x16 blocks, 256 accumulator registers. Weight rows are the MFMA "A"
// operand so that a lane ends up with runs of 4 consecutive output columns of
// one token row. A tile with fewer rows multiplies fewer token blocks, so its
// time follows its rows.
//
// Replaces, for this regime, the reference's moeKernel
// (src/hip/kernel/moeKernel.h:37-107) and its TILE_M=1 GEMV tiles
// (src/hip/kernel/tasks/internal/gemmImpl/basicGemmTileImpl.h:14-94).
#include <type_traits>

#define FMOE_PARAMS_IN_KERNARG 1
#include "moe_device.h"

namespace fmoe {

typedef float f32x16 __attribute__((ext_vector_type(16)));


constexpr int JT_MAX = 10;         // 32-row token blocks of the tallest row tile
constexpr int TM_MAX = 32 * JT_MAX;  // 320 token rows
constexpr int TN = 256;            // weight rows per tile
constexpr int KS = 64;             // k per LDS stage
constexpr int ROWB = KS * 2;       // bytes of a row per stage: one 128-byte line
constexpr int T_THREADS = 256;
constexpr int WAVES = T_THREADS / 64;  // one per SIMD
constexpr int NLD = 8;             // 8-row loads per wave, operand and stage
constexpr int G1_COLS = TN / 2;    // h columns per gate/up task
constexpr int RT_TOK = 32;         // tokens per scatter task
constexpr int CMB_TOK = 8;         // tokens per combine task

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
// core: V_MFMA_F32_16X16X4_F32 and V_MFMA_F32_32X32X2_F32 add their four / two
// products to the accumulator one after the other in k order (checked bit for bit
// against a CPU fmaf chain), and a product of two bf16 values is exact in float, so
// every step is the oracle's acc = fmaf(x, w, acc).
// A task is 16 or 32 tokens x a slab of 128 experts. With 16 tokens a wave carries two
// 16x16 chains (experts 16w..16w+15 and 64+16w..64+16w+15); with 32 tokens one 32x32
// chain (experts 32w..32w+31), which does the work of four 16x16 chains with half the
// operand reads and permutes per multiply-add, and in less time: with every CU on the
// float matrix core the chip holds ~56 cycles per 1024 multiply-adds in the 32x32 shape
// against ~70 in the 16x16 shape (32 nominal for both).
// All waves load: 64 k of the token rows and the 128 expert rows per stage,
// four stages deep, with coalesced direct-to-LDS loads. Stage rows are 144 bytes
// (128 of data, 16 of padding), so the 16-byte reads of 16 rows at one k fall
// into different banks. 16x16: lane l multiplies row l % 16 of both operands at
// k = 4*s + l/16: of the eight bf16 a 16-byte read brings, elements l/16 and
// 4 + l/16. 32x32: row l % 32 at k = 2*s + l/32: elements l/32, 2 + l/32, 4 + l/32,
// 6 + l/32. Each is moved into the upper half of a zero word by one byte permute.
// Then selection as in refTopk.h:36-58 / refMoeGate.h:27-30.
constexpr int RT16_TOK = 16;  // tokens of the small router task; the large one has twice as many
constexpr int RT_ROW_BYTES = 144;
constexpr int RT_STAGES = 4;
constexpr int RT_NL = 6;                                  // loads per wave and stage
constexpr int RT_STAGE_BYTES = WAVES * RT_NL * 1024;      // 24 KiB
constexpr int RT_NROWS = 2 * RT16_TOK + 128;
static_assert(RT_NROWS * 9 <= WAVES * RT_NL * 64, "router stage too small");
constexpr int ROUTER_LDS_BYTES = RT_STAGES * RT_STAGE_BYTES + 2 * RT16_TOK * MAX_EXPERTS * 4 + WAVES * MAX_TOPK * 8;

__device__ __forceinline__ void load_to_lds_addr(const unsigned char* addr, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :
               : "v"(addr), "s"(lds_addr)
               : "memory");
}

template <int NB>  // 1: 16 tokens, 16x16 chains; 2: 32 tokens, 32x32 chains
__device__ __noinline__ void tiled_router_task(ParamsRef pv, int blk) {
  constexpr int NTOK = NB * RT16_TOK;
  constexpr int NROWS = NTOK + 128;
  constexpr int NW = NB == 2 ? 1 : 2;  // expert rows a lane reads
  ParamsRef p = uniform_params(pv);
  const int T = uni(p.T), E = uni(p.E), H = uni(p.H);
  const unsigned char* tokens = uni(reinterpret_cast<const unsigned char*>(p.tokens));
  const unsigned char* gate = uni(reinterpret_cast<const unsigned char*>(p.gate));
  const float* bias = uni(p.bias);
  unsigned* keys = reinterpret_cast<unsigned*>(lds_raw + RT_STAGES * RT_STAGE_BYTES);  // [NTOK][MAX_EXPERTS]
  double* sel = reinterpret_cast<double*>(keys + NTOK * MAX_EXPERTS);              // WAVES x MAX_TOPK
  const unsigned lds_addr = uni(static_cast<unsigned>(
      reinterpret_cast<size_t>((FMOE_L3 unsigned char*)lds_raw)));
  const int tid = threadIdx.x;
  const int wave = uni(tid >> 6), lane = tid & 63;
  const int t0 = uni(blk) * NTOK;
  const int nsteps = H >> 6;
  // slot g of a stage (16 bytes): position g % 9 of row g / 9 (position 8 is padding);
  // rows 0..NTOK-1 are the tokens, the next 128 the experts of the slab; slots past the last row repeat it
  const int r16 = lane & 15, kq = lane >> 4;    // 16x16: row and k quarter
  const int r32 = lane & 31, kh = lane >> 5;    // 32x32: row and k half
  const unsigned pick = NB == 2 ? (kh == 0 ? 0x01000C0Cu : 0x03020C0Cu)
                                : (kq == 0   ? 0x01000C0Cu
                                   : kq == 1 ? 0x03020C0Cu
                                   : kq == 2 ? 0x05040C0Cu
                                             : 0x07060C0Cu);
  const int xoff = (NB == 2 ? r32 : r16) * RT_ROW_BYTES;
  const int woff0 = (NB == 2 ? NTOK + 32 * wave + r32 : NTOK + 16 * wave + r16) * RT_ROW_BYTES;
  const int woff1 = (NTOK + 64 + 16 * wave + r16) * RT_ROW_BYTES;  // 16x16 only
  for (int e0 = 0; e0 < E; e0 += 128) {
    const unsigned char* src[RT_NL];
#pragma unroll
    for (int i = 0; i < RT_NL; ++i) {
      const int g = (wave * RT_NL + i) * 64 + lane;
      const int row = min(g / 9, NROWS - 1);
      const int pos = min(g % 9, 7);
      const unsigned char* base =
          row < NTOK ? tokens + static_cast<size_t>(min(t0 + row, T - 1)) * H * 2
                     : gate + static_cast<size_t>(min(e0 + row - NTOK, E - 1)) * H * 2;
      src[i] = base + pos * 16;
    }
    auto issue = [&](int step) {  // past the last step: the last one again, into a stage nobody reads
      const size_t koff = static_cast<size_t>(min(step, nsteps - 1)) * 128;
      const unsigned st = lds_addr + (step & (RT_STAGES - 1)) * RT_STAGE_BYTES + wave * (RT_NL * 1024);
#pragma unroll
      for (int i = 0; i < RT_NL; ++i) load_to_lds_addr(src[i] + koff, st + i * 1024);
    };
    f32x4 acc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};  // 16x16
    f32x16 big;                                                               // 32x32
#pragma unroll
    for (int i = 0; i < 16; ++i) big[i] = 0.f;
    // Operands of half a stage (32 k): four 16-byte chunks of the token row and of the
    // expert rows. While the 16 matrix instructions of one half run, the next half is
    // read, one chunk of each row after every four; the scheduling barriers keep the
    // reads from being gathered in front of their first use.
    struct Half {
      uint4 a[4], w[NW][4];
    };
    auto read_chunk = [&](Half& h, const unsigned char* hb, int c4) {
      h.a[c4] = *reinterpret_cast<const uint4*>(hb + xoff + 16 * c4);
      h.w[0][c4] = *reinterpret_cast<const uint4*>(hb + woff0 + 16 * c4);
      if constexpr (NB == 1) h.w[1][c4] = *reinterpret_cast<const uint4*>(hb + woff1 + 16 * c4);
    };
    auto sel1 = [&](unsigned v) { return __uint_as_float(__builtin_amdgcn_perm(v, v, pick)); };
    auto chain_and_read = [&](const Half& h, Half& nx, const unsigned char* nb) {
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) {
        if constexpr (NB == 2) {
          big = __builtin_amdgcn_mfma_f32_32x32x2f32(sel1(h.a[c4].x), sel1(h.w[0][c4].x), big, 0, 0, 0);
          big = __builtin_amdgcn_mfma_f32_32x32x2f32(sel1(h.a[c4].y), sel1(h.w[0][c4].y), big, 0, 0, 0);
          big = __builtin_amdgcn_mfma_f32_32x32x2f32(sel1(h.a[c4].z), sel1(h.w[0][c4].z), big, 0, 0, 0);
          big = __builtin_amdgcn_mfma_f32_32x32x2f32(sel1(h.a[c4].w), sel1(h.w[0][c4].w), big, 0, 0, 0);
        } else {
          const float xl = __uint_as_float(__builtin_amdgcn_perm(h.a[c4].y, h.a[c4].x, pick));
          const float xh = __uint_as_float(__builtin_amdgcn_perm(h.a[c4].w, h.a[c4].z, pick));
#pragma unroll
          for (int j = 0; j < NW; ++j)
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                xl, __uint_as_float(__builtin_amdgcn_perm(h.w[j][c4].y, h.w[j][c4].x, pick)), acc[j], 0, 0, 0);
#pragma unroll
          for (int j = 0; j < NW; ++j)
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                xh, __uint_as_float(__builtin_amdgcn_perm(h.w[j][c4].w, h.w[j][c4].z, pick)), acc[j], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        read_chunk(nx, nb, c4);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
#pragma unroll
    for (int st = 0; st < RT_STAGES; ++st) issue(st);
    wait_vm<(RT_STAGES - 1) * RT_NL>();
    __builtin_amdgcn_s_barrier();  // stage 0 is in
    asm volatile("" ::: "memory");
    Half h0, h1;
#pragma unroll
    for (int c4 = 0; c4 < 4; ++c4) read_chunk(h0, lds_raw, c4);
    for (int st = 0; st < nsteps; ++st) {
      chain_and_read(h0, h1, lds_raw + (st & (RT_STAGES - 1)) * RT_STAGE_BYTES + 64);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // this wave no longer reads stage st
      wait_vm<(RT_STAGES - 2) * RT_NL>();                 // its loads of stage st+1 are in
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      issue(st + RT_STAGES);
      // after the last step this reads a stage that is being refilled; the values are never used
      chain_and_read(h1, h0, lds_raw + ((st + 1) & (RT_STAGES - 1)) * RT_STAGE_BYTES);
    }
    wait_vm<0>();                  // nothing may land in a stage after this slab
    __builtin_amdgcn_s_barrier();  // the stages may be refilled for the next slab
    asm volatile("" ::: "memory");
    if constexpr (NB == 2) {
      // big[i] of lane l: token 8*(i/4) + 4*(l/32) + i%4, expert e0 + 32*wave + l%32
      const int e = e0 + 32 * wave + r32;
      const float bv = (bias != nullptr && e < E) ? as_global(bias)[e] : 0.0f;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float x = bias != nullptr ? __fadd_rn(big[i], bv) : big[i];
        const int tl = 8 * (i >> 2) + 4 * kh + (i & 3);
        if (e < MAX_EXPERTS) keys[tl * MAX_EXPERTS + e] = ordered_bits(x, e < E);
      }
    } else {
      // acc[j][v] of lane l: token 4*(l/16) + v, expert e0 + 64*j + 16*wave + l%16
      const int ea = e0 + 16 * wave + r16, eb = ea + 64;
      const float bva = (bias != nullptr && ea < E) ? as_global(bias)[ea] : 0.0f;
      const float bvb = (bias != nullptr && eb < E) ? as_global(bias)[eb] : 0.0f;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        float xa = acc[0][v], xb = acc[1][v];
        if (bias != nullptr) {
          xa = __fadd_rn(xa, bva);
          xb = __fadd_rn(xb, bvb);
        }
        if (ea < MAX_EXPERTS) keys[(4 * kq + v) * MAX_EXPERTS + ea] = ordered_bits(xa, ea < E);
        if (eb < MAX_EXPERTS) keys[(4 * kq + v) * MAX_EXPERTS + eb] = ordered_bits(xb, eb < E);
      }
    }
  }
  __syncthreads();
  // selection: every wave takes its share of the tokens
  double* lex = sel + wave * MAX_TOPK;
  for (int i = 0; i < NTOK / WAVES; ++i) {
    const int tl = wave * (NTOK / WAVES) + i;
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
// Final scan: one wave turns the totals into row offsets and the row-tile table
// (an expert's rows in as few tiles of at most TM_MAX rows as possible, of equal size).
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
      // balanced tiles of at most TM_MAX rows, whole 32-row blocks
      const int nt = (c + TM_MAX - 1) / TM_MAX;
      const int per = nt > 0 ? ((c + nt - 1) / nt + 31) / 32 * 32 : 0;
      const int tincl = wave_inclusive_scan(nt);
      const int toff = tile_base + tincl - nt;
      if (e < r.E) {
        stc(&r.expert_offset[e], off);
        int done = 0;
        for (int i = 0; i < nt; ++i) {
          const int left = c - done;
          const int tr = min(per, left);
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
// Operands go HBM/L2 -> LDS directly (global_load_lds_dwordx4: lane l's 16 bytes
// land at LDS base + 16*l, from any global address), in stages of 64 k: one
// 128-byte line of every operand row, so every request uses whole cache lines
// whatever the row pitch. Two stages; no register staging, no LDS write
// instructions, almost no vector-ALU work in the loop.
//
// One wave per SIMD, each with 64 weight rows x all token rows of the tile:
// acc[2][JT] blocks of 32x32. The first 8 token blocks' accumulators fill the
// 256 accumulator registers a[0:255]; a tile of 257..320 rows (JT 9, 10) keeps
// the last blocks' in v[...]. Per 16 k a wave reads 2 weight and JT token
// fragments (16 bytes per lane each) for 2*JT matrix instructions. A tile's
// time follows its rows down to about 160; below that the 32 load round trips
// of its k-loop set it.
//
// LDS stage layout: rows of 128 bytes, unpadded, weight rows 0..255 then token
// rows. Row R keeps its eight 16-byte chunks permuted: chunk C sits at position
// C ^ ((R >> 1) & 7), so the 16 rows a quarter-wave reads together at one k fall
// into 16 different 16-byte bank groups. One wave-wide load fills 8 rows; lane
// l brings the chunk that belongs at position l & 7 of row l >> 3.
//
// The matrix instructions are written as assembly with the accumulator pinned
// to its register file: 256 accumulators fill a[0:255] exactly, and the
// compiler's own choice moved parts of them in and out of v[...] (it also
// chose the vector-register form of the instruction, which cannot reach a[...]).
// The first instruction of every accumulator takes the constant 0 as its
// addend, so nothing zeroes them.
template <bool INIT, bool IN_V>
__device__ __forceinline__ void mma32(const uint4& a, const uint4& b, f32x16& c) {
  typedef unsigned v4u __attribute__((ext_vector_type(4)));
  const v4u av = {a.x, a.y, a.z, a.w}, bv = {b.x, b.y, b.z, b.w};
  if (IN_V) {
    if (INIT) {
      asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=v"(c) : "v"(av), "v"(bv));
    } else {
      asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(av), "v"(bv));
    }
  } else {
    if (INIT) {
      asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=a"(c) : "v"(av), "v"(bv));
    } else {
      asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(av), "v"(bv));
    }
  }
}

constexpr int ntl_of(int jt) { return jt > 8 ? 10 : 8; }            // 8-row token loads per wave and stage
constexpr int stage_bytes_of(int jt) { return (TN + 4 * 8 * ntl_of(jt)) * ROWB; }
constexpr int TILE_LDS_BYTES = 2 * stage_bytes_of(JT_MAX);          // 147456
// behind the stages: the tile's destination rows and gate weights for the down epilogue
constexpr int SIDE_OFF = TILE_LDS_BYTES;
constexpr int SIDE_BYTES = TM_MAX * 8;
// and behind those one 16-byte line of words a GEMM task leaves for the worker loop: the ticket it
// drew for the workgroup's next task. They live in
// the dynamic block because a file-scope LDS variable written from a function that is not
// inlined landed on top of the dynamic block's first bytes.
constexpr int NOTE_OFF = SIDE_OFF + SIDE_BYTES;
constexpr int NOTE_BYTES = 16;
__device__ __forceinline__ unsigned* task_notes() { return reinterpret_cast<unsigned*>(lds_raw + NOTE_OFF); }
constexpr int EPI_LD = TN * 2 + 16;              // bytes per row of the down epilogue's staging slab
static_assert(128 * EPI_LD <= TILE_LDS_BYTES, "epilogue slab exceeds the stage buffers");

struct TileOperands {
  const unsigned char* wbase;  // uniform: the weight matrix (or this wave's packed slice) the offsets are relative to
  const unsigned char* tbase;  // uniform: tokens, or h
  unsigned wstride;            // uniform: bytes from one stage's weights to the next
  bool wpacked;                // uniform: the weights come from the packed layout (see packed_run_offset)
  unsigned woff[NLD];          // this lane's 16 bytes of weight load q at stage 0
  unsigned toff[10];           // the same for the token rows
};

// Stage row (within its operand) that this lane's part of load q belongs to when a wave
// issues `per_wave` loads per stage, and the byte offset inside the row's 128-byte line of
// the chunk it brings.
__device__ __forceinline__ int stage_row(int per_wave, int q) {
  return ((threadIdx.x >> 6) * per_wave + q) * 8 + ((threadIdx.x & 63) >> 3);
}
__device__ __forceinline__ unsigned stage_chunk_bytes(int row) {
  return static_cast<unsigned>(((threadIdx.x & 7) ^ ((row >> 1) & 7)) << 4);
}

struct Frag {
  uint4 a[2];
  uint4 b[JT_MAX];
};

// acc[i][j] = W-block i (32 of this wave's 64 weight rows) x token-block j, j < JT, over
// nstages * 64 k (nstages >= 2). Token rows from 32*JT on are neither loaded nor multiplied.
//
// A stage is 4 sub-steps of 16 k; a sub-step is NS = max(8, JT) slots; a slot is one pair of
// matrix instructions and, behind it, the LDS reads and global loads the schedule puts there:
//  * the fragments of sub-step u+1 are read under sub-step u, one token block per slot
//  * hand-over in sub-step 3 after BAR pairs: this wave's reads of stage s have returned and
//    its loads of stage s+1 have landed, then the workgroup barrier; from there on the next
//    stage's first fragments are read and the loads of stage s+2 go out into the buffer just
//    left, one per slot, the rest under the next stage's first sub-steps. (Measured on all
//    256 CUs: all 16 loads behind the barrier at once, barrier in front of the sub-step: 51 us
//    per 256x256x2048 tile; this schedule: 48 us.)
//
// Bookkeeping rides along: at the first hand-over (every memory operation this wave issued
// before it, the previous task's stores included, has completed there anyway) thread 0
// signals the previous task's completion on `pend` (if any) and draws the workgroup's next
// ticket from `queue` into `next`, so neither trip to memory is waited for between tasks.
template <int JT, typename AfterFirstLoads>
__device__ __forceinline__ void tile_gemm(const TileOperands& op, int nstages, f32x16 (&acc)[2][JT_MAX],
                                          unsigned* pend, unsigned* queue, unsigned& next,
                                          AfterFirstLoads after_first_loads) {
  const int lane = threadIdx.x & 63, wave = uni(threadIdx.x >> 6);
  const int r32 = lane & 31, kq = lane >> 5;
  const unsigned lds_addr = uni(static_cast<unsigned>(
      reinterpret_cast<size_t>((FMOE_L3 unsigned char*)lds_raw)));
  constexpr int TROWS = 32 * JT;
  constexpr int NTL = ntl_of(JT);
  constexpr int STG = stage_bytes_of(JT);
  constexpr int NS = JT > 8 ? JT : 8;  // slots per sub-step
  constexpr int NRD = 2 + JT;          // fragment reads per sub-step
  constexpr int BAR = 2;               // pairs of sub-step 3 in front of the hand-over
  constexpr int AFTER = NS - BAR;      // slots of sub-step 3 behind it
  constexpr int RPS = (NRD + AFTER - 1) / AFTER;  // reads of the next stage's first fragments per slot there

  int fo[4];  // per-lane fragment offsets of the four 16-k sub-steps
#pragma unroll
  for (int u = 0; u < 4; ++u) fo[u] = r32 * ROWB + (((2 * u + kq) ^ ((r32 >> 1) & 7)) << 4);

  auto issue_one = [&](int s, int q) {  // q: 0..7 weights, 8..8+NTL-1 tokens
    const unsigned st = uni(static_cast<int>(lds_addr + (s & 1) * STG));
    if (q < NLD) {
      load_to_lds(op.woff[q], op.wbase + static_cast<size_t>(s) * op.wstride, st + (wave * 64 + q * 8) * ROWB);
    } else if (q < NLD + NTL) {
      const int qq = q - NLD;
      if ((NTL == 8 && JT == 8) || (wave * NTL + qq) * 8 < TROWS)
        load_to_lds(op.toff[qq], op.tbase + static_cast<size_t>(s) * ROWB,
                    st + TN * ROWB + ((wave * NTL + qq) * 8) * ROWB);
    }
  };
  // weight fragments: from row-major stage rows as the token fragments, or, when the wave's
  // weight rows keep the packed order (eight runs [k-step 0..1][block 0..3] of [chunk][row]),
  // row r32 of 32-row block i = row r32 % 16 of run block 2i + r32 / 16, chunk 2*(u % 2) + kq
  // of k-step u / 2
  int ao[4];
#pragma unroll
  for (int u = 0; u < 4; ++u)
    ao[u] = op.wpacked ? ((u >> 1) * 4 + (r32 >> 4)) * 1024 + (((2 * (u & 1) + kq) * 16 + (r32 & 15)) << 4)
                       : fo[u];
  const int ablock = uni(op.wpacked ? 2048 : 32 * ROWB);  // bytes from weight block 0 to block 1
  auto read_n = [&](Frag& f, int s, int u, int r) {  // r-th of the NRD reads of a sub-step
    const unsigned char* st = lds_raw + (s & 1) * STG + fo[u];
    if (r < 2) {
      f.a[r] = *reinterpret_cast<const uint4*>(lds_raw + (s & 1) * STG + wave * (64 * ROWB) + r * ablock + ao[u]);
    } else if (r < NRD) {
      f.b[r - 2] = *reinterpret_cast<const uint4*>(st + TN * ROWB + ((r - 2) * 32) * ROWB);
    }
  };
  auto pair = [&](auto init_tag, const Frag& cur, int j) {
    constexpr bool INIT = decltype(init_tag)::value;
    if (j < JT) {
      if (j < 8) {
        mma32<INIT, false>(cur.a[0], cur.b[j], acc[0][j]);
        mma32<INIT, false>(cur.a[1], cur.b[j], acc[1][j]);
      } else {
        mma32<INIT, true>(cur.a[0], cur.b[j], acc[0][j]);
        mma32<INIT, true>(cur.a[1], cur.b[j], acc[1][j]);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  auto bookkeeping = [&]() {
    if (threadIdx.x == 0) {
      if (pend != nullptr) (void)add_relaxed(pend, 1u);
      next = add_relaxed(queue, 1u);
    }
  };

  Frag f0, f1;
#pragma unroll
  for (int q = 0; q < NLD + NTL; ++q) issue_one(0, q);
#pragma unroll
  for (int q = 0; q < NLD + NTL; ++q) issue_one(1, q);
  // Loads to registers that the task still needs go out here, behind the loads to LDS: a
  // load to registers that is still on its way when a younger load to LDS is issued may not
  // deliver its data (seen with 16-byte loads; the register kept its old content). Every
  // later load to LDS follows a wait for all outstanding loads.
  after_first_loads();
  // stage 0 has landed, then everybody's. (The wait is for everything this wave has asked
  // for, stage 1 and the loads to registers included: the two kinds of load are not counted
  // in order with each other, so a count that leaves stage 1 in flight would not say that
  // stage 0 is in.)
  wait_vm<0>();
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
#pragma unroll
  for (int r = 0; r < NRD; ++r) read_n(f0, 0, 0, r);

  auto stage = [&](int s, auto first_tag, auto early_tag, auto late_tag, auto next_tag) {
    constexpr bool EARLY = decltype(early_tag)::value;  // the tail of stage s+1's loads is still to go out
    constexpr bool LATE = decltype(late_tag)::value;    // stage s+2 exists
    constexpr bool NEXT = decltype(next_tag)::value;    // stage s+1 exists
    using No = std::false_type;
#pragma unroll
    for (int u = 0; u < 3; ++u) {
      const Frag& cur = (u & 1) ? f1 : f0;
      Frag& nxt = (u & 1) ? f0 : f1;
#pragma unroll
      for (int j = 0; j < NS; ++j) {
        if (u == 0) {
          pair(first_tag, cur, j);
        } else {
          pair(No{}, cur, j);
        }
        if (EARLY) issue_one(s + 1, AFTER + NS * u + j);
        if (j == 0) {
          read_n(nxt, s, u + 1, 0);
          read_n(nxt, s, u + 1, 1);
        }
        read_n(nxt, s, u + 1, 2 + j);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#pragma unroll
    for (int j = 0; j < NS; ++j) {
      if (j == BAR) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (NEXT) {
          wait_vm<0>();
          __builtin_amdgcn_s_barrier();
          asm volatile("" ::: "memory");
          if (decltype(first_tag)::value) bookkeeping();
        }
      }
      pair(No{}, f1, j);
      if (j >= BAR) {
        if (LATE) issue_one(s + 2, j - BAR);
        if (NEXT) {
#pragma unroll
          for (int r = (j - BAR) * RPS; r < (j - BAR + 1) * RPS; ++r) read_n(f0, s + 1, 0, r);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  using Yes = std::true_type;
  using No = std::false_type;
  if (nstages > 2) {
    stage(0, Yes{}, No{}, Yes{}, Yes{});
  } else {
    stage(0, Yes{}, No{}, No{}, Yes{});
  }
  int s = 1;
  for (; s + 2 < nstages; ++s) stage(s, No{}, Yes{}, Yes{}, Yes{});
  if (s + 1 < nstages) {
    stage(s, No{}, Yes{}, No{}, Yes{});
    ++s;
  }
  stage(s, No{}, No{}, No{}, No{});
  // the compiler does not see matrix instructions in the assembly above: keep the wait states
  // between the last of them and the first read of an accumulator
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
  __syncthreads();  // the stages are free for the epilogue
}

// The same product when the weights come from the packed layout, on a deeper pipeline that
// keeps its depth in registers instead of LDS.
//
// A wave's 64 weight rows are its own: no other wave reads them. So they do not go through
// LDS at all: every fragment (32 rows x 16 k, 16 bytes per lane) is one global load straight
// into the registers the matrix instruction reads, four 256-byte segments of the packed runs
// per instruction. Two register sets: the fragments of stage s+2 are requested into the
// registers of stage s as soon as its sub-step is through, two stages (about 2 us) before
// they are needed. The token rows, which all four waves read, still meet in LDS, but they
// travel global -> registers -> LDS (ds_write_b128) instead of straight to LDS: a wave
// requests its JT loads of 8 rows of stage s+3 during stage s, into the registers whose
// previous content (stage s+1) it has just written to LDS. Two LDS buffers of 4 KiB per
// 32-row block, written one stage before they are read. Half the LDS traffic of the version
// above is gone (no weight rows written, no weight fragments read), the hand-over between
// two stages waits for LDS only (this wave's writes of stage s+1 and reads of stage s, then
// the workgroup barrier), and every global load has 1.75 to 2 stages to arrive.
//
// Loads straight to LDS are not used here on purpose: a load to registers that was still
// outstanding when a younger load-to-LDS was issued did not deliver its data (the register
// kept its old content; measured, deterministic), and the two kinds are not counted in order
// with each other either. With one kind of load only, completion is in order and how many
// younger loads may stay in flight at each wait is a constant of the schedule: every wave
// issues the same loads in the same order. direct_wait() counts them from the list of what
// a stage issues (which also covers the last stages, where loads of stages that do not exist
// are left out):
//   sub-step 0: weights (s+1, sub-step 3); sub-step 1: weights (s+2, sub-step 0), then the
//   token rows of stage s+3; sub-step 2, 3: weights (s+2, sub-step 1, 2).
// The loads in front of the loop are issued in the same order, as if by stages -2 and -1.
constexpr int DIRECT_GROUPS = 5;
constexpr int DIRECT_JT_MAX = 8;     // taller tiles do not leave the registers for it
constexpr int DIRECT_MIN_STAGES = 4;
// Loads that group g (in issue order) of a stage with r stages after it puts out.
constexpr int direct_group(int jt, int r, int g) {
  switch (g) {
    case 0: return r >= 1 ? 2 : 0;
    case 2: return r >= 3 ? jt : 0;
    default: return r >= 2 ? 2 : 0;
  }
}
// Loads issued after group g0 of the stage `back` stages before the present one (which has
// r stages after it) and before group g1 of the present stage: those may still be in flight
// when everything up to and including that group has to have landed.
constexpr int direct_in_flight(int jt, int r, int back, int g0, int g1) {
  int n = 0;
  for (int b = back; b >= 0; --b) {
    const int lo = b == back ? g0 + 1 : 0;
    const int hi = b == 0 ? g1 : DIRECT_GROUPS;
    for (int g = lo; g < hi; ++g) n += direct_group(jt, r + b, g);
  }
  return n;
}
// wait in front of sub-step w of a stage with r stages after it: its weight fragments and,
// for sub-step 0, the token rows of the next stage, which that sub-step writes to LDS
constexpr int direct_wait(int jt, int r, int w) {
  switch (w) {
    case 0: return direct_in_flight(jt, r, 2, 2, 0);
    case 1: return direct_in_flight(jt, r, 2, 3, 1);
    case 2: return direct_in_flight(jt, r, 2, 4, 3);
    default: return direct_in_flight(jt, r, 1, 0, 4);
  }
}

typedef unsigned v4u_t __attribute__((ext_vector_type(4)));

template <bool INIT>
__device__ __forceinline__ void mma32v(const v4u_t& av, const uint4& b, f32x16& c) {
  const v4u_t bv = {b.x, b.y, b.z, b.w};
  if (INIT) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=a"(c) : "v"(av), "v"(bv));
  } else {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(av), "v"(bv));
  }
}

// 16 bytes per lane from base + off into the registers of `dst`; completion is tracked by
// hand (wait_vm), so the compiler must not believe it knows when the value is there: the
// operand is read-write, which keeps the value in one place from the load to its last use.
__device__ __forceinline__ void load_fragment(v4u_t& dst, unsigned off, const unsigned char* base) {
  asm volatile("global_load_dwordx4 %0, %1, %2" : "+v"(dst) : "v"(off), "s"(base) : "memory");
}
// 16 bytes per lane from registers to LDS (byte address `lds_off`)
__device__ __forceinline__ void store_fragment(unsigned lds_off, const v4u_t& src) {
  asm volatile("ds_write_b128 %0, %1" : : "v"(lds_off), "v"(src) : "memory");
}

template <int JT>
__device__ __forceinline__ void tile_gemm_direct(const TileOperands& op, int nstages, f32x16 (&acc)[2][JT_MAX],
                                                 unsigned* pend, unsigned* queue, unsigned& next) {
  static_assert(JT <= DIRECT_JT_MAX, "tile too tall for the register-staged pipeline");
  constexpr int NS = 8;                           // slots per sub-step
  constexpr int BAR = 2;                          // pairs of sub-step 3 in front of the hand-over
  constexpr int AFTER = NS - BAR;
  constexpr int STG = 32 * JT * ROWB;             // token rows of one stage
  constexpr int RPS = (JT + AFTER - 1) / AFTER;   // reads of the next stage's first fragments per slot behind the hand-over
  static_assert(2 * STG <= TILE_LDS_BYTES, "token stages exceed the tile's LDS");
  const int lane = threadIdx.x & 63, wave = uni(threadIdx.x >> 6);
  const int r32 = lane & 31, kq = lane >> 5;
  const unsigned lds_addr = uni(static_cast<unsigned>(
      reinterpret_cast<size_t>((FMOE_L3 unsigned char*)lds_raw)));

  int fo[4];  // per-lane token fragment offsets of the four 16-k sub-steps
#pragma unroll
  for (int u = 0; u < 4; ++u) fo[u] = r32 * ROWB + (((2 * u + kq) ^ ((r32 >> 1) & 7)) << 4);
  // weight fragment (sub-step u, 32-row block i) of stage s in the wave's packed slice:
  // 8192*s + 4096*(u/2) + 2048*i + 512*(u%2), plus this lane's part
  const unsigned aoff = static_cast<unsigned>(((r32 >> 4) << 10) + (kq << 8) + ((r32 & 15) << 4));
  // where this lane's 16 bytes of the wave's token load q belong in a stage buffer: the
  // eight rows of load q are one run of 1 KiB, lane l at 16*l
  const unsigned wr_off = lds_addr + static_cast<unsigned>((wave * JT) * 1024 + lane * 16);

  v4u_t as[2][4][2];   // weight fragments: [stage parity][sub-step][block]
  v4u_t bs[2][JT];     // token rows on their way to LDS: [stage parity][load]
#pragma unroll
  for (int p = 0; p < 2; ++p) {
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < 2; ++i) as[p][u][i] = v4u_t{0u, 0u, 0u, 0u};
#pragma unroll
    for (int q = 0; q < JT; ++q) bs[p][q] = v4u_t{0u, 0u, 0u, 0u};
  }
  uint4 bf[2][JT_MAX];

  auto issue_a = [&](int s, int u, int i, v4u_t& dst) {
    load_fragment(dst, aoff, op.wbase + static_cast<size_t>(s) * 8192 + ((u >> 1) * 4096 + i * 2048 + (u & 1) * 512));
  };
  auto issue_b = [&](int s, int q, v4u_t& dst) {  // q-th token load of this wave for stage s
    load_fragment(dst, op.toff[q], op.tbase + static_cast<size_t>(s) * ROWB);
  };
  auto write_b = [&](int buf, int q, const v4u_t& src) { store_fragment(wr_off + buf * STG + q * 1024, src); };
  auto read_b = [&](int buf, int u, int j) {
    return *reinterpret_cast<const uint4*>(
        __builtin_assume_aligned(lds_raw + buf * STG + fo[u] + j * (32 * ROWB), 16));
  };
  auto pair = [&](auto init_tag, const v4u_t (&a)[2], const uint4 (&b)[JT_MAX], int j) {
    constexpr bool INIT = decltype(init_tag)::value;
    if (j < JT) {
      mma32v<INIT>(a[0], b[j], acc[0][j]);
      mma32v<INIT>(a[1], b[j], acc[1][j]);
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- in front of the loop. First what stage 0 needs at once: its token rows, its weight
  // fragments, and the token rows of stage 1 (which stage 0 writes to LDS).
#pragma unroll
  for (int q = 0; q < JT; ++q) issue_b(0, q, bs[0][q]);
#pragma unroll
  for (int i = 0; i < 2; ++i) issue_a(0, 0, i, as[0][0][i]);
#pragma unroll
  for (int q = 0; q < JT; ++q) issue_b(1, q, bs[1][q]);
#pragma unroll
  for (int u = 1; u < 4; ++u)
#pragma unroll
    for (int i = 0; i < 2; ++i) issue_a(0, u, i, as[0][u][i]);
  // Everything requested so far has landed, and so have the stores of the previous task's
  // epilogue (loads and stores do not complete in order with each other, so only a wait for
  // all of them covers the stores): behind the workgroup barrier thread 0 may signal that
  // task's completion, and draws the ticket of the task after this one.
  wait_vm<0>();
#pragma unroll
  for (int q = 0; q < JT; ++q) write_b(0, q, bs[0][q]);
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  if (threadIdx.x == 0) {
    if (pend != nullptr) (void)add_relaxed(pend, 1u);
    next = add_relaxed(queue, 1u);
  }
  // then what stage -1 would have issued
#pragma unroll
  for (int i = 0; i < 2; ++i) issue_a(1, 0, i, as[1][0][i]);
#pragma unroll
  for (int q = 0; q < JT; ++q) issue_b(2, q, bs[0][q]);
#pragma unroll
  for (int u = 1; u < 3; ++u)
#pragma unroll
    for (int i = 0; i < 2; ++i) issue_a(1, u, i, as[1][u][i]);
#pragma unroll
  for (int j = 0; j < JT; ++j) bf[0][j] = read_b(0, 0, j);

  // One stage. P: its parity (which weight registers it multiplies, which LDS buffer it
  // reads). R: stages after it, 3 meaning 3 or more.
  auto stage = [&](auto par_tag, auto rem_tag, auto first_tag, int s) {
    constexpr int P = decltype(par_tag)::value;
    constexpr int R = decltype(rem_tag)::value;
    constexpr bool A2 = R >= 2, A13 = R >= 1, B3 = R >= 3, NEXT = R >= 1;
    using No = std::false_type;
#pragma unroll
    for (int u = 0; u < 3; ++u) {
      if (u == 0) wait_vm<direct_wait(JT, R, 0)>();
      if (u == 1) wait_vm<direct_wait(JT, R, 1)>();
      if (u == 2) wait_vm<direct_wait(JT, R, 2)>();
      const uint4 (&cur)[JT_MAX] = bf[u & 1];
      uint4 (&nxt)[JT_MAX] = bf[(u + 1) & 1];
#pragma unroll
      for (int j = 0; j < NS; ++j) {
        if (u == 0) {
          pair(first_tag, as[P][u], cur, j);
        } else {
          pair(No{}, as[P][u], cur, j);
        }
        if (u == 0) {
          if (j < 2 && A13) issue_a(s + 1, 3, j, as[1 - P][3][j]);
          if (j < JT && NEXT) write_b(1 - P, j, bs[1 - P][j]);   // token rows of stage s+1
        } else if (u == 1) {
          if (j == 0 && A2) {
            issue_a(s + 2, 0, 0, as[P][0][0]);
            issue_a(s + 2, 0, 1, as[P][0][1]);
          }
          if (j < JT && B3) issue_b(s + 3, j, bs[1 - P][j]);
        } else if (j < 2 && A2) {
          issue_a(s + 2, 1, j, as[P][1][j]);
        }
        if (j < JT) nxt[j] = read_b(P, u + 1, j);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    wait_vm<direct_wait(JT, R, 3)>();
#pragma unroll
    for (int j = 0; j < NS; ++j) {
      if (j == BAR) {
        // this wave no longer reads this stage's buffer and has written its part of the next
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (NEXT) {
          __builtin_amdgcn_s_barrier();
          asm volatile("" ::: "memory");
        }
      }
      pair(No{}, as[P][3], bf[1], j);
      if (j < 2 && A2) issue_a(s + 2, 2, j, as[P][2][j]);
      if (j >= BAR && NEXT) {
#pragma unroll
        for (int r = (j - BAR) * RPS; r < (j - BAR + 1) * RPS; ++r)
          if (r < JT) bf[0][r] = read_b(1 - P, 0, r);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  using Yes = std::true_type;
  using No = std::false_type;
  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;
  using R3 = std::integral_constant<int, 3>;
  // nstages is even and at least 4; stages with 3 or more after them: nstages - 3 (odd)
  stage(P0{}, R3{}, Yes{}, 0);
  int s = 1;
  for (; s + 3 < nstages; s += 2) {
    stage(P1{}, R3{}, No{}, s);
    stage(P0{}, R3{}, No{}, s + 1);
  }
  stage(P1{}, std::integral_constant<int, 2>{}, No{}, s);
  stage(P0{}, std::integral_constant<int, 1>{}, No{}, s + 1);
  stage(P1{}, std::integral_constant<int, 0>{}, No{}, s + 2);
  // the compiler does not see matrix instructions in the assembly above: keep the wait states
  // between the last of them and the first read of an accumulator
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
  wait_vm<0>();
  __syncthreads();  // the stages are free for the epilogue
}

// Weights in the packed layout (the streaming variant's: per wave task and 32-k step four
// runs of 1 KiB, one per 16-row block, each [16-byte chunk 0..3][row 0..15]). This wave's 64
// stage rows are exactly one packed task: gate/up task (expert, 32 h columns) = gate blocks
// 0,1 and up blocks 2,3; down task (expert, 64 output columns) = blocks 0..3. A stage of 64 k
// is two 32-k steps, i.e. eight runs, and load q of the wave copies run (k-step q / 4, block
// q % 4) as it is: eight whole lines read by consecutive lanes. (Permuting the chunks into the
// row-major stage layout on the way in made every 16 lanes touch 8 lines: prefill 798 -> 867 us.)
// So with packed weights the wave's weight rows keep the packed order in LDS, and only the
// fragment reads differ: see tile_gemm.
static_assert(G1_NB == 2 && G2_NB == 4, "the tiled variant reads the packed layout as 32+32-row and 64-row tasks");
__device__ __forceinline__ unsigned packed_run_offset(int q) {
  return static_cast<unsigned>((q >> 2) * 4096 + (q & 3) * 1024 + (threadIdx.x & 63) * 16);
}

// One GEMM tile task, gate/up or down, for a row tile of up to 32*JT rows.
//
// gate/up: h[row, n0 .. n0+128) (test/singleGPU/cpp/moe/reference/refExpertFFN1.h:51-65).
// h is [T*K, I] row-major, rows in permuted order. Wave w holds gate rows n0+32w.. and the
// matching up rows, so SiLU(gate)*up happens in registers; the tile's 128 columns leave
// through LDS as 256-byte row segments.
//
// down: y[t*K+slot, n0 .. n0+256) = h[row] . W2[e]^T (refFullMoe.h:58-65,
// src/hip/kernel/tasks/ffn2Task.h:37-40), bf16, through LDS as 512-byte row segments, 128
// rows at a time. The rows' destinations are fetched when the task starts and parked in LDS
// behind the stages, so the epilogue waits for no memory. The slot's gate weight is applied
// by the combine task, which has instruction slots to spare; here every instruction of the
// epilogue is one the matrix cores wait for.
template <int JT, bool down>
__device__ __forceinline__ void tile_task(ParamsRef p, int expert, int row0, int rows, int nblk, unsigned* pend,
                                          unsigned* queue) {
  const int H = uni(p.H), I = uni(p.I), K = uni(p.K);
  const int wave = uni(threadIdx.x >> 6), lane = threadIdx.x & 63;
  constexpr int NTL = ntl_of(JT);
  // packed weights and at least four stages: the deeper pipeline (tile_gemm_direct), where a
  // wave brings JT token loads per stage instead of NTL
  const bool direct = JT <= DIRECT_JT_MAX &&
                      uni(((down ? p.ffn2_packed : p.ffn1_packed) != nullptr && (down ? I : H) >= DIRECT_MIN_STAGES * KS) ? 1 : 0) != 0;
  const int tl_per_wave = direct ? JT : NTL;
  const int* perm = uni(p.perm) + row0;
  const int n0 = uni(nblk) * (down ? TN : G1_COLS);
  TileOperands op;
  int side_dst[2] = {-1, -1};
  int nstages;
  if (down) {
    nstages = I / KS;
    const bool packed = uni(p.ffn2_packed != nullptr ? 1 : 0) != 0;
    if (packed) {
      const size_t task = static_cast<size_t>(expert) * (H / 64) + (n0 / 64 + wave);
      op.wbase = uni(reinterpret_cast<const unsigned char*>(p.ffn2_packed)) + task * (static_cast<size_t>(I / 32) * 4096);
      op.wstride = 8192u;
      op.wpacked = true;
    } else {
      op.wpacked = false;
      op.wbase = uni(reinterpret_cast<const unsigned char*>(p.ffn2)) + (static_cast<size_t>(expert) * H + n0) * I * 2;
      op.wstride = static_cast<unsigned>(ROWB);
    }
    op.tbase = uni(reinterpret_cast<const unsigned char*>(p.h)) + static_cast<size_t>(row0) * I * 2;
#pragma unroll
    for (int q = 0; q < NLD; ++q) {
      const int row = stage_row(NLD, q);
      op.woff[q] = packed ? packed_run_offset(q)
                          : static_cast<unsigned>(row) * static_cast<unsigned>(I * 2) + stage_chunk_bytes(row);
    }
#pragma unroll
    for (int q = 0; q < NTL; ++q) {
      const int row = stage_row(tl_per_wave, q);
      op.toff[q] = static_cast<unsigned>(min(row, rows - 1)) * static_cast<unsigned>(I * 2) + stage_chunk_bytes(row);
    }
  } else {
    nstages = H / KS;
    const bool packed = uni(p.ffn1_packed != nullptr ? 1 : 0) != 0;
    if (packed) {
      const size_t task = static_cast<size_t>(expert) * (I / 32) + (n0 / 32 + wave);
      op.wbase = uni(reinterpret_cast<const unsigned char*>(p.ffn1_packed)) + task * (static_cast<size_t>(H / 32) * 4096);
      op.wstride = 8192u;
      op.wpacked = true;
    } else {
      op.wpacked = false;
      op.wbase = uni(reinterpret_cast<const unsigned char*>(p.ffn1)) + static_cast<size_t>(expert) * 2 * I * H * 2;
      op.wstride = static_cast<unsigned>(ROWB);
    }
    op.tbase = uni(reinterpret_cast<const unsigned char*>(p.tokens));
#pragma unroll
    for (int q = 0; q < NLD; ++q) {
      const int row = stage_row(NLD, q);
      // weight stage rows 64w..64w+31: gate rows n0+32w.., 64w+32..64w+63: up rows I+n0+32w..
      const int wl = row & 63;
      const int wrow = (wl < 32 ? n0 : I + n0 - 32) + 32 * wave + wl;
      op.woff[q] = packed ? packed_run_offset(q)
                          : static_cast<unsigned>(wrow) * static_cast<unsigned>(H * 2) + stage_chunk_bytes(row);
    }
#pragma unroll
    for (int q = 0; q < NTL; ++q) {
      const int row = stage_row(tl_per_wave, q);
      const int tok = ldc(&perm[min(row, rows - 1)]) / K;
      op.toff[q] = static_cast<unsigned>(tok) * static_cast<unsigned>(H * 2) + stage_chunk_bytes(row);
    }
  }
  f32x16 acc[2][JT_MAX];
  unsigned next = 0u;
  // down: where the tile's rows go (token, slot), fetched while the k-loop runs
  auto load_side = [&]() {
    if (down) {
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const int r = static_cast<int>(threadIdx.x) + k * T_THREADS;
        side_dst[k] = r < rows ? ldc(&perm[r]) : -1;
      }
    }
  };
  if (direct) {
    load_side();
    if constexpr (JT <= DIRECT_JT_MAX) tile_gemm_direct<JT>(op, nstages, acc, pend, queue, next);
  } else {
    tile_gemm<JT>(op, nstages, acc, pend, queue, next, load_side);
  }
  if (threadIdx.x == 0) task_notes()[0] = next;  // the epilogue's barriers publish it

  const int r32 = lane & 31, kq = lane >> 5;
  unsigned char* slab = lds_raw;
  if (!down) {
    constexpr int LD = G1_COLS * 2 + 16;  // slab row pitch in bytes
#pragma unroll
    for (int j = 0; j < JT; ++j)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        float hv[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) hv[v] = silu_mul_fast(acc[0][j][g4 * 4 + v], acc[1][j][g4 * 4 + v]);
        uint2 pk;
        pk.x = pack_bf16(hv[0], hv[1]);
        pk.y = pack_bf16(hv[2], hv[3]);
        *reinterpret_cast<uint2*>(slab + (j * 32 + r32) * LD + (wave * 32 + g4 * 8 + kq * 4) * 2) = pk;
      }
    __syncthreads();
    // 16 lanes store one row's 256 bytes; a wave stores 4 rows per instruction
    unsigned char* h = uni(reinterpret_cast<unsigned char*>(p.h)) + (static_cast<size_t>(row0) * I + n0) * 2;
    // (the reads of a batch first, then its stores: a store's assembly orders memory
    // operations around it, and one LDS round trip per store would add up to microseconds)
    constexpr int NIT = 8 * JT / WAVES, BATCH = 8;
#pragma unroll
    for (int it0 = 0; it0 < NIT; it0 += BATCH) {
      uint4 v[BATCH];
#pragma unroll
      for (int u = 0; u < BATCH; ++u) {
        const int row = ((it0 + u) * WAVES + wave) * 4 + (lane >> 4);
        if (it0 + u < NIT) v[u] = *reinterpret_cast<const uint4*>(slab + row * LD + (lane & 15) * 16);
      }
#pragma unroll
      for (int u = 0; u < BATCH; ++u) {
        const int row = ((it0 + u) * WAVES + wave) * 4 + (lane >> 4);
        if (it0 + u < NIT && row < rows)
          st16_through(h + static_cast<size_t>(row) * I * 2 + (lane & 15) * 16, v[u]);
      }
    }
    __syncthreads();  // the slab is stage memory again
  } else {
    int* sdst = reinterpret_cast<int*>(lds_raw + SIDE_OFF);
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int r = static_cast<int>(threadIdx.x) + k * T_THREADS;
      if (r < TM_MAX) sdst[r] = side_dst[k];
    }
    __syncthreads();
    unsigned char* y = uni(reinterpret_cast<unsigned char*>(p.y)) + n0 * 2;
#pragma unroll
    for (int part = 0; part < (JT + 3) / 4; ++part) {
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        const int j = part * 4 + jj;
        if (j < JT) {
#pragma unroll
          for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
              uint2 pk;
              pk.x = pack_bf16(acc[i][j][g4 * 4 + 0], acc[i][j][g4 * 4 + 1]);
              pk.y = pack_bf16(acc[i][j][g4 * 4 + 2], acc[i][j][g4 * 4 + 3]);
              *reinterpret_cast<uint2*>(slab + (jj * 32 + r32) * EPI_LD +
                                        (wave * 64 + i * 32 + g4 * 8 + kq * 4) * 2) = pk;
            }
        }
      }
      __syncthreads();
      // 32 lanes store one row's 512 bytes at the row's (token, slot); a wave stores 2 rows per instruction
      constexpr int BATCH = 8;
#pragma unroll
      for (int it0 = 0; it0 < 128 / (2 * WAVES); it0 += BATCH) {
        uint4 v[BATCH];
        int dst[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
          const int lr = ((it0 + u) * WAVES + wave) * 2 + (lane >> 5);  // row inside this part
          const int row = part * 128 + lr;
          dst[u] = row < 32 * JT ? sdst[row] : -1;
          v[u] = *reinterpret_cast<const uint4*>(slab + lr * EPI_LD + (lane & 31) * 16);
        }
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
          if (dst[u] >= 0) st16_through(y + static_cast<size_t>(dst[u]) * H * 2 + (lane & 31) * 16, v[u]);
      }
      __syncthreads();
    }
  }
}

// one straight-line instantiation per number of live token blocks
__device__ __noinline__ void tiled_gemm_task(ParamsRef pv, const TileDesc& tile_in, int nblk, int down_in,
                                             unsigned* pend_in, unsigned* queue_in) {
  ParamsRef p = uniform_params(pv);
  unsigned* pend = uni(pend_in);
  unsigned* queue = uni(queue_in);
  const int expert = uni(tile_in.expert), row0 = uni(tile_in.row0), rows = uni(tile_in.rows);
  const bool down = uni(down_in) != 0;
  const int jt = (rows + 31) >> 5;
  if (jt > 9) {
    if (down) tile_task<10, true>(p, expert, row0, rows, nblk, pend, queue); else tile_task<10, false>(p, expert, row0, rows, nblk, pend, queue);
  } else if (jt > 8) {
    if (down) tile_task<9, true>(p, expert, row0, rows, nblk, pend, queue); else tile_task<9, false>(p, expert, row0, rows, nblk, pend, queue);
  } else if (jt > 7) {
    if (down) tile_task<8, true>(p, expert, row0, rows, nblk, pend, queue); else tile_task<8, false>(p, expert, row0, rows, nblk, pend, queue);
  } else if (jt > 6) {
    if (down) tile_task<7, true>(p, expert, row0, rows, nblk, pend, queue); else tile_task<7, false>(p, expert, row0, rows, nblk, pend, queue);
  } else if (jt > 4) {
    if (down) tile_task<6, true>(p, expert, row0, rows, nblk, pend, queue); else tile_task<6, false>(p, expert, row0, rows, nblk, pend, queue);
  } else if (jt > 2) {
    if (down) tile_task<4, true>(p, expert, row0, rows, nblk, pend, queue); else tile_task<4, false>(p, expert, row0, rows, nblk, pend, queue);
  } else {
    if (down) tile_task<2, true>(p, expert, row0, rows, nblk, pend, queue); else tile_task<2, false>(p, expert, row0, rows, nblk, pend, queue);
  }
}

constexpr int TILED_LDS_BYTES =
    NOTE_OFF + NOTE_BYTES > ROUTER_LDS_BYTES ? NOTE_OFF + NOTE_BYTES : ROUTER_LDS_BYTES;

// combine: out[t] = sum over slots, in slot order, of w[t,slot] * y[t*K+slot]
// (refFullMoe.h:35,62-65): y holds each slot's down-projection row rounded to bf16; weight
// and sum are float, one fused multiply-add per slot, then one rounding to bf16.
//
// One item = 8 columns of one token; a unit = the rows of up to 8 slots of one item (16
// bytes each). A thread walks through its units with the loads of the next CMB_D - 1 units
// in flight while it sums the present one: with one wave per SIMD nothing else covers the
// summing, and a thread that loads everything and then sums everything leaves the memory
// pipeline idle half of the time (4.4 TB/s; measured with four items loaded at once).
constexpr int CMB_D = 3;  // units of a thread: one being summed, the others in flight
constexpr int CMB_RUN = 8;  // units of one straight-line run (30B shape: one task)
// Every thread of the task walks through the same number of units with unconditional loads
// (a thread without an item of its own repeats the task's last one and stores nothing; slots
// past K repeat slot K-1 and are not summed), so control flow is uniform and every wave has
// the same loads in flight. The loads are issued from assembly and waited for by count
// (left to itself the compiler waited for all but one unit's loads before every sum).
// Stores are not counted: they may complete out of order with the loads, and leaving them
// out of the count only makes a wait longer, never shorter.
__device__ __forceinline__ void load_once(v4u_t& dst, unsigned off, const unsigned char* base) {
  asm volatile("global_load_dwordx4 %0, %1, %2 nt" : "=v"(dst) : "v"(off), "s"(base) : "memory");
}
template <bool RESIDUAL>
__device__ __forceinline__ void combine_units(const unsigned short* y, const unsigned short* residual,
                                              unsigned short* out, const float* wts, const unsigned char* flag,
                                              int t0, int nitems, int cpr, int H, int K) {
  constexpr int LPU = RESIDUAL ? 9 : 8;  // loads per unit
  const int tid = threadIdx.x;
  const int nchunks = uni((K + 7) >> 3);  // units per item
  const int nunits = uni(((nitems + T_THREADS - 1) / T_THREADS) * nchunks);
  v4u_t v[CMB_D][8];
  v4u_t rv[CMB_D];
  // the task's rows of y and of the residual (uniform); a lane's offsets inside them fit 32 bits
  const unsigned char* ybase = uni(reinterpret_cast<const unsigned char*>(y + static_cast<size_t>(t0) * K * H));
  const unsigned char* rbase = uni(reinterpret_cast<const unsigned char*>(residual + static_cast<size_t>(t0) * H));
  auto where = [&](int unit, int& tl, int& col, int& k0, bool& live) {
    const int item = unit / nchunks;  // uniform
    k0 = (unit - item * nchunks) << 3;
    const int it = tid + item * T_THREADS;
    live = it < nitems;
    const int itc = min(it, nitems - 1);
    tl = itc / cpr;
    col = (itc - tl * cpr) << 3;
  };
  auto issue = [&](int unit, v4u_t (&dst)[8], v4u_t& rdst) {
    int tl, col, k0;
    bool live;
    where(unit, tl, col, k0, live);
    const unsigned yoff = static_cast<unsigned>((tl * K * H + col) * 2);
#pragma unroll
    for (int k = 0; k < 8; ++k) load_once(dst[k], yoff, ybase + static_cast<size_t>(min(k0 + k, K - 1)) * H * 2);
    if (RESIDUAL) load_once(rdst, static_cast<unsigned>((tl * H + col) * 2), rbase);
  };
  float s[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) s[i] = 0.0f;
  auto consume = [&](int unit, const v4u_t (&src)[8], const v4u_t& rsrc) {
    int tl, col, k0;
    bool live;
    where(unit, tl, col, k0, live);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int kk = min(k0 + k, K - 1);
      // a slot without an expert holds rows nobody wrote: they are not looked at
      const bool use = k0 + k < K && flag[tl * K + kk] != 0;
      const float w = wts[tl * K + kk];
      float f[8];
      unpack<BF16>(make_uint4(src[k].x, src[k].y, src[k].z, src[k].w), f);
#pragma unroll
      for (int i = 0; i < 8; ++i) s[i] = use ? __fmaf_rn(f[i], w, s[i]) : s[i];
    }
    if (k0 + 8 >= K) {  // the item's last unit (uniform)
      if (RESIDUAL) {  // output = input row + layer, the row added last
        float f[8];
        unpack<BF16>(make_uint4(rsrc.x, rsrc.y, rsrc.z, rsrc.w), f);
#pragma unroll
        for (int i = 0; i < 8; ++i) s[i] += f[i];
      }
      if (live)
        st16(out + static_cast<size_t>(t0 + tl) * H + col,
             u32x4{pack_bf16(s[0], s[1]), pack_bf16(s[2], s[3]), pack_bf16(s[4], s[5]), pack_bf16(s[6], s[7])});
#pragma unroll
      for (int i = 0; i < 8; ++i) s[i] = 0.0f;
    }
  };
  // Units go in straight-line runs of CMB_RUN (no loop-carried registers: a value that is
  // still on its way from memory must never be copied), the rest one by one.
  auto run = [&](auto n_tag, int u0) {
    constexpr int N = decltype(n_tag)::value;
#pragma unroll
    for (int d = 0; d + 1 < CMB_D && d < N; ++d) issue(u0 + d, v[d], rv[d]);
#pragma unroll
    for (int d = 0; d < N; ++d) {
      if (d + CMB_D - 1 < N) {
        issue(u0 + d + CMB_D - 1, v[(d + CMB_D - 1) % CMB_D], rv[(d + CMB_D - 1) % CMB_D]);
        wait_vm<(CMB_D - 1) * LPU>();
      } else if (d + 2 < N && CMB_D > 3) {
        wait_vm<2 * LPU>();
      } else if (d + 1 < N) {
        wait_vm<LPU>();
      } else {
        wait_vm<0>();
      }
      __builtin_amdgcn_sched_barrier(0);
      consume(u0 + d, v[d % CMB_D], rv[d % CMB_D]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  int u0 = 0;
  for (; u0 + CMB_RUN <= nunits; u0 += CMB_RUN) run(std::integral_constant<int, CMB_RUN>{}, u0);
  for (; u0 < nunits; ++u0) run(std::integral_constant<int, 1>{}, u0);
}

__device__ __noinline__ void tiled_combine_task(ParamsRef pv, int blk) {
  ParamsRef p = uniform_params(pv);
  const int H = uni(p.H), K = uni(p.K), T = uni(p.T), E = uni(p.E), W = uni(p.W);
  unsigned short* out = uni(reinterpret_cast<unsigned short*>(p.out));
  const unsigned short* y = uni(reinterpret_cast<const unsigned short*>(p.y));
  const unsigned short* residual = uni(reinterpret_cast<const unsigned short*>(p.residual));
  const int* topk_idx = uni(p.topk_idx);
  const float* topk_w = uni(p.topk_w);
  unsigned long long* masks = uni(p.masks);
  const int tid = threadIdx.x;
  const int t0 = uni(blk) * CMB_TOK;
  const int ntok = uni(min(CMB_TOK, T - t0));
  // which (token, slot) pairs of this task hold an expert, and their gate weights: one load each
  float* wts = reinterpret_cast<float*>(lds_raw);                      // [CMB_TOK * MAX_TOPK]
  unsigned char* flag = lds_raw + CMB_TOK * MAX_TOPK * sizeof(float);  // [CMB_TOK * MAX_TOPK]
  if (tid < ntok * K) {
    flag[tid] = ldc(&topk_idx[static_cast<size_t>(t0) * K + tid]) >= 0 ? 1 : 0;
    wts[tid] = ldc(&topk_w[static_cast<size_t>(t0) * K + tid]);
  }
  __syncthreads();
  const int cpr = H >> 3;  // items per token
  if (residual != nullptr) {
    combine_units<true>(y, residual, out, wts, flag, t0, ntok * cpr, cpr, H, K);
  } else {
    combine_units<false>(y, residual, out, wts, flag, t0, ntok * cpr, cpr, H, K);
  }
  for (int tl = 0; tl < ntok; ++tl) {
    const int t = t0 + tl;
    if ((t & 63) == 0) {
      for (int e = tid; e < E; e += T_THREADS) stc(&masks[static_cast<size_t>(e) * W + (t >> 6)], 0ull);
    }
  }
  __syncthreads();  // flag[] and wts[] are reused by the next task
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
  // router tasks: 16 tokens each while one round of them covers the batch, 32 beyond that
  // (a task of 32 takes longer than one of 16, but less than two of them)
  const bool rt2 = (T + RT16_TOK - 1u) / RT16_TOK > gridDim.x;
  const unsigned rt_tok = rt2 ? 2u * RT16_TOK : 1u * RT16_TOK;
  const unsigned n_rt = (T + rt_tok - 1u) / rt_tok;
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
      st16(reinterpret_cast<char*>(r) + 32,
           u32x4{static_cast<unsigned>(t_end), static_cast<unsigned>(t_end >> 32), 0u, 0u});
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
      if (rt2) {
        tiled_router_task<2>(p, static_cast<int>(tk));
      } else {
        tiled_router_task<1>(p, static_cast<int>(tk));
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
    // The first ticket of a queue is drawn on its own; every task then draws its successor
    // while it runs, and its own completion is signalled under the next task (`pend`), so a
    // workgroup goes from one task's last store to the next task's first load without a trip
    // to memory. A completion that is still pending is signalled at once (after waiting for
    // the stores) when the next task has to wait for a dependency or there is no next task:
    // nobody may wait on a counter that a waiting workgroup holds back.
    if (threadIdx.x == 0) sh.ticket = add_relaxed(&ctl->xq[q].v, 1u);
    __syncthreads();
    unsigned j = sh.ticket;
    __syncthreads();
    unsigned* pend = nullptr;
    auto flush = [&]() {
      if (pend != nullptr) {
        fence_release();
        __syncthreads();
        if (threadIdx.x == 0) (void)add_relaxed(pend, 1u);
        pend = nullptr;
      }
    };
    while (ok) {
      const long long t_fetch = p.trace ? wall_clock64() : 0;
      if (j >= q1 + q2) break;
      long long t_ready = 0;
      if (j < q1) {
        const unsigned m = lo + j / nt1;
        if (p.trace) t_ready = wall_clock64();
        const TileDesc tile = ld_tile(&p.mtiles[m]);
        tiled_gemm_task(p, tile, static_cast<int>(j % nt1), 0, pend, &ctl->xq[q].v);
        pend = &p.g1_done[m].v;
        trace(t_dyn0 + lo * nt1 + j, 3, m, t_fetch, t_ready);
        j = task_notes()[0];
      } else {
        const unsigned jj = j - q1;
        const unsigned m = lo + jj / nt2;
        const TileDesc tile = ld_tile(&p.mtiles[m]);  // in flight while thread 0 looks at the counter
        if (pend != nullptr) {
          if (threadIdx.x == 0) sh.ok = ld_relaxed(&p.g1_done[m].v) >= nt1 ? 1u : 0u;
          __syncthreads();
          const bool ready = sh.ok != 0u;
          __syncthreads();
          if (!ready) flush();
        }
        ok = wg_wait_ge(p, &p.g1_done[m].v, nt1, &sh);
        if (ok) {
          if (p.trace) t_ready = wall_clock64();
          tiled_gemm_task(p, tile, static_cast<int>(jj % nt2), 1, pend, &ctl->xq[q].v);
          pend = &ctl->g2_done.v;
          trace(t_dyn0 + nm * nt1 + lo * nt2 + jj, 4, m, t_fetch, t_ready);
          j = task_notes()[0];
        }
      }
    }
    flush();
  }

  // ---- combine tasks from the last global counter
  if (ok && n2_total != 0u) ok = wg_wait_ge(p, &ctl->g2_done.v, n2_total, &sh);
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
    const unsigned err = ldc(&ctl->error.v);
    if (err != 0u) {
      recover_after_error(p, err, static_cast<int>(threadIdx.x), T_THREADS);
      __syncthreads();
    }
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
// y of the tiled variant: one bf16 row of H per (token, slot)
size_t tiled_y_bytes(size_t rows, size_t hidden) { return rows * hidden * 2; }

hipError_t launch_tiled_kernel(const Params& p, int grid, hipStream_t stream) {
  hipLaunchKernelGGL(moe_tiled_kernel, dim3(grid), dim3(T_THREADS), TILED_LDS_BYTES, stream, p);
  return hipGetLastError();
}

hipError_t prepare_tiled_kernel() {
  return hipFuncSetAttribute(reinterpret_cast<const void*>(moe_tiled_kernel),
                             hipFuncAttributeMaxDynamicSharedMemorySize, TILED_LDS_BYTES);
}

hipError_t tiled_kernel_occupancy(int* per_cu) {
  return hipOccupancyMaxActiveBlocksPerMultiprocessor(per_cu, moe_tiled_kernel, T_THREADS, TILED_LDS_BYTES);
}

}  // namespace fmoe
