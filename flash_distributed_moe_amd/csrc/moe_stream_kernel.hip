// Persistent MoE kernel, weight-streaming ("skinny") variant for gfx950.
//
// One workgroup per CU; every wave of every workgroup is an independent worker
// that draws task tickets from one counter in HBM. A ticket number decodes to a
// task; tasks only depend on tasks with smaller tickets, so a worker that
// holds a ticket can always wait for its dependencies: whoever holds them is
// already running. Stages (ticket order):
//   router   token t: logits in the oracle's summation order, top-k, softmax
//            over the winners, one bit per (expert, token) in `masks`
//   scan     per-expert counts / offsets from the bit masks, row-tile table
//   scatter  token t: permuted row of each of its slots (stable by token id)
//   gate/up  (row tile, 32 columns): h = silu(x.W1^T) * (x.W3^T), MFMA 16x16
//   down     (row tile, 64 columns): y = w * (h.W2^T)
//   combine  (token, 256 columns): out = sum over slots of y, in slot order
// Weights stream HBM -> registers -> MFMA with no reuse across waves, which is
// the right shape when an expert sees at most a few dozen rows (decode).
// The down projection reads h rows that other workers wrote, so its B operand
// uses coherent loads.
//
// Replaces, for this regime, the reference's moeKernel
// (src/hip/kernel/moeKernel.h:37-107), its task executors
// (src/hip/kernel/tasks/*.h) and its queue (src/hip/taskSystem/*.h).
#define FMOE_PARAMS_IN_KERNARG 1
#include "moe_device.h"

namespace fmoe {

// --------------------------------------------------------------------- router
// Follows the CPU MoE of the reference: logits accumulate the products one at a
// time in ascending k in float (test/singleGPU/cpp/moe/reference/refGemm.h:21-24),
// winners are the k largest with ties to the lower index
// (refTopk.h:36-58), weights are a softmax over the winners in double
// (refMoeGate.h:27-30, refSoftmax.h:19-52). For bf16 inputs each product is
// exact in float, so the fused multiply-add below rounds exactly as mul+add.
//
// The logits are computed by "dot" tasks: one wave takes 8 tokens x 8 experts,
// one (token, expert) chain per lane. Token rows and expert rows arrive with
// fully coalesced 16-byte loads, are converted to float once and staged in the
// wave's private LDS slice in k-chunks, and feed one sequential chain per lane
// (k ascending). Each chain ends as a 64-bit candidate key in HBM. A "select"
// task per token waits for all of the token's expert groups and picks the
// winners.
constexpr int ROUTER_KC = 256;   // k-chunk staged in LDS
constexpr int ROUTER_LD = ROUTER_KC + 4;  // LDS row stride in floats (bank spread)
constexpr int ROUTER_LDS_FLOATS = 2 * ROUTER_EXP * ROUTER_LD;  // per wave

extern __shared__ __align__(16) float lds_dyn[];  // ROUTER_LDS_FLOATS per wave

template <typename DT>
__device__ __noinline__ void router_dot_task(ParamsRef pv, int tg, int eg) {
  ParamsRef p = uniform_params(pv);
  typedef typename DT::elem elem;
  constexpr int EPV = DT::EPV;
  constexpr int CH_ROW = ROUTER_KC / EPV;               // 16-byte chunks per staged row
  constexpr int NLD = ROUTER_EXP * CH_ROW / 64;         // loads per lane per tile and chunk
  // Params is reached through a generic reference; keep what the loops need in
  // registers so that LDS stores do not force reloads.
  const int H = p.H, E = p.E, T = p.T;
  const int lane = lane_id();
  const int ti = lane >> 3, ei = lane & 7;
  const int t = tg * ROUTER_TOK + ti;
  const int e = eg * ROUTER_EXP + ei;
  float* ws = lds_dyn + (threadIdx.x >> 6) * ROUTER_LDS_FLOATS;  // [ROUTER_EXP][ROUTER_LD]
  float* xs = ws + ROUTER_EXP * ROUTER_LD;                       // [ROUTER_TOK][ROUTER_LD]
  const elem* gate = reinterpret_cast<const elem*>(p.gate);
  const elem* tokens = reinterpret_cast<const elem*>(p.tokens);

  // PF k-chunks of global loads are in flight ahead of the chunk being consumed
  constexpr int PF = 1;  // deeper prefetch measured slower (registers)
  uint4 wr[PF][NLD], xr[PF][NLD];
  auto issue = [&](uint4(&wq)[NLD], uint4(&xq)[NLD], int c0) {  // global -> registers
    if (c0 >= H) return;
    const int ch_row = min(ROUTER_KC, H - c0) / EPV;
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      // no branches around the loads: rows past the tile (short last chunk)
      // re-read the last row and are dropped when staging
      const int c = i * 64 + lane;
      const int row = min(c / ch_row, ROUTER_EXP - 1), col = c % ch_row;
      const int er = min(eg * ROUTER_EXP + row, E - 1);
      const int tr = min(tg * ROUTER_TOK + row, T - 1);
      wq[i] = ld16(gate + static_cast<size_t>(er) * H + c0 + col * EPV);
      xq[i] = ld16(tokens + static_cast<size_t>(tr) * H + c0 + col * EPV);
    }
  };
  auto stage = [&](const uint4(&wq)[NLD], const uint4(&xq)[NLD], int n) {  // -> float rows in LDS
    const int ch_row = n / EPV;
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int c = i * 64 + lane;
      const int row = c / ch_row, col = c % ch_row;
      if (row < ROUTER_EXP) {
        float wf[EPV], xf[EPV];
        unpack<DT>(wq[i], wf);
        unpack<DT>(xq[i], xf);
#pragma unroll
        for (int q = 0; q < EPV; q += 4) {
          *reinterpret_cast<float4*>(ws + row * ROUTER_LD + col * EPV + q) =
              make_float4(wf[q], wf[q + 1], wf[q + 2], wf[q + 3]);
          *reinterpret_cast<float4*>(xs + row * ROUTER_LD + col * EPV + q) =
              make_float4(xf[q], xf[q + 1], xf[q + 2], xf[q + 3]);
        }
      }
    }
  };

  float acc = 0.0f;
  const float* wrow = ws + ei * ROUTER_LD;
  const float* xrow = xs + ti * ROUTER_LD;
  auto consume = [&](int n) {
    // 32 k per block; the next block's LDS reads are in flight while this
    // block's chain runs (n is a multiple of 64)
    float4 wa[8], xa[8], wb[8], xb[8];
    auto lds_load = [&](float4(&w)[8], float4(&x)[8], int k) {
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        w[q] = *reinterpret_cast<const float4*>(wrow + k + 4 * q);
        x[q] = *reinterpret_cast<const float4*>(xrow + k + 4 * q);
      }
    };
    auto chain = [&](const float4(&w)[8], const float4(&x)[8]) {
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        if constexpr (EPV == 8) {
          acc = __builtin_fmaf(x[q].x, w[q].x, acc);
          acc = __builtin_fmaf(x[q].y, w[q].y, acc);
          acc = __builtin_fmaf(x[q].z, w[q].z, acc);
          acc = __builtin_fmaf(x[q].w, w[q].w, acc);
        } else {
          acc = __fadd_rn(acc, __fmul_rn(x[q].x, w[q].x));
          acc = __fadd_rn(acc, __fmul_rn(x[q].y, w[q].y));
          acc = __fadd_rn(acc, __fmul_rn(x[q].z, w[q].z));
          acc = __fadd_rn(acc, __fmul_rn(x[q].w, w[q].w));
        }
      }
    };
    if (n == ROUTER_KC) {
      // full chunk: straight-line code, so the two register sets simply
      // alternate and no copies are needed between blocks
      lds_load(wa, xa, 0);
#pragma unroll
      for (int k = 0; k < ROUTER_KC; k += 64) {
        lds_load(wb, xb, k + 32);
        chain(wa, xa);
        if (k + 64 < ROUTER_KC) lds_load(wa, xa, k + 64);
        chain(wb, xb);
      }
    } else {
      for (int k = 0; k < n; k += 32) {
        lds_load(wa, xa, k);
        chain(wa, xa);
      }
    }
  };

#pragma unroll
  for (int j = 0; j < PF; ++j) issue(wr[j], xr[j], j * ROUTER_KC);
  for (int c0 = 0; c0 < H; c0 += PF * ROUTER_KC) {
#pragma unroll
    for (int j = 0; j < PF; ++j) {
      const int cj = c0 + j * ROUTER_KC;
      if (cj < H) {
        const int n = min(ROUTER_KC, H - cj);
        stage(wr[j], xr[j], n);
        lds_wave_sync();
        issue(wr[j], xr[j], cj + PF * ROUTER_KC);
        consume(n);
        lds_wave_sync();
      }
    }
  }

  const bool valid = (t < T) && (e < E);
  if (valid) {
    float v = acc;
    if (p.bias != nullptr) v = __fadd_rn(v, as_global(p.bias)[e]);
    stc(&p.cand[static_cast<size_t>(t) * E + e], make_key(v, e, true));
  }
  fence_release();
  if (ei == 0 && t < T) add_relaxed(&p.tok_arrive[t], 1u);
}

// The same chains on the matrix core, for bf16 layers: V_MFMA_F32_16X16X4_F32 adds
// its four products to the accumulator one after the other in k order, one
// rounding each, so a chain of them is the same sequential sum (and a dependent
// chain issues back to back, 32 cycles an instruction: 512 of them for H = 2048
// against 2048 dependent FMAs on the vector unit). A whole workgroup takes 16
// tokens x 16 experts: wave 0 only multiplies, waves 1..4 prepare its operands so
// that it has nothing else to do: they load 32 bytes of a row (16 k), widen them
// to float and leave them in LDS in the order the instruction wants them: the 16
// k of a group as [k % 4][row][k / 4], so lane l of the multiplying wave (row
// l % 16, k % 4 = l / 16) reads its operand of four consecutive instructions with
// one 16-byte read at 16 * l. Two stages of DOT16_KC k; one workgroup barrier per
// stage; the preparing waves hold the loads of eight stages in registers.
// Called by all eight waves of the workgroup.
constexpr int DOT16_GROUPS = DOT16_KC / 16;             // 16-k groups per stage
constexpr int DOT16_OP_BYTES = DOT16_GROUPS * 1024;     // one operand of one stage
constexpr int DOT16_STAGE_BYTES = 2 * DOT16_OP_BYTES;   // expert rows, then token rows
constexpr int DOT16_AHEAD = 8;                          // stages whose loads are in flight together (even)

__device__ __noinline__ void router_dot16_task(ParamsRef pv, int tg, int eg) {
  ParamsRef p = uniform_params(pv);
  const int H = p.H, E = p.E, T = p.T;
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int nc = H / DOT16_KC;
  unsigned char* lds = reinterpret_cast<unsigned char*>(lds_dyn);
  auto barrier = [] {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  if (wave == 0) {
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
    const unsigned char* mine = lds + lane * 16;
    float4 wc, xc, wn, xn;
    barrier();  // stage 0 is written
    wc = *reinterpret_cast<const float4*>(mine);
    xc = *reinterpret_cast<const float4*>(mine + DOT16_OP_BYTES);
    for (int c = 0; c < nc; ++c) {
      const unsigned char* st = mine + (c & 1) * DOT16_STAGE_BYTES;
      const unsigned char* st_next = mine + ((c + 1) & 1) * DOT16_STAGE_BYTES;
#pragma unroll
      for (int g = 0; g < DOT16_GROUPS; ++g) {
        if (g + 1 < DOT16_GROUPS) {
          wn = *reinterpret_cast<const float4*>(st + (g + 1) * 1024);
          xn = *reinterpret_cast<const float4*>(st + DOT16_OP_BYTES + (g + 1) * 1024);
        } else {
          // every read of this stage has returned: the stage may be refilled, and
          // the next one is complete once the others have arrived too
          barrier();
          if (c + 1 < nc) {
            wn = *reinterpret_cast<const float4*>(st_next);
            xn = *reinterpret_cast<const float4*>(st_next + DOT16_OP_BYTES);
          }
        }
        // the reads of the next group go out before this group's instructions, not after
        __builtin_amdgcn_sched_barrier(0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wc.x, xc.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wc.y, xc.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wc.z, xc.z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wc.w, xc.w, acc, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        wc = wn;
        xc = xn;
      }
    }
    // acc[v] of lane l: expert 16*eg + 4*(l/16) + v, token 16*tg + l%16
    const int t = tg * 16 + (lane & 15);
    const int e0 = eg * 16 + 4 * (lane >> 4);
    if (t < T) {
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int e = e0 + v;
        if (e < E) {
          float x = acc[v];
          if (p.bias != nullptr) x = __fadd_rn(x, as_global(p.bias)[e]);
          stc(&p.cand[static_cast<size_t>(t) * E + e], make_key(x, e, true));
        }
      }
    }
    fence_release();
    if (lane < 16 && t < T) add_relaxed(&p.tok_arrive[t], 1u);
  } else if (wave <= 4) {
    // lane -> (row, group): four lanes cover 128 contiguous bytes of a row
    const int hl = (wave - 1) * 64 + lane;
    const int row = (hl & 63) >> 2;
    const int g = (hl >> 6) * 4 + (hl & 3);
    const unsigned short* wsrc = reinterpret_cast<const unsigned short*>(p.gate) +
                                 static_cast<size_t>(min(eg * 16 + row, E - 1)) * H + g * 16;
    const unsigned short* xsrc = reinterpret_cast<const unsigned short*>(p.tokens) +
                                 static_cast<size_t>(min(tg * 16 + row, T - 1)) * H + g * 16;
    unsigned char* dst = lds + g * 1024 + row * 16;
    struct Regs {
      uint4 w0, w1, x0, x1;
    };
    auto load = [&](Regs& r, int c) {
      const int k = min(c, nc - 1) * DOT16_KC;  // past the end: the last stage again, never written
      r.w0 = ld16(wsrc + k);
      r.w1 = ld16(wsrc + k + 8);
      r.x0 = ld16(xsrc + k);
      r.x1 = ld16(xsrc + k + 8);
    };
    auto widen = [](unsigned char* d, const uint4& a, const uint4& b) {
      // k % 4 = 0 and 1: low and high halves of the even words; 2 and 3: of the odd words
      *reinterpret_cast<uint4*>(d) = make_uint4(a.x << 16, a.z << 16, b.x << 16, b.z << 16);
      *reinterpret_cast<uint4*>(d + 256) =
          make_uint4(a.x & 0xFFFF0000u, a.z & 0xFFFF0000u, b.x & 0xFFFF0000u, b.z & 0xFFFF0000u);
      *reinterpret_cast<uint4*>(d + 512) = make_uint4(a.y << 16, a.w << 16, b.y << 16, b.w << 16);
      *reinterpret_cast<uint4*>(d + 768) =
          make_uint4(a.y & 0xFFFF0000u, a.w & 0xFFFF0000u, b.y & 0xFFFF0000u, b.w & 0xFFFF0000u);
    };
    // The loads of DOT16_AHEAD stages go out together (straight-line code, so each
    // stage waits for exactly its own four): a load takes 2 to 3 us to come back
    // here, three times what the multiplying wave spends on a stage.
    for (int c0 = 0; c0 < nc; c0 += DOT16_AHEAD) {
      Regs r[DOT16_AHEAD];
#pragma unroll
      for (int i = 0; i < DOT16_AHEAD; ++i) load(r[i], c0 + i);
#pragma unroll
      for (int i = 0; i < DOT16_AHEAD; ++i) {
        if (c0 + i < nc) {
          unsigned char* d = dst + (i & 1) * DOT16_STAGE_BYTES;
          widen(d, r[i].w0, r[i].w1);
          widen(d + DOT16_OP_BYTES, r[i].x0, r[i].x1);
          barrier();  // the stage is written; the multiplying wave is done with the one before
        }
      }
    }
    barrier();  // the multiplying wave has read everything: the LDS is free again
  } else {
    for (int c = 0; c <= nc; ++c) barrier();
  }
}

// All expert groups of token t have left their keys: pick the winners.
__device__ __noinline__ void router_select_task(ParamsRef pv, int t) {
  ParamsRef p = uniform_params(pv);
  constexpr int MAXEPL = MAX_EXPERTS / 64;
  const int lane = lane_id();
  unsigned val[MAXEPL];  // the ordered logit bits are the upper half of a candidate key
#pragma unroll
  for (int j = 0; j < MAXEPL; ++j) {
    const int e = lane + 64 * j;
    val[j] = e < p.E ? static_cast<unsigned>(ldc(&p.cand[static_cast<size_t>(t) * p.E + e]) >> 32) : 0u;
  }
  if (lane == 0) stc(&p.tok_arrive[t], 0u);
  router_select_max(p, t, val,
                    reinterpret_cast<double*>(lds_dyn + (threadIdx.x >> 6) * ROUTER_LDS_FLOATS));
  const unsigned old = wave_arrive(&p.ctl->router_done.v);
  if (p.early && old == static_cast<unsigned>(p.T) - 1u) broadcast_flag(p, FLAG_ROUTED);
}

// ------------------------------------------------------------- scan / scatter
// Expert counts and offsets from the selection bit masks, and the table of row
// tiles. The permutation this defines is the stable sort of (token, slot) by
// expert id: inside an expert, rows ascend by token id. The reference has no
// permutation stage (it runs one GEMV per (token, slot)); this is the
// token-grouping the streaming and tiled GEMMs need. For small batches the same
// wave also writes the permutation.
__device__ __noinline__ void scan_task(ParamsRef pv) {
  ParamsRef p = uniform_params(pv);
  const RouteTables r = route_tables(p);
  const int fuse = p.fuse_scatter;
  Control* ctl = p.ctl;
  const int lane = lane_id();
  const int epl = (r.E + 63) >> 6;
  const int wact = (r.T + 63) >> 6;
  int base = 0, tile_base = 0;
  for (int j = 0; j < epl; ++j) {
    const int e = lane + 64 * j;
    int c = 0;
    if (e < r.E) {
      const unsigned long long* m = r.masks + static_cast<size_t>(e) * r.W;
      int* wp = r.word_prefix + static_cast<size_t>(e) * r.W;
      for (int w = 0; w < wact; ++w) {
        stc(&wp[w], c);
        c += __popcll(ldc(&m[w]));
      }
    }
    const int incl = wave_inclusive_scan(c);
    const int off = base + incl - c;
    const int nt = (c + SKINNY_MT - 1) / SKINNY_MT;
    const int tincl = wave_inclusive_scan(nt);
    const int toff = tile_base + tincl - nt;
    if (e < r.E) {
      stc(&r.expert_count[e], c);
      stc(&r.expert_offset[e], off);
      for (int i = 0; i < nt; ++i) {
        if (toff + i < r.max_mtiles) {
          stc16(&r.mtiles[toff + i],
                make_uint4(static_cast<unsigned>(e), static_cast<unsigned>(off + i * SKINNY_MT),
                           static_cast<unsigned>(min(SKINNY_MT, c - i * SKINNY_MT)), nt > 1 ? 1u : 0u));
        }
      }
    }
    base += __shfl(incl, 63, 64);
    tile_base += __shfl(tincl, 63, 64);
  }
  if (lane == 0) {
    stc(&r.expert_offset[r.E], base);
    if (tile_base > r.max_mtiles) {
      or_relaxed(&ctl->error.v, ERR_CAPACITY);
      tile_base = 0;
    }
    stc(&ctl->n_mtiles.v, static_cast<unsigned>(tile_base));
  }
  fence_release();
  broadcast_flag(p, FLAG_SCAN);
  if (fuse) {
    // offsets and prefixes were written by other lanes of this wave; the
    // release above has waited for those stores
    const int n = r.T * r.K;
    constexpr int B = 8;  // entries per lane whose loads are in flight together
    for (int i0 = lane; i0 < n; i0 += 64 * B) {
      int ee[B], off[B], pre[B];
      unsigned long long mm[B];
      float ww[B];
#pragma unroll
      for (int b = 0; b < B; ++b) {
        const int i = i0 + 64 * b;
        ee[b] = i < n ? ldc(&r.topk_idx[i]) : -1;
      }
#pragma unroll
      for (int b = 0; b < B; ++b) {
        if (ee[b] >= 0) {
          const int i = i0 + 64 * b;
          const int wd = (i / r.K) >> 6;
          mm[b] = ldc(&r.masks[static_cast<size_t>(ee[b]) * r.W + wd]);
          off[b] = ldc(&r.expert_offset[ee[b]]);
          pre[b] = ldc(&r.word_prefix[static_cast<size_t>(ee[b]) * r.W + wd]);
          ww[b] = ldc(&r.topk_w[i]);
        }
      }
#pragma unroll
      for (int b = 0; b < B; ++b) {
        if (ee[b] >= 0) {
          const int i = i0 + 64 * b;
          const int t = i / r.K;
          const int pos = off[b] + pre[b] + __popcll(mm[b] & ((1ull << (t & 63)) - 1ull));
          stc(&r.perm[pos], i);
          stc(&r.row_w[pos], ww[b]);
        }
      }
    }
    fence_release();
    broadcast_flag(p, FLAG_PERM);
  }
}

// Small batches (every mask word, its prefix and every expert's offset fit the
// wave's LDS slice): the same wave also writes the permutation, looking the
// per-expert data up in LDS, so the whole stage costs two trips to memory — the
// loads of masks and routing at the start, the stores at the end.
static_assert(SCAN_LDS_WORDS * 12 + MAX_EXPERTS * 4 <= ROUTER_LDS_FLOATS * 4, "scan tables exceed the wave's LDS");

__device__ __noinline__ void scan_scatter_small_task(ParamsRef pv) {
  ParamsRef p = uniform_params(pv);
  const RouteTables r = route_tables(p);
  Control* ctl = p.ctl;
  const int lane = lane_id();
  const int epl = (r.E + 63) >> 6;
  const int wact = (r.T + 63) >> 6;
  const int n = r.T * r.K;
  unsigned long long* lmask = reinterpret_cast<unsigned long long*>(lds_dyn + (threadIdx.x >> 6) * ROUTER_LDS_FLOATS);
  int* lpre = reinterpret_cast<int*>(lmask + SCAN_LDS_WORDS);
  int* loff = lpre + SCAN_LDS_WORDS;
  constexpr int B = 8;  // routing entries per lane in flight together
  // first round of routing entries: independent of the masks, fetched alongside them
  int ee[B];
  float ww[B];
#pragma unroll
  for (int b = 0; b < B; ++b) {
    const int i = lane + 64 * b;
    ee[b] = i < n ? ldc(&r.topk_idx[i]) : -1;
    ww[b] = i < n ? ldc(&r.topk_w[i]) : 0.0f;
  }
  int base = 0, tile_base = 0;
  for (int j = 0; j < epl; ++j) {
    const int e = lane + 64 * j;
    int c = 0;
    if (e < r.E) {
      const unsigned long long* m = r.masks + static_cast<size_t>(e) * r.W;
      int* wp = r.word_prefix + static_cast<size_t>(e) * r.W;
      for (int w0 = 0; w0 < wact; w0 += 4) {
        unsigned long long mv[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) mv[q] = w0 + q < wact ? ldc(&m[w0 + q]) : 0ull;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          if (w0 + q < wact) {
            stc(&wp[w0 + q], c);
            lmask[e * wact + w0 + q] = mv[q];
            lpre[e * wact + w0 + q] = c;
            c += __popcll(mv[q]);
          }
        }
      }
    }
    const int incl = wave_inclusive_scan(c);
    const int off = base + incl - c;
    // early mode: expert e owns tile e, empty or not, and the tile holds all of the
    // expert's rows (the tasks walk through it SKINNY_MT rows at a time)
    const int nt = p.early ? (e < r.E ? 1 : 0) : (c + SKINNY_MT - 1) / SKINNY_MT;
    const int tincl = wave_inclusive_scan(nt);
    const int toff = tile_base + tincl - nt;
    if (e < r.E) {
      loff[e] = off;
      stc(&r.expert_count[e], c);
      stc(&r.expert_offset[e], off);
      for (int i = 0; i < nt; ++i) {
        if (toff + i < r.max_mtiles) {
          stc16(&r.mtiles[toff + i],
                make_uint4(static_cast<unsigned>(e), static_cast<unsigned>(off + i * SKINNY_MT),
                           static_cast<unsigned>(p.early ? c : min(SKINNY_MT, c - i * SKINNY_MT)),
                           c > SKINNY_MT ? 1u : 0u));
        }
      }
    }
    base += __shfl(incl, 63, 64);
    tile_base += __shfl(tincl, 63, 64);
  }
  if (lane == 0) {
    stc(&r.expert_offset[r.E], base);
    if (tile_base > r.max_mtiles) {
      or_relaxed(&ctl->error.v, ERR_CAPACITY);
      tile_base = 0;
    }
    stc(&ctl->n_mtiles.v, static_cast<unsigned>(tile_base));
  }
  lds_wave_sync();
  for (int i0 = lane; i0 < n; i0 += 64 * B) {
    if (i0 != lane) {
#pragma unroll
      for (int b = 0; b < B; ++b) {
        const int i = i0 + 64 * b;
        ee[b] = i < n ? ldc(&r.topk_idx[i]) : -1;
        ww[b] = i < n ? ldc(&r.topk_w[i]) : 0.0f;
      }
    }
#pragma unroll
    for (int b = 0; b < B; ++b) {
      if (ee[b] >= 0) {
        const int i = i0 + 64 * b;
        const int t = i / r.K;
        const int wi = ee[b] * wact + (t >> 6);
        const int pos = loff[ee[b]] + lpre[wi] + __popcll(lmask[wi] & ((1ull << (t & 63)) - 1ull));
        stc(&r.perm[pos], i);
        stc(&r.row_w[pos], ww[b]);
      }
    }
  }
  fence_release();
  broadcast_flag(p, FLAG_SCAN);
  broadcast_flag(p, FLAG_PERM);
  lds_wave_sync();
}

__device__ void scatter_task(ParamsRef p, int t) {
  const RouteTables r = route_tables(p);
  const int lane = lane_id();
  if (lane < r.K) scatter_entry(r, t * r.K + lane);
  const unsigned old = wave_arrive(&p.ctl->perm_done.v);
  if (old == static_cast<unsigned>(r.T) - 1u) broadcast_flag(p, FLAG_PERM);
}

// Wave-uniform bounded wait for this workgroup's copy of a phase flag. Only one
// wave of the workgroup polls HBM; the others watch a word in LDS that the
// polling wave sets (1 = flag seen, 2 = failed).
__device__ __forceinline__ bool wait_flag(ParamsRef p, int which, unsigned* lds_flag,
                                          unsigned* lds_poller) {
  int ok = 1;
  if (lane_id() == 0) {
    while (true) {
      const unsigned f = __hip_atomic_load(&lds_flag[which], __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_WORKGROUP);
      if (f != 0u) {
        ok = f == 1u;
        break;
      }
      if (__hip_atomic_exchange(&lds_poller[which], 1u, __ATOMIC_RELAXED,
                                __HIP_MEMORY_SCOPE_WORKGROUP) == 0u) {
        // this wave polls for the workgroup
        const unsigned* g = &p.wgflags[blockIdx.x].f[which];
        const long long t0 = wall_clock64();
        unsigned spins = 0;
        unsigned res = 1u;
        while (ld_relaxed(g) == 0u) {
          if ((++spins & 31u) == 0u && ld_relaxed(&p.ctl->error.v) != 0u) {
            res = 2u;
            break;
          }
          if (wall_clock64() - t0 > p.spin_limit) {
            or_relaxed(&p.ctl->error.v, ERR_TIMEOUT);
            res = 2u;
            break;
          }
          __builtin_amdgcn_s_sleep(16);
        }
        __hip_atomic_store(&lds_flag[which], res, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        ok = res == 1u;
        break;
      }
      __builtin_amdgcn_s_sleep(8);
    }
  }
  ok = __builtin_amdgcn_readfirstlane(ok);
  fence_acquire();
  return ok != 0;
}

// ------------------------------------------------- streaming 16x16 MFMA sweep
// acc[i][r] += A_i (16 weight rows) . B_r (16 token rows)^T over `ksteps` steps
// of 4*EPV elements. ap[i] / bp[r] already point at this lane's row and
// k-offset. Each round issues U steps' worth of 16-byte loads and then feeds
// the MFMAs; the other waves of the CU keep HBM busy meanwhile. `pre` runs once
// after the first round's weight loads are in flight and before any B row is
// touched (the down projection waits for its h rows there).
//
// transpose_a (the caller's row-major weights): a fragment wants lane l to hold row l % 16,
// 16-byte chunk l / 16 of a 64-byte row segment, which read that way makes every lane of a
// load touch a line of its own.
// So lane l loads chunk l % 4 of row l / 4 instead, four neighbouring lanes one contiguous
// 64-byte segment, and the fragment is put right in registers afterwards: lane l takes the
// four dwords of lane 4 * (l % 16) + l / 16 (ds_bpermute_b32: the LDS crossbar, no LDS memory).
__device__ __forceinline__ uint4 fragment_from_row_order(const uint4& v, int pull_from) {
  uint4 r;
  r.x = static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(pull_from, static_cast<int>(v.x)));
  r.y = static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(pull_from, static_cast<int>(v.y)));
  r.z = static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(pull_from, static_cast<int>(v.z)));
  r.w = static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(pull_from, static_cast<int>(v.w)));
  return r;
}
// row and 16-byte chunk (of the 64-byte segment of one k-step) that this lane loads of a
// 16-row weight block in the caller's row-major layout
__device__ __forceinline__ int row_order_row() { return lane_id() >> 2; }
__device__ __forceinline__ int row_order_chunk() { return lane_id() & 3; }

template <typename DT, int NA, int RB, int U, bool COH_B, bool transpose_a, bool once_a, typename Pre>
__device__ __forceinline__ bool stream_mma(const typename DT::elem* const (&ap)[NA],
                                           const typename DT::elem* const (&bp)[RB], int ksteps,
                                           int astep, f32x4 (&acc)[NA][RB], Pre pre,
                                           const void* bbase = nullptr, unsigned bbytes = 0) {
  // astep: elements between one k-step's A fragment and the next (4*EPV in the
  // caller's row-major layout, NA*64*EPV in the packed layout)
  constexpr int KS = 4 * DT::EPV;
  uint4 a[U][NA], b[U][RB];
  // COH_B: the B rows (inside [bbase, bbase + bbytes)) were written by other
  // workers during this launch and are read at agent scope
  const CoherentBuffer cb = coherent_buffer(bbase, bbytes);
  auto ld_b = [&](const typename DT::elem* q) {
    if (COH_B) {
      return ld16_agent(cb, static_cast<unsigned>(reinterpret_cast<const char*>(q) -
                                                  reinterpret_cast<const char*>(bbase)));
    }
    return ld16(q);
  };

  auto load_a = [&](int s) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int i = 0; i < NA; ++i) {
        // once_a: the weights have no other reader in this launch, so they pass through the
        // caches without staying (non-temporal). Not for row-major rows, which are read half a
        // line at a time: the other half comes with the next k-step and must find the line still
        // cached (with the hint it was fetched again: 64 tokens 300 -> 273 us). Not for an
        // expert with several row tiles either, whose tasks read the same weights at about the
        // same time (bf16, 30B shape, streaming variant forced: 1024 tokens 538 -> 485 us, 4096
        // tokens 1638 -> 1433 us with ordinary loads).
        a[u][i] = once_a ? ld16_once(ap[i] + static_cast<size_t>(s + u) * astep)
                         : ld16(ap[i] + static_cast<size_t>(s + u) * astep);
      }
  };
  auto load_b = [&](int s) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int r = 0; r < RB; ++r) {
        const typename DT::elem* q = bp[r] + static_cast<size_t>(s + u) * KS;
        b[u][r] = ld_b(q);
      }
  };
  const int pull_from = (((lane_id() & 15) << 2) | (lane_id() >> 4)) << 2;
  auto load_step = [&](int u, int s) {  // the loads of k-step s into slot u
#pragma unroll
    for (int i = 0; i < NA; ++i)
      a[u][i] = once_a ? ld16_once(ap[i] + static_cast<size_t>(s) * astep)
                       : ld16(ap[i] + static_cast<size_t>(s) * astep);
#pragma unroll
    for (int r = 0; r < RB; ++r) b[u][r] = ld_b(bp[r] + static_cast<size_t>(s) * KS);
  };
  auto mma_step = [&](int u) {
    if (transpose_a) {
#pragma unroll
      for (int i = 0; i < NA; ++i) a[u][i] = fragment_from_row_order(a[u][i], pull_from);
    }
#pragma unroll
    for (int i = 0; i < NA; ++i)
#pragma unroll
      for (int r = 0; r < RB; ++r) acc[i][r] = mma16<DT>(a[u][i], b[u][r], acc[i][r]);
  };

  // One block of 16 rows (ROLL): the window of U k-steps is filled once; from then on a slot
  // is asked for again as soon as its matrix instructions have read it, so the wave keeps
  // U - 1 steps' loads in flight all the time instead of a burst per round that drains
  // before the next one (a bare read loop of the same loads on all CUs: 4.7 TB/s in bursts,
  // 6.3 TB/s refilled slot by slot). With more row blocks the bursts do better (two blocks:
  // 256 tokens 272 -> 275 us, 235B shape 853 -> 867 us with refills), and so they do on
  // row-major weights (64 tokens 272 against 275 us: a line's second half, asked for one
  // step after the first, misses more often behind a steady stream of other requests).
  constexpr bool ROLL = RB == 1 && !transpose_a;
  auto mma = [&]() {
#pragma unroll
    for (int u = 0; u < U; ++u) mma_step(u);
  };
  const int main_steps = (ksteps / U) * U;
  int s = 0;
  if (main_steps > 0) {
    load_a(0);
    __builtin_amdgcn_sched_barrier(0);
    if (!pre()) return false;
    load_b(0);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (ROLL) {
      auto round = [&]() {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          mma_step(u);
          __builtin_amdgcn_sched_barrier(0);
          load_step(u, s + U + u);
          __builtin_amdgcn_sched_barrier(0);
        }
        s += U;
      };
      // The first round stands in front of the loop: the window's first loads were issued
      // operand by operand (every weight load, then every token load), later ones step by
      // step, and the compiler counts the loads a step may leave in flight from both orders
      // wherever the two meet (with the first round inside the loop every round's first step
      // waited until 7 loads were left of 40).
      if (s + 2 * U <= main_steps) {
        round();
        asm volatile("; end of the first round" ::: "memory");  // keeps it apart from the loop
        while (s + 2 * U <= main_steps) round();
      }
      mma();
      s += U;
    } else {
      mma();
      s = U;
      for (; s < main_steps; s += U) {
        __builtin_amdgcn_sched_barrier(0);
        load_a(s);
        load_b(s);
        __builtin_amdgcn_sched_barrier(0);
        mma();
      }
    }
  } else {
    if (!pre()) return false;
  }
  for (; s < ksteps; ++s) {  // remainder when ksteps is not a multiple of U
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      uint4 av = once_a ? ld16_once(ap[i] + static_cast<size_t>(s) * astep)
                        : ld16(ap[i] + static_cast<size_t>(s) * astep);
      if (transpose_a) av = fragment_from_row_order(av, pull_from);
#pragma unroll
      for (int r = 0; r < RB; ++r) {
        const typename DT::elem* q = bp[r] + static_cast<size_t>(s) * KS;
        acc[i][r] = mma16<DT>(av, ld_b(q), acc[i][r]);
      }
    }
  }
  return true;
}

// Steps per load round, by rows blocks of the tile: keeps a round near 32-40
// loads of 16 bytes per lane.
template <int NA, int RB>
struct RoundSteps {
  static constexpr int value = RB == 1 ? (NA <= 2 ? 16 : 8) : (RB == 2 ? (NA <= 2 ? 8 : 4) : 4);
};

// -------------------------------------------------------------------- gate/up
// h[row, n0 .. n0+16*G1_NB) for the rows of one tile. Follows
// refExpertFFN1.h:51-65 (two GEMMs against the [2I,H] expert matrix, then
// SiLU(gate) * up), accumulated on MFMA in float.
// The row tile of expert e read off the top-k table alone: its rows are the
// entries i = token*K + slot that name e, in ascending i (the order the
// permutation gives them), and its first row is the number of entries that name
// a lower expert. Lanes 0..15 (and their copies in the other lane groups) get
// the entry of row min(lane & 15, rows - 1). The table is read 512 entries at a time.
template <int RB>
__device__ __forceinline__ void tile_from_topk(ParamsRef p, int e, int& row0, int& rows,
                                               int (&entry)[RB]) {
  const int lane = lane_id();
  const int r16 = lane & 15;
  const int n = p.T * p.K;
  int cnt = 0, lt = 0;
  int idx[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) idx[r] = 0;
  constexpr int B = 8;  // entries per lane in flight together
  for (int i0 = 0; i0 < n; i0 += 64 * B) {
    int ee[B];
#pragma unroll
    for (int b = 0; b < B; ++b) {
      const int i = i0 + 64 * b + lane;
      ee[b] = i < n ? ldc(&p.topk_idx[i]) : -1;
    }
#pragma unroll
    for (int b = 0; b < B; ++b) {
      const unsigned long long m = __ballot(ee[b] == e);
      lt += __popcll(__ballot(ee[b] >= 0 && ee[b] < e));
      const int pc = __popcll(m);
#pragma unroll
      for (int r = 0; r < RB; ++r) {
        const int want = r * 16 + r16;  // this lane keeps the entries of rows r16, 16 + r16, ...
        if (want >= cnt && want < cnt + pc) {
          unsigned long long mm = m;
          for (int j = cnt; j < want; ++j) mm &= mm - 1ull;
          idx[r] = i0 + 64 * b + static_cast<int>(__builtin_ctzll(mm));
        }
      }
      cnt += pc;
    }
  }
  row0 = lt;
  rows = cnt;
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    // row r*16 + r16, or the last row when the tile is shorter: held by lane (row % 16) as entry row / 16
    const int row = max(min(r * 16 + r16, cnt - 1), 0);
    int v = 0;
#pragma unroll
    for (int q = 0; q < RB; ++q) {
      const int got = __shfl(idx[q], row & 15, 64);
      if ((row >> 4) == q) v = got;
    }
    entry[r] = v;
  }
}

// EARLY (small batches: every expert owns the row tile of its own index, empty
// or not, so tile -> weights is known at launch): the task is taken before the
// routing exists. It issues its first round of weight loads at once, then waits
// until every token's top-k entries are final and reads its rows off that table
// (the scan and the permutation are only needed by the down tasks), so one round
// of HBM latency and transfer per worker, and the scan, are off the critical path.
// Returns 0: done (or the tile is empty), 1: the wait failed, 2 (EARLY only):
// the tile has more than 16*RB rows, nothing was written, and the caller runs
// the task again from the tile table with more row blocks.
template <typename DT, int RB, bool EARLY>
__device__ __forceinline__ int gateup_body(ParamsRef p, TileDesc& tile, int nblk,
                                           unsigned* lds_flag, unsigned* lds_poller) {
  typedef typename DT::elem elem;
  constexpr int EPV = DT::EPV;
  constexpr int NA = 2 * G1_NB;
  constexpr int U = RoundSteps<NA, RB>::value;
  const int lane = lane_id();
  const int r16 = lane & 15, g = lane >> 4;
  const int n0 = nblk * (16 * G1_NB);

  const elem* ap[NA];
  int astep = 4 * EPV;
  if (p.ffn1_packed != nullptr) {
    // this task's slice: [k-step][NA blocks][64 lanes][EPV]
    const size_t task = static_cast<size_t>(tile.expert) * (p.I / (16 * G1_NB)) + nblk;
    const elem* base = reinterpret_cast<const elem*>(p.ffn1_packed) +
                       task * (static_cast<size_t>(p.H / (4 * EPV)) * NA * 64 * EPV);
#pragma unroll
    for (int i = 0; i < NA; ++i) ap[i] = base + (i * 64 + lane) * EPV;
    astep = NA * 64 * EPV;
  } else {
    const elem* w13 = reinterpret_cast<const elem*>(p.ffn1) +
                      static_cast<size_t>(tile.expert) * 2 * p.I * p.H;
    const int wr = row_order_row(), wc = row_order_chunk();
#pragma unroll
    for (int b = 0; b < G1_NB; ++b) {
      ap[b] = w13 + static_cast<size_t>(n0 + 16 * b + wr) * p.H + wc * EPV;                // gate
      ap[G1_NB + b] = w13 + static_cast<size_t>(p.I + n0 + 16 * b + wr) * p.H + wc * EPV;  // up
    }
  }
  const bool row_major = p.ffn1_packed == nullptr;
  const elem* bp[RB];
  auto token_rows = [&] {
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      const int row = min(r * 16 + r16, tile.rows - 1);
      const int tok = ldc(&p.perm[tile.row0 + row]) / p.K;
      bp[r] = reinterpret_cast<const elem*>(p.tokens) + static_cast<size_t>(tok) * p.H + g * EPV;
    }
  };
  if (!EARLY) token_rows();
  f32x4 acc[NA][RB];
#pragma unroll
  for (int i = 0; i < NA; ++i)
#pragma unroll
    for (int r = 0; r < RB; ++r) acc[i][r] = f32x4{0.f, 0.f, 0.f, 0.f};

  int status = 0;
  auto before_rows = [&] {
    if (EARLY) {
      if (!wait_flag(p, FLAG_ROUTED, lds_flag, lds_poller)) {
        status = 1;
        return false;
      }
      int entry[RB];
      tile_from_topk<RB>(p, tile.expert, tile.row0, tile.rows, entry);
      if (tile.rows == 0) return false;
      if (tile.rows > 16 * RB) {
        status = 2;
        return false;
      }
#pragma unroll
      for (int r = 0; r < RB; ++r)
        bp[r] = reinterpret_cast<const elem*>(p.tokens) + static_cast<size_t>(entry[r] / p.K) * p.H + g * EPV;
    }
    return true;
  };
  // (two instantiations: a run-time switch inside the sweep cost the packed path 6 %)
  const bool ran =
      row_major ? stream_mma<DT, NA, RB, U, false, true, false>(ap, bp, p.H / (4 * EPV), astep, acc, before_rows)
      : tile.shared != 0
          ? stream_mma<DT, NA, RB, U, false, false, false>(ap, bp, p.H / (4 * EPV), astep, acc, before_rows)
          : stream_mma<DT, NA, RB, U, false, false, true>(ap, bp, p.H / (4 * EPV), astep, acc, before_rows);
  if (!ran) return status;

#pragma unroll
  for (int r = 0; r < RB; ++r) {
    const int row = r * 16 + r16;
    if (row < tile.rows) {
#pragma unroll
      for (int b = 0; b < G1_NB; ++b) {
        float hv[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) hv[v] = silu_mul(acc[b][r][v], acc[G1_NB + b][r][v]);
        const size_t off = static_cast<size_t>(tile.row0 + row) * p.I + n0 + 16 * b + 4 * g;
        if constexpr (EPV == 8) {
          const unsigned lo = f2bf(hv[0]) | (f2bf(hv[1]) << 16);
          const unsigned hi = f2bf(hv[2]) | (f2bf(hv[3]) << 16);
          stc(reinterpret_cast<unsigned long long*>(reinterpret_cast<unsigned short*>(p.h) + off),
              static_cast<unsigned long long>(lo) | (static_cast<unsigned long long>(hi) << 32));
        } else {
          stc16(reinterpret_cast<float*>(p.h) + off,
                make_uint4(__float_as_uint(hv[0]), __float_as_uint(hv[1]), __float_as_uint(hv[2]),
                           __float_as_uint(hv[3])));
        }
      }
    }
  }
  return 0;
}

template <typename DT, int RB>
__device__ __noinline__ void gateup_task(ParamsRef pv, int expert, int row0, int rows, int nblk, int shared) {
  // (the row tile arrives as three integers: a struct by value makes the callee save
  // and restore every callee-saved register it touches, a struct by reference costs
  // a trip to the caller's private memory)
  ParamsRef p = uniform_params(pv);
  TileDesc tile;
  tile.expert = expert;
  tile.row0 = row0;
  tile.rows = rows;
  tile.shared = __builtin_amdgcn_readfirstlane(shared);
  gateup_body<DT, RB, false>(p, tile, nblk, nullptr, nullptr);
}

// the rows of the expert's tile are worked out inside, once the routing is known
template <typename DT, int RB>
__device__ __noinline__ int gateup_early_task(ParamsRef pv, int expert, int nblk,
                                              unsigned* lds_flag, unsigned* lds_poller) {
  ParamsRef p = uniform_params(pv);
  TileDesc tile;
  tile.expert = expert;
  tile.row0 = 0;
  tile.rows = 0;
  tile.shared = 0;
  return gateup_body<DT, RB, true>(p, tile, nblk, lds_flag, lds_poller);
}

// ----------------------------------------------------------------------- down
// y[t*K+slot, n0 .. n0+16*G2_NB) = w * (h[row] . W2[e]^T): refFullMoe.h:58-65
// with the gate weight applied before the slot sum, as the reference GPU path
// does (src/hip/kernel/tasks/ffn2Task.h:37-40). The weight rows do not depend
// on h, so their first loads are issued before the wait for the tile's
// gate/up tasks. Returns false if that wait failed.
template <typename DT, int RB>
__device__ __noinline__ bool down_task(ParamsRef pv, int expert, int row0, int rows, int nblk, int shared,
                                       unsigned* dep, unsigned dep_target) {
  ParamsRef p = uniform_params(pv);
  TileDesc tile;
  tile.expert = expert;
  tile.row0 = row0;
  tile.rows = rows;
  tile.shared = __builtin_amdgcn_readfirstlane(shared);
  typedef typename DT::elem elem;
  constexpr int EPV = DT::EPV;
  constexpr int NA = G2_NB;
  constexpr int U = RoundSteps<NA, RB>::value;
  const int lane = lane_id();
  const int r16 = lane & 15, g = lane >> 4;
  const int n0 = nblk * (16 * G2_NB);

  const elem* ap[NA];
  int astep = 4 * EPV;
  if (p.ffn2_packed != nullptr) {
    const size_t task = static_cast<size_t>(tile.expert) * (p.H / (16 * G2_NB)) + nblk;
    const elem* base = reinterpret_cast<const elem*>(p.ffn2_packed) +
                       task * (static_cast<size_t>(p.I / (4 * EPV)) * NA * 64 * EPV);
#pragma unroll
    for (int i = 0; i < NA; ++i) ap[i] = base + (i * 64 + lane) * EPV;
    astep = NA * 64 * EPV;
  } else {
    const elem* w2 =
        reinterpret_cast<const elem*>(p.ffn2) + static_cast<size_t>(tile.expert) * p.H * p.I;
    const int wr = row_order_row(), wc = row_order_chunk();
#pragma unroll
    for (int b = 0; b < NA; ++b)
      ap[b] = w2 + static_cast<size_t>(n0 + 16 * b + wr) * p.I + wc * EPV;
  }
  const bool row_major = p.ffn2_packed == nullptr;
  // the part of h this tile reads (uniform; the offsets inside it fit 32 bits)
  const size_t hrow0 = static_cast<size_t>(tile.row0);
  const elem* hbase = uniform_ptr(reinterpret_cast<const elem*>(p.h) + hrow0 * p.I);
  const unsigned hbytes = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(
      tile.rows * p.I * static_cast<int>(sizeof(elem))));
  const elem* bp[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    const int row = min(r * 16 + r16, tile.rows - 1);
    const size_t hrow = static_cast<size_t>(tile.row0 + row);
    bp[r] = reinterpret_cast<const elem*>(p.h) + hrow * p.I + g * EPV;
  }
  // gate weight and destination of this lane's rows: fetched now, so that their
  // latency is spent under the weight stream and not in the epilogue
  float roww[RB];
  int dstrow[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    const int row = min(r * 16 + r16, tile.rows - 1);
    roww[r] = ldc(&p.row_w[tile.row0 + row]);
    dstrow[r] = ldc(&p.perm[tile.row0 + row]);
  }
  f32x4 acc[NA][RB];
#pragma unroll
  for (int i = 0; i < NA; ++i)
#pragma unroll
    for (int r = 0; r < RB; ++r) acc[i][r] = f32x4{0.f, 0.f, 0.f, 0.f};

  // The h rows are read at agent scope: two gate/up tasks, possibly on different
  // XCDs, each write half of a 128-byte line of h, so this XCD's L2 may hold a
  // line one of its own tasks wrote before the other half existed.
  auto wait_for_rows = [&] { return wave_wait_ge(dep, dep_target, p.ctl, p.spin_limit); };
  const bool ok =
      row_major ? stream_mma<DT, NA, RB, U, true, true, false>(ap, bp, p.I / (4 * EPV), astep, acc, wait_for_rows,
                                                               hbase, hbytes)
      : tile.shared != 0
          ? stream_mma<DT, NA, RB, U, true, false, false>(ap, bp, p.I / (4 * EPV), astep, acc, wait_for_rows,
                                                          hbase, hbytes)
          : stream_mma<DT, NA, RB, U, true, false, true>(ap, bp, p.I / (4 * EPV), astep, acc, wait_for_rows,
                                                         hbase, hbytes);
  if (!ok) return false;

  float* const ybase = p.y + n0 + 4 * g;
  const size_t ystride = static_cast<size_t>(p.H);
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    const int row = r * 16 + r16;
    if (row < tile.rows) {
      const float w = roww[r];
      float* const yrow = ybase + static_cast<size_t>(dstrow[r]) * ystride;
#pragma unroll
      for (int b = 0; b < NA; ++b) {
        st16_through(yrow + 16 * b,
              make_uint4(__float_as_uint(acc[b][r][0] * w), __float_as_uint(acc[b][r][1] * w),
                         __float_as_uint(acc[b][r][2] * w), __float_as_uint(acc[b][r][3] * w)));
      }
    }
  }
  return true;
}

// -------------------------------------------------------------------- combine
// out[t, c0..c0+256) = sum over slots, in slot order, of the weighted rows
// (refFullMoe.h:35,62-65; src/hip/kernel/tasks/internal/reduceBlock.h:35-53).
template <typename DT>
__device__ void combine_task(ParamsRef p, int t, int chunk) {
  const int lane = lane_id();
  const int c = chunk * COMBINE_COLS + lane * 4;
  if (c < p.H) {
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    // eight slots at a time: their validity and their rows are loaded together
    // (one memory latency per group instead of two per slot), then added in slot order
    for (int k0 = 0; k0 < p.K; k0 += 8) {
      int idx[8];
      uint4 v[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const int kk = min(k0 + k, p.K - 1);
        idx[k] = ldc(&p.topk_idx[static_cast<size_t>(t) * p.K + kk]);
        v[k] = ld16_once(p.y + (static_cast<size_t>(t) * p.K + kk) * p.H + c);
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        if (k0 + k < p.K && idx[k] >= 0) {
          s.x += __uint_as_float(v[k].x);
          s.y += __uint_as_float(v[k].y);
          s.z += __uint_as_float(v[k].z);
          s.w += __uint_as_float(v[k].w);
        }
      }
    }
    const size_t off = static_cast<size_t>(t) * p.H + c;
    if (p.residual != nullptr) {  // output = input row + layer, the row added last
      if constexpr (DT::EPV == 8) {
        const unsigned long long xx = *as_global(
            reinterpret_cast<const unsigned long long*>(reinterpret_cast<const unsigned short*>(p.residual) + off));
        const uint2 x = make_uint2(static_cast<unsigned>(xx), static_cast<unsigned>(xx >> 32));
        s.x += bf16_lo(x.x);
        s.y += bf16_hi(x.x);
        s.z += bf16_lo(x.y);
        s.w += bf16_hi(x.y);
      } else {
        const uint4 x = ld16(reinterpret_cast<const float*>(p.residual) + off);
        s.x += __uint_as_float(x.x);
        s.y += __uint_as_float(x.y);
        s.z += __uint_as_float(x.z);
        s.w += __uint_as_float(x.w);
      }
    }
    if constexpr (DT::EPV == 8) {
      uint2 pk;
      pk.x = f2bf(s.x) | (f2bf(s.y) << 16);
      pk.y = f2bf(s.z) | (f2bf(s.w) << 16);
      *reinterpret_cast<uint2*>(reinterpret_cast<unsigned short*>(p.out) + off) = pk;
    } else {
      *reinterpret_cast<float4*>(reinterpret_cast<float*>(p.out) + off) = s;
    }
  }
  // the selection masks are dead once the permutation is written: clear this
  // token block's words for the next launch
  if (chunk == 0 && (t & 63) == 0) {
    for (int e = lane; e < p.E; e += 64) stc(&p.masks[static_cast<size_t>(e) * p.W + (t >> 6)], 0ull);
  }
}

// The combine items slot, slot + n_workers, ... of one worker (a function of its
// own so that the worker loop's registers are not shared with it).
template <typename DT>
__device__ __noinline__ void combine_items(ParamsRef pv, unsigned slot, unsigned nc,
                                           unsigned ncomb, unsigned worker, unsigned id0,
                                           long long t_fetch) {
  ParamsRef p = uniform_params(pv);
  const int lane = lane_id();
  for (unsigned q = slot; q < nc; q += static_cast<unsigned>(p.n_workers)) {
    const long long t_item = p.trace ? wall_clock64() : 0;
    combine_task<DT>(p, static_cast<int>(q / ncomb), static_cast<int>(q % ncomb));
    const unsigned id = id0 + q;
    if (p.trace && lane == 0 && id < p.trace_cap) {
      const long long t_end = wall_clock64();
      TraceRec* r = p.trace + id;
      st16(r, u32x4{id, 5u, worker, q / ncomb});
      st16(reinterpret_cast<char*>(r) + 16,
           u32x4{static_cast<unsigned>(t_fetch), static_cast<unsigned>(t_fetch >> 32),
                 static_cast<unsigned>(t_item), static_cast<unsigned>(t_item >> 32)});
      st16(reinterpret_cast<char*>(r) + 32,
           u32x4{static_cast<unsigned>(t_end), static_cast<unsigned>(t_end >> 32), 0u, 0u});
    }
  }
}

// ---------------------------------------------------------------- worker loop
// Nothing the tasks are called with lives in the wave's private memory: the
// launch parameters are read in place (ParamsRef), a row tile travels as three
// integers. A trip to private memory goes through the vector memory pipeline,
// behind the weight loads of all eight waves, and cost every task several
// microseconds (30B shape, T = 64: 263 -> 230 us without them).
// disable_tail_calls: once no argument points into the caller's frame the
// compiler marks the task calls as possible tail calls, and a function with such
// a call site loses the treatment local functions get here (no callee-saved
// registers, the caller knows what the callee clobbers): every task would save
// and restore some fifty registers through private memory. The attribute
// keeps the marks off.
template <typename DT>
__global__ __launch_bounds__(512) __attribute__((disable_tail_calls)) void moe_stream_kernel(
    const Params params) {
  ParamsRef p = kernel_params();
  __shared__ unsigned lds_flag[4];
  __shared__ unsigned lds_poller[4];
  if (threadIdx.x < 4) {
    lds_flag[threadIdx.x] = 0u;
    lds_poller[threadIdx.x] = 0u;
  }
  __syncthreads();
  const int lane = lane_id();
  const int wave_in_group = threadIdx.x >> 6;
  const int waves_per_group = blockDim.x >> 6;
  Control* ctl = p.ctl;
  const unsigned T = static_cast<unsigned>(p.T);
  // dot tasks: 8 x 8 chains per wave, or (dot16) 16 x 16 per workgroup; those are
  // not drawn, workgroup b < n_dot runs number b before its waves take tickets
  const bool dot16 = p.dot16 != 0;
  const unsigned dot_side = dot16 ? 16u : static_cast<unsigned>(ROUTER_EXP);
  static_assert(ROUTER_EXP == ROUTER_TOK, "square dot tasks");
  const unsigned n_eg = (static_cast<unsigned>(p.E) + dot_side - 1u) / dot_side;
  const unsigned n_tg = (T + dot_side - 1u) / dot_side;
  const unsigned n_dot = n_tg * n_eg;
  const unsigned n_router = n_dot + T;  // dot tasks, then one select task per token
  const unsigned t_scan = n_router;
  const unsigned t_scatter0 = n_router + 1u;
  const unsigned nt1 = static_cast<unsigned>(p.I / (16 * G1_NB));
  const unsigned t_dyn0 = t_scatter0 + (p.fuse_scatter ? 0u : T);
  const unsigned nt2 = static_cast<unsigned>(p.H / (16 * G2_NB));
  const unsigned ncomb = static_cast<unsigned>((p.H + COMBINE_COLS - 1) / COMBINE_COLS);
  const unsigned worker = blockIdx.x * waves_per_group + wave_in_group;
  unsigned n1 = 0, n2 = 0, nc = 0;
  bool have_dyn = false, perm_ready = false;
  if (p.early) {  // one row tile per expert: the task counts do not depend on the routing
    n1 = static_cast<unsigned>(p.E) * nt1;
    n2 = static_cast<unsigned>(p.E) * nt2;
    nc = T * ncomb;
    have_dyn = true;
  }

  // The first ticket of every worker is fixed (wave w of every workgroup before
  // wave w+1 of any, so the first tasks spread over all CUs); the shared counter
  // hands out the tickets after those.
  const unsigned n_workers = static_cast<unsigned>(p.n_workers);
  bool first = true;
  const unsigned n_skip = dot16 ? n_dot : 0u;
  unsigned first_tk = n_skip + static_cast<unsigned>(wave_in_group) * gridDim.x + blockIdx.x;
  unsigned dyn_base = n_skip + n_workers;  // tickets below this are handed out statically
  unsigned late_lo = 0xFFFFFFFFu, late_skip = 0u;  // early mode: static tickets [late_lo, late_lo + late_skip)
  if (p.early) {
    // The other workers start streaming weights at once, and a routing task
    // whose loads queue behind those in its CU's memory pipeline runs a third
    // slower. So the routing tasks sit together on the first workgroups: dot
    // tasks on waves 0..3 (one per SIMD), select and scan tasks on waves 4..7.
    // Workers of those workgroups without a routing task take dynamic tickets.
    const unsigned nr = max(dot16 ? n_dot : (n_dot + 3u) / 4u, (T + 4u) / 4u);
    const unsigned rest = gridDim.x - nr;
    dyn_base = n_router + 1u + 8u * rest;
    if (n1 >= 8u * rest) {
      late_skip = 4u * rest;
      late_lo = t_dyn0 + n1 - late_skip;
      dyn_base = t_dyn0 + late_skip;
    }
    if (blockIdx.x >= nr) {
      first_tk = n_router + 1u + static_cast<unsigned>(wave_in_group) * rest + (blockIdx.x - nr);
      // A CU's waves 4..7 stream at half the rate of waves 0..3 while both run, so
      // their first tasks end last of all (140-155 us against 70-80 at T = 64 on
      // the 30B shape). They take the gate/up tasks of the last experts, whose down
      // tasks are drawn last anyway; the tickets in between are drawn by the waves
      // that finish first.
      if (late_skip != 0u && wave_in_group >= 4)
        first_tk = late_lo + (static_cast<unsigned>(wave_in_group) - 4u) * rest + (blockIdx.x - nr);
    } else {
      const unsigned q = blockIdx.x * 4u + (static_cast<unsigned>(wave_in_group) & 3u);
      if (wave_in_group < 4) {
        first_tk = q;
        first = !dot16 && q < n_dot;
      } else {
        first_tk = n_dot + q;  // q == T: the scan
        first = q <= T;
      }
    }
  }

  if (dot16 && blockIdx.x < n_dot) {
    const long long t0 = p.trace ? wall_clock64() : 0;
    router_dot16_task(p, static_cast<int>(blockIdx.x / n_eg), static_cast<int>(blockIdx.x % n_eg));
    if (p.trace && threadIdx.x == 0 && blockIdx.x < p.trace_cap) {
      const long long t1 = wall_clock64();
      TraceRec* r = p.trace + blockIdx.x;
      st16(r, u32x4{blockIdx.x, 0u, worker, blockIdx.x});
      st16(reinterpret_cast<char*>(r) + 16,
           u32x4{static_cast<unsigned>(t0), static_cast<unsigned>(t0 >> 32),
                 static_cast<unsigned>(t0), static_cast<unsigned>(t0 >> 32)});
      st16(reinterpret_cast<char*>(r) + 32,
           u32x4{static_cast<unsigned>(t1), static_cast<unsigned>(t1 >> 32), 0u, 0u});
    }
  }

  while (true) {
    const long long t_fetch = p.trace ? wall_clock64() : 0;
    unsigned tk = first_tk;
    if (!first) {
      if (lane == 0) tk = dyn_base + add_relaxed(&ctl->ticket.v, 1u);
      tk = __builtin_amdgcn_readfirstlane(tk);
      if (tk >= late_lo) tk += late_skip;  // early mode: over the late waves' static tickets
    }
    first = false;
    unsigned kind = 0, aux = 0;
    long long t_ready = 0;

    if (tk < n_dot) {
      kind = 0;
      aux = tk;
      if (p.trace) t_ready = wall_clock64();
      router_dot_task<DT>(p, static_cast<int>(tk / n_eg), static_cast<int>(tk % n_eg));
    } else if (tk < n_router) {
      kind = 6;
      aux = tk - n_dot;
      if (!wave_wait_ge(&p.tok_arrive[aux], n_eg, ctl, p.spin_limit)) break;
      if (p.trace) t_ready = wall_clock64();
      router_select_task(p, static_cast<int>(aux));
    } else if (tk == t_scan) {
      kind = 1;
      if (!wave_wait_ge(&ctl->router_done.v, T, ctl, p.spin_limit)) break;
      if (p.trace) t_ready = wall_clock64();
      if (p.fuse_scatter && p.E * ((p.T + 63) >> 6) <= SCAN_LDS_WORDS) {
        scan_scatter_small_task(p);
      } else {
        scan_task(p);
      }
    } else if (tk < t_dyn0) {
      kind = 2;
      aux = tk - t_scatter0;
      if (!wait_flag(p, FLAG_SCAN, lds_flag, lds_poller)) break;
      if (p.trace) t_ready = wall_clock64();
      scatter_task(p, static_cast<int>(aux));
    } else {
      if (!have_dyn) {
        if (!wait_flag(p, FLAG_SCAN, lds_flag, lds_poller)) break;
        const unsigned nm = ldc(&ctl->n_mtiles.v);
        n1 = nm * nt1;
        n2 = nm * nt2;
        nc = T * ncomb;
        have_dyn = true;
      }
      const unsigned j = tk - t_dyn0;
      if (j < n1 && p.early) {
        kind = 3;
        aux = j / nt1;  // tile = expert
        if (p.trace) t_ready = wall_clock64();
        const int nblk = static_cast<int>(j % nt1);
        TileDesc tile;
        tile.expert = static_cast<int>(aux);
        tile.row0 = 0;
        tile.rows = 0;
        tile.shared = 0;
        // (p.early is the number of 16-row blocks an early task carries)
        const int st = p.early == 1
                           ? gateup_early_task<DT, 1>(p, tile.expert, nblk, lds_flag, lds_poller)
                           : gateup_early_task<DT, 2>(p, tile.expert, nblk, lds_flag, lds_poller);
        if (st == 1) break;
        if (st == 2) {
          if (!perm_ready) {
            if (!wait_flag(p, FLAG_PERM, lds_flag, lds_poller)) break;
            perm_ready = true;
          }
          tile = ld_tile(&p.mtiles[aux]);
          for (int r0 = 0; r0 < tile.rows; r0 += SKINNY_MT) {
            const int rc = min(SKINNY_MT, tile.rows - r0);
            if (rc <= 16) {
              gateup_task<DT, 1>(p, tile.expert, tile.row0 + r0, rc, nblk, 1);
            } else if (rc <= 32) {
              gateup_task<DT, 2>(p, tile.expert, tile.row0 + r0, rc, nblk, 1);
            } else {
              gateup_task<DT, 4>(p, tile.expert, tile.row0 + r0, rc, nblk, 1);
            }
          }
        }
        wave_arrive(&p.g1_done[aux].v);
      } else if (j < n1) {
        kind = 3;
        aux = j / nt1;
        if (!perm_ready) {
          if (!wait_flag(p, FLAG_PERM, lds_flag, lds_poller)) break;
          perm_ready = true;
        }
        if (p.trace) t_ready = wall_clock64();
        const TileDesc tile = ld_tile(&p.mtiles[aux]);
        const int nblk = static_cast<int>(j % nt1);
        if (tile.rows <= 16) {
          gateup_task<DT, 1>(p, tile.expert, tile.row0, tile.rows, nblk, tile.shared);
        } else if (tile.rows <= 32) {
          gateup_task<DT, 2>(p, tile.expert, tile.row0, tile.rows, nblk, tile.shared);
        } else {
          gateup_task<DT, 4>(p, tile.expert, tile.row0, tile.rows, nblk, tile.shared);
        }
        wave_arrive(&p.g1_done[aux].v);
      } else if (j < n1 + n2) {
        kind = 4;
        aux = (j - n1) / nt2;
        const int nblk = static_cast<int>((j - n1) % nt2);
        if (p.early && !perm_ready) {  // nothing has waited for the tile table yet
          if (!wait_flag(p, FLAG_PERM, lds_flag, lds_poller)) break;
          perm_ready = true;
        }
        if (p.trace) t_ready = wall_clock64();
        const TileDesc tile = ld_tile(&p.mtiles[aux]);
        bool ok;
        {
          // the task reads its rows' gate weights and destinations up front
          if (!perm_ready) {
            if (!wait_flag(p, FLAG_PERM, lds_flag, lds_poller)) break;
            perm_ready = true;
          }
          unsigned* dep = &p.g1_done[aux].v;
          // early mode keeps the tiles of unused experts (no rows) and gives an expert
          // one tile however many rows it holds; otherwise this is a single pass
          if (tile.rows == 0) {
            ok = true;
          } else if (tile.rows <= 16) {
            ok = down_task<DT, 1>(p, tile.expert, tile.row0, tile.rows, nblk, tile.shared, dep, nt1);
          } else if (tile.rows <= 32) {
            ok = down_task<DT, 2>(p, tile.expert, tile.row0, tile.rows, nblk, tile.shared, dep, nt1);
          } else if (tile.rows <= SKINNY_MT) {
            ok = down_task<DT, 4>(p, tile.expert, tile.row0, tile.rows, nblk, tile.shared, dep, nt1);
          } else {
            ok = true;
            for (int r0 = 0; ok && r0 < tile.rows; r0 += SKINNY_MT) {
              const int rc = min(SKINNY_MT, tile.rows - r0);
              if (rc <= 16) {
                ok = down_task<DT, 1>(p, tile.expert, tile.row0 + r0, rc, nblk, 1, dep, nt1);
              } else if (rc <= 32) {
                ok = down_task<DT, 2>(p, tile.expert, tile.row0 + r0, rc, nblk, 1, dep, nt1);
              } else {
                ok = down_task<DT, 4>(p, tile.expert, tile.row0 + r0, rc, nblk, 1, dep, nt1);
              }
            }
          }
        }
        if (!ok) break;
        const unsigned old = wave_arrive(&ctl->g2_done.v);
        if (old == n2 - 1u) broadcast_flag(p, FLAG_G2);
      } else {
        // Every gate/up and down ticket has been handed out. The combine items
        // need no order among themselves, so they are not ticketed one by one (a
        // counter hands out only about 90 million tickets a second, which is what
        // short combine tasks ran at). This last ticket of the worker is its
        // arrival number instead: it takes items slot, slot + n_workers, ..., so
        // the workers that run out of down tasks first do the combining, and one
        // without an item leaves at once instead of spinning beside waves that
        // still run down tasks.
        const unsigned slot = j - n1 - n2;
        if (slot >= nc) break;
        if (n2 != 0u && !wait_flag(p, FLAG_G2, lds_flag, lds_poller)) break;
        combine_items<DT>(p, slot, nc, ncomb, worker, t_dyn0 + n1 + n2, t_fetch);
        break;
      }
    }
    if (p.trace && lane == 0 && tk < p.trace_cap) {
      const long long t_end = wall_clock64();
      TraceRec* r = p.trace + tk;  // 48 bytes: four words, then four 64-bit times
      st16(r, u32x4{tk, kind, worker, aux});
      st16(reinterpret_cast<char*>(r) + 16,
           u32x4{static_cast<unsigned>(t_fetch), static_cast<unsigned>(t_fetch >> 32),
                 static_cast<unsigned>(t_ready), static_cast<unsigned>(t_ready >> 32)});
      st16(reinterpret_cast<char*>(r) + 32,
           u32x4{static_cast<unsigned>(t_end), static_cast<unsigned>(t_end >> 32), 0u, 0u});
    }
  }

  // The last worker out returns every counter to zero for the next launch.
  unsigned last = 0;
  if (lane == 0) {
    last = (add_relaxed(&ctl->exit_count.v, 1u) == static_cast<unsigned>(p.n_workers) - 1u)
               ? 1u
               : 0u;
  }
  last = __builtin_amdgcn_readfirstlane(last);
  if (last) {
    const unsigned err = ldc(&ctl->error.v);
    if (err != 0u) recover_after_error(p, err, lane, 64);
    // (early mode: one row tile per expert, known without a trip to memory)
    unsigned nm = p.early ? static_cast<unsigned>(p.E)
                          : min(ldc(&ctl->n_mtiles.v), static_cast<unsigned>(p.max_mtiles));
    for (unsigned i = lane; i < nm; i += 64) stc(&p.g1_done[i].v, 0u);
    for (int g = lane; g < p.n_groups; g += 64) {
      stc(&p.wgflags[g].f[FLAG_SCAN], 0u);
      stc(&p.wgflags[g].f[FLAG_PERM], 0u);
      stc(&p.wgflags[g].f[FLAG_G2], 0u);
      stc(&p.wgflags[g].f[FLAG_ROUTED], 0u);
    }
    if (lane == 0) {
      stc(&ctl->launches.v, ldc(&ctl->launches.v) + 1u);
      stc(&ctl->router_done.v, 0u);
      stc(&ctl->perm_done.v, 0u);
      stc(&ctl->g2_done.v, 0u);
      stc(&ctl->n_mtiles.v, 0u);
      stc(&ctl->exit_count.v, 0u);
      stc(&ctl->ticket.v, 0u);
    }
  }
}

// ------------------------------------------------------------ weight packing
// dst chunk c (16 bytes) of the packed gate/up or down weights <- its source.
// which = 0: ffn1 [E,2I,H] -> tasks of 2*G1_NB blocks (gate blocks, then up
// blocks); which = 1: ffn2 [E,H,I] -> tasks of G2_NB blocks.
template <typename DT>
__global__ void pack_weights_kernel(const void* src_, void* dst_, int E, int H, int I, int which) {
  typedef typename DT::elem elem;
  constexpr int EPV = DT::EPV;
  const elem* src = reinterpret_cast<const elem*>(src_);
  const int K = which == 0 ? H : I;            // contraction length
  const int NA = which == 0 ? 2 * G1_NB : G2_NB;
  const int nb = which == 0 ? G1_NB : G2_NB;   // 16-row blocks per output slab
  const int ntask = which == 0 ? I / (16 * G1_NB) : H / (16 * G2_NB);
  const int ksteps = K / (4 * EPV);
  const size_t per_task = static_cast<size_t>(ksteps) * NA * 64;
  const size_t total = static_cast<size_t>(E) * ntask * per_task;
  for (size_t c = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; c < total;
       c += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const int lane = static_cast<int>(c & 63);
    const int a = static_cast<int>((c >> 6) % NA);
    const int ks = static_cast<int>((c / (64 * NA)) % ksteps);
    const size_t task = c / per_task;
    const int nblk = static_cast<int>(task % ntask);
    const int e = static_cast<int>(task / ntask);
    const int r16 = lane & 15, g = lane >> 4;
    size_t row;
    if (which == 0) {
      const int n0 = nblk * 16 * nb;
      row = static_cast<size_t>(e) * 2 * I + (a < nb ? n0 + 16 * a + r16 : I + n0 + 16 * (a - nb) + r16);
    } else {
      row = static_cast<size_t>(e) * H + nblk * 16 * nb + 16 * a + r16;
    }
    const uint4 v = ld16(src + row * K + static_cast<size_t>(ks) * 4 * EPV + g * EPV);
    st16(reinterpret_cast<char*>(dst_) + c * 16, u32x4{v.x, v.y, v.z, v.w});
  }
}

hipError_t pack_weights(const void* src, void* dst, int dtype, int E, int H, int I, int which,
                        hipStream_t stream) {
  if (dtype == DT_BF16) {
    hipLaunchKernelGGL(pack_weights_kernel<BF16>, dim3(4096), dim3(256), 0, stream, src, dst, E, H, I,
                       which);
  } else {
    hipLaunchKernelGGL(pack_weights_kernel<F32>, dim3(4096), dim3(256), 0, stream, src, dst, E, H, I,
                       which);
  }
  return hipGetLastError();
}

template __global__ void moe_stream_kernel<F32>(const Params);
template __global__ void moe_stream_kernel<BF16>(const Params);

hipError_t launch_stream_kernel(const Params& p, int dtype, int grid, hipStream_t stream) {
  const size_t lds = static_cast<size_t>(8) * ROUTER_LDS_FLOATS * sizeof(float);
  if (dtype == DT_BF16) {
    hipLaunchKernelGGL(moe_stream_kernel<BF16>, dim3(grid), dim3(512), lds, stream, p);
  } else {
    hipLaunchKernelGGL(moe_stream_kernel<F32>, dim3(grid), dim3(512), lds, stream, p);
  }
  return hipGetLastError();
}

hipError_t prepare_stream_kernel() {
  const size_t max_lds = static_cast<size_t>(8) * ROUTER_LDS_FLOATS * sizeof(float);
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(moe_stream_kernel<BF16>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize,
                                     static_cast<int>(max_lds));
  if (e != hipSuccess) return e;
  return hipFuncSetAttribute(reinterpret_cast<const void*>(moe_stream_kernel<F32>),
                             hipFuncAttributeMaxDynamicSharedMemorySize,
                             static_cast<int>(max_lds));
}

hipError_t stream_kernel_occupancy(int dtype, int* per_cu) {
  const size_t lds = static_cast<size_t>(8) * ROUTER_LDS_FLOATS * sizeof(float);
  return dtype == DT_BF16
             ? hipOccupancyMaxActiveBlocksPerMultiprocessor(per_cu, moe_stream_kernel<BF16>, 512, lds)
             : hipOccupancyMaxActiveBlocksPerMultiprocessor(per_cu, moe_stream_kernel<F32>, 512, lds);
}

}  // namespace fmoe
