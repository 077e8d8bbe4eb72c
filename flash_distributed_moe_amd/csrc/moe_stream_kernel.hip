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
//
// Replaces, for this regime, the reference's moeKernel
// (src/hip/kernel/moeKernel.h:37-107), its task executors
// (src/hip/kernel/tasks/*.h) and its queue (src/hip/taskSystem/*.h).
#include <float.h>
#include <hip/hip_runtime.h>

#include "moe_params.h"

namespace fmoe {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct F32 {
  typedef float elem;
  static constexpr int EPV = 4;  // elements per 16-byte vector
};
struct BF16 {
  typedef unsigned short elem;
  static constexpr int EPV = 8;
};

// ------------------------------------------------------------------ helpers
__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }

__device__ __forceinline__ unsigned ld_relaxed(const unsigned* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void fence_acquire() {
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}
__device__ __forceinline__ void fence_release() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
}
__device__ __forceinline__ unsigned add_relaxed(unsigned* p, unsigned v) {
  return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// All lanes' earlier stores become visible device-wide, then the counter moves.
__device__ __forceinline__ void wave_signal(unsigned* counter) {
  fence_release();
  if (lane_id() == 0) add_relaxed(counter, 1u);
}

// Wave-uniform bounded wait for *p >= target. False on time-out or when
// another worker has raised an error; the caller then leaves the loop.
__device__ __forceinline__ bool wave_wait_ge(const unsigned* p, unsigned target,
                                             Control* ctl, long long limit) {
  int ok = 1;
  if (lane_id() == 0) {
    if (ld_relaxed(p) < target) {
      const long long t0 = wall_clock64();
      while (ld_relaxed(p) < target) {
        if (ld_relaxed(&ctl->error) != 0u) {
          ok = 0;
          break;
        }
        if (wall_clock64() - t0 > limit) {
          __hip_atomic_fetch_or(&ctl->error, ERR_TIMEOUT, __ATOMIC_RELAXED,
                                __HIP_MEMORY_SCOPE_AGENT);
          ok = 0;
          break;
        }
        __builtin_amdgcn_s_sleep(8);
      }
    }
  }
  ok = __builtin_amdgcn_readfirstlane(ok);
  fence_acquire();
  return ok != 0;
}

__device__ __forceinline__ uint4 ld16(const void* p) {
  return *reinterpret_cast<const uint4*>(p);
}

__device__ __forceinline__ float bf16_lo(unsigned u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(unsigned u) {
  return __uint_as_float(u & 0xFFFF0000u);
}
// float -> bfloat16 bits, round to nearest even (NaN stays NaN).
__device__ __forceinline__ unsigned f2bf(float f) {
  unsigned u = __float_as_uint(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u >> 16) | 0x40u;
  u += 0x7FFFu + ((u >> 16) & 1u);
  return u >> 16;
}

template <typename DT>
__device__ __forceinline__ void unpack(const uint4& v, float (&f)[DT::EPV]);
template <>
__device__ __forceinline__ void unpack<F32>(const uint4& v, float (&f)[4]) {
  f[0] = __uint_as_float(v.x);
  f[1] = __uint_as_float(v.y);
  f[2] = __uint_as_float(v.z);
  f[3] = __uint_as_float(v.w);
}
template <>
__device__ __forceinline__ void unpack<BF16>(const uint4& v, float (&f)[8]) {
  f[0] = bf16_lo(v.x);
  f[1] = bf16_hi(v.x);
  f[2] = bf16_lo(v.y);
  f[3] = bf16_hi(v.y);
  f[4] = bf16_lo(v.z);
  f[5] = bf16_hi(v.z);
  f[6] = bf16_lo(v.w);
  f[7] = bf16_hi(v.w);
}

// One 16x16 accumulate step over the k-range a 16-byte fragment pair covers.
// Lane l holds row (l & 15) of its operand at k-offset (l >> 4) * EPV; the
// result lane l holds D[4*(l>>4) + v][l & 15], v = 0..3.
template <typename DT>
__device__ __forceinline__ f32x4 mma16(const uint4& a, const uint4& b, f32x4 c);
template <>
__device__ __forceinline__ f32x4 mma16<BF16>(const uint4& a, const uint4& b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                 __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x4 mma16<F32>(const uint4& a, const uint4& b, f32x4 c) {
  c = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a.x), __uint_as_float(b.x), c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a.y), __uint_as_float(b.y), c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a.z), __uint_as_float(b.z), c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a.w), __uint_as_float(b.w), c, 0, 0, 0);
  return c;
}

__device__ __forceinline__ unsigned long long wave_max_u64(unsigned long long v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const unsigned long long o = __shfl_xor(v, off, 64);
    v = o > v ? o : v;
  }
  return v;
}

__device__ __forceinline__ int wave_inclusive_scan(int v) {
  const int lane = lane_id();
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int o = __shfl_up(v, off, 64);
    if (lane >= off) v += o;
  }
  return v;
}

// --------------------------------------------------------------------- router
// Follows the CPU MoE of the reference: logits accumulate the products one at a
// time in ascending k in float (test/singleGPU/cpp/moe/reference/refGemm.h:21-24),
// winners are the k largest with ties to the lower index
// (refTopk.h:36-58), weights are a softmax over the winners in double
// (refMoeGate.h:27-30, refSoftmax.h:19-52). For bf16 inputs each product is
// exact in float, so the fused multiply-add below rounds exactly as mul+add.
template <typename DT>
__device__ void router_task(const Params& p, int t) {
  typedef typename DT::elem elem;
  constexpr int EPV = DT::EPV;
  constexpr int MAXEPL = MAX_EXPERTS / 64;
  const int lane = lane_id();
  const int epl = (p.E + 63) >> 6;

  const elem* x = reinterpret_cast<const elem*>(p.tokens) + static_cast<size_t>(t) * p.H;
  const elem* wrow[MAXEPL];
  float acc[MAXEPL];
#pragma unroll
  for (int j = 0; j < MAXEPL; ++j) {
    int e = lane + 64 * j;
    e = e < p.E ? e : p.E - 1;
    wrow[j] = reinterpret_cast<const elem*>(p.gate) + static_cast<size_t>(e) * p.H;
    acc[j] = 0.0f;
  }

#pragma unroll 2
  for (int k0 = 0; k0 < p.H; k0 += EPV) {
    float xf[EPV];
    unpack<DT>(ld16(x + k0), xf);
#pragma unroll
    for (int j = 0; j < MAXEPL; ++j) {
      if (j < epl) {
        float wf[EPV];
        unpack<DT>(ld16(wrow[j] + k0), wf);
#pragma unroll
        for (int i = 0; i < EPV; ++i) {
          if constexpr (EPV == 8) {
            acc[j] = __builtin_fmaf(xf[i], wf[i], acc[j]);
          } else {
            acc[j] = __fadd_rn(acc[j], __fmul_rn(xf[i], wf[i]));
          }
        }
      }
    }
  }

  // Candidate keys: (order-preserving value bits, inverted index) so that the
  // wave maximum is the largest value and, among equals, the lowest index.
  // Values that the reference's strict '>' against lowest() never admits
  // (NaN, -inf, -FLT_MAX) get key 0.
  unsigned long long key[MAXEPL];
#pragma unroll
  for (int j = 0; j < MAXEPL; ++j) {
    const int e = lane + 64 * j;
    float v = acc[j];
    if (p.bias != nullptr && e < p.E) v = __fadd_rn(v, p.bias[e]);
    const bool valid = (j < epl) && (e < p.E) && (v > -FLT_MAX);
    unsigned u = __float_as_uint(v);
    u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
    key[j] = valid ? ((static_cast<unsigned long long>(u) << 32) |
                      static_cast<unsigned long long>(0xFFFFFFFFu - static_cast<unsigned>(e)))
                   : 0ull;
  }

  int my_idx = -1;
  float my_val = -FLT_MAX;
  for (int s = 0; s < p.K; ++s) {
    unsigned long long best = key[0];
#pragma unroll
    for (int j = 1; j < MAXEPL; ++j) best = key[j] > best ? key[j] : best;
    best = wave_max_u64(best);
    int e = -1;
    float v = -FLT_MAX;
    if (best != 0ull) {
      e = static_cast<int>(0xFFFFFFFFu - static_cast<unsigned>(best & 0xFFFFFFFFull));
      unsigned u = static_cast<unsigned>(best >> 32);
      u = (u & 0x80000000u) ? (u & 0x7FFFFFFFu) : ~u;
      v = __uint_as_float(u);
#pragma unroll
      for (int j = 0; j < MAXEPL; ++j)
        if (e == lane + 64 * j) key[j] = 0ull;
    }
    if (lane == s) {
      my_idx = e;
      my_val = v;
    }
  }

  // softmax over the K winners (descending, so the first is the maximum)
  const double v0 = static_cast<double>(__shfl(my_val, 0, 64));
  const double ex = lane < p.K ? exp(static_cast<double>(my_val) - v0) : 0.0;
  double sum = 0.0;
  for (int s = 0; s < p.K; ++s) sum += __shfl(ex, s, 64);
  if (lane < p.K) {
    float w;
    if (sum <= 0.0) {
      w = static_cast<float>(1.0 / static_cast<double>(p.K));
    } else {
      w = static_cast<float>(ex / sum);
    }
    p.topk_idx[static_cast<size_t>(t) * p.K + lane] = my_idx;
    p.topk_w[static_cast<size_t>(t) * p.K + lane] = w;
    if (my_idx >= 0) {
      __hip_atomic_fetch_or(&p.masks[static_cast<size_t>(my_idx) * p.W + (t >> 6)],
                            1ull << (t & 63), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  wave_signal(&p.ctl->router_done);
}

// ----------------------------------------------------------------------- scan
// Expert counts and offsets from the selection bit masks, and the table of row
// tiles. The permutation this defines is the stable sort of (token, slot) by
// expert id: inside an expert, rows ascend by token id. The reference has no
// permutation stage (it runs one GEMV per (token, slot)); this is the
// token-grouping the streaming and tiled GEMMs need.
__device__ void scan_task(const Params& p) {
  constexpr int MAXEPL = MAX_EXPERTS / 64;
  const int lane = lane_id();
  const int epl = (p.E + 63) >> 6;
  const int wact = (p.T + 63) >> 6;
  int base = 0, tile_base = 0;
  for (int j = 0; j < epl; ++j) {
    const int e = lane + 64 * j;
    int c = 0;
    if (e < p.E) {
      const unsigned long long* m = p.masks + static_cast<size_t>(e) * p.W;
      int* wp = p.word_prefix + static_cast<size_t>(e) * p.W;
      for (int w = 0; w < wact; ++w) {
        wp[w] = c;
        c += __popcll(m[w]);
      }
    }
    const int incl = wave_inclusive_scan(c);
    const int off = base + incl - c;
    const int nt = (c + SKINNY_MT - 1) / SKINNY_MT;
    const int tincl = wave_inclusive_scan(nt);
    const int toff = tile_base + tincl - nt;
    if (e < p.E) {
      p.expert_count[e] = c;
      p.expert_offset[e] = off;
      for (int i = 0; i < nt; ++i) {
        if (toff + i < p.max_mtiles) {
          TileDesc d;
          d.expert = e;
          d.row0 = off + i * SKINNY_MT;
          d.rows = min(SKINNY_MT, c - i * SKINNY_MT);
          d.pad = 0;
          p.mtiles[toff + i] = d;
        }
      }
    }
    base += __shfl(incl, 63, 64);
    tile_base += __shfl(tincl, 63, 64);
  }
  if (lane == 0) {
    p.expert_offset[p.E] = base;
    if (tile_base > p.max_mtiles) {
      __hip_atomic_fetch_or(&p.ctl->error, ERR_CAPACITY, __ATOMIC_RELAXED,
                            __HIP_MEMORY_SCOPE_AGENT);
      tile_base = 0;
    }
    p.ctl->n_mtiles = static_cast<unsigned>(tile_base);
  }
  wave_signal(&p.ctl->scan_done);
}

// -------------------------------------------------------------------- scatter
__device__ void scatter_task(const Params& p, int t) {
  const int lane = lane_id();
  if (lane < p.K) {
    const int e = p.topk_idx[static_cast<size_t>(t) * p.K + lane];
    if (e >= 0) {
      const int wd = t >> 6;
      const unsigned long long m = p.masks[static_cast<size_t>(e) * p.W + wd];
      const unsigned long long below = m & ((1ull << (t & 63)) - 1ull);
      const int pos = p.expert_offset[e] + p.word_prefix[static_cast<size_t>(e) * p.W + wd] +
                      __popcll(below);
      p.perm[pos] = t * p.K + lane;
      p.row_w[pos] = p.topk_w[static_cast<size_t>(t) * p.K + lane];
    }
  }
  wave_signal(&p.ctl->perm_done);
}

// ------------------------------------------------- streaming 16x16 MFMA sweep
// acc[i][r] += A_i (16 weight rows) . B_r (16 token rows)^T over `ksteps` steps
// of 4*EPV elements. ap[i] / bp[r] already point at this lane's row and
// k-offset. Fragments are double-buffered in registers, U steps per buffer, so
// the next buffer's loads are in flight while the current one feeds the MFMAs.
template <typename DT, int NA, int RB, int U>
__device__ __forceinline__ void stream_mma(const typename DT::elem* const (&ap)[NA],
                                           const typename DT::elem* const (&bp)[RB], int ksteps,
                                           f32x4 (&acc)[NA][RB]) {
  constexpr int KS = 4 * DT::EPV;
  uint4 a0[U][NA], b0[U][RB], a1[U][NA], b1[U][RB];

  auto load = [&](uint4(&a)[U][NA], uint4(&b)[U][RB], int s) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int i = 0; i < NA; ++i) a[u][i] = ld16(ap[i] + static_cast<size_t>(s + u) * KS);
#pragma unroll
      for (int r = 0; r < RB; ++r) b[u][r] = ld16(bp[r] + static_cast<size_t>(s + u) * KS);
    }
  };
  auto mma = [&](uint4(&a)[U][NA], uint4(&b)[U][RB]) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int i = 0; i < NA; ++i)
#pragma unroll
        for (int r = 0; r < RB; ++r) acc[i][r] = mma16<DT>(a[u][i], b[u][r], acc[i][r]);
  };

  const int main_steps = (ksteps / U) * U;
  int s = 0;
  if (main_steps > 0) {
    load(a0, b0, 0);
    for (; s + 2 * U <= main_steps; s += 2 * U) {
      load(a1, b1, s + U);
      mma(a0, b0);
      if (s + 2 * U < main_steps) load(a0, b0, s + 2 * U);
      mma(a1, b1);
    }
    if (s < main_steps) {
      mma(a0, b0);
      s += U;
    }
  }
  for (; s < ksteps; ++s) {  // remainder when ksteps is not a multiple of U
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const uint4 a = ld16(ap[i] + static_cast<size_t>(s) * KS);
#pragma unroll
      for (int r = 0; r < RB; ++r)
        acc[i][r] = mma16<DT>(a, ld16(bp[r] + static_cast<size_t>(s) * KS), acc[i][r]);
    }
  }
}

__device__ __forceinline__ float silu_mul(float a, float b) {
  // a * sigmoid(a) * b with the sign-split sigmoid of
  // test/singleGPU/cpp/moe/reference/refExpertFFN1.h:12-21,45
  float s;
  if (a >= 0.0f) {
    s = 1.0f / (1.0f + __expf(-a));
  } else {
    const float e = __expf(a);
    s = e / (1.0f + e);
  }
  return a * s * b;
}

// -------------------------------------------------------------------- gate/up
// h[row, n0 .. n0+32) for the rows of one tile. Follows
// refExpertFFN1.h:51-65 (two GEMMs against the [2I,H] expert matrix, then
// SiLU(gate) * up), accumulated on MFMA in float.
template <typename DT, int RB>
__device__ void gateup_task(const Params& p, const TileDesc& tile, int nblk) {
  typedef typename DT::elem elem;
  constexpr int EPV = DT::EPV;
  constexpr int NA = 2 * G1_NB;
  constexpr int U = RB >= 4 ? 1 : (RB == 2 ? 2 : 3);
  const int lane = lane_id();
  const int r16 = lane & 15, g = lane >> 4;
  const int n0 = nblk * (16 * G1_NB);

  const elem* w13 = reinterpret_cast<const elem*>(p.ffn1) +
                    static_cast<size_t>(tile.expert) * 2 * p.I * p.H;
  const elem* ap[NA];
#pragma unroll
  for (int b = 0; b < G1_NB; ++b) {
    ap[b] = w13 + static_cast<size_t>(n0 + 16 * b + r16) * p.H + g * EPV;            // gate rows
    ap[G1_NB + b] = w13 + static_cast<size_t>(p.I + n0 + 16 * b + r16) * p.H + g * EPV;  // up rows
  }
  const elem* bp[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    const int row = min(r * 16 + r16, tile.rows - 1);
    const int tok = p.perm[tile.row0 + row] / p.K;
    bp[r] = reinterpret_cast<const elem*>(p.tokens) + static_cast<size_t>(tok) * p.H + g * EPV;
  }
  f32x4 acc[NA][RB];
#pragma unroll
  for (int i = 0; i < NA; ++i)
#pragma unroll
    for (int r = 0; r < RB; ++r) acc[i][r] = f32x4{0.f, 0.f, 0.f, 0.f};

  stream_mma<DT, NA, RB, U>(ap, bp, p.H / (4 * EPV), acc);

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
          uint2 pk;
          pk.x = f2bf(hv[0]) | (f2bf(hv[1]) << 16);
          pk.y = f2bf(hv[2]) | (f2bf(hv[3]) << 16);
          *reinterpret_cast<uint2*>(reinterpret_cast<unsigned short*>(p.h) + off) = pk;
        } else {
          *reinterpret_cast<float4*>(reinterpret_cast<float*>(p.h) + off) =
              make_float4(hv[0], hv[1], hv[2], hv[3]);
        }
      }
    }
  }
}

// ----------------------------------------------------------------------- down
// y[t*K+slot, n0 .. n0+64) = w * (h[row] . W2[e]^T): refFullMoe.h:58-65 with the
// gate weight applied before the slot sum, as the reference GPU path does
// (src/hip/kernel/tasks/ffn2Task.h:37-40).
template <typename DT, int RB>
__device__ void down_task(const Params& p, const TileDesc& tile, int nblk) {
  typedef typename DT::elem elem;
  constexpr int EPV = DT::EPV;
  constexpr int NA = G2_NB;
  constexpr int U = RB >= 4 ? 1 : (RB == 2 ? 2 : 3);
  const int lane = lane_id();
  const int r16 = lane & 15, g = lane >> 4;
  const int n0 = nblk * (16 * G2_NB);

  const elem* w2 =
      reinterpret_cast<const elem*>(p.ffn2) + static_cast<size_t>(tile.expert) * p.H * p.I;
  const elem* ap[NA];
#pragma unroll
  for (int b = 0; b < NA; ++b) ap[b] = w2 + static_cast<size_t>(n0 + 16 * b + r16) * p.I + g * EPV;
  const elem* bp[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    const int row = min(r * 16 + r16, tile.rows - 1);
    bp[r] = reinterpret_cast<const elem*>(p.h) + static_cast<size_t>(tile.row0 + row) * p.I + g * EPV;
  }
  f32x4 acc[NA][RB];
#pragma unroll
  for (int i = 0; i < NA; ++i)
#pragma unroll
    for (int r = 0; r < RB; ++r) acc[i][r] = f32x4{0.f, 0.f, 0.f, 0.f};

  stream_mma<DT, NA, RB, U>(ap, bp, p.I / (4 * EPV), acc);

#pragma unroll
  for (int r = 0; r < RB; ++r) {
    const int row = r * 16 + r16;
    if (row < tile.rows) {
      const float w = p.row_w[tile.row0 + row];
      const size_t dst = static_cast<size_t>(p.perm[tile.row0 + row]) * p.H;
#pragma unroll
      for (int b = 0; b < NA; ++b) {
        *reinterpret_cast<float4*>(p.y + dst + n0 + 16 * b + 4 * g) =
            make_float4(acc[b][r][0] * w, acc[b][r][1] * w, acc[b][r][2] * w, acc[b][r][3] * w);
      }
    }
  }
}

// -------------------------------------------------------------------- combine
// out[t, c0..c0+256) = sum over slots, in slot order, of the weighted rows
// (refFullMoe.h:35,62-65; src/hip/kernel/tasks/internal/reduceBlock.h:35-53).
template <typename DT>
__device__ void combine_task(const Params& p, int t, int chunk) {
  const int lane = lane_id();
  const int c = chunk * COMBINE_COLS + lane * 4;
  if (c < p.H) {
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int k = 0; k < p.K; ++k) {
      if (p.topk_idx[static_cast<size_t>(t) * p.K + k] < 0) continue;
      const float4 v =
          *reinterpret_cast<const float4*>(p.y + (static_cast<size_t>(t) * p.K + k) * p.H + c);
      s.x += v.x;
      s.y += v.y;
      s.z += v.z;
      s.w += v.w;
    }
    const size_t off = static_cast<size_t>(t) * p.H + c;
    if constexpr (DT::EPV == 8) {
      uint2 pk;
      pk.x = f2bf(s.x) | (f2bf(s.y) << 16);
      pk.y = f2bf(s.z) | (f2bf(s.w) << 16);
      *reinterpret_cast<uint2*>(reinterpret_cast<unsigned short*>(p.out) + off) = pk;
    } else {
      *reinterpret_cast<float4*>(reinterpret_cast<float*>(p.out) + off) = s;
    }
  }
  // the selection masks are dead once every scatter task has run: clear this
  // token block's words for the next launch
  if (chunk == 0 && (t & 63) == 0) {
    for (int e = lane; e < p.E; e += 64) p.masks[static_cast<size_t>(e) * p.W + (t >> 6)] = 0ull;
  }
}

// ---------------------------------------------------------------- worker loop
template <typename DT>
__global__ __launch_bounds__(512) void moe_stream_kernel(const Params p) {
  const int lane = lane_id();
  Control* ctl = p.ctl;
  const unsigned T = static_cast<unsigned>(p.T);
  const unsigned t_scan = T, t_scatter0 = T + 1u, t_dyn0 = 2u * T + 1u;
  const unsigned nt1 = static_cast<unsigned>(p.I / (16 * G1_NB));
  const unsigned nt2 = static_cast<unsigned>(p.H / (16 * G2_NB));
  const unsigned ncomb = static_cast<unsigned>((p.H + COMBINE_COLS - 1) / COMBINE_COLS);
  unsigned n1 = 0, n2 = 0, nc = 0;
  bool have_dyn = false, perm_ready = false, g2_ready = false;

  while (true) {
    unsigned tk = 0;
    if (lane == 0) tk = add_relaxed(&ctl->ticket, 1u);
    tk = __builtin_amdgcn_readfirstlane(tk);

    if (tk < T) {
      router_task<DT>(p, static_cast<int>(tk));
    } else if (tk == t_scan) {
      if (!wave_wait_ge(&ctl->router_done, T, ctl, p.spin_limit)) break;
      scan_task(p);
    } else if (tk < t_dyn0) {
      if (!wave_wait_ge(&ctl->scan_done, 1u, ctl, p.spin_limit)) break;
      scatter_task(p, static_cast<int>(tk - t_scatter0));
    } else {
      if (!have_dyn) {
        if (!wave_wait_ge(&ctl->scan_done, 1u, ctl, p.spin_limit)) break;
        const unsigned nm = ctl->n_mtiles;
        n1 = nm * nt1;
        n2 = nm * nt2;
        nc = T * ncomb;
        have_dyn = true;
      }
      const unsigned j = tk - t_dyn0;
      if (j < n1) {
        if (!perm_ready) {
          if (!wave_wait_ge(&ctl->perm_done, T, ctl, p.spin_limit)) break;
          perm_ready = true;
        }
        const TileDesc tile = p.mtiles[j / nt1];
        const int nblk = static_cast<int>(j % nt1);
        if (tile.rows <= 16) {
          gateup_task<DT, 1>(p, tile, nblk);
        } else if (tile.rows <= 32) {
          gateup_task<DT, 2>(p, tile, nblk);
        } else {
          gateup_task<DT, 4>(p, tile, nblk);
        }
        wave_signal(&p.g1_done[j / nt1]);
      } else if (j < n1 + n2) {
        const unsigned m = (j - n1) / nt2;
        const int nblk = static_cast<int>((j - n1) % nt2);
        if (!wave_wait_ge(&p.g1_done[m], nt1, ctl, p.spin_limit)) break;
        const TileDesc tile = p.mtiles[m];
        if (tile.rows <= 16) {
          down_task<DT, 1>(p, tile, nblk);
        } else if (tile.rows <= 32) {
          down_task<DT, 2>(p, tile, nblk);
        } else {
          down_task<DT, 4>(p, tile, nblk);
        }
        wave_signal(&ctl->g2_done);
      } else if (j < n1 + n2 + nc) {
        if (!g2_ready) {
          if (!wave_wait_ge(&ctl->g2_done, n2, ctl, p.spin_limit)) break;
          g2_ready = true;
        }
        const unsigned q = j - n1 - n2;
        combine_task<DT>(p, static_cast<int>(q / ncomb), static_cast<int>(q % ncomb));
      } else {
        break;
      }
    }
  }

  // The last worker out returns every counter to zero for the next launch.
  unsigned last = 0;
  if (lane == 0) {
    last = (__hip_atomic_fetch_add(&ctl->exit_count, 1u, __ATOMIC_ACQ_REL,
                                   __HIP_MEMORY_SCOPE_AGENT) ==
            static_cast<unsigned>(p.n_workers) - 1u)
               ? 1u
               : 0u;
  }
  last = __builtin_amdgcn_readfirstlane(last);
  if (last) {
    const unsigned nm = min(ctl->n_mtiles, static_cast<unsigned>(p.max_mtiles));
    for (unsigned i = lane; i < nm; i += 64) p.g1_done[i] = 0u;
    if (lane == 0) {
      ctl->launches = ctl->launches + 1u;
      ctl->router_done = 0u;
      ctl->scan_done = 0u;
      ctl->perm_done = 0u;
      ctl->g2_done = 0u;
      ctl->n_mtiles = 0u;
      ctl->exit_count = 0u;
      ctl->ticket = 0u;
    }
  }
}

template __global__ void moe_stream_kernel<F32>(const Params);
template __global__ void moe_stream_kernel<BF16>(const Params);

hipError_t launch_stream_kernel(const Params& p, int dtype, int grid, hipStream_t stream) {
  if (dtype == DT_BF16) {
    hipLaunchKernelGGL(moe_stream_kernel<BF16>, dim3(grid), dim3(512), 0, stream, p);
  } else {
    hipLaunchKernelGGL(moe_stream_kernel<F32>, dim3(grid), dim3(512), 0, stream, p);
  }
  return hipGetLastError();
}

}  // namespace fmoe
