// Device helpers shared by the streaming and the tiled MoE kernels: coherent
// data access between workers, bounded waits, bf16 packing, the router's
// selection step and the permutation rule.
#pragma once
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
// Coherence between workers. MI355X has eight XCDs with one L2 each, and an
// agent-scope release/acquire fence writes back / invalidates a whole L2: with
// two thousand waves signalling, each fence costs tens of microseconds. So
// nothing here uses those fences. Every value one worker produces for another
// (routing tables, h, y, counters) is written and read with agent-scope relaxed
// atomic accesses of 4 or 8 bytes, which go through to the memory-side
// coherence point; a producer waits for its stores (workgroup-scope release =
// wait for outstanding memory operations) and then bumps a counter, a consumer
// polls the counter and then loads. Inputs (tokens, weights) are never written
// while the kernel runs and use ordinary cached loads.
__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }
// The launch parameters where the dispatch put them: the kernels take one
// argument, a Params by value, which starts the kernel-argument segment.
#if defined(FMOE_PARAMS_IN_KERNARG)
__device__ __forceinline__ ParamsRef kernel_params() {
#if defined(__HIP_DEVICE_COMPILE__)
  return *(const __attribute__((address_space(4))) Params*)__builtin_amdgcn_kernarg_segment_ptr();
#else
  return *static_cast<const Params*>(nullptr);
#endif
}
#endif

// Every pointer in Params is HBM: saying so lets the compiler emit global_*
// instead of flat_* memory instructions (flat ones also count as LDS traffic).
#define FMOE_GLOBAL __attribute__((address_space(1)))
template <typename T>
__device__ __forceinline__ FMOE_GLOBAL T* as_global(T* p) {
  return (FMOE_GLOBAL T*)p;
}

__device__ __forceinline__ unsigned ldc(const unsigned* p) {
  return __hip_atomic_load(as_global(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ int ldc(const int* p) {
  return __hip_atomic_load(as_global(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float ldc(const float* p) {
  return __uint_as_float(__hip_atomic_load(as_global(reinterpret_cast<const unsigned*>(p)),
                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
__device__ __forceinline__ unsigned long long ldc(const unsigned long long* p) {
  return __hip_atomic_load(as_global(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void stc(unsigned* p, unsigned v) {
  __hip_atomic_store(as_global(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void stc(int* p, int v) {
  __hip_atomic_store(as_global(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void stc(float* p, float v) {
  __hip_atomic_store(as_global(reinterpret_cast<unsigned*>(p)), __float_as_uint(v),
                     __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void stc(unsigned long long* p, unsigned long long v) {
  __hip_atomic_store(as_global(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// 16 coherent bytes as two 8-byte accesses
__device__ __forceinline__ uint4 ldc16(const void* p) {
  const unsigned long long* q = reinterpret_cast<const unsigned long long*>(p);
  const unsigned long long a = ldc(q), b = ldc(q + 1);
  return make_uint4(static_cast<unsigned>(a), static_cast<unsigned>(a >> 32),
                    static_cast<unsigned>(b), static_cast<unsigned>(b >> 32));
}
__device__ __forceinline__ void stc16(void* p, const uint4& v) {
  unsigned long long* q = reinterpret_cast<unsigned long long*>(p);
  stc(q, static_cast<unsigned long long>(v.x) | (static_cast<unsigned long long>(v.y) << 32));
  stc(q + 1, static_cast<unsigned long long>(v.z) | (static_cast<unsigned long long>(v.w) << 32));
}
// 16 bytes written through to device-coherent memory (agent scope): visible to
// every XCD once the store has completed, with no cache write-back needed.
__device__ __forceinline__ void st16_through(void* p, const uint4& v) {
  typedef unsigned v4u __attribute__((ext_vector_type(4)));
  const v4u d = {v.x, v.y, v.z, v.w};
  // The two idle cycles after the store are the wait states the hardware needs
  // before a vector instruction may overwrite the data registers of a store
  // wider than 8 bytes; the compiler inserts them for its own stores, but does
  // not look inside assembly.
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(p), "v"(d) : "memory");
}
__device__ __forceinline__ TileDesc ld_tile(const TileDesc* t) {
  const uint4 v = ldc16(t);
  TileDesc d;
  d.expert = static_cast<int>(v.x);
  d.row0 = static_cast<int>(v.y);
  d.rows = static_cast<int>(v.z);
  d.shared = static_cast<int>(v.w);
  return d;
}

__device__ __forceinline__ unsigned ld_relaxed(const unsigned* p) {
  return __hip_atomic_load(as_global(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Ordering only (no cache maintenance): later loads stay after the poll that
// precedes this / earlier stores have completed before the counter moves.
__device__ __forceinline__ void fence_acquire() {
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}
__device__ __forceinline__ void fence_release() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_waitcnt(0);  // every outstanding store has reached the coherence point
}
__device__ __forceinline__ unsigned add_relaxed(unsigned* p, unsigned v) {
  return __hip_atomic_fetch_add(as_global(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_relaxed(unsigned* p, unsigned v) {
  __hip_atomic_store(as_global(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void or_relaxed(unsigned* p, unsigned v) {
  __hip_atomic_fetch_or(as_global(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void or_relaxed(unsigned long long* p, unsigned long long v) {
  __hip_atomic_fetch_or(as_global(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// All lanes' earlier coherent stores have completed, then the counter moves.
// Returns the counter's previous value to every lane.
__device__ __forceinline__ unsigned wave_arrive(unsigned* counter) {
  fence_release();
  unsigned old = 0;
  if (lane_id() == 0) old = add_relaxed(counter, 1u);
  return __builtin_amdgcn_readfirstlane(old);
}

// Called by the worker that completed a phase (after wave_arrive told it so, or
// after its own release fence): raises the phase flag of every workgroup.
__device__ __forceinline__ void broadcast_flag(ParamsRef p, int which) {
  const int n = p.n_groups;
  WgFlags* flags = p.wgflags;
  for (int g = lane_id(); g < n; g += 64) st_relaxed(&flags[g].f[which], 1u);
}

// A launch that raised an error bit (a bounded wait ran out, the tile table overflowed) has
// left counters, masks and outputs in an arbitrary state. The last worker to leave makes
// the failure visible and the launcher usable again without any help from the host, which
// may be replaying a captured graph and never look: every element of `out` becomes NaN,
// the workspace's zero region returns to zero (the count of completed launches apart), and
// the bits are added to the launcher's word in pinned host memory, where the next Launch
// finds them. `tid` of `nthreads` threads of that worker call this; nobody else is running.
__device__ __forceinline__ void recover_after_error(ParamsRef p, unsigned err, int tid, int nthreads) {
  unsigned* ws = reinterpret_cast<unsigned*>(p.ctl);
  const unsigned launches_word =
      static_cast<unsigned>(reinterpret_cast<unsigned*>(&p.ctl->launches.v) - ws);
  const unsigned nz = p.zero_words;
  for (unsigned i = tid; i < nz; i += nthreads)
    if (i != launches_word) stc(&ws[i], 0u);
  const size_t nout = static_cast<size_t>(p.T) * p.H * p.elem_bytes / 4;
  const unsigned nan_word = p.elem_bytes == 2 ? 0x7FC07FC0u : 0x7FC00000u;
  unsigned* out = reinterpret_cast<unsigned*>(p.out);
  for (size_t i = tid; i < nout; i += nthreads) stc(&out[i], nan_word);
  if (tid == 0 && p.host_error != nullptr)
    __hip_atomic_fetch_or(as_global(p.host_error), err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Wave-uniform bounded wait for *p >= target. False on time-out or when
// another worker has raised an error; the caller then leaves the loop.
__device__ __forceinline__ bool wave_wait_ge(const unsigned* p, unsigned target,
                                             Control* ctl, long long limit) {
  int ok = 1;
  if (lane_id() == 0) {
    if (ld_relaxed(p) < target) {
      const long long t0 = wall_clock64();
      unsigned spins = 0;
      while (ld_relaxed(p) < target) {
        if ((++spins & 31u) == 0u && ld_relaxed(&ctl->error.v) != 0u) {
          ok = 0;
          break;
        }
        if (wall_clock64() - t0 > limit) {
          or_relaxed(&ctl->error.v, ERR_TIMEOUT);
          ok = 0;
          break;
        }
        __builtin_amdgcn_s_sleep(16);
      }
    }
  }
  ok = __builtin_amdgcn_readfirstlane(ok);
  fence_acquire();
  return ok != 0;
}

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 ld16(const void* p) {
  const u32x4 v = *as_global(reinterpret_cast<const u32x4*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}
// a pointer that is the same in every lane, pinned to scalar registers
template <typename T>
__device__ __forceinline__ T* uniform_ptr(T* ptr) {
  const unsigned long long v = reinterpret_cast<unsigned long long>(ptr);
  const unsigned lo = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(v));
  const unsigned hi = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(v >> 32));
  return reinterpret_cast<T*>((static_cast<unsigned long long>(hi) << 32) | lo);
}
// The launch parameters as a function that is not inlined receives them: arguments
// arrive in vector registers, and only a pointer known to be uniform gets scalar loads.
__device__ __forceinline__ ParamsRef uniform_params(ParamsRef p) {
#if defined(__HIP_DEVICE_COMPILE__) && defined(FMOE_PARAMS_IN_KERNARG)
  const unsigned long long v = (unsigned long long)&p;
  const unsigned lo = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(v));
  const unsigned hi = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(v >> 32));
  return *(const __attribute__((address_space(4))) Params*)((static_cast<unsigned long long>(hi) << 32) | lo);
#else
  return p;
#endif
}
// 16 bytes read at agent scope (one instruction; an atomic load carries 8 at
// most): the load bypasses whatever this XCD's L2 holds for the line, so it sees
// what other XCDs have written through. `base` is uniform, `off` < `bytes`.
struct CoherentBuffer {
  __amdgpu_buffer_rsrc_t rsrc;
};
__device__ __forceinline__ CoherentBuffer coherent_buffer(const void* base, unsigned bytes) {
  CoherentBuffer b;
  b.rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, static_cast<int>(bytes), 0x00020000);
  return b;
}
__device__ __forceinline__ uint4 ld16_agent(const CoherentBuffer& b, unsigned off) {
  const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(b.rsrc, static_cast<int>(off), 0, 16 /* sc1 */);
  return make_uint4(v.x, v.y, v.z, v.w);
}
// 16 bytes that are used once (expert weights): marked non-temporal, so that
// they do not push the token rows and the routing tables out of the L2
__device__ __forceinline__ uint4 ld16_once(const void* p) {
  const u32x4 v = __builtin_nontemporal_load(as_global(reinterpret_cast<const u32x4*>(p)));
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void st16(void* p, const u32x4& v) {
  *as_global(reinterpret_cast<u32x4*>(p)) = v;
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

// two floats to packed bf16 (round to nearest even) with the hardware converter
__device__ __forceinline__ unsigned pack_bf16(float lo, float hi) {
  typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
  typedef float f2 __attribute__((ext_vector_type(2)));
  const f2 v = {lo, hi};
  return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf2));
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
// (order-preserving value bits, inverted index): the maximum key is the largest
// value and, among equals, the lowest index. Values the reference's strict '>'
// against lowest() never admits (NaN, -inf, -FLT_MAX) get key 0.
__device__ __forceinline__ unsigned long long make_key(float v, int e, bool in_range) {
  const bool valid = in_range && (v > -FLT_MAX);
  unsigned u = __float_as_uint(v);
  u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  return valid ? ((static_cast<unsigned long long>(u) << 32) |
                  static_cast<unsigned long long>(0xFFFFFFFFu - static_cast<unsigned>(e)))
               : 0ull;
}

// Orders this wave's LDS writes before its later LDS reads (other lanes' data)
// without waiting for global loads that are still in flight.
__device__ __forceinline__ void lds_wave_sync() {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_wave_barrier();
}

// Order-preserving image of a logit: greater float <=> greater unsigned. Values
// the reference's strict '>' against lowest() never admits (NaN, -inf,
// -FLT_MAX) and experts out of range map to 0, which never wins.
__device__ __forceinline__ unsigned ordered_bits(float v, bool in_range) {
  const unsigned u = __float_as_uint(v);
  return (in_range && v > -FLT_MAX) ? ((u & 0x80000000u) ? ~u : (u | 0x80000000u)) : 0u;
}
__device__ __forceinline__ float from_ordered_bits(unsigned u) {
  return __uint_as_float((u & 0x80000000u) ? (u & 0x7FFFFFFFu) : ~u);
}

// Maximum over the wave, in a scalar register: four cross-lane steps inside
// each row of 16 lanes, then the four row results.
__device__ __forceinline__ unsigned wave_max_u32(unsigned v) {
  auto step = [](unsigned x, unsigned moved) { return x > moved ? x : moved; };
  v = step(v, static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0xB1, 0xF, 0xF, true)));   // lane ^ 1
  v = step(v, static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x4E, 0xF, 0xF, true)));   // lane ^ 2
  v = step(v, static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x141, 0xF, 0xF, true)));  // mirror in 8
  v = step(v, static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x140, 0xF, 0xF, true)));  // mirror in 16
  const unsigned r0 = __builtin_amdgcn_readlane(static_cast<int>(v), 0);
  const unsigned r1 = __builtin_amdgcn_readlane(static_cast<int>(v), 16);
  const unsigned r2 = __builtin_amdgcn_readlane(static_cast<int>(v), 32);
  const unsigned r3 = __builtin_amdgcn_readlane(static_cast<int>(v), 48);
  const unsigned a = r0 > r1 ? r0 : r1, b = r2 > r3 ? r2 : r3;
  return a > b ? a : b;
}

// Top-k and gate weights of one token, by K rounds of "take the greatest logit
// that is left, the lowest expert index among equals" (refTopk.h:36-58 keeps the
// first of equal values because it compares with a strict '>'). val[j] is
// ordered_bits of expert lane + 64*j. lex: MAX_TOPK doubles of LDS private to
// the wave.
__device__ __forceinline__ void router_select_max(ParamsRef p, int t,
                                                  unsigned (&val)[MAX_EXPERTS / 64], double* lex) {
  constexpr int MAXEPL = MAX_EXPERTS / 64;
  const int lane = lane_id();
  const int K = p.K;
  int my_idx = -1;
  unsigned my_bits = 0u, top_bits = 0u;
  for (int s = 0; s < K; ++s) {
    unsigned m = val[0];
#pragma unroll
    for (int j = 1; j < MAXEPL; ++j) m = val[j] > m ? val[j] : m;
    const unsigned best = wave_max_u32(m);
    if (s == 0) top_bits = best;
    if (best == 0u) break;  // fewer admissible experts than K: the remaining slots stay -1
    int e = -1;
#pragma unroll
    for (int j = 0; j < MAXEPL; ++j) {
      if (e < 0) {
        const unsigned long long owners = __ballot(val[j] == best);
        if (owners != 0ull) {
          const int owner = __ffsll(static_cast<long long>(owners)) - 1;
          e = owner + 64 * j;
          if (lane == owner) val[j] = 0u;
        }
      }
    }
    if (lane == s) {
      my_idx = e;
      my_bits = best;
    }
  }
  // softmax over the K winners (descending, so the first is the maximum)
  const float my_val = my_bits != 0u ? from_ordered_bits(my_bits) : -FLT_MAX;
  const float v0f = top_bits != 0u ? from_ordered_bits(top_bits) : -FLT_MAX;
  const double ex = lane < K ? exp(static_cast<double>(my_val) - static_cast<double>(v0f)) : 0.0;
  if (lane < K) lex[lane] = ex;
  lds_wave_sync();
  double sum = 0.0;
  for (int s = 0; s < K; ++s) sum += lex[s];
  if (lane < K) {
    const float w = sum <= 0.0 ? static_cast<float>(1.0 / static_cast<double>(K))
                               : static_cast<float>(ex / sum);
    stc(&p.topk_idx[static_cast<size_t>(t) * K + lane], my_idx);
    stc(&p.topk_w[static_cast<size_t>(t) * K + lane], w);
    if (my_idx >= 0) {
      or_relaxed(&p.masks[static_cast<size_t>(my_idx) * p.W + (t >> 6)], 1ull << (t & 63));
    }
  }
  lds_wave_sync();
}

// ------------------------------------------------------------- scan / scatter
// The tables the scan and scatter tasks work on, held in registers (Params is
// reached through a generic reference, which every store would force the
// compiler to re-read).
struct RouteTables {
  int T, E, K, W, max_mtiles;
  int* topk_idx;
  float* topk_w;
  unsigned long long* masks;
  int* word_prefix;
  int* expert_count;
  int* expert_offset;
  int* perm;
  float* row_w;
  TileDesc* mtiles;
};
__device__ __forceinline__ RouteTables route_tables(ParamsRef p) {
  RouteTables r;
  r.T = p.T;
  r.E = p.E;
  r.K = p.K;
  r.W = p.W;
  r.max_mtiles = p.max_mtiles;
  r.topk_idx = p.topk_idx;
  r.topk_w = p.topk_w;
  r.masks = p.masks;
  r.word_prefix = p.word_prefix;
  r.expert_count = p.expert_count;
  r.expert_offset = p.expert_offset;
  r.perm = p.perm;
  r.row_w = p.row_w;
  r.mtiles = p.mtiles;
  return r;
}

// Permuted row of assignment i = t*K+slot: rows of one expert ascend by token.
__device__ __forceinline__ void scatter_entry(const RouteTables& r, int i) {
  const int e = ldc(&r.topk_idx[i]);
  if (e >= 0) {
    const int t = i / r.K;
    const int wd = t >> 6;
    const unsigned long long m = ldc(&r.masks[static_cast<size_t>(e) * r.W + wd]);
    const unsigned long long below = m & ((1ull << (t & 63)) - 1ull);
    const int pos = ldc(&r.expert_offset[e]) +
                    ldc(&r.word_prefix[static_cast<size_t>(e) * r.W + wd]) + __popcll(below);
    stc(&r.perm[pos], i);
    stc(&r.row_w[pos], ldc(&r.topk_w[i]));
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
// The same function with the hardware exponential and reciprocal (1 ulp each):
// a * b / (1 + 2^(-a * log2 e)), six instructions per element. Where 2^(...) overflows
// (a < -88.7) the reciprocal of infinity is 0 and the result the signed zero that the
// exact value (|a * b| * 1e-38 at most) rounds to next to any other term.
__device__ __forceinline__ float silu_mul_fast(float a, float b) {
  const float e = __builtin_amdgcn_exp2f(a * -1.44269504088896340736f);
  return a * __builtin_amdgcn_rcpf(1.0f + e) * b;
}


}  // namespace fmoe
