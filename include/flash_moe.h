/* C ABI of the MI355X fused MoE layer (libflashMoe.so).
 *
 * Plain pointers and sizes only; every pointer named "device" is HBM owned by
 * the caller. This is the layer the C++ interface in iMoeKernelLauncher.h and
 * any foreign-function binding (ctypes, cgo, JNI ...) sit on. All functions
 * return a hipError_t value as int (0 = hipSuccess) and never throw.
 *
 * What each entry point replaces in the reference (paths relative to the
 * reference checkout):
 *   flashMoeCreate      CreateLauncher  -> MoeKernelLauncher::Init
 *                       (src/moeKernelLauncher.cpp:33-46,
 *                        src/hip/launcher/moeKernelLauncher.hip:96-187), with the
 *                       compile-time shape of src/hip/common/metadata.h:7-13
 *                       turned into run-time fields
 *   flashMoeLaunch      IMoeKernelLauncher::Launch
 *                       (include/iMoeKernelLauncher.h:12-13,
 *                        src/hip/launcher/moeKernelLauncher.hip:58-93,207-212)
 *   flashMoeDestroy     DestroyLauncher -> MoeKernelLauncher::Deinit
 *                       (src/moeKernelLauncher.cpp:49-55,
 *                        src/hip/launcher/moeKernelLauncher.hip:190-204)
 *   flashMoeReadRouting no counterpart: copies the router's decisions out so
 *                       that tests can compare them bit for bit, as the
 *                       reference's stage test does for its gate
 *                       (test/singleGPU/cpp/moe/internal/moeGateTest.hip:62-109)
 *   flashMoeStatus      no counterpart: the reference asserts on the device
 *                       (src/hip/utils/hipDeviceUtils.h:12); here a bounded wait
 *                       that runs out raises a flag the host can read
 */
#ifndef FLASH_MOE_H_
#define FLASH_MOE_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct FlashMoeLauncher FlashMoeLauncher; /* opaque */

enum { FLASH_MOE_F32 = 0, FLASH_MOE_BF16 = 1 };

/* Scheduling variant. AUTO picks by rows per expert. */
enum { FLASH_MOE_SCHED_AUTO = 0, FLASH_MOE_SCHED_STREAM = 1, FLASH_MOE_SCHED_TILED = 2 };

/* The packed weight layout: contiguous 1 KiB runs (16 rows x 32 k) in the order
 * the kernels' tasks read them, which the streaming (small-batch) variant reads
 * front to back and the tiled variant loads as whole cache lines; same size as
 * the row-major tensors. Three ways to use it:
 *  FLASH_MOE_FLAG_PACK_WEIGHTS      at create the library copies the caller's
 *      row-major expert weights into a packed second copy in its workspace
 *      (+3*E*H*I elements of device memory). The caller's tensors stay the external
 *      format and must stay valid: a launch reads whichever form is faster for its
 *      batch (bf16: always the copy; float32: the caller's tensors from 16 rows an
 *      expert on). After changing them call flashMoeRefreshWeights.
 *  FLASH_MOE_FLAG_WEIGHTS_PREPACKED ffn1_weights / ffn2_weights already hold the
 *      packed layout (made by flashMoePackWeights into buffers of the caller's, or
 *      by flashMoePackWeightsInPlace): no second copy anywhere; the row-major form
 *      need not exist any more.
 *  neither                          launches read the caller's row-major tensors. */
enum { FLASH_MOE_FLAG_PACK_WEIGHTS = 1, FLASH_MOE_FLAG_WEIGHTS_PREPACKED = 2 };

/* Optional steps at the layer's edges (neither exists in the reference, whose
 * layer is gate + experts only, test/singleGPU/cpp/moe/reference/refFullMoe.h:9-70;
 * with neither flag the layer computes exactly that):
 *  FLASH_MOE_FLAG_RMSNORM   the router and the experts see rmsnorm(tokens) instead
 *      of tokens: xn[t,k] = (x[t,k] * float(1/sqrt(mean_k x[t,k]^2 + norm_eps))) *
 *      norm_weight[k], rounded to the layer dtype. A small kernel in front of the
 *      layer's kernel writes xn into the workspace (+max_tokens*H elements).
 *      The mean of squares is taken in double. For bfloat16 rows that sum is exact
 *      in any order, so xn (and the routing after it) is reproducible bit for bit
 *      by a CPU restatement. For float32 rows the squares are exact in double but
 *      their sum is rounded at every addition, in the kernel's order (64 strided
 *      partial sums, then a butterfly across the wave): another order can differ
 *      in the last bits of the double, which changes the float scale only when it
 *      lies within about 2^-29 ulp of a rounding boundary (about one row in 10^8);
 *      such a row's xn differs by one float ulp from the restatement's.
 *  FLASH_MOE_FLAG_RESIDUAL  output = tokens + layer(...): the un-normalised input
 *      row is added to the sum over the slots (last, in float) before the one
 *      rounding to the layer dtype. Works in place like everything else.
 * Together: output = x + moe(rmsnorm(x)), a pre-norm transformer block's MoE half. */
enum { FLASH_MOE_FLAG_RMSNORM = 4, FLASH_MOE_FLAG_RESIDUAL = 8 };

typedef struct FlashMoeLayerDesc {
  int experts;      /* E, 1..256 */
  int hidden;       /* H, multiple of 64 */
  int intermediate; /* I, multiple of 32 */
  int top_k;        /* k, 1..min(E,32) */
  int dtype;        /* FLASH_MOE_F32 or FLASH_MOE_BF16: weights, tokens, output */
  int max_tokens;   /* largest tokens_num a launch may pass */
  int sched;        /* FLASH_MOE_SCHED_* */
  int flags;        /* FLASH_MOE_FLAG_* bits */
  const void* gate_weights;  /* device, [E,H] row-major */
  const void* ffn1_weights;  /* device, [E,2I,H]: rows 0..I-1 gate proj, I..2I-1 up proj */
  const void* ffn2_weights;  /* device, [E,H,I] */
  const float* router_bias;  /* device, [E] float added to the logits, or NULL */
  const void* norm_weight;   /* device, [H] in the layer dtype; read with FLASH_MOE_FLAG_RMSNORM only */
  double norm_eps;           /* added to the mean square; read with FLASH_MOE_FLAG_RMSNORM only */
} FlashMoeLayerDesc;

/* Device bytes flashMoeCreate would allocate for this description. */
int flashMoeWorkspaceBytes(const FlashMoeLayerDesc* desc, size_t* bytes);

/* Allocates the workspace on the current device and synchronises `stream`.
 * Weights are borrowed and must outlive the launcher. On failure *out is left
 * untouched. hipErrorUnknown: max_tokens beyond capacity;
 * hipErrorInvalidValue: anything else wrong with the description. */
int flashMoeCreate(FlashMoeLauncher** out, const FlashMoeLayerDesc* desc, void* stream);

/* Packs expert weights for FLASH_MOE_FLAG_WEIGHTS_PREPACKED. which = 0: src is
 * ffn1 [experts, 2I, H]; which = 1: src is ffn2 [experts, H, I]; row-major,
 * dtype FLASH_MOE_F32 or FLASH_MOE_BF16, device memory. flashMoePackWeights writes
 * the packed form to dst (same size, must not overlap src), enqueued on `stream`.
 * flashMoePackWeightsInPlace rewrites the tensor where it lies, one expert at a
 * time through a staging buffer of one expert's matrix that it allocates and
 * frees; it waits for `stream`. No counterpart in the reference, which reads the
 * caller's layout only (src/hip/launcher/moeKernelLauncher.hip:107-109). */
int flashMoePackWeights(int dtype, int experts, int hidden, int intermediate, int which,
                        const void* src, void* dst, void* stream);
int flashMoePackWeightsInPlace(int dtype, int experts, int hidden, int intermediate, int which,
                               void* weights, void* stream);

/* Re-reads the caller's expert weights into the packed copy (no-op without
 * FLASH_MOE_FLAG_PACK_WEIGHTS). Enqueued on `stream`. No counterpart in the
 * reference, which keeps no copy of the weights
 * (src/hip/launcher/moeKernelLauncher.hip:107-109). */
int flashMoeRefreshWeights(FlashMoeLauncher* l, void* stream);

/* Enqueues one forward pass on `stream` and returns without waiting.
 * tokens, output: device [tokens_num, H] in the layer dtype; output may alias
 * tokens. Launches on one launcher must be ordered on one stream (its waits
 * happen inside the kernel, against its own workspace).
 * hipErrorUnknown when tokens_num > max_tokens, or when an earlier launch failed
 * on the device (see flashMoeStatus): then nothing is enqueued. */
int flashMoeLaunch(FlashMoeLauncher* l, const void* tokens, void* output, int tokens_num,
                   void* stream);

/* One forward pass that allocates nothing: for callers that cannot call
 * hipMalloc (code under HIP graph capture, tight serving loops, harnesses that
 * forbid it). It has no counterpart in the reference, whose launcher allocates
 * its buffers in Init (src/hip/launcher/moeKernelLauncher.hip:147-165). Same
 * kernels and results as flashMoeCreate + flashMoeLaunch on the same inputs, but
 * the workspace is a static device array of FLASH_MOE_NOALLOC_SCRATCH_BYTES that
 * every device the library runs on holds until the process ends. `desc` is read
 * as in flashMoeCreate (weights borrowed for the duration of the launch; every
 * flag but FLASH_MOE_FLAG_PACK_WEIGHTS is honoured: the array has no room for a
 * packed weight copy, weights the caller has packed in place are fine); the
 * workspace is laid out for tokens_num alone, and with FLASH_MOE_SCHED_AUTO the
 * variant is the one flashMoeLaunch would take if its workspace fits, else the
 * streaming one.
 * A failure on the device (a dependency wait that ran out, a row-tile table that
 * overflowed) is not returned by any call of this entry point: the launch's output
 * is all NaN, the array is usable again, and the error bits (as in flashMoeStatus)
 * are added to a word that flashMoeNoAllocStatus reads and clears.
 * Cost when unused: the array is part of the library's code object, so every
 * process that loads the library holds FLASH_MOE_NOALLOC_SCRATCH_BYTES (+256) of
 * device memory on each device it touches, whether or not it calls this.
 * hipErrorUnknown when tokens_num > desc->max_tokens or when that batch needs
 * more workspace than the array holds (bf16, top-8, 128 experts: 847 tokens of
 * the H2048/I768 shape with the streaming variant and 1447 with the tiled one,
 * 426 and 733 of H4096/I1536); nothing is enqueued then.
 * Enqueues a small clearing kernel and the layer's kernel on `stream`, waits
 * for nothing, calls no hipMalloc/hipFree. The first call on a device looks up
 * the array's address and the device's properties (make it outside a graph
 * capture). All calls on a device share the one array: calls that may overlap
 * on a device (two streams, two threads) race; order them on one stream. */
#define FLASH_MOE_NOALLOC_SCRATCH_BYTES (64u << 20)
int flashMoeLaunchNoAlloc(const FlashMoeLayerDesc* desc, const void* tokens, void* output,
                          int tokens_num, void* stream);

/* Waits for `stream`, then reports and clears the error bits that launches of
 * flashMoeLaunchNoAlloc on the current device have raised since the last call
 * (1 = a dependency wait timed out, 2 = tile table overflow; 0 = none). Not for
 * use under graph capture (it copies one word to the host). */
int flashMoeNoAllocStatus(unsigned* error_bits, void* stream);

/* Frees the workspace; synchronises `stream`. */
int flashMoeDestroy(FlashMoeLauncher* l, void* stream);

/* After a launch of tokens_num tokens: waits for `stream`, then copies the
 * routing of that launch to host arrays (any may be NULL):
 * topk_idx [T,k], topk_w [T,k], expert_counts [E], expert_offsets [E+1],
 * perm [T*k] (permuted row -> t*k+slot; only the first expert_offsets[E] are
 * meaningful). */
int flashMoeReadRouting(FlashMoeLauncher* l, int tokens_num, int* topk_idx, float* topk_w,
                        int* expert_counts, int* expert_offsets, int* perm, void* stream);

/* After a launch of tokens_num tokens: waits for `stream`, then copies the
 * expert stage's intermediate rows to the host: h [tokens_num*top_k, I] in the
 * layer dtype, row r = SiLU(gate proj) * (up proj) of permuted row r (perm[r] of
 * flashMoeReadRouting names its token and slot; rows from expert_offsets[E] on
 * are unused). No counterpart in the reference's library; it is what lets a
 * test compare the gate/up stage alone with the CPU reference, as the
 * reference's stage test does
 * (test/singleGPU/cpp/moe/internal/moeExpertFFN1Test.hip:58-106). */
int flashMoeReadIntermediate(FlashMoeLauncher* l, int tokens_num, void* h, void* stream);

/* After a launch of tokens_num tokens: waits for `stream`, then copies the down
 * projection's rows, as the combine step reads them, to the host:
 * y [tokens_num*top_k, H], row t*top_k+slot = h[row of (t, slot)] . W2[expert]^T.
 * The two variants keep them differently, which *elem_dtype and *weighted report:
 * the streaming variant float32, already multiplied by the slot's gate weight
 * (FLASH_MOE_F32, 1), the tiled variant bfloat16, unweighted (FLASH_MOE_BF16, 0).
 * `y` must hold 4 bytes per element either way. Rows of slots without an expert
 * are undefined. hipErrorInvalidValue if the launcher's workspace keeps fewer rows
 * than asked for (the streaming variant of an AUTO launcher that hands larger
 * batches to the tiled one). No counterpart in the reference's library; it lets a
 * test check the down projection and its scaling apart from the slot sum, as
 * the reference's stage tests do
 * (test/singleGPU/cpp/moe/internal/moeExpertsTests.hip:389-475). */
int flashMoeReadDownRows(FlashMoeLauncher* l, int tokens_num, void* y, int* elem_dtype, int* weighted,
                         void* stream);

/* Device-side failures. A dependency wait inside the kernel is bounded (see
 * flashMoeSetWaitLimitMs); when one runs out, or the row-tile table overflows,
 * the launch ends normally, its last worker fills the launch's output with NaN,
 * returns the workspace to its initial state (so later launches and graph
 * replays work) and adds the error bits to a word in pinned host memory. The
 * first flashMoeLaunch made after that kernel has finished launches nothing and
 * returns hipErrorUnknown (the reference aborts in a device assert instead,
 * src/hip/utils/hipDeviceUtils.h:12); the launch after it runs normally.
 * flashMoeStatus waits for `stream`, reports the bits raised since it was last
 * called (1 = a dependency wait timed out, 2 = tile table overflow), including
 * those a Launch has already reported, and the number of completed launches. */
int flashMoeStatus(FlashMoeLauncher* l, unsigned* error_bits, unsigned* launches, void* stream);

/* Bound on a single dependency wait inside the kernel, in milliseconds
 * (default 2000). A wait that runs out raises error bit 1 and ends the launch. */
int flashMoeSetWaitLimitMs(FlashMoeLauncher* l, double ms);

/* Task timeline for profiling (no counterpart in the reference, whose only
 * timing aid is the host-side hipEvent helper of
 * test/singleGPU/cpp/benchmarks/benchmarkUtils.h:26-52). Enable allocates
 * `capacity` 48-byte records (0 frees them and turns tracing off); a traced
 * launch writes one record per task, indexed by ticket:
 *   { u32 ticket, kind, worker, aux; i64 t_fetch, t_ready, t_end, pad }
 * kind: 0 router dot, 1 scan, 2 scatter, 3 gate/up, 4 down, 5 combine, 6 router
 * select; times in
 * ticks of the 100 MHz device wall clock. Read waits for `stream`, copies up to
 * max_records records to the host and marks all records unused (all bits set). */
int flashMoeTraceEnable(FlashMoeLauncher* l, unsigned capacity);
int flashMoeTraceRead(FlashMoeLauncher* l, void* records, unsigned max_records, void* stream);

/* Which scheduling variant a launch of tokens_num tokens would use. */
int flashMoeSchedFor(FlashMoeLauncher* l, int tokens_num);

const char* flashMoeVersion(void);

/* Binary interface revision, for bindings that were built against another header.
 * History: 1 = first release; 2 = FlashMoeLayerDesc grew by norm_weight and norm_eps
 * (16 bytes at the end; flashMoeCreate reads the whole struct, so a caller built
 * against revision 1 must be rebuilt), flashMoeSetDenseSmallBatch became a no-op;
 * 3 = flashMoeAbi, flashMoeReadDownRows, flashMoeNoAllocStatus added (symbol version
 * LIBFLASHMOE_MI355X_0.3), nothing changed or removed. *desc_bytes (may be NULL)
 * receives sizeof(FlashMoeLayerDesc) as the library was built: a binding compares it
 * with its own before it passes a description. */
#define FLASH_MOE_ABI_VERSION 3
int flashMoeAbi(int* version, size_t* desc_bytes);

/* Retained for binaries built against revision 1: the dense small-batch mode it
 * switched measured slower at every batch size and no longer exists. Does nothing,
 * returns hipSuccess. */
int flashMoeSetDenseSmallBatch(FlashMoeLauncher* l, int enable);

#ifdef __cplusplus
}
#endif
#endif /* FLASH_MOE_H_ */
