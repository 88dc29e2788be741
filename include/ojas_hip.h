/*
 * ojas_hip.h — C ABI of the MI355X (gfx950) backend for Ojas Engine's quantized-matmul path.
 *
 * This is the boundary a Rust `ojas-hip` crate binds with `extern "C"`: plain pointers, sizes and
 * integer status codes; no C++ types, no exceptions, nothing allocated by the caller is retained
 * after a call returns.  Each entry names the reference interface it stands in for (paths are
 * relative to the reference tree).
 *
 * Two seams are exported, as in the reference:
 *   1. the kernel seam  — `Device` + `KernelRuntime` (crates/ojas-core/src/lib.rs:26-40,
 *      crates/ojas-core/src/kernel.rs:67-81; CUDA implementation
 *      crates/ojas-cuda/src/device.rs:418-537): families of kernels loaded by name, dispatched
 *      by canonical entry name with positional buffers then u32 constants;
 *   2. the op seam      — `CudaSsm::mm(x, &Lin, y, m, accum)`
 *      (crates/ojas-cuda/src/qwen35.rs:146-201, :644-702) and the MoE expert FFN
 *      (crates/ojas-cpu/src/cpu_glm.rs:519-597, crates/ojas-cuda/src/kernels/moe.rs:45-125).
 *
 * Threading: one HIP stream per device handle; a handle is used from one thread at a time
 * (the reference's decoder is not Sync either, crates/ojas-core/src/device_fault.rs:19-20).
 * Every call is asynchronous on that stream unless stated; `ojh_submit` and `ojh_download`
 * synchronise.
 *
 * Errors: every function returns OJH_OK (0) or a negative status; `ojh_last_error()` returns a
 * thread-local message for the last failure.  Nothing aborts or throws across this boundary.
 */
#ifndef OJAS_HIP_H
#define OJAS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OJH_ABI_VERSION 1

enum {
    OJH_OK = 0,
    OJH_ERR_ARG = -1,        /* bad argument / shape the kernel cannot take */
    OJH_ERR_HIP = -2,        /* a HIP runtime call failed (message has the HIP error) */
    OJH_ERR_NOT_LOADED = -3, /* kernel or family not loaded: call ojh_ensure_family first */
    OJH_ERR_UNSUPPORTED = -4,/* format / combination without a kernel */
    OJH_ERR_BOUNDS = -5,     /* a buffer is too small for what the kernel would touch */
    OJH_ERR_NO_DEVICE = -6
};

/* GGUF tensor types handled by this path (crates/ojas-formats/src/gguf.rs:563-591). */
enum { OJH_F16 = 1 /* plain f16 rows: the `gemm_mm_f16*` entries only (ojh_lin_create does not take it) */, OJH_Q4_0 = 2, OJH_Q4_1 = 3, OJH_Q5_0 = 6, OJH_Q5_1 = 7, OJH_Q8_0 = 8, OJH_Q2_K = 10, OJH_Q3_K = 11, OJH_Q4_K = 12, OJH_Q5_K = 13, OJH_Q6_K = 14,
       OJH_IQ4_NL = 20, OJH_IQ4_XS = 23,
       /* the grid-codebook formats (gguf.rs:840-1041): decoders and f32-activation matvecs for all seven; IQ2_XXS and
        * IQ3_XXS also on int8 activations, which is what matvec_kq runs for them (cpu_math.rs:1177-1178) */
       OJH_IQ2_XXS = 16, OJH_IQ2_XS = 17, OJH_IQ3_XXS = 18, OJH_IQ1_S = 19, OJH_IQ3_S = 21, OJH_IQ2_S = 22, OJH_IQ1_M = 29,
       /* MXFP4 as the reference packs it for its native matvec: { u8 e8m0 scale; u8 qs[16] } = 17 bytes per 32 weights,
        * weight 2j the low and 2j+1 the high nibble of qs[j]; 139 is the reference's synthetic id (this is a safetensors
        * format, not a GGUF type: crates/ojas-core/src/quant_src.rs:91-95, crates/ojas-formats/src/mxfp4.rs).  f32
        * activations only, no MFMA tile. */
       OJH_MXFP4 = 139 };

/* Element type of an activation buffer handed to ojh_mm. */
enum { OJH_X_F32 = 0, OJH_X_BF16 = 1, OJH_X_F16 = 2 };

/* Arithmetic contract of a matmul.
 *   OJH_ACT_Q8K — activations quantized to int8 per 256 (quant_q8k), integer dots: the arithmetic
 *                 of the CPU reference `matvec_kq` (crates/ojas-cpu/src/cpu_math.rs:1145-1189).
 *                 Q8_0, IQ4_NL and IQ4_XS weights always take f32 activations, as `dot_q80`,
 *                 `dot_iq4nl` and `dot_iq4xs` do (:971-981, :993-1010, :943-967): asking for
 *                 OJH_ACT_Q8K on IQ4 rows is refused, and no MFMA tile reads them (every token
 *                 count runs on the matvec entries).  The same holds for the legacy 32-weight
 *                 blocks Q4_0, Q4_1, Q5_0, Q5_1 and for Q2_K and Q3_K, which the reference runs on
 *                 its GPU path only (f32 activations against the weights of `dequant_to_f16`'s
 *                 arms :653-703 and :730-795).  Of the grid-codebook formats IQ2_XXS and IQ3_XXS
 *                 take this contract (dot_iq2xxs_q8k / dot_iq3xxs_q8k, :1057-1128: what matvec_kq
 *                 runs for them, and what OJH_ACT_AUTO picks at every token count); IQ3_S and
 *                 IQ2_S are f32-activation rows on the CPU path (dot_iq3s, dot_iq2s) and IQ2_XS,
 *                 IQ1_S, IQ1_M exist on the reference's GPU path only: those five refuse it.  No
 *                 MFMA tile reads a grid-codebook format.
 *   OJH_ACT_FLOAT — activations kept in floating point (f32 for the GEMV, rounded to f16 into the
 *                 MFMA tile for the GEMM): the contract of the reference's GPU kernels
 *                 (crates/ojas-core/src/quant_src.rs:779-867, crates/ojas-cuda/src/kernels/gemm_q.rs:1-56).
 *                 In the tile a Q4_K weight is the binary16 fma qa*q + qb with qa = f16(d*sc),
 *                 qb = f16(-dmin*m): the bits the reference's `gemm_mm_q4l` multiplies
 *                 (gemm_q.rs:104-140 over crates/ojas-formats/src/quant.rs:187-222); Q6_K and Q8_0
 *                 weights are the bits of `dequant_to_f16`.
 *   OJH_ACT_FLOAT_EXACT — as OJH_ACT_FLOAT, but a Q4_K weight too enters the tile as the bits of
 *                 `dequant_to_f16` (crates/ojas-formats/src/gguf.rs:612-1116); a slower tile.
 *   OJH_ACT_Q8_1 — Q8_0 rows only, f32 activations: quantized to int8 per 32 values (`quantize_q8_1`), integer dots
 *                 against the blocks as the file stores them, token by token: the arithmetic of the reference's GPU
 *                 decode path for Q8_0 models (crates/ojas-cuda/src/kernels/gemv_q8.rs:152-215, gemv.rs:33-52; its
 *                 own bar 1e-2 of the output peak against the dequantized dot).  Never chosen by OJH_ACT_AUTO.
 *   OJH_ACT_AUTO  — OJH_ACT_Q8K for K-quant GEMV-shaped calls, OJH_ACT_FLOAT above the crossover. */
enum { OJH_ACT_AUTO = 0, OJH_ACT_Q8K = 1, OJH_ACT_FLOAT = 2, OJH_ACT_FLOAT_EXACT = 3, OJH_ACT_Q8_1 = 4 };

typedef struct ojh_gguf ojh_gguf;     /* an open GGUF file: metadata + tensor index */
typedef struct ojh_device ojh_device; /* one GPU + one stream + loaded families */
typedef struct ojh_buf ojh_buf;       /* device allocation with a known size */
typedef struct ojh_lin ojh_lin;       /* a weight matrix W[N,K] in its GGUF block bytes */
typedef struct ojh_graph ojh_graph;   /* a recorded chain of dispatches, replayable */
typedef struct ojh_expert_cache ojh_expert_cache; /* device arena of expert slots, LRU */

/* Mirrors `Caps` (crates/ojas-core/src/kernel.rs:26-41). */
typedef struct ojh_caps {
    int32_t tier;            /* 0 = C, 1 = B, 2 = A (matrix units) */
    int32_t f16_compute;
    uint32_t simd_width;     /* 64 */
    int32_t unified_memory;  /* 0 */
    uint64_t max_buffer;
    uint32_t compute_units;
    uint32_t clock_mhz;
    uint64_t total_memory;
    char arch[32];           /* "gfx950..." */
    const char *features;    /* comma-separated: "mfma_bf16,mfma_f16,mfma_i8,dot4_i8,wave64" */
} ojh_caps;

/* ---- device lifetime ---------------------------------------------------------------------- */
/* `CudaGpu::new` (crates/ojas-cuda/src/device.rs:91-131). Fails with OJH_ERR_NO_DEVICE when no
 * gfx950 GPU is visible: there is no CPU fallback behind this library. */
int ojh_open(int ordinal, ojh_device **out);
int ojh_close(ojh_device *dev);
/* `Device::name` (crates/ojas-core/src/lib.rs:31). */
const char *ojh_name(const ojh_device *dev);
/* `KernelRuntime::caps` (crates/ojas-core/src/kernel.rs:72). */
int ojh_caps_get(const ojh_device *dev, ojh_caps *out);
const char *ojh_last_error(void);
int ojh_abi_version(void);

/* ---- buffers: `Device::alloc / upload / read` (crates/ojas-core/src/lib.rs:36-39,
 *      crates/ojas-cuda/src/device.rs:448-476, byte forms :341-389) --------------------------- */
int ojh_alloc(ojh_device *dev, size_t bytes, ojh_buf **out);
int ojh_free(ojh_device *dev, ojh_buf *buf);
/* Wrap device memory owned by someone else (e.g. a tensor of the host framework); not freed. */
int ojh_wrap(ojh_device *dev, void *device_ptr, size_t bytes, ojh_buf **out);
size_t ojh_buf_bytes(const ojh_buf *buf);
void *ojh_buf_ptr(const ojh_buf *buf);
/* Synchronous with respect to the host buffer: it may be reused as soon as the call returns. */
int ojh_upload(ojh_device *dev, ojh_buf *dst, size_t dst_off, const void *host, size_t bytes);
/* Waits for the device stream, then copies. */
int ojh_download(ojh_device *dev, const ojh_buf *src, size_t src_off, void *host, size_t bytes);
int ojh_memset0(ojh_device *dev, ojh_buf *dst, size_t off, size_t bytes);

/* ---- kernel seam: `KernelRuntime` (crates/ojas-core/src/kernel.rs:67-81) -------------------- */
/* Load the family's gfx950 code object (built offline). Families: "dequant", "gemv",
 * "gemv_q8k", "gemm", "moe".  Idempotent. */
int ojh_ensure_family(ojh_device *dev, const char *family);
/* 1 if `name` resolved in a loaded family, 0 otherwise (never an error). */
int ojh_has_kernel(const ojh_device *dev, const char *name);
/* The family that defines `name` in this build's manifest, or NULL. */
const char *ojh_kernel_family(const char *name);
/* Manifest walk for structural tests: returns the number of kernels; fills name/family/counts
 * of entry i when i is in range (crates/ojas-core/src/kernel.rs:43-58 `KernelSpec`). */
int ojh_manifest(int i, const char **name, const char **family, int *n_bufs, int *n_consts);
/* wave64 launch shape for a kernel at a problem size. The reference's callers carry 32-lane
 * tables (crates/ojas-core/src/quant_src.rs:83-111); on gfx950 the library owns them. */
int ojh_launch_shape(const ojh_device *dev, const char *name, uint32_t K, uint32_t N, uint32_t M,
                     uint32_t grid[3], uint32_t block[3]);
/* `dispatch(enc, name, bufs, consts, grid, block)`: buffers (with byte offsets) first, then u32
 * constants, in the kernel's documented order.  Buffer sizes are checked against what the kernel
 * touches at these constants before anything is launched. */
int ojh_dispatch(ojh_device *dev, const char *name, int n_bufs, ojh_buf *const *bufs,
                 const uint64_t *offsets, int n_consts, const uint32_t *consts,
                 const uint32_t grid[3], const uint32_t block[3]);
/* `submit(enc)`: wait for everything dispatched so far. */
int ojh_submit(ojh_device *dev);

/* Record-and-replay of a chain of dispatches (the reference's encoder is a chain submitted as a
 * unit, crates/ojas-core/src/kernel.rs:73-80; its `Caps.features` names "cuda_graphs" for the
 * same purpose, :38-40).  Between begin and end every dispatch / ojh_mm* / ojh_quant_q8k call is
 * recorded instead of run; calls that synchronise or allocate (alloc, free, upload, download,
 * submit, a scratch buffer that has to grow) fail with OJH_ERR_ARG — run the chain once eagerly
 * first.  `ojh_graph_launch` replays the chain on the device's stream with one host call: by
 * default from a native loop over the recorded launches, or as an instantiated hipGraph when
 * OJAS_HIP_REPLAY=graph is set in the environment at `ojh_capture_begin`.
 * A chain keeps the device addresses it was recorded with, including those of the library's own
 * scratch buffers (ojh_mm, ojh_matmul_q8, ojh_moe_ffn stage activations there).  While any chain of
 * a device is alive, a scratch buffer that a later eager call outgrows is kept (parked) rather than
 * freed, so replays stay valid; the parked memory is released when the last chain is freed.  Buffers
 * the caller passed in must outlive the chain, as with any recorded pointer.
 * If a call fails between begin and end, call `ojh_capture_end` all the same: it ends the recording
 * (its own result may be an error in hipGraph mode, where a failed HIP call invalidates the capture)
 * and the device runs eagerly again. */
int ojh_capture_begin(ojh_device *dev);
int ojh_capture_end(ojh_device *dev, ojh_graph **out);
int ojh_graph_launch(ojh_device *dev, ojh_graph *graph);
int ojh_graph_free(ojh_device *dev, ojh_graph *graph);

/* Event timing on the device's stream (the reference times kernels the same way,
 * crates/ojas-cuda/tests/prefill_gemm_q.rs:262-283). `ojh_timer_stop` synchronises. */
int ojh_timer_start(ojh_device *dev);
int ojh_timer_stop(ojh_device *dev, float *elapsed_ms);
/* A pool of OJH_MAX_MARKS events for timing individual launches inside a longer region:
 * `ojh_mark` records event `slot` on the stream; `ojh_mark_elapsed` waits for `b` and returns the
 * time from `a` to `b`. */
#define OJH_MAX_MARKS 8192
int ojh_mark(ojh_device *dev, int slot);
int ojh_mark_elapsed(ojh_device *dev, int a, int b, float *elapsed_ms);

/* ---- op seam ------------------------------------------------------------------------------ */
/* `Lin::load` (crates/ojas-cuda/src/qwen35.rs:174-201): keep the tensor in its GGUF block bytes.
 * `raw` is host memory of n * row_bytes(type, k) bytes and is copied before the call returns. */
int ojh_lin_create(ojh_device *dev, uint32_t ggml_type, uint32_t n, uint32_t k, const void *raw,
                   ojh_lin **out);
/* Same, over block bytes already resident in `raw` at `off` (borrowed, not freed). */
int ojh_lin_wrap(ojh_device *dev, uint32_t ggml_type, uint32_t n, uint32_t k, ojh_buf *raw,
                 size_t off, ojh_lin **out);
int ojh_lin_free(ojh_device *dev, ojh_lin *lin);
size_t ojh_row_bytes(uint32_t ggml_type, uint32_t k); /* 0 for an unknown type / ragged k */

/* `CudaSsm::mm(x, w, y, m, accum)` (crates/ojas-cuda/src/qwen35.rs:644-702):
 * y[m][N] (=, +=) x[m][K] . W^T, f32 result.  Chooses GEMV / small-M / MFMA tile / split-K.
 * `bias` (f32[N]) may be NULL. */
int ojh_mm(ojh_device *dev, const ojh_buf *x, size_t x_off, int x_dtype, const ojh_lin *w,
           ojh_buf *y, size_t y_off, const ojh_buf *bias, uint32_t m, int accum, int act_mode);

/* `ojh_mm` with OJH_ACT_Q8K for callers that cannot allocate device memory — code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.
 * The int8 activations and their per-256 scales are staged in a static device array of
 * `ojh_noalloc_scratch_bytes()` bytes (1 MiB of activations + their scales) that each GPU holds
 * until the process ends, so the call allocates and frees nothing; the launches and results are
 * those of `ojh_mm(..., OJH_ACT_Q8K)` bit for bit below 17 tokens; from there `ojh_mm` may take a
 * prefill tile or K slices that stage more in library scratch, which this entry never does (Q4_K stays
 * on the few-token kernels, Q6_K / Q5_K take their 128-token tile unsliced: the same integer sums, the
 * f32 terms equal to rounding).  K-quant weights (Q4_K, Q5_K, Q6_K), f32 or bf16
 * activations, m * K <= OJH_NOALLOC_MAX_ACT (OJH_ERR_BOUNDS beyond); the families "gemv_q8k" and
 * "gemm_q8k" must already be loaded (OJH_ERR_NOT_LOADED otherwise: loading allocates).  Every
 * handle on one GPU shares that GPU's array: calls that overlap on one GPU race. */
#define OJH_NOALLOC_MAX_ACT (1u << 20)
int ojh_mm_noalloc(ojh_device *dev, const ojh_buf *x, size_t x_off, int x_dtype, const ojh_lin *w,
                   ojh_buf *y, size_t y_off, const ojh_buf *bias, uint32_t m, int accum);
size_t ojh_noalloc_scratch_bytes(void);

/* The same product from activations that are already quantized (`ojh_quant_q8k`): one
 * quantization feeds every projection that reads the same vector (q/k/v, gate/up), the split the
 * reference's CUDA path makes between `quantize_q8_1` and `gemv_q80_dp4a`
 * (crates/ojas-cuda/src/kernels/gemv.rs:37-53, gemv_q8.rs:178-292). K-quant weights only. */
int ojh_mm_q8k(ojh_device *dev, const ojh_buf *xq, const ojh_buf *xscales, const ojh_lin *w, ojh_buf *y,
               size_t y_off, const ojh_buf *bias, uint32_t m, int accum);

/* One to four projections of the same quantized vector in ONE launch: ys[i] = xq . ws[i]^T, each
 * Lin its own allocation, all with the same K.  The reference's fused q/k/v and gate/up launches
 * (`qkv_q80_dp4a`, `ffn_gu_q80_dp4a`: crates/ojas-core/src/kernels/gemv_q8.rs:229-260) take one
 * pointer per projection in the same way.  Results are bit-identical to `count` calls of
 * `ojh_mm_q8k`.  Q4_K, Q5_K and Q6_K tensors may be mixed in one call (a Q4_K_M file keeps attention v and
 * the feed-forward down in Q6_K): still one launch, every row in its own format's arithmetic; other formats
 * run as that many launches.
 * `y_offs` (bytes) may be NULL. */
int ojh_mm_q8k_multi(ojh_device *dev, const ojh_buf *xq, const ojh_buf *xscales, int count,
                     const ojh_lin *const *ws, ojh_buf *const *ys, const size_t *y_offs);

/* One stage of a decode layer in ONE launch: ys[i] (=, +=) x . ws[i]^T for one to four projections of the same
 * f32 vector x[K] (q/k/v, gate/up, or a single o / down / head), the vector quantized as `quant_q8k` does inside the
 * launch — the reference's CUDA decode path fuses the same steps (`qkv_q80_dp4a`, `ffn_gu_q80_dp4a` after
 * `quantize_q8_1`, crates/ojas-cuda/src/kernels/gemv_q8.rs:178-260).  Bit-identical to `ojh_quant_q8k` followed by
 * `ojh_mm_q8k` per projection (OJH_ACT_Q8K arithmetic); `accum` adds onto every y.  Q4_K tensors with K <= 16384 take
 * the single launch; other K-quant formats or longer rows run as a quantizer launch plus the per-format launches.
 * `y_offs` (bytes) may be NULL. */
int ojh_mm_multi(ojh_device *dev, const ojh_buf *x, size_t x_off, int count, const ojh_lin *const *ws,
                 ojh_buf *const *ys, const size_t *y_offs, int accum);

/* A decode step's dependent stages in ONE launch.  Each stage is what `ojh_mm_multi` computes — one to four
 * Q4_K projections of one f32 vector, quantized as `quant_q8k` does — and a stage may read what an earlier stage
 * of the same call wrote (x of stage s = a y of stage s-1, or the residual an earlier stage accumulated onto):
 * q/k/v -> o -> gate/up -> down -> output head, or a feed-forward block norm -> gate/up -> SiLU*up -> down.  The
 * reference fuses neighbouring projections per launch (`qkv_q80_dp4a`, `ffn_gu_q80_dp4a`,
 * crates/ojas-cuda/src/kernels/gemv_q8.rs:229-260) and still pays dispatches per dependent stage; here the grid
 * is the concatenation of all stages' workgroups (per stage a few quantizer workgroups, then the row workgroups
 * of the separate launch), the hardware hands them out in index order, and what one workgroup hands to another
 * travels as {value, launch tag} pairs that the reader polls a bounded number of times.  The arithmetic of a
 * stage starts only after every element of its input has arrived.  Results are bit-identical to the same stages
 * run as separate `ojh_mm_multi` (and, for the prologues, `ojh_ffn_gu_q8k` / `ojh_rmsnorm_quant_q8k`) launches.
 * Measured on MI355X the single launch is SLOWER than the separate launches for the 8B decode step (the waits'
 * round trips run through a memory system the other workgroups keep saturated); the separate launches stay the
 * library's default path and this entry point is for callers that need one launch.
 *
 * `prologue` says how the stage's input is formed from `x` (and `x2`) before it is quantized:
 *   OJH_CHAIN_X_PLAIN     x
 *   OJH_CHAIN_X_SILU_MUL  silu(x) * x2        (x = gate projection, x2 = up projection; cpu_math.rs:486)
 *   OJH_CHAIN_X_GELU_MUL  gelu_tanh(x) * x2   (cpu_math.rs:497-501)
 *   OJH_CHAIN_X_RMSNORM   x * (1 / sqrt(mean(x^2) + eps)) * x2, x2 = the norm's weights (cpu_math.rs:456-460;
 *                         the mean of squares is summed in f64 and rounded once, as ojh_rmsnorm_quant_q8k does)
 * Limits: 1..OJH_CHAIN_MAX_STAGES stages; Q4_K tensors; all tensors of a stage share K, K % 256 == 0,
 * K <= 16384; a stage's x / x2 must not overlap its own outputs; an input that lies inside an output of an
 * earlier stage is followed inside the launch, one that only straddles such an output is refused; a stage that
 * accumulates onto an output of an earlier stage must take that whole vector and depend on that stage through
 * its inputs.  Waits are bounded (OJAS_HIP_CHAIN_SPIN looks, default 2^22, or `ojh_chain_spin_limit`): if one
 * gives up, every kernel still exits and the next `ojh_submit` / `ojh_download` on the device returns
 * OJH_ERR_HIP; outputs of chain calls since the last successful one are then undefined.  The call is
 * asynchronous like every other launch and can be recorded (`ojh_capture_begin`, the library's own replay; a
 * captured hipGraph would freeze the launch tag and is refused) after one eager call. */
#define OJH_CHAIN_MAX_STAGES 8
enum { OJH_CHAIN_X_PLAIN = 0, OJH_CHAIN_X_SILU_MUL = 1, OJH_CHAIN_X_GELU_MUL = 2, OJH_CHAIN_X_RMSNORM = 3 };
typedef struct ojh_chain_stage {
    const ojh_buf *x;      /* f32[K] input */
    size_t x_off;          /* bytes */
    const ojh_buf *x2;     /* second operand of the prologue, NULL for OJH_CHAIN_X_PLAIN */
    size_t x2_off;
    int prologue;          /* OJH_CHAIN_X_* */
    float eps;             /* OJH_CHAIN_X_RMSNORM */
    int count;             /* 1..4 projections reading this input */
    const ojh_lin *ws[4];
    ojh_buf *ys[4];        /* f32[ws[i]->n] each */
    size_t y_offs[4];      /* bytes */
    int accum;             /* ys[i] += instead of = */
} ojh_chain_stage;
int ojh_decode_chain(ojh_device *dev, const ojh_chain_stage *stages, int n_stages);
/* Timestamps of the chain launches that follow, for profiling: `buf` receives, per stage, when the stage's first
 * quantizer workgroup started, had its input (i.e. the rows it waited for were done) and had published it, as
 * the 100 MHz counter's value, u64 [OJH_CHAIN_MAX_STAGES][3]; NULL switches it off.  The buffer must outlive the
 * launches (also recorded ones). */
int ojh_chain_trace(ojh_device *dev, ojh_buf *buf);
/* Polls a chain's waits may take from now on (0: every wait gives up at once — the failure path, for tests). */
int ojh_chain_spin_limit(ojh_device *dev, uint32_t polls);

/* Decode-layer epilogues around the matvec (the reference fuses the same steps on its GPU path:
 * `rmsnorm_q8` / `quantize_q8_1` and `ffn_gu_q80_dp4a`, crates/ojas-cuda/src/kernels/gemv.rs:37-53,
 * gemv_q8.rs:246-260).
 *   ojh_rmsnorm_quant_q8k: per row of x (f32 [m][k], k <= 16384), xn = x * rsqrt(mean(x^2) + eps) * gamma
 *     (`rmsnorm`, crates/ojas-cpu/src/cpu_math.rs:456-460) quantized as `quant_q8k` does, in one
 *     launch; `xn` (f32 [m][k]) may be NULL when only the quantized form is needed.
 *   ojh_ffn_gu_q8k: out[n] = act(gate[n] . x) * (up[n] . x) from one quantized vector; act 0 = SiLU
 *     (cpu_math.rs:486), 1 = GELU tanh form (:497-501).  Q4_K, Q5_K or Q6_K tensors of equal shape (the two
 *     may differ in format); each dot has the bits of that format's matvec. */
int ojh_rmsnorm_quant_q8k(ojh_device *dev, const ojh_buf *x, size_t x_off, const ojh_buf *gamma, float eps,
                          uint32_t m, uint32_t k, ojh_buf *q, ojh_buf *scales, ojh_buf *xn);
int ojh_ffn_gu_q8k(ojh_device *dev, const ojh_buf *xq, const ojh_buf *xscales, const ojh_lin *gate,
                   const ojh_lin *up, ojh_buf *out, size_t out_off, int act);

/* `relayout_q4k_q4l` (crates/ojas-formats/src/quant.rs:192-222) on the device: n rows of k Q4_K
 * weights -> nibble pairs `nib` [n*k/2], f16 `qa` = d*sc and `qb` = -dmin*m per 32 weights
 * [n*k/32 each].  Bit-exact with the reference.  The library's own prefill GEMM does not need
 * it (it forms qa / qb in the tile from the raw blocks); it serves callers that keep Q4L. */
int ojh_relayout_q4k_q4l(ojh_device *dev, const ojh_buf *raw, size_t raw_off, uint32_t n, uint32_t k,
                         ojh_buf *nib, ojh_buf *qa, ojh_buf *qb);

/* The row-int8 representation of the reference's CPU models (`W::Q8`,
 * crates/ojas-cpu/src/cpu_math.rs:14-23).  `ojh_q8rows_from_f16` is the load-time requantization
 * `q8_rows_from_f16` (crates/ojas-formats/src/quant.rs:16-39): binary16 weights [n][k] -> int8
 * [n][k] + one f32 scale per row.  `ojh_matmul_q8` is `matmul(w, xs, m)` (cpu_math.rs:187-289):
 * every row of x (f32 [m][k]) quantized per whole vector (`quant_row_i8`, :174-179), integer
 * dots, y[m][n] = bias + acc*sw*sx rounded operation by operation — bit-identical to the CPU
 * path.  `bias` (f32[n]) may be NULL.  K must be a multiple of 16. */
int ojh_q8rows_from_f16(ojh_device *dev, const ojh_buf *w16, size_t w_off, uint32_t n, uint32_t k,
                        ojh_buf *q, ojh_buf *scale);
int ojh_matmul_q8(ojh_device *dev, const ojh_buf *x, size_t x_off, const ojh_buf *wq, const ojh_buf *wscale,
                  const ojh_buf *bias, ojh_buf *y, size_t y_off, uint32_t n, uint32_t k, uint32_t m);

/* `dequant_to_f16` (crates/ojas-formats/src/gguf.rs:612-1116) on the device: `n_weights`
 * weights of `raw` -> binary16 bit patterns in `out`. Bit-exact with the reference. */
int ojh_dequant_f16(ojh_device *dev, uint32_t ggml_type, const ojh_buf *raw, size_t raw_off,
                    size_t n_weights, ojh_buf *out, size_t out_off);

/* `quant_q8k` (crates/ojas-cpu/src/cpu_math.rs:539-563) for m rows of k activations:
 * q int8 [m][ceil(k/256)*256], scales f32 [m][ceil(k/256)]. */
int ojh_quant_q8k(ojh_device *dev, const ojh_buf *x, size_t x_off, int x_dtype, uint32_t m,
                  uint32_t k, ojh_buf *q, ojh_buf *scales);

/* Router: softmax over `n_expert` logits per token, top-`ksel` (lowest index wins ties),
 * renormalised (crates/ojas-cuda/src/kernels/moe.rs:45-70). idx u32[T][ksel], wgt f32[T][ksel]. */
int ojh_moe_route(ojh_device *dev, const ojh_buf *logits, uint32_t n_tokens, uint32_t n_expert,
                  uint32_t ksel, ojh_buf *idx, ojh_buf *wgt);

/* Expert FFN over all (token, slot) assignments, grouped by expert
 * (crates/ojas-cpu/src/cpu_glm.rs:551-582; per-assignment GPU form
 * crates/ojas-metal/src/kernels/moe.rs:199-272):
 *   y[t] (+)= sum_j wgt[t][j] * Wd_e( silu(Wg_e x[t]) * (Wu_e x[t]) ),  e = idx[t][j].
 * gate/up: n_expert stacked Q4_K matrices [n_ff][d]; down: n_expert stacked [d][n_ff], Q4_K, Q5_K or Q6_K.
 * Or gate+up and down each one of Q8_0, IQ4_XS, IQ4_NL: f32 activations meet the raw rows as dot_q80 /
 * dot_iq4xs / dot_iq4nl do (crates/ojas-cpu/src/cpu_math.rs:943-1010) through the reference's own expert
 * kernels moe_gu_<fmt> / moe_down_<fmt> (crates/ojas-cuda/src/kernels/moe.rs:75-125, moe_iq.rs:64-112),
 * one launch each over all tokens; there act_mode is OJH_ACT_AUTO or OJH_ACT_FLOAT and d, n_ff are
 * whole blocks of the formats.  Under OJH_ACT_AUTO a batch of such experts (4 assignments per expert on
 * average for Q8_0, IQ4_NL and IQ4_XS, 8 where a tensor is in a grid codebook; d and n_ff multiples of 64) is grouped by expert on the f16 matrix tile:
 * activations and silu * up rounded to f16, f32 accumulate, within 1e-3 of the output peak of the f32
 * products; OJH_ACT_FLOAT keeps the per-assignment kernels at every batch size.  K-quant experts take the same two launches under OJH_ACT_FLOAT
 * (`moe_gu_q4k`, `moe_down_{q4k,q5k,q6k}`: f32 activations against the dequantized weights, the
 * reference's GPU expert kernels for those formats, crates/ojas-core/src/quant_src.rs:174-179);
 * OJH_ACT_AUTO and OJH_ACT_Q8K keep the CPU path's int8-activation arithmetic for them.
 * Expert indices must be below n_expert (one that is not never reads outside the tensors; what
 * it contributes is unspecified). Up to 2 tokens run as two launches addressed
 * by assignment (bit-identical to the grouped integer-dot pipeline) when d <= 8192, n_ff <= 2048,
 * ksel <= 64 and ksel * n_ff <= 32768 (beyond that the grouped pipeline serves them; forcing the
 * two-launch form with OJAS_HIP_MOE=3 then returns OJH_ERR_UNSUPPORTED); larger batches are grouped
 * by expert, on int8 MFMA from three to four assignments per expert (sums associate differently there:
 * last ulps). Environment: OJAS_HIP_MOE = 1 / 2 / 3 forces MFMA / grouped dots / the decode
 * form, OJAS_HIP_MOE_DEC_TOKENS moves the 8. */
int ojh_moe_ffn(ojh_device *dev, const ojh_buf *x, uint32_t n_tokens, uint32_t d, uint32_t n_ff,
                uint32_t n_expert, uint32_t ksel, const ojh_buf *idx, const ojh_buf *wgt,
                const ojh_lin *gate, const ojh_lin *up, const ojh_lin *down, ojh_buf *y,
                int accum, int act_mode);

/* Router and expert FFN in one call: logits [n_tokens][n_expert] f32 -> idx, wgt [n_tokens][ksel] (written: softmax,
 * top ksel, renormalised — ojh_moe_route's arithmetic, the same bits) -> y as ojh_moe_ffn.  For up to 2 tokens over
 * Q4_K gate / up experts (the decode form of ojh_moe_ffn and its limits) the router runs inside the gate/up launch:
 * two launches per layer and token instead of three; every other case is ojh_moe_route followed by ojh_moe_ffn.
 * The op-level seam of the reference takes router logits or (idx, wgt) alike (ojas-cuda moe.rs:45-125 run back to
 * back by its decoders); OJAS_HIP_MOE_ROUTE_FUSE=0 keeps the router a launch of its own. */
int ojh_moe_ffn_routed(ojh_device *dev, const ojh_buf *x, uint32_t n_tokens, uint32_t d, uint32_t n_ff,
                       uint32_t n_expert, uint32_t ksel, const ojh_buf *logits, ojh_buf *idx, ojh_buf *wgt,
                       const ojh_lin *gate, const ojh_lin *up, const ojh_lin *down, ojh_buf *y, int accum,
                       int act_mode);

/* The same over streamed experts: the matrices of assignment a = (token, slot) start at byte
 * offset off_*[a] (u64, 16-byte aligned) of their arena, wherever the caller's expert cache put
 * them (crates/ojas-cuda/src/kernels/moe.rs:133-174 `moe_{gu,down}_*_slots`,
 * crates/ojas-cuda/src/expert_cache.rs). Q4_K experts, the two-launch form at any token count;
 * d <= 8192, n_ff <= 2048, ksel <= 64, ksel * n_ff <= 32768. An offset at which a whole expert
 * does not fit is clamped to the last one at which it does. */
int ojh_moe_ffn_slots(ojh_device *dev, const ojh_buf *x, uint32_t n_tokens, uint32_t d, uint32_t n_ff,
                      uint32_t ksel, const ojh_buf *arena_gate, const ojh_buf *off_gate,
                      const ojh_buf *arena_up, const ojh_buf *off_up, const ojh_buf *arena_down,
                      const ojh_buf *off_down, const ojh_buf *wgt, ojh_buf *y, int accum);

/* ---- resident expert cache ----------------------------------------------------------------------
 * `ExpertCache` (crates/ojas-cuda/src/expert_cache.rs:34-152): a device arena of budget / expert_bytes
 * (at least one) fixed-size slots.  `gather` makes every requested expert resident — hits are re-ticked,
 * misses take a free slot or evict the least recently used one and are filled through `load`, which
 * writes one expert's bytes into page-locked staging (where a caller does its pread from the model
 * file) — and returns one byte offset into the arena per request, in the order asked: what
 * ojh_moe_ffn_slots and the `_slots` kernels take.  More distinct experts in one call than the arena
 * has slots is refused (OJH_ERR_BOUNDS), not absorbed.  Copies are queued on the device's stream: work
 * queued afterwards sees them, work queued before has finished with the slot.  Two staging buffers
 * alternate, so `load` of one miss overlaps the copy of the previous one.  Not while a chain is being
 * recorded.  With dev = NULL the cache keeps the books only (no arena, `load` unused): hit rates of a
 * routing trace under a budget, without a GPU.  Destroy a cache before closing its device. */
typedef struct ojh_gather_stats {
    uint64_t hits, misses, bytes_streamed, evictions;
} ojh_gather_stats;
/* Fill dst[0 .. bytes) with expert `id`; return 0, or non-zero to abort the gather. */
typedef int (*ojh_expert_load_fn)(void *user, uint32_t id, void *dst, size_t bytes);
int ojh_expert_cache_create(ojh_device *dev, size_t budget_bytes, size_t expert_bytes, ojh_expert_cache **out);
int ojh_expert_cache_destroy(ojh_expert_cache *cache);
uint32_t ojh_expert_cache_slots(const ojh_expert_cache *cache);
size_t ojh_expert_cache_resident_bytes(const ojh_expert_cache *cache);   /* slots * expert_bytes */
ojh_buf *ojh_expert_cache_arena(ojh_expert_cache *cache);                /* owned by the cache */
int ojh_expert_cache_gather(ojh_expert_cache *cache, const uint32_t *ids, size_t n, ojh_expert_load_fn load,
                            void *user, uint64_t *offsets);
int ojh_expert_cache_stats(const ojh_expert_cache *cache, ojh_gather_stats *out);

/* ---- GGUF files -> device (no GPU needed for the reader itself) --------------------------------
 * `Gguf::open` / `tensor_meta` / `read_tensor_raw` (crates/ojas-formats/src/gguf.rs:100-206, 297-339,
 * 440-452, 551-556): versions 2 and 3, the reference's header limits, `general.alignment`, extents
 * validated against the file length.  Split models (split.count > 1) are refused.
 * `ojh_gguf_tensor_meta`: dims padded with 1 to four entries; `bytes` is 0 for a type whose on-disk
 * size this reader does not know (`stored_bytes`, gguf.rs:563-591). */
int ojh_gguf_open(const char *path, ojh_gguf **out);
int ojh_gguf_close(ojh_gguf *g);
int ojh_gguf_tensor_count(const ojh_gguf *g);
const char *ojh_gguf_tensor_name(const ojh_gguf *g, int i);
int ojh_gguf_tensor_meta(const ojh_gguf *g, const char *name, uint32_t *ggml_type, uint32_t *n_dims,
                         uint64_t dims[4], uint64_t *file_offset, uint64_t *bytes);
int ojh_gguf_meta_u64(const ojh_gguf *g, const char *key, uint64_t *out);
int ojh_gguf_meta_str(const ojh_gguf *g, const char *key, char *out, size_t cap);
int ojh_gguf_read_raw(ojh_gguf *g, const char *name, void *dst, uint64_t cap);

/* `Lin::load` (crates/ojas-cuda/src/qwen35.rs:174-201): the named tensors, which must share K
 * (dims[0]) and the GGUF type, stacked along N into one device allocation in the file's own
 * block bytes (Q8_0 / Q4_K / Q6_K with K a whole number of blocks; anything else is refused —
 * the reference dequantizes such groups to f16, which is outside this library).  The file is
 * streamed through a pinned staging buffer; no host copy of the tensor is kept. */
int ojh_lin_load(ojh_device *dev, ojh_gguf *g, const char *const *names, int count, ojh_lin **out);

#ifdef __cplusplus
}
#endif
#endif
