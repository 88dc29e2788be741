// Internal declarations shared by the host-side translation units of libojas_hip.so.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <map>
#include <string>
#include <vector>

#include "../../include/ojas_hip.h"

struct ojh_buf {
    void *ptr = nullptr;
    size_t bytes = 0;
    bool owned = false;
};

struct ojh_lin {
    uint32_t type = 0, n = 0, k = 0;
    size_t row_bytes = 0;
    ojh_buf *raw = nullptr;  // block bytes
    size_t off = 0;
    bool owns_raw = false;
};

// One recorded launch.
struct ojh_command {
    hipFunction_t fn = nullptr;
    std::vector<void *> ptrs;
    std::vector<uint32_t> consts;
    std::vector<uint8_t> blob;   // a kernel whose arguments are one struct: its bytes, passed as the argument buffer
    int tag_offset = -1;         // ... and where in it every launch writes a fresh 32-bit tag (-1: nowhere)
    uint32_t grid[3] = {1, 1, 1}, block[3] = {1, 1, 1};
};

// A recorded chain: either a command list replayed from a native loop, or an instantiated hipGraph.
struct ojh_graph {
    std::vector<ojh_command> list;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
};

// Scratch the op-level entry points keep per device (quantized activations, MoE staging).
struct ojh_scratch {
    ojh_buf *buf = nullptr;
};

struct ojh_device {
    int ordinal = 0;
    hipStream_t stream = nullptr;
    hipDeviceProp_t prop{};
    std::string name;
    std::map<std::string, hipModule_t> modules;      // family -> code object
    std::map<std::string, hipFunction_t> functions;  // entry name -> function
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    std::vector<hipEvent_t> marks;  // lazily created, indexed by slot
    // named scratch buffers, grown on demand
    std::map<std::string, ojh_buf *> scratch;
    int gemv_rows_override = 0;  // OJAS_HIP_GEMV_R
    uint32_t gemm_min_m = 32;    // OJAS_HIP_GEMM_MIN_M: rows from which ojh_mm takes the MFMA tile
    int gemm_split_override = 0; // OJAS_HIP_GEMM_SPLIT
    int q80_lds = 1;             // OJAS_HIP_Q80_LDS: 0 = never take the LDS-staged Q8_0 matvec
    uint32_t q80_lds_min_n = 8192;  // OJAS_HIP_Q80_LDS_MIN_N: rows from which it is taken (weights from HBM, K = 4096: 14336 rows 15.3 against 17.8 us, 4096 rows 7.9 against 7.0)
    uint32_t q80_lds_bpc = 0;       // OJAS_HIP_Q80_LDS_BPC: workgroups per CU its grid is sized for (0: 2 or 3 by K chunking)
    uint32_t q6k_mf_min_m = 5;   // OJAS_HIP_Q6K_MF_MIN_M: tokens from which Q6_K rows (fewer than 32768) go to the int8 matrix cores
    uint32_t q6k_ml_min_m = 2;   // OJAS_HIP_Q6K_ML_MIN_M: ... with the rows copied through LDS (32768 rows or more)
    int q6k_ml = 1;              // OJAS_HIP_Q6K_ML: 0 = keep those rows on direct loads (gemv_q8k_q6k_mf)
    uint32_t px_bpc = 0;         // OJAS_HIP_PX_BPC: workgroups per CU for the grid-stride head matvec (0: 8)
    int px = 1;                  // OJAS_HIP_PX: 0 = never take it
    uint32_t q4k_ml_min_m = 2;   // OJAS_HIP_Q4K_ML_MIN_M: tokens from which long Q4_K matrices (32768 rows or more) take the LDS-copy form (0: never)
    uint32_t rms_threads = 0;    // OJAS_HIP_RMS_THREADS: block size of rmsnorm_q8k (256 or 1024; 0: by the number of rows)
    uint32_t q4k_xt_split = 1;   // OJAS_HIP_Q4K_XT_SPLIT: K slices of the 64-row int8 tile when its tiles leave CUs idle (0: never, 1: chosen, n: n)
    uint32_t q4k_xt_min_m = 1;   // OJAS_HIP_Q4K_XT_MIN_M: tokens from which Q4_K rows take the 128-token int8 tile (0: never, 1: by shape)
    bool q4k_xt64 = false;       // OJAS_HIP_Q4K_XT64=1: that tile always in its 64-row form
    bool no_scratch = false;     // set around calls that may not allocate (ojh_mm_noalloc): paths that need library scratch are skipped
    uint32_t q8row_mt_min_m = 1; // OJAS_HIP_Q8ROW_MT_MIN_M: tokens from which ojh_matmul_q8 takes the int8 matrix tile (0: never, 1: measured default, n: n)
    uint32_t iq4_tile = 5;       // OJAS_HIP_IQ4_TILE: tokens from which IQ4_NL / IQ4_XS rows run on the tile through their own loaders instead of the decode pass (0: never)
    uint32_t iq4_tile_cap = 128; // OJAS_HIP_IQ4_TILE_CAP: tokens up to which Q3_K rows take their loader
    uint32_t gemm_few = 32;      // OJAS_HIP_GEMM_FEW: tokens up to which Q8_0 / IQ4 / legacy / MXFP4 / Q2_K / Q3_K batches take `gemm_few_*` instead of the LDS-staged tile (0: never; at most 64)
    uint32_t moe_few = 128;       // OJAS_HIP_MOE_FEW: average assignments per expert up to which the grouped products of Q8_0 / IQ4 experts run on `moe_few_*` (0: never)
    uint32_t moe_mm_tile = 1;    // OJAS_HIP_MOE_MM_TILE: assignments per expert (average) from which Q8_0 experts run on the grouped f16 matrix tile under OJH_ACT_AUTO (0: never, 1: measured default, n: n)
    uint32_t moe_down_gs = 1;    // OJAS_HIP_MOE_DOWN_GS: assignments per expert (average) from which Q5_K / Q6_K down tensors run on the int8 matrix tile (0: never, 1: measured default, n: n)
    bool q8row_dec = true;       // OJAS_HIP_Q8ROW_DEC=0: 1 to 8 tokens on the per-row kernel instead of the one that stages the tokens in LDS
    uint32_t q8row_t128_min_m = 1; // OJAS_HIP_Q8ROW_T128_MIN_M: tokens from which that tile covers 128 tokens (0: never, 1: measured default, n: n)
    uint32_t q8row_split = 1;    // OJAS_HIP_Q8ROW_SPLIT: K slices of that tile (0: never, 1: by shape, n: n)
    uint32_t deq_big_m = 1024;   // OJAS_HIP_DEQ_BIG_M: tokens from which Q6_K rows of a large matrix are decoded into scratch ahead of the f16 tile (Q5_K / Q8_0 rows from twice as many; 0: never)
    uint32_t deq_min_m = 1;      // OJAS_HIP_DEQ_MIN_M: tokens from which a format without a tile of its own is decoded into scratch and multiplied on the f16 tile (0: never, 1: by matrix size, n: n)
    uint32_t q80_tile_min_m = 1; // OJAS_HIP_Q80_TILE_MIN_M: tokens from which OJH_ACT_AUTO sends Q8_0 rows to the f16 tile (0: GEMM_MIN_M, 1: by shape, n: n)
    int gemm_m128 = 128;         // OJAS_HIP_GEMM_M128: tokens up to which Q5_K / Q6_K / Q8_0 batches take the 128-token f16 tile (0: never)
    uint32_t kq_gs_split = 1;    // OJAS_HIP_KQ_GS_SPLIT: K slices of that tile (0: never, 1: chosen, n: n)
    uint32_t kq_gs_min_m = 1;    // OJAS_HIP_KQ_GS_MIN_M: tokens from which Q6_K / Q5_K rows take the 128-row x 64-token int8 tile (0: never, 1: by shape)
    uint32_t q4k_mf_min_m = 5;   // OJAS_HIP_Q4K_MF_MIN_M: tokens from which Q4_K rows go to the int8 matrix cores
    int moe_mode = 0;            // OJAS_HIP_MOE: 0 = by batch size, 1 = matrix cores always, 2 = grouped integer dots always,
                                 // 3 = per-assignment decode form always, 4 = matrix cores in the workgroup-per-tile form always
    uint32_t moe_dec_tokens = 2; // OJAS_HIP_MOE_DEC_TOKENS: the decode form serves up to this many tokens (128 experts, top 8, weights from HBM: 2 tokens 21.0 against 23.3 us grouped, 3 tokens 27.4 against 25.9, 8 tokens 59 against 38)
    int gemm_bdk = 1;            // OJAS_HIP_GEMM_BDK: 0 never takes the 64-row tile whose waves split K, 2 takes it wherever the 128-token tile would run
    bool gemm_sr = false;        // OJAS_HIP_GEMM_SR=1: K slices of the prefill tile meet in scratch, added in slice order (reproducible bits), instead of in f32 atomics
    bool moe_route_fuse = true;  // OJAS_HIP_MOE_ROUTE_FUSE=0: ojh_moe_ffn_routed keeps the router a launch of its own
    bool moe_fuse = true;        // OJAS_HIP_MOE_FUSE=0: the grouped pipeline keeps its quantizer and grouping launches apart
    bool gemm_exact = false;     // OJAS_HIP_GEMM_EXACT: Q4_K prefill through the tile that holds dequant_to_f16 bits
    bool fused_quant = false;    // OJAS_HIP_FUSED_QUANT=1: ojh_mm (m = 1, Q4_K) quantizes x inside the matvec launch
    uint32_t fq_blocks_per_cu = 8; // OJAS_HIP_FQ_BLOCKS: blocks per CU the fused-quantizer matvec aims for
    uint32_t fq_threads = 1024;    // OJAS_HIP_FQ_THREADS: threads per workgroup of ojh_mm_multi's launch (256, 512, 1024)
    int fq_rows = 0;               // OJAS_HIP_FQ_ROWS: rows per wave of ojh_mm_multi's launch (0: by row count)
    int fq_multi = 1;              // OJAS_HIP_FQ_MULTI: 0 = ojh_mm_multi always quantizes in a launch of its own, 2 = never
    uint32_t fq_multi_blocks = 1;  // OJAS_HIP_FQ_MULTI_BLOCKS: workgroups per CU of its single launch
    bool capturing = false;      // between ojh_capture_begin and ojh_capture_end
    bool capture_hip_graph = false;
    std::vector<ojh_command> recorded;
    // Recorded chains hold raw pointers into the scratch buffers.  While any chain of this device is alive, a scratch
    // buffer that has to grow is parked here instead of freed, and released when the last chain is.
    int live_graphs = 0;
    std::vector<ojh_buf *> parked;
    // the single-launch decode chain (ojh_chain.cpp): its counters on the device, the word a wait that gave up sets
    // (pinned host memory the kernels write to), the number of polls a wait may take
    uint32_t *chain_status = nullptr;
    uint32_t chain_spin = 1u << 22;    // OJAS_HIP_CHAIN_SPIN
    uint32_t chain_tag = 0;            // the last launch's tag (never 0)
    void *chain_trace = nullptr;       // ojh_chain_trace: timestamps of the next chain launches go here
    void *noalloc_scratch = nullptr;   // this GPU's copy of the static scratch array of ojh_mm_noalloc (ojh_noalloc.cpp)
};

// ---- errors ------------------------------------------------------------------------------------
int ojh_fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
#define OJH_HIP(call)                                                                              \
    do {                                                                                           \
        hipError_t e_ = (call);                                                                    \
        if (e_ != hipSuccess)                                                                      \
            return ojh_fail(OJH_ERR_HIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e_),   \
                            __FILE__, __LINE__);                                                   \
    } while (0)

// ---- manifest ----------------------------------------------------------------------------------
struct ojh_block_format {
    uint32_t type, bytes, weights;
    const char *tag;
};
const ojh_block_format *ojh_format(uint32_t ggml_type);
bool ojh_float_rows(uint32_t ggml_type);   // the CPU path reads f32 activations for this format
size_t ojh_block_align(const ojh_block_format *f);
uint32_t ojh_matmul_q8row_slices(const ojh_device *dev, uint32_t K, uint32_t N, uint32_t M);  // K slices of the row-int8 tile (1: whole)
uint32_t ojh_gemm_q8k_gs_slices(const ojh_device *dev, uint32_t K, uint32_t N, uint32_t M);   // K slices of the Q6_K / Q5_K int8 tile (1: whole)
uint32_t ojh_gemm_sr_slices(uint32_t K, uint32_t nsplit);   // K slices of the `_sr` tiles that hold a super-block
bool ojh_grid_type(uint32_t ggml_type);    // a grid-codebook format: its kernels live in the family "iq_grid"
bool ojh_float_only(uint32_t ggml_type);   // ... and only the f32-activation matvecs exist for it

// What a kernel touches at given constants. Returns OJH_OK or fails with a message.
typedef int (*ojh_check_fn)(const struct ojh_kernel_spec *spec, const uint32_t *consts,
                            const uint32_t grid[3], const uint32_t block[3], size_t need[16],
                            size_t align[16]);
typedef int (*ojh_shape_fn)(const struct ojh_kernel_spec *spec, const ojh_device *dev, uint32_t K,
                            uint32_t N, uint32_t M, uint32_t grid[3], uint32_t block[3]);

struct ojh_kernel_spec {
    const char *name;
    const char *family;
    int n_bufs, n_consts;
    uint32_t type;       // GGUF type the kernel reads, 0 if none
    int rows_per_wave;   // for the row-parallel matvecs
    ojh_check_fn check;
    ojh_shape_fn shape;
    // Expert kernels whose reference argument list carries no expert count: buffers 1 .. expert_bufs are
    // expert tensors, need[] is one expert's bytes, and the dispatcher appends min(extent / need) as a
    // trailing constant so that an index past the tensors multiplies nothing instead of reading past them.
    int expert_bufs = 0;
    int bound_first = 1;   // index of the first such buffer (0 for a table that is the first argument)
    // Streamed-expert kernels: buffers 1 .. arena_bufs are cache arenas addressed by byte offsets, need[] is one
    // expert's bytes, and the dispatcher appends, per arena, the last offset at which an expert still fits.
    int arena_bufs = 0;
};
const std::vector<ojh_kernel_spec> &ojh_manifest_table();
const ojh_kernel_spec *ojh_find_kernel(const char *name);

// ---- helpers -----------------------------------------------------------------------------------
int ojh_scratch_get(ojh_device *dev, const char *name, size_t bytes, ojh_buf **out);
// ... a slot whose kernels leave zeros behind: cleared whenever it is (re)allocated
int ojh_scratch_get_zeroed(ojh_device *dev, const char *name, size_t bytes, ojh_buf **out);
int ojh_launch(ojh_device *dev, const char *name, const std::vector<void *> &ptrs,
               const std::vector<uint32_t> &consts, const uint32_t grid[3], const uint32_t block[3]);
// a kernel that takes one struct as its argument list
int ojh_launch_blob(ojh_device *dev, const char *name, const void *args, size_t bytes, const uint32_t grid[3],
                    const uint32_t block[3], int tag_offset = -1);
int ojh_chain_check_status(ojh_device *dev);   // after a synchronisation: did a chain's bounded wait give up? (ojh_chain.cpp)
// shared by ojh_mm / ojh_mm_q8k / ojh_mm_noalloc (ojh_ops.cpp)
int ojh_mm_checks(const char *who, const ojh_lin *w, ojh_buf *y, size_t y_off, const ojh_buf *bias, uint32_t m, int accum,
                  const ojh_block_format **fmt);
int ojh_quant_q8k_launch(ojh_device *dev, const void *x, int x_dtype, uint32_t m, uint32_t k, void *q, void *scales);
int ojh_mm_q8k_launch(ojh_device *dev, void *xq, void *xs, const ojh_lin *w, const ojh_block_format *f, void *yp,
                      const ojh_buf *bias, uint32_t m, int accum, bool sides_ready = false);
bool ojh_q4k_xt_taken(const ojh_device *dev, const ojh_lin *w, uint32_t m, const void *wp);
int ojh_noalloc_setup(ojh_device *dev);   // resolves the static scratch array on the current GPU (ojh_noalloc.cpp)
void ojh_gemm_q8k_tiles(const ojh_device *dev, uint32_t K, uint32_t N, uint32_t M, uint32_t *rw, uint32_t *rt);   // row tiles per workgroup / per wave of gemm_q8k_q4k_mf
uint32_t ojh_moe_mt_groups(const ojh_device *dev, uint32_t N, uint32_t E, uint32_t per_cu);   // workgroups per expert of those entries
uint64_t ojh_moe_mt_lds(uint32_t K);                // LDS bytes of moe_{gu,down}_q4k_mt (ojh_manifest.cpp)
uint64_t ojh_gemm_q8k_mk_lds(uint32_t K, uint32_t M);   // LDS bytes of gemm_q8k_q4k_mk (ojh_manifest.cpp)
uint64_t ojh_gemm_q8k_ml_lds(uint32_t K);           // LDS bytes of gemm_q8k_q4k_ml (ojh_manifest.cpp)
uint64_t ojh_q6k_mk_lds(uint32_t K, uint32_t M);   // LDS bytes of gemv_q8k_q6k_mk (ojh_manifest.cpp)
uint64_t ojh_q6k_ml_lds(uint32_t K, uint32_t M);   // LDS bytes of gemv_q8k_q6k_ml (ojh_manifest.cpp)
uint32_t ojh_q80_lds_kc(uint32_t K);   // chunks of K for gemv_nat_q80_lds, 0 if none (ojh_manifest.cpp)
