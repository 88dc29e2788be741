/*
 * TEST INFRASTRUCTURE — CPU restatement of the reference's quantized-matmul arithmetic.
 *
 * This library is the checker the HIP kernels are compared against.  It is never part of the
 * shipped product path: only the test-suite, the smoke check and the CPU-baseline leg of the
 * benchmark may load it.
 *
 * Every function cites the reference source (paths relative to the reference tree) whose
 * arithmetic it restates.  Build with -ffp-contract=off: the reference is Rust, which never
 * fuses a multiply with an add.
 *
 * How each function is pinned (a function without such a check would say "parity unpinned"):
 *   dequant Q4_K/Q5_K/Q6_K  FNV-1a digests held by crates/ojas-formats/tests/quant_formats.rs:38-40
 *   dequant Q2_K/Q3_K       the digests of the same table (quant_formats.rs:36-37), weight-by-weight numpy restatement
 *   dequant IQ4_NL/IQ4_XS   the digests of the same table (quant_formats.rs:45,48), one-hot codes vs the codebook
 *   dequant Q8_0            closed form of crates/ojas-formats/tests/rows.rs:13-18
 *   dequant Q4_0/Q4_1/Q5_0/Q5_1  closed forms only (d * (q - 8 | 16), d * q + m, nibble halves, the fifth-bit field):
 *                           the reference's tests hold no digest for the legacy 32-weight blocks
 *   f16 <-> f32             the digests above + exhaustive comparison with IEEE binary16 (numpy)
 *   quant_q8k               invariants (max|q|=127, bsums, half-away rounding, |x-s*q|<=s/2)
 *   dequant IQ2_XXS/IQ2_XS/IQ2_S/IQ3_XXS/IQ3_S/IQ1_S/IQ1_M   (ojas_oracle_iq.c) the digests of the same table
 *                           (quant_formats.rs:41-44,46-47,49), closed forms on hand-built blocks; the packed codebooks
 *                           by a digest of every published table (tests/golden/iq_grid_digests.json)
 *   dequant MXFP4           the hand-computed blocks of crates/ojas-core/src/quant_src.rs:1376-1420 and
 *                           crates/ojas-formats/src/mxfp4.rs:127-160 (codebook sweep, scales 2^2 and 2^-1, e8m0 table)
 *   dot_q80                 f64 dot over the dequantized row, brute force at K=32
 *   dot_iq2xxs/iq3xxs/iq2s/iq3s   f64 dot over the exactly decoded row, one-hot activations
 *   dot_iq2xxs_q8k/iq3xxs_q8k     identity dot(row, quant(x)) == sum xs * sum w * q in f64
 *   dot_iq4nl / dot_iq4xs   f64 dot over the dequantized row (the check of cpu_math.rs:1206-1285), one-hot activations
 *   dot_q4k/q5k/q6k         identity dot(row, quant(x)) == sum dequant(row)*(scale*q) in f64,
 *                           one-hot activations (pins nibble / sub-block order)
 *   relayout_q4k_q4l        qa*nib+qb == dequant up to the two f16 roundings, one-hot blocks
 *   gemv_q8_rows            numpy f64 product on the generators of crates/ojas-cuda/tests/conformance.rs:248-268 (q8_rows,
 *                           tvec), all-ones rows (y = scale * sum x), one-hot activations
 *   quantize_q8_pertoken    invariants (max|q| = 127, d = amax / 127, ties to even at x = 0.5 d and 1.5 d, zero tokens -> d = 0, q = 0)
 *   moe_topk                softmax + stable sort closed form (numpy)
 *   moe_ffn                 composition of the above
 * The f32 association order inside dot_q4k / dot_q6k is pinned by the source text only; it
 * moves the last ulp, far below the 1e-3 parity bar.
 */
#ifndef OJAS_ORACLE_H
#define OJAS_ORACLE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GGUF type ids (crates/ojas-formats/src/gguf.rs:563-591). */
enum { OJO_Q4_0 = 2, OJO_Q4_1 = 3, OJO_Q5_0 = 6, OJO_Q5_1 = 7, OJO_Q8_0 = 8, OJO_Q2_K = 10, OJO_Q3_K = 11, OJO_Q4_K = 12, OJO_Q5_K = 13, OJO_Q6_K = 14,
       OJO_IQ4_NL = 20, OJO_IQ4_XS = 23,
       OJO_MXFP4 = 139, /* the reference's synthetic id for 17-byte MXFP4 blocks (crates/ojas-core/src/quant_src.rs:91-95) */
       OJO_IQ2_XXS = 16, OJO_IQ2_XS = 17, OJO_IQ3_XXS = 18, OJO_IQ1_S = 19, OJO_IQ3_S = 21, OJO_IQ2_S = 22, OJO_IQ1_M = 29 };

/* IEEE binary16 <-> binary32, round-to-nearest-even, subnormals kept
 * (crate half 2.7.1; call sites gguf.rs:602-608). */
float    ojo_f16_to_f32(uint16_t h);
uint16_t ojo_f32_to_f16(float f);
/* bf16 round-to-nearest-even of an f32 (activation rounding of the prefill GEMM). */
uint16_t ojo_f32_to_bf16(float f);
float    ojo_bf16_to_f32(uint16_t h);

/* (block bytes, weights per block); returns 0 on unknown type (synth.rs:12-21). */
int ojo_block_shape(uint32_t ty, uint32_t *bytes, uint32_t *weights);

/* Seeded synthetic blocks (crates/ojas-formats/src/synth.rs:29-64). out: nb*block_bytes. */
int ojo_synth_blocks(uint32_t ty, size_t nb, uint8_t *out);

/* dequant_to_f16 (gguf.rs:612-1116; arms :704-709, :1042-1059, :1060-1085, :1086-1108).
 * n = number of weights; out = n binary16 bit patterns. */
int ojo_dequant_to_f16(const uint8_t *b, uint32_t ty, size_t n, uint16_t *out);
/* Same decoders evaluated exactly in double (no f32/f16 rounding), as
 * crates/ojas-models/examples/q6k_gate.rs:60-110 does. */
int ojo_dequant_to_f64(const uint8_t *b, uint32_t ty, size_t n, double *out);

/* FNV-1a-64 over the ASCII of "%.6f" of every f16 value
 * (crates/ojas-formats/tests/quant_formats.rs:20-31). */
uint64_t ojo_digest_f16(const uint16_t *v, size_t n);

/* quant_q8k (crates/ojas-cpu/src/cpu_math.rs:539-563). k need not be a multiple of 256;
 * q has ceil(k/256)*256 entries, scales ceil(k/256), bsums ceil(k/256)*8. */
void ojo_quant_q8k(const float *x, size_t k, float *scales, int8_t *q, int32_t *bsums);

/* Row dots (cpu_math.rs:971-981, :609-635, :638-670, :674-722). */
float ojo_dot_q80(const uint8_t *row, const float *x, size_t k);
float ojo_dot_iq4nl(const uint8_t *row, const float *x, size_t k);
float ojo_dot_iq4xs(const uint8_t *row, const float *x, size_t k);
float ojo_dot_q4k(const uint8_t *row, size_t k, const float *scales, const int8_t *q, const int32_t *bsums);
float ojo_dot_q5k(const uint8_t *row, size_t k, const float *scales, const int8_t *q, const int32_t *bsums);
float ojo_dot_q6k(const uint8_t *row, size_t k, const float *scales, const int8_t *q, const int32_t *bsums);

/* Grid-codebook formats (ojas_oracle_iq.c): one 256-weight block as the f32 values the reference rounds to f16 and
 * exactly in double; the f32-activation dots (cpu_math.rs:728-757, :884-913, :915-941, :1023-1052) and the
 * int8-activation dots (:1057-1128); a published codebook expanded from its packed form. */
int    ojo_iq_is_grid_type(uint32_t ty);
void   ojo_iq_block(uint32_t ty, const uint8_t *blk, float *of, double *od);
size_t ojo_iq_grid_bytes(int which, uint8_t *out);
float  ojo_dot_iq2xxs(const uint8_t *row, const float *x, size_t k);
float  ojo_dot_iq3xxs(const uint8_t *row, const float *x, size_t k);
float  ojo_dot_iq2s(const uint8_t *row, const float *x, size_t k);
float  ojo_dot_iq3s(const uint8_t *row, const float *x, size_t k);
float  ojo_dot_iq_grid(uint32_t ty, const uint8_t *row, const float *x, size_t k);
float  ojo_dot_iq2xxs_q8k(const uint8_t *row, size_t k, const float *scales, const int8_t *q);
float  ojo_dot_iq3xxs_q8k(const uint8_t *row, size_t k, const float *scales, const int8_t *q);

/* matvec_kq (cpu_math.rs:1145-1189): 8-row work stealing over `threads` workers. */
int ojo_matvec_kq(const uint8_t *raw, uint32_t ty, size_t n, size_t k, const float *x,
                  int threads, float *y);

/* Row-int8 path every dense CPU model runs (cpu_math.rs:174-179, :187-274, :404-415)
 * and its load-time requantizer (crates/ojas-formats/src/quant.rs:16-39). */
void ojo_quantize_q8_1(const float *x, size_t k, int8_t *q8, float *d8, float *d8sum);
/* The reference GPU decoder's row-int8 matvec and its per-token quantizer (crates/ojas-cuda/src/kernels/gemv_q8.rs:31-55,
 * gemv.rs:57-74). */
void ojo_gemv_q8_rows(const int8_t *w, const float *scale, const float *x, size_t k, size_t n, float *y);
void ojo_quantize_q8_pertoken(const float *x, size_t m, size_t k, int8_t *q8, float *d8);
double ojo_row_q80_dp4a(const uint8_t *row, const int8_t *q8, const float *d8, size_t k);
void ojo_gemv_q80_dp4a(const uint8_t *w, const int8_t *q8, const float *d8, size_t k, size_t n, float *y);
float ojo_quant_row_i8(const float *row, size_t k, int8_t *q);
void  ojo_q8_rows_from_f16(const uint16_t *w16, size_t n, size_t k, int8_t *q, float *scale);
void  ojo_matmul_q8(const int8_t *wq, const float *wscale, size_t n, size_t k,
                    const float *xs, size_t m, const float *bias, int threads, float *ys);

/* relayout_q4k_q4l (crates/ojas-formats/src/quant.rs:192-222). */
void ojo_relayout_q4k_q4l(const uint8_t *w, size_t k, size_t n, uint8_t *nib, uint16_t *qa, uint16_t *qb);

/* The f16 weights the reference's GPU prefill kernel multiplies for Q4_K tensors relaid to Q4L:
 * binary16 fma(qa, q, qb) per weight (crates/ojas-cuda/src/kernels/gemm_q.rs:104-140 over the
 * relayout above).  `out` is [n][k] binary16 bit patterns in the tensor's own weight order. */
void ojo_q4l_weights_f16(const uint8_t *w, size_t k, size_t n, uint16_t *out);

/* The GPU-test oracle: y = x * dequant(W)^T accumulated in double
 * (crates/ojas-cuda/tests/conformance.rs:798-803, tests/prefill_gemm_q.rs:116-130).
 *   wmode: 0 = weights exact (double), 1 = weights rounded to f16 as dequant_to_f16 stores them,
 *          2 = Q4_K weights as the Q4L GPU kernel forms them (ojo_q4l_weights_f16)
 *   xmode: 0 = x as given, 1 = x rounded to f16, 2 = x rounded to bf16
 * x is [m][k] f32, y is [m][n] double. */
int ojo_matmul_ref(const uint8_t *raw, uint32_t ty, size_t n, size_t k, const float *x, size_t m,
                   int wmode, int xmode, int threads, double *y);

/* rmsnorm (crates/ojas-cpu/src/cpu_math.rs:456-460) and the FFN activation functions
 * (silu :486, gelu tanh form :497-501). */
void  ojo_rmsnorm(const float *x, const float *w, size_t k, float eps, float *y);
float ojo_ffn_act(float g, int act);

/* Router: softmax, ksel argmax passes with strict '>', lowest index wins, renormalise
 * (crates/ojas-cuda/src/kernels/moe.rs:45-70; oracle crates/ojas-cuda/tests/conformance.rs:385-392). */
void ojo_moe_topk(const float *logits, int n_expert, int ksel, uint32_t *idx, float *wgt);
void ojo_moe_topk_nonorm(const float *lg, int E, int ksel, uint32_t *idx, float *wgt);
void ojo_moe_topk_v3(const float *lg, const float *bias, int E, int ksel, float rscale, int norm, uint32_t *idx, float *wgt);

/* Expert FFN for T tokens (crates/ojas-cpu/src/cpu_glm.rs:551-582; silu cpu_math.rs:486):
 * for each token t and slot j (in slot order): act = silu(Wg_e x) * (Wu_e x);
 * y[t] += wgt[t][j] * (Wd_e act).   y must be initialised by the caller.
 *   mode 0: every matvec is matvec_kq (int8 activations, the CPU path)
 *   mode 1: every matvec is dequant-in-double dot (the GPU-test convention); y stays f32.
 * gate/up: [E][n_ff][d] rows of type ty_gu; down: [E][d][n_ff] rows of type ty_d. */
int ojo_moe_ffn(const float *x, size_t T, size_t d, size_t n_ff, int n_expert, int ksel,
                const uint32_t *idx, const float *wgt,
                const uint8_t *gate, const uint8_t *up, uint32_t ty_gu,
                const uint8_t *down, uint32_t ty_d, int mode, int threads, float *y);

#ifdef __cplusplus
}
#endif
#endif
