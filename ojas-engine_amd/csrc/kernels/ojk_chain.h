// Argument block of the single-launch decode chain (kernel `decode_chain_q4k`, family "chain"), shared by the host
// side that fills it and the kernel that reads it from its kernarg segment.  Plain C layout: pointers first, then
// 32-bit words.
#pragma once
#include <stdint.h>

#define OJK_CHAIN_MAX_STAGES 8
#define OJK_CHAIN_THREADS 256u      // four waves per workgroup
#define OJK_CHAIN_MAX_K 16384u
#define OJK_CHAIN_QSEGS 4u          // 256-element segments of a stage's input one quantizer workgroup converts
#define OJK_CHAIN_REPLICAS 64u      // copies of a stage's {scale, tag} table: the row workgroups poll different lines

// How a stage's f32 input vector is formed before it is quantized per 256 (quant_q8k).
enum {
    OJK_CHAIN_X_PLAIN = 0,      // x
    OJK_CHAIN_X_SILU_MUL = 1,   // silu(x) * x2       (the gate / up pair of a feed-forward block)
    OJK_CHAIN_X_GELU_MUL = 2,   // gelu_tanh(x) * x2
    OJK_CHAIN_X_RMSNORM = 3,    // x * (1 / sqrt(mean(x^2) + eps)) * x2    (x2 = the norm's weights)
};

// A value one workgroup hands to another inside the launch travels as a pair {value, tag}, written and read as
// one 8-byte access: the tag names the launch that wrote the value, so a reader knows whether it has arrived.
struct ojk_chain_pair {
    float value;
    uint32_t tag;
};

struct ojk_chain_stage {
    const void *x;          // f32[K], or ojk_chain_pair[K] when bit 0 of `tagged` is set
    const void *x2;         // second operand of the prologue, likewise (bit 1)
    const void *w[4];       // Q4_K rows of up to four tensors sharing x (unused slots repeat the last)
    void *y[4];             // f32 outputs, one per tensor
    struct ojk_chain_pair *xchg[4];         // where tensor i's results also go as pairs (a later stage reads them), or NULL
    const struct ojk_chain_pair *addsrc[4]; // accumulating stage: the old values as pairs of an earlier stage, or NULL (read y)
    signed char *xq;                        // K bytes: this stage's quantized input
    struct ojk_chain_pair *xs;              // [OJK_CHAIN_REPLICAS][64]: {scale of segment i, tag}
    uint32_t ends[4];       // cumulative row counts: tensor i owns stacked rows ends[i-1] .. ends[i]-1
    uint32_t K;
    uint32_t prologue;
    uint32_t accum;         // y += W x instead of y = W x
    uint32_t eps_bits;      // RMS norm epsilon, as float bits
    uint32_t tagged;
    uint32_t rows_per_wave; // 1 or 2
    uint32_t wg_first;      // the stage's first workgroup: n_quant quantizer workgroups, then its row workgroups
    uint32_t n_quant;
};

struct ojk_chain_args {
    struct ojk_chain_stage st[OJK_CHAIN_MAX_STAGES];
    uint32_t *abort_word;   // device word: set by a wait that gave up, the other waits stop at their next look at it
    uint32_t *status;       // host-visible word: set to 1 + stage index when a bounded wait gives up
    uint64_t *trace;        // optional: OJK_CHAIN_TRACE_EVENTS timestamps (100 MHz counter) per stage
    uint32_t nstages;
    uint32_t spin_cap;      // looks a wait may take before it gives up (0: gives up at once)
    uint32_t tag;           // this launch's tag: never 0, never the tag of an earlier launch of the device
    uint32_t pad_;
};

// trace[stage * OJK_CHAIN_TRACE_EVENTS + event], written by the stage's first quantizer workgroup
#define OJK_CHAIN_TRACE_EVENTS 3u
enum {
    OJK_CHAIN_T_QUANT_ENTER = 0,    // it starts
    OJK_CHAIN_T_QUANT_ARRIVED = 1,  // it has the stage's whole input (the norm) or its own part of it: the rows it waited for are done
    OJK_CHAIN_T_QUANT_DONE = 2,     // it has published its segments
};
