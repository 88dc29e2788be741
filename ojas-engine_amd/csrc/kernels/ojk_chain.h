// Argument block of the single-launch decode chain (kernel `decode_chain_q4k`, family "chain"), shared by the host
// side that fills it and the kernel that reads it from its kernarg segment.  Plain C layout, no padding surprises:
// pointers first, then 32-bit words.
#pragma once
#include <stdint.h>

#define OJK_CHAIN_MAX_STAGES 8
#define OJK_CHAIN_THREADS 1024u     // one workgroup of sixteen waves per compute unit
#define OJK_CHAIN_WAVES 16u
#define OJK_CHAIN_MAX_K 16384u

// How a stage's f32 input vector is formed before it is quantized per 256 (quant_q8k).
enum {
    OJK_CHAIN_X_PLAIN = 0,      // x
    OJK_CHAIN_X_SILU_MUL = 1,   // silu(x) * x2       (the gate / up pair of a feed-forward block)
    OJK_CHAIN_X_GELU_MUL = 2,   // gelu_tanh(x) * x2
    OJK_CHAIN_X_RMSNORM = 3,    // x * (1 / sqrt(mean(x^2) + eps)) * x2    (x2 = the norm's weights)
};

// Words of the device-side state block (uint32 each), zero when allocated and never reset: eight 64-bit launch
// counters on separate 128-byte lines (workgroup b adds one to counter b % 8 when it starts), and the abort word.
#define OJK_CHAIN_SYNC_TICKET(g) ((g) * 32u)
#define OJK_CHAIN_SYNC_ABORT 256u   // set by a workgroup whose wait gave up: the others stop waiting too; the host clears it
#define OJK_CHAIN_SYNC_WORDS 288u

// A result that a later stage of the same launch reads travels as a pair {value, tag}, written and read as one
// 8-byte access: the tag says which launch wrote the value, so a reader knows whether it has arrived.
struct ojk_chain_pair {
    float value;
    uint32_t tag;
};

struct ojk_chain_stage {
    const void *x;          // f32[K], or ojk_chain_pair[K] when bit 0 of `tagged` is set
    const void *x2;         // second operand of the prologue, likewise (bit 1)
    const void *w[4];       // Q4_K rows of up to four tensors sharing x (unused slots repeat the last)
    void *y[4];             // f32 outputs, one per tensor
    struct ojk_chain_pair *xchg[4];   // where tensor i's results go as pairs for later stages, NULL if none reads them
    uint32_t ends[4];       // cumulative row counts: tensor i owns stacked rows ends[i-1] .. ends[i]-1
    uint32_t K;
    uint32_t prologue;
    uint32_t accum;         // y += W x instead of y = W x
    uint32_t eps_bits;      // RMS norm epsilon, as float bits
    uint32_t tagged;
    uint32_t pad_;
};

struct ojk_chain_args {
    struct ojk_chain_stage st[OJK_CHAIN_MAX_STAGES];
    uint32_t *sync;         // OJK_CHAIN_SYNC_WORDS words
    uint32_t *status;       // host-visible word: set to 1 + stage index when a bounded wait gives up
    uint64_t *trace;        // optional: OJK_CHAIN_TRACE_EVENTS timestamps (100 MHz counter) per workgroup and stage
    uint32_t nstages;
    uint32_t spin_cap;      // polls a wait may take before it gives up (0: gives up at once)
};

// trace[(workgroup * OJK_CHAIN_MAX_STAGES + stage) * OJK_CHAIN_TRACE_EVENTS + event], written by the workgroup's first wave
#define OJK_CHAIN_TRACE_EVENTS 4u
enum {
    OJK_CHAIN_T_ENTER = 0,     // the wave turns to the stage's input
    OJK_CHAIN_T_ARRIVED = 1,   // its part of the input has arrived
    OJK_CHAIN_T_INPUT = 2,     // the whole input is quantized in LDS
    OJK_CHAIN_T_ROWS = 3,      // the wave's rows are done and stored
};
