// Interface between the decode step's host code (decode.hip) and the persistent
// whole-step kernel (decode_persist.hip).
#pragma once

#include "int4_kernels.hpp"

namespace l2 {

// Attended rows per attention block and the longest history the persistent
// step takes (24 blocks of 128 rows); longer histories use the launch sequence.
constexpr int kPBlockRows = 128;
constexpr int kPMaxBlocks = 24;
constexpr int kPMaxRows = kPBlockRows * kPMaxBlocks; // 3072
constexpr int kPPartStride = kRopeHeadSize + 2;     // 128 partial outputs, block max, block sum
constexpr int kPWaves = 8;                           // wavefronts per workgroup, one workgroup per compute unit: 256 registers each
constexpr int kPUnits = kPWaves / 4;                 // attention units (4 wavefronts, one block of a head) per workgroup
constexpr int kPersistSpinLimit = 1 << 21;           // unsuccessful polls (about a microsecond each) before a wait gives up

// Ints of the decoder's device-resident state block (shared with decode.hip).
constexpr int kStateInts = 8;
constexpr int kStatePos = 0;      // position of the step
constexpr int kStatePrompt = 1;   // first position whose token is generated
constexpr int kStateAdvance = 2;  // 1: the sampling kernel advances the position
constexpr int kStateSlots = 3;    // token slots (context length)
constexpr int kSpareTokenSlot = 4;
constexpr int kStateSerial = 5;   // counts persistent steps (bumped right before each, by nothing else): their hand-over tags derive from it
constexpr int kStateError = 6;    // set by the persistent step when a bounded wait gave up

struct PersistLayer { // one per layer, in device memory
    QW q, k, v, o, gate, up, down;
    const uint16_t* rms_att;
    const uint16_t* rms_ffn;
};

struct PersistArgs {
    const PersistLayer* layers;
    int n_layers, dim, hidden, n_heads, vocab, seq_len;
    int ws_d, ss_d, zs_d; // per-row sizes of a dim-input tensor
    int ws_h, ss_h, zs_h; // of a hidden-input tensor
    float eps, scale;
    const uint16_t* embedding; // layer 0 input: row tokens[pos] ...
    const int* tokens;
    const uint16_t* x_in;      // ... or, when embedding is null, this vector
    const uint16_t* rms_final;
    const uint16_t* classifier; // null: stop after the last layer and write the residual stream to x_out
    uint16_t* logits;
    uint16_t* x_out;
    uint16_t* kcache; // [layer][seq_len][dim]
    uint16_t* vcache;
    int* state;
    // tagged hand-over buffers (zero-initialised once)
    uint32_t* ll_x0;   // [dim]       layer input
    uint32_t* ll_qkv;  // [3 dim]     q, k, v of the step's position, unrotated
    uint32_t* ll_att;  // [dim]       attention output
    uint32_t* ll_x1;   // [dim]       residual stream after the o-projection
    uint32_t* ll_h;    // [hidden]    SwiGLU output
    unsigned long long* ll_part; // [n_heads][kPMaxBlocks][kPPartStride] attention partials
    int skip_attention; // 1: the o-projection consumes q directly (mat-vec chain without attention)
    int spin_limit;     // polls before a wait gives up and raises the error flag
#ifdef L2_PERSIST_TRACE
    // diagnostic build (make TRACE=1): wavefront 0 of workgroups 0, 1, 100 and 255 stores the
    // 100 MHz clock at every phase boundary, kPTracePoints records per layer and workgroup
    unsigned long long* trace;
#endif
};
constexpr int kPTracePoints = 16;

// Index of the kernel instantiation that fits the shapes on `num_cus` compute units, or -1.
int persist_variant(int dim, int hidden, int n_heads, int num_cus);
// Bytes of the hand-over buffers, and their placement inside one zeroed allocation.
size_t persist_scratch_bytes(int dim, int hidden, int n_heads);
void persist_bind_scratch(PersistArgs& a, void* base);
int persist_launch(int variant, const PersistArgs& a, int num_cus);

} // namespace l2
