// Persistent decode kernel (decode_mega.hip): argument blocks and launcher.
#pragma once

#include "mesh_common.hpp"

namespace mesh {

// One matrix (or gate/up pair) of a GEMV phase.
struct MegaPart {
    const uint8_t *W0, *W1;        // tiled K-quant matrices; W1 is the "up" matrix of a SwiGLU pair, else null
    int type;                      // ggml type of W0 (and W1): q4_K or q6_K
    int M;                         // rows
    int begin;                     // first tile-row in the phase's concatenated tile-row index
    int ldy;
    float *y;                      // output [B][ldy] (replica 0)
    const float *bias;             // f32 or null
    int n_rep;                     // copies of the output to write (1, or MEGA_REPLICAS for vectors every workgroup reads)
    size_t y_rep_stride;           // floats between replicas
};

// One GEMV phase: y_p = W_p . f(x) for up to three matrices that share the activations.
struct MegaPhase {
    MegaPart part[3];
    int n_part;
    int total_rows;                // tile-rows (16 rows each) over all parts
    const float *x;                // activations [B][ldx] (replica 0)
    size_t x_rep_stride;           // floats between replicas
    int ldx, K;
    const float *norm_w;           // fused RMS norm weight or null
    int epi;                       // GemvEpilogue; EPI_RESIDUAL adds into y in place
};

struct MegaLayer {
    MegaPhase ph[4];               // q/k/v, o, gate/up, down
    uint16_t *kc, *vc;             // this layer's KV cache of the session
};

struct MegaArgs {
    const MegaLayer *layers;       // device array
    int n_layers;
    int B;                         // tokens, each in its own sequence (1..4)
    int E;
    int n_head, n_kv, group, n_rot, rope_mode, n_ctx, n_splits;
    float eps, attn_scale;
    // exchange buffers (device memory, sized for 4 tokens): projection outputs, attention output, split partials
    float *x;                      // hidden state [replica][B][E]; the caller fills replica 0
    size_t x_rep_stride, attn_rep_stride;
    const float *q, *k, *v;
    float *attn, *part, *ml;
    float *rope_cs, *rope_sn;      // [B][64] cos / sin of pos * inv_freq, filled by the launcher (ordinary device memory)
    const int32_t *pos, *seq;      // device, [B]
    const float *inv_freq;
    unsigned *bar;                 // grid-barrier counter
    unsigned bar_base;             // its value when this launch starts
    int *abort_flag;               // set by any workgroup whose barrier wait times out
    unsigned spin_limit;
};

constexpr int MEGA_SPLITS_MAX = 32;
constexpr int MEGA_BATCH_MAX = 4;
constexpr int MEGA_REPLICAS = 8;

// LDS bytes a launch needs for column count nb (1, 2 or 4) over the phases of `layer` on a grid of `grid` workgroups
size_t mega_smem_bytes(const MegaLayer &layer, int nb, int group, int grid);
// grid workgroups must all be resident (launched cooperatively); returns a mesh_status
int decode_mega(const MegaArgs &a, int grid, size_t smem, hipStream_t stream);
int mega_barriers_per_launch(int n_layers);
bool mega_group_supported(int group);

}  // namespace mesh
