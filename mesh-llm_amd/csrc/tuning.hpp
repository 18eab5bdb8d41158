// Every switch that picks between kernels or moves a dispatch threshold, in one table.
//
// A stage holds one copy, fixed at mesh_stage_open: the process default (the table below, overridden ONCE per process by
// the environment variable MESH_TUNING="name=value,name=value"), then mesh_stage_opts.tuning in the same syntax.  Each
// session starts from its stage's copy; mesh_session_set_option changes the switches marked SESSION between decode
// calls.  The ones marked STAGE decide what the stage and its sessions allocate and cannot change afterwards.  Nothing
// else in the library reads the environment for tuning.
#pragma once

#include <cstddef>
#include <cstdint>
#include <string>

namespace mesh {

struct Tuning {
    // --- STAGE: fixed at mesh_stage_open
    int gemm_layout = 1;           // stages that can be handed prefill-sized calls keep a GEMM-layout copy of their projections
    int gemm_min_tokens = 17;      // calls with at least this many tokens take the large-tile MFMA GEMM
    int skinny_min_tokens = 0;     // ... and at least this many the skinny MFMA GEMM; 0 = 4 with skinny_f16, 5 without
    // --- SESSION: mesh_session_set_option
    int gemm_splitk = 1;           // GEMM launches too narrow to fill the chip split K over workgroups
    int chunk_kv16 = 1;            // long prefill chunks over a quantised cache decode a layer's rows once into an f16 copy
    int gemv_rope = 1;             // RoPE and the KV append in the q/k/v projection's epilogue (0: their own kernel)
    int xq_handover = 1;           // the gate/up mat-vec leaves the FFN vector quantised for the down projection
    int skinny_f16 = 1;            // calls of skinny_min_tokens..gemm_min_tokens-1 tokens on the f16 matrix cores (0: integer, 16-bit activations)
    int skinny_norm_fused = 1;     // f16 skinny GEMM: the RMS norms ride in the launches around them (0: a norm launch of their own)
    int skinny_pair = 1;           // skinny GEMMs: q4_K q/k and a q6_K v projection as one launch (0: one launch per type)
    int skinny_f16_wide = 1;       // batches of gemm_min_tokens..32 decode steps stay on the f16 skinny GEMM, 32 columns per pass (0: large-tile GEMM)
    int gemm_fused = 1;            // q/k/v and gate/up of a prefill call as one GEMM launch each
    int gemm_xdirect = 1;          // the prefill GEMM reads k8-major activations directly (0: row-major staged through LDS)
    int gemm_big = 1;              // the 256-row tile for wide projections of long calls
    int gemm_narrow = 1;           // the 64-token tile for calls of at most 64 tokens
    int attn_chunk_ksplit = 1;     // a prefill chunk's key walks split over workgroups when the grid would not fill the chip
    int attn_mma_min_tokens = 1;   // decode attention on the matrix cores from this many tokens (below: the all-f32 kernel)
    int attn_split_target = 0;     // workgroups a decode attention launch aims at; 0 = 256, 512 for quantised rows of 64+ (token, head) pairs
    int moe_group = 1;             // (token, slot) pairs grouped by expert (0: every pair its own product)
    int moe_router_tail = 1;       // small decode batches: the router launch's last workgroup routes and groups (0: a second launch)
    int moe_fuse_quant = 1;        // the expert combine step quantises for the next layer's projections
    int moe_gemm = 1;              // prefill-sized expert products as tiles of the large-tile GEMM
    int moe_gemm_min_pairs = 4;    // ... from this many pairs per expert on average
    int grouped_oversub = 8;       // grouped expert mat-vec: workgroups per compute unit and item
    int graphs = 0;                // decode steps of up to 32 tokens replayed from captured HIP graphs

    int skinny_from() const { return skinny_min_tokens > 0 ? skinny_min_tokens : (skinny_f16 ? 4 : 5); }
};

enum TuningLevel { TUNE_STAGE = 0, TUNE_SESSION = 1 };

struct TuningField {
    const char *name;
    int Tuning::*field;
    int lo, hi;
    TuningLevel level;
};
// the table, ended by a null name
const TuningField *tuning_fields();

// MESH_OK, or MESH_ERR_INVALID with the message set: unknown name, value outside [lo, hi], or a STAGE switch when
// `session_only` is set.
int tuning_set(Tuning &t, const char *name, int value, bool session_only);
int tuning_get(const Tuning &t, const char *name, int *value);
// "name=value,name=value" (spaces ignored); stops at the first bad entry
int tuning_parse(Tuning &t, const char *text, const char *what);
// table defaults with MESH_TUNING applied; read once.  A bad MESH_TUNING makes mesh_stage_open fail with its message.
int tuning_process_default(Tuning &out);
// "name=value,..." of every switch
std::string tuning_describe(const Tuning &t);

}  // namespace mesh
