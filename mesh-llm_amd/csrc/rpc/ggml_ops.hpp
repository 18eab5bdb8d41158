// ggml operation ids as they appear in the `op` field of a serialized tensor.
//
// FROM MEMORY, UNVERIFIABLE OFFLINE.  The enum lives in ggml.h of llama.cpp@45155597
// (third_party/llama.cpp/upstream.txt:1), which is not vendored; the reference tree shows exactly one value, GGML_OP_NONE = 0
// (third_party/llama.cpp/patches/0002-rpc-add-direct-peer-tensor-transfers.patch:1406).  The numbering below is the
// upstream enum as of late 2025 as best recalled, and it shifts whenever upstream inserts an operation.  Nothing in the
// server's decisions depends on it: a graph is recognised by the names of its weight tensors and the shapes around them
// (rpc_graph.cpp); this table only turns op numbers into words in log lines, with the number printed beside the word.
#pragma once

#include <cstdint>

namespace mesh_rpc {

constexpr uint32_t GGML_OP_NONE = 0;      // the one value the reference tree itself states: a leaf (weight, input, cache)

inline const char *ggml_op_name_guess(uint32_t op) {
    static const char *const names[] = {
        "NONE", "DUP", "ADD", "ADD_ID", "ADD1", "ACC", "SUB", "MUL", "DIV", "SQR", "SQRT", "LOG", "SIN", "COS", "SUM", "SUM_ROWS", "MEAN",
        "ARGMAX", "COUNT_EQUAL", "REPEAT", "REPEAT_BACK", "CONCAT", "SILU_BACK", "NORM", "RMS_NORM", "RMS_NORM_BACK", "GROUP_NORM",
        "L2_NORM", "MUL_MAT", "MUL_MAT_ID", "OUT_PROD", "SCALE", "SET", "CPY", "CONT", "RESHAPE", "VIEW", "PERMUTE", "TRANSPOSE",
        "GET_ROWS", "GET_ROWS_BACK", "SET_ROWS", "DIAG", "DIAG_MASK_INF", "DIAG_MASK_ZERO", "SOFT_MAX", "SOFT_MAX_BACK", "ROPE",
        "ROPE_BACK", "CLAMP", "CONV_TRANSPOSE_1D", "IM2COL", "IM2COL_BACK", "IM2COL_3D", "CONV_2D", "CONV_3D", "CONV_2D_DW",
        "CONV_TRANSPOSE_2D", "POOL_1D", "POOL_2D", "POOL_2D_BACK", "UPSCALE", "PAD", "PAD_REFLECT_1D", "ROLL", "ARANGE",
        "TIMESTEP_EMBEDDING", "ARGSORT", "LEAKY_RELU", "FLASH_ATTN_EXT", "FLASH_ATTN_BACK", "SSM_CONV", "SSM_SCAN", "WIN_PART",
        "WIN_UNPART", "GET_REL_POS", "ADD_REL_POS", "RWKV_WKV6", "GATED_LINEAR_ATTN", "RWKV_WKV7", "UNARY", "MAP_CUSTOM1", "MAP_CUSTOM2",
        "MAP_CUSTOM3", "CUSTOM", "CROSS_ENTROPY_LOSS", "CROSS_ENTROPY_LOSS_BACK", "OPT_STEP_ADAMW", "OPT_STEP_SGD", "GLU",
    };
    return op < sizeof(names) / sizeof(names[0]) ? names[op] : "?";
}

}  // namespace mesh_rpc
