// Shared by the MoE decode kernels (moe.hip, moe_persist.hip).
#pragma once
#include "mk_common.h"

// Expert id of a routed pair.  When the table states its size, an id outside it selects entry 0 with routing weight 0:
// the pair then adds nothing to the token's row (the pointer arrays are never read out of bounds).  The reference
// would panic on such an index; a caller that wants to know asks mk_dev_moe_count_bad_ids (moe.hip).
__device__ __forceinline__ int mk_checked_expert(int e, size_t n_experts, bool &ok) {
    ok = n_experts == 0 || (unsigned)e < (unsigned)n_experts;
    return ok ? e : 0;
}

// Integer dot of one 32-block: 32 e2m1 weights (16 bytes) against 32 q8 values held as 16 f16 pairs.  Every product is
// a multiple of 0.5 below 2^15, so the f32 sum is exact: the result is half of q8::block_dot (src/q8.rs:170-202).
__device__ __forceinline__ float mk_dot32_fp4_f16(const mk_i4 w, const mk_h2 *xr) {
    float h = 0.0f;
#pragma unroll
    for (int d = 0; d < 4; d++) {
        uint32_t wd = (uint32_t)w[d];
        h = __builtin_amdgcn_fdot2(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(wd, 1.0f, 0), xr[d * 4 + 0], h, false);
        h = __builtin_amdgcn_fdot2(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(wd, 1.0f, 1), xr[d * 4 + 1], h, false);
        h = __builtin_amdgcn_fdot2(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(wd, 1.0f, 2), xr[d * 4 + 2], h, false);
        h = __builtin_amdgcn_fdot2(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(wd, 1.0f, 3), xr[d * 4 + 3], h, false);
    }
    return h;
}

struct FusedArgs {
    mk_expert_table tab;
    const int32_t *ids;
    const float *weights;
    const float *x;
    int topk, shared, per, d, inter, act_kind, ds_rule;
    float limit;
    float *af;   // [P][inter]  activation values in f32 (the down kernel forms their q8 blocks)
    float *out;  // [B][d]
};

enum { MK_MOE_STAGE_ALL = 0, MK_MOE_STAGE_ACT = 1, MK_MOE_STAGE_FROM_ACT = 2 };

// moe_persist.hip: the one-launch expert section (one resident workgroup per CU) over a table that carries the packed
// copies (tab.w13t, tab.w2t).
//   stage ALL       x -> out                      (a.af unused; the activation values go through `lines`)
//   stage ACT       x -> a.af, nothing else
//   stage FROM_ACT  a.af -> out
// lines: [P][inter] 8-byte units of the caller's workspace.
bool mk_moe_persist_takes(size_t B, size_t d, size_t inter, int per);
size_t mk_moe_persist_lines_bytes(size_t P, size_t inter);
int mk_moe_persist_launch(const FusedArgs &a, size_t B, int stage, void *lines, hipStream_t st);
