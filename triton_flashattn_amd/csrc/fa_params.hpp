// Kernel argument blocks (host fills them from the C-ABI structs after validation).
#pragma once
#include <stdint.h>

namespace fa {

// strides in elements; index 0 = batch, 1 = sequence, 2 = head (the head-dim stride is 1)
struct Strides3 {
    int64_t b, s, h;
};
// bias / dbias: (B, H, M, N), any strides
struct Strides4 {
    int64_t b, h, m, n;
};

// keys of a row-broadcast bias that the forward and dQ kernels keep in LDS (as fp32)
constexpr int kRowBiasKeys = 4096;

struct FwdParams {
    const void* q;
    const void* k;
    const void* v;
    const void* bias;
    void* o;
    float* lse;  // (B, H, M)
    Strides3 sq, sk, sv, so;
    Strides4 sbias;
    int B, H, M, N;
    float sm_scale;
    int bias_vec;  // bias rows may be read with aligned 16-byte loads
    int n_mtiles;
    // Keys split between n_splits work-groups per query tile (1 = no split): split s takes
    // keys_per_split keys (a multiple of the kernel's step) and writes its output, in fp32,
    // and its LSE to part_o (n_splits, B*H, M, D) / part_lse (n_splits, B*H, M);
    // fa_fwd_merge_kernel combines them.
    int n_splits, keys_per_split;
    void* part_o;
    float* part_lse;
    int row_bias_kind;  // 0, or the element kind (1 bool, 2 fp16, 3 bf16, 4 fp32) of a bias with stride 0 along M
                        // whose keys (of one split) fit the kernel's LDS row: staged once, not streamed
};

struct BwdParams {
    const void* q;
    const void* k;
    const void* v;
    const void* o;
    const void* dout;
    const void* bias;
    const float* lse;  // (B, H, M)
    float* delta;      // (B, H, M)        workspace
    float* partials;   // workspace behind delta: reduced-dBias partial sums (see fa_bwd_kernel)
    void* dq;
    void* dk;
    void* dv;
    void* dbias;
    Strides3 sq, sk, sv, so, sdo, sdq, sdk, sdv;
    Strides4 sbias, sdbias;
    int B, H, M, N;
    float sm_scale;
    int n_ntiles;   // key tiles of the dK/dV kernel
    int waves_per_role;  // 32-key blocks per key tile of the dK/dV kernel
    int n_mtiles;   // query tiles of the dQ kernel
    int bias_vec;   // bias rows may be read with aligned 16-byte loads
    int dbias_vec;  // dbias rows may be written with aligned 16-byte stores
    // dQ kernel: keys split between dq_splits work-groups per query tile (1 = no split), each over
    // dq_keys_per_split keys, their shares of dq in fp32 in part_dq (dq_splits, B*H, M, D);
    // fa_bwd_dq_sum_kernel adds them up
    int dq_splits, dq_keys_per_split;
    void* part_dq;
    int row_bias_kind;  // 0, or the element kind (1 bool, 2 fp16, 3 bf16, 4 fp32) of a bias with stride 0 along M:
                        // the dK/dV kernel reads it as one value per key, the dQ kernel stages it in LDS
    int dq_makes_delta; // the dQ kernel runs before the dK/dV kernel and forms delta itself (and stores it),
                        // in place of fa_bwd_prep_kernel and bit for bit like it
};

}  // namespace fa
