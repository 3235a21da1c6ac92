// C ABI of libfa_mi355.so (declared in include/fa_mi355.h): argument validation and dispatch.
// Host code only; the kernels live in fa_fwd.hip and fa_bwd.hip.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <initializer_list>
#include <mutex>

#include "../../include/fa_mi355.h"
#include "fa_params.hpp"

namespace fa {
// one object file per head dimension defines these (fa_fwd.hip, fa_bwd.hip with -DFA_HEAD_DIM)
template <int D> hipError_t launch_fwd_d(const FwdParams& p, int dtype, int bias, bool causal, hipStream_t st);
template <int D> hipError_t launch_bwd_d(const BwdParams& p, int dtype, int bias, bool causal, int dbias, int stages, hipStream_t st);
#define FA_DECLARE_D(D)                                                                                         \
    template <> hipError_t launch_fwd_d<D>(const FwdParams& p, int dtype, int bias, bool causal, hipStream_t st); \
    template <> hipError_t launch_bwd_d<D>(const BwdParams& p, int dtype, int bias, bool causal, int dbias, int stages, hipStream_t st);
FA_DECLARE_D(16)
FA_DECLARE_D(32)
FA_DECLARE_D(64)
FA_DECLARE_D(128)
FA_DECLARE_D(256)
#undef FA_DECLARE_D

static hipError_t launch_fwd(const FwdParams& p, int D, int dtype, int bias, bool causal, hipStream_t st) {
    switch (D) {
        case 16: return launch_fwd_d<16>(p, dtype, bias, causal, st);
        case 32: return launch_fwd_d<32>(p, dtype, bias, causal, st);
        case 64: return launch_fwd_d<64>(p, dtype, bias, causal, st);
        case 128: return launch_fwd_d<128>(p, dtype, bias, causal, st);
        case 256: return launch_fwd_d<256>(p, dtype, bias, causal, st);
    }
    return hipErrorNotSupported;
}
static hipError_t launch_bwd(const BwdParams& p, int D, int dtype, int bias, bool causal, int dbias, int stages, hipStream_t st) {
    switch (D) {
        case 16: return launch_bwd_d<16>(p, dtype, bias, causal, dbias, stages, st);
        case 32: return launch_bwd_d<32>(p, dtype, bias, causal, dbias, stages, st);
        case 64: return launch_bwd_d<64>(p, dtype, bias, causal, dbias, stages, st);
        case 128: return launch_bwd_d<128>(p, dtype, bias, causal, dbias, stages, st);
        case 256: return launch_bwd_d<256>(p, dtype, bias, causal, dbias, stages, st);
    }
    return hipErrorNotSupported;
}
// query rows per work-group of the forward and dQ kernels; keys per work-group of the dK/dV kernel
static int fwd_block_m() { return 128; }
static int bwd_block_n(int D) { return D > 128 ? 64 : 128; }  // keys per tile of the dK/dV kernel
}  // namespace fa

// Scratch of fa_bwd_noalloc: delta, one float per (batch, head, query row), in the first half; the
// partial sums of a reduced dbias in the second.  Every GPU the library
// runs on holds its own copy of this array until the process ends.  In host code the name is only
// a handle; the device address comes from hipGetSymbolAddress (scratch_on_current_device).
static __device__ __align__(256) float scratch[2 * FA_NOALLOC_MAX_ROWS];

namespace fa {

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static float* g_scratch_ptr[kMaxDevices];  // device address of `scratch`, per device

// Address of this device's copy of `scratch`, looked up once per device with that device current.
// This function has external linkage on purpose: the compiler gives a static device variable a
// symbol the runtime can find only when a host function with external linkage refers to it.
float* scratch_on_current_device() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
        g_scratch_ptr[dev] = static_cast<float*>(ptr);
    }
    return g_scratch_ptr[dev];
}

}  // namespace fa

namespace {

bool head_dim_ok(int d) { return d == 16 || d == 32 || d == 64 || d == 128 || d == 256; }

int check_problem(const fa_problem& p) {
    if (p.B < 1 || p.H < 1 || p.M < 1 || p.N < 1) return FA_ERR_SHAPE;
    if (!head_dim_ok(p.D)) return FA_ERR_HEAD_DIM;
    if (p.dtype != FA_F16 && p.dtype != FA_BF16) return FA_ERR_DTYPE;
    if (p.bias_dtype < FA_BIAS_NONE || p.bias_dtype > FA_BIAS_ALIBI) return FA_ERR_DTYPE;
    if (p.causal && p.M != p.N) return FA_ERR_SHAPE;
    // row indices times four (the LSE and delta vectors) are formed in 32 bits
    if (p.M >= (1 << 28) || p.N >= (1 << 28)) return FA_ERR_SHAPE;
    // a grid is one-dimensional: tiles * B * H must fit in 31 bits
    if ((int64_t)((p.M + 63) / 64 + (p.N + 63) / 64) * p.B * p.H >= (1ll << 31)) return FA_ERR_SHAPE;
    return FA_OK;
}

// 16-byte rule for a (B, seq, H, D) tensor of 2-byte elements; strides of extent-1 dims are free
// (FA_OK, FA_ERR_HEAD_STRIDE or FA_ERR_LAYOUT)
int qkv_layout(const void* ptr, const int64_t s[4], int nb, int ns, int nh) {
    if (s[3] != 1) return FA_ERR_HEAD_STRIDE;
    if (reinterpret_cast<uintptr_t>(ptr) % 16 != 0) return FA_ERR_LAYOUT;
    if (nb > 1 && s[0] % 8 != 0) return FA_ERR_LAYOUT;
    if (ns > 1 && s[1] % 8 != 0) return FA_ERR_LAYOUT;
    if (nh > 1 && s[2] % 8 != 0) return FA_ERR_LAYOUT;
    // the kernels form 32-bit byte offsets inside a tile of up to 128 rows
    if (ns > 1 && (s[1] < 0 || s[1] >= (1 << 23))) return FA_ERR_LAYOUT;
    return FA_OK;
}
// the first complaint among several tensors
int first_bad(std::initializer_list<int> sts) {
    for (int s : sts)
        if (s != FA_OK) return s;
    return FA_OK;
}

fa::Strides3 s3(const int64_t s[4]) { return fa::Strides3{s[0], s[1], s[2]}; }
fa::Strides4 s4(const int64_t s[4]) { return fa::Strides4{s[0], s[1], s[2], s[3]}; }

int bias_elem_size(int bias_dtype) {
    switch (bias_dtype) {
        case FA_BIAS_BOOL: return 1;
        case FA_BIAS_F16:
        case FA_BIAS_BF16: return 2;
        case FA_BIAS_F32: return 4;
    }
    return 0;
}

// rows of bias may be fetched with aligned 16-byte loads
bool bias_vec_ok(const void* ptr, const int64_t s[4], const fa_problem& p) {
    int es = bias_elem_size(p.bias_dtype);
    if (es == 0) return false;
    if (p.N > 1 && s[3] != 1) return false;
    if (reinterpret_cast<uintptr_t>(ptr) % 16 != 0) return false;
    if (p.B > 1 && (s[0] * es) % 16 != 0) return false;
    if (p.H > 1 && (s[1] * es) % 16 != 0) return false;
    if (p.M > 1 && (s[2] * es) % 16 != 0) return false;
    // A copy fetches whole 16-byte chunks: either the rows are whole chunks, or the row stride leaves
    // room for the last one (a padded row pitch, or a column slice of a wider tensor), so that the
    // bytes behind the last key of a row are readable; the kernels mask what they read there and write
    // a partial chunk of dbias element by element.
    const int64_t row_bytes = (int64_t)p.N * es, padded = (row_bytes + 15) & ~(int64_t)15;
    if (row_bytes != padded && !(p.M > 1 && s[2] * es >= padded)) return false;
    // one (batch, head) slice is addressed through a 32-bit buffer descriptor
    if (s[2] < 0 || (int64_t)(p.M - 1) * s[2] * es + padded >= (1ll << 31)) return false;
    return true;
}

size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

// With FA_MI355_VERBOSE set in the environment, says once per process on stderr when a bias cannot
// take the 16-byte copy path and the kernels fall back to reading or writing it element by element
// (much slower; the rules are in the header).
void note_slow_bias(const char* what, const void* ptr, const int64_t s[4], const fa_problem& p) {
    static std::atomic<bool> said{false};
    if (!std::getenv("FA_MI355_VERBOSE") || said.exchange(true)) return;
    std::fprintf(stderr,
                 "libfa_mi355: %s takes the element-wise path (pointer %p, strides %lld/%lld/%lld/%lld elements, N = %d): "
                 "needs unit key stride, 16-byte aligned base and B/H/M strides, rows of whole 16-byte chunks (or a "
                 "row stride that covers the last chunk) and (batch, head) slices below 2 GiB\n",
                 what, ptr, (long long)s[0], (long long)s[1], (long long)s[2], (long long)s[3], p.N);
}

// the two parts of the backward scratch, in floats: delta, and the partial sums of a reduced
// dbias (column sums per (batch, head, key), or slope gradients per (batch, head, key tile, wave))
size_t delta_floats(const fa_problem& p) { return (size_t)p.B * p.H * p.M; }
size_t partial_floats(const fa_problem& p) {
    const size_t tiles4 = (size_t)((p.N + fa::bwd_block_n(p.D) - 1) / fa::bwd_block_n(p.D)) * (fa::bwd_block_n(p.D) / 32);
    return (size_t)p.B * p.H * ((size_t)p.N > tiles4 ? (size_t)p.N : tiles4);
}

// Compute units of the current device (looked up once per device; 256, an MI355X, when no device
// can be asked: the size queries must also work where no GPU is present).
int compute_units() {
    static std::atomic<int> cached[fa::kMaxDevices];
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= fa::kMaxDevices) return 256;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

// Keys of a query tile split between work-groups when the query tiles alone leave the GPU half empty
// (fewer than two work-groups per CU): as many splits as it takes to get there, at most four, each
// with at least 16 steps of the K/V stream.  The answer depends on the current device (its CU
// count): a size query and the launch it sizes must run with the same device current.
struct FwdSplit {
    int n_splits, keys_per_split;
};
FwdSplit fwd_split(const fa_problem& p) {
    if (p.causal) return {1, 0};
    const int64_t wgs = (int64_t)((p.M + fa::fwd_block_m() - 1) / fa::fwd_block_m()) * p.B * p.H;
    const int64_t full = 2 * (int64_t)compute_units();
    if (wgs >= full) return {1, 0};
    const int bk = p.bias_dtype == FA_BIAS_NONE ? 64 : 32;  // keys per step of the forward kernel
    const int n_steps = (p.N + bk - 1) / bk;
    int s = (int)(full / wgs);
    s = s > 4 ? 4 : s;
    while (s > 1 && n_steps / s < 16) s--;
    if (s <= 1) return {1, 0};
    return {s, ((n_steps + s - 1) / s * bk + 63) / 64 * 64};  // whole steps of either kernel tiling
}

// the shares of dq of a dQ kernel that splits its keys like the forward (0 when it does not)
size_t dq_share_bytes(const fa_problem& p) {
    const FwdSplit s = fwd_split(p);
    return s.n_splits <= 1 ? 0 : align256((size_t)s.n_splits * p.B * p.H * p.M * p.D * sizeof(float));
}

// How dbias is laid out: 0 none, 1 dense (B, H, M, N), 2 reduced in the kernels; -1 = not acceptable
int dbias_mode(const fa_bwd_args* a) {
    const fa_problem& p = a->p;
    if (!a->dbias) return 0;
    if (p.bias_dtype == FA_BIAS_ALIBI) return 2;
    const int64_t* s = a->dbias_strides;
    const bool red_b = p.B > 1 && s[0] == 0, red_h = p.H > 1 && s[1] == 0, red_m = p.M > 1 && s[2] == 0;
    if (!red_b && !red_h && !red_m) return 1;
    // a reduction over batches or heads alone would need an (M, N) accumulator per output slice
    if (!red_m && p.M > 1) return -1;
    if (p.N > 1 && s[3] == 0) return -1;
    return 2;
}

}  // namespace

extern "C" {

int fa_abi_version(void) { return FA_ABI_VERSION; }

const char* fa_strerror(int status) {
    switch (status) {
        case FA_OK: return "ok";
        case FA_ERR_NULL: return "a required pointer is NULL";
        case FA_ERR_SHAPE: return "bad shape: a dimension is < 1, too large, or causal with M != N";
        case FA_ERR_HEAD_DIM: return "head dimension must be one of 16, 32, 64, 128, 256";
        case FA_ERR_DTYPE: return "unsupported dtype / bias dtype (or dbias requested for a bool bias)";
        case FA_ERR_LAYOUT:
            return "layout: head-dim stride must be 1 and pointers/strides 16-byte aligned; a dbias broadcast over "
                   "batches or heads must be broadcast over the query rows too";
        case FA_ERR_WORKSPACE: return "workspace is NULL, misaligned or smaller than fa_bwd_workspace_bytes()";
        case FA_ERR_UNSUPPORTED: return "combination not built into this library";
        case FA_ERR_LAUNCH: return "HIP kernel launch failed";
        case FA_ERR_TOO_LARGE: return "fa_bwd_noalloc: the problem exceeds FA_NOALLOC_MAX_ROWS";
        case FA_ERR_HEAD_STRIDE:
            return "the head-dim stride of q, k, v, o, do, dq, dk and dv must be 1: make the tensor contiguous first";
    }
    return "unknown status";
}

size_t fa_fwd_workspace_bytes(const fa_problem* p) {
    if (!p || check_problem(*p) != FA_OK) return 0;
    const FwdSplit s = fwd_split(*p);
    if (s.n_splits <= 1) return 0;
    const size_t rows = (size_t)p->B * p->H * p->M;
    return align256((size_t)s.n_splits * rows * p->D * sizeof(float)) + align256((size_t)s.n_splits * rows * sizeof(float));
}

int fa_fwd(const fa_fwd_args* a, void* stream) {
    if (!a) return FA_ERR_NULL;
    const fa_problem& p = a->p;
    int st = check_problem(p);
    if (st != FA_OK) return st;
    if (!a->q || !a->k || !a->v || !a->o || !a->lse) return FA_ERR_NULL;
    if ((p.bias_dtype != FA_BIAS_NONE) != (a->bias != nullptr)) return FA_ERR_NULL;
    st = first_bad({qkv_layout(a->q, a->q_strides, p.B, p.M, p.H), qkv_layout(a->k, a->k_strides, p.B, p.N, p.H),
                    qkv_layout(a->v, a->v_strides, p.B, p.N, p.H), qkv_layout(a->o, a->o_strides, p.B, p.M, p.H)});
    if (st != FA_OK) return st;

    fa::FwdParams k{};
    k.q = a->q; k.k = a->k; k.v = a->v; k.bias = a->bias; k.o = a->o; k.lse = a->lse;
    k.sq = s3(a->q_strides); k.sk = s3(a->k_strides); k.sv = s3(a->v_strides); k.so = s3(a->o_strides);
    k.B = p.B; k.H = p.H; k.M = p.M; k.N = p.N;
    k.sm_scale = p.sm_scale;
    if (a->bias && p.bias_dtype != FA_BIAS_ALIBI) {
        k.sbias = s4(a->bias_strides);
        k.bias_vec = bias_vec_ok(a->bias, a->bias_strides, p) ? 1 : 0;
        if (!k.bias_vec) note_slow_bias("bias", a->bias, a->bias_strides, p);
    }
    k.n_mtiles = (p.M + fa::fwd_block_m() - 1) / fa::fwd_block_m();
    k.n_splits = 1;
    if (a->workspace) {
        const size_t need = fa_fwd_workspace_bytes(&p);
        if (need > 0) {
            if (a->workspace_bytes < need || reinterpret_cast<uintptr_t>(a->workspace) % 256 != 0) return FA_ERR_WORKSPACE;
            const FwdSplit s = fwd_split(p);
            const size_t rows = (size_t)p.B * p.H * p.M;
            k.n_splits = s.n_splits;
            k.keys_per_split = s.keys_per_split;
            k.part_o = a->workspace;
            k.part_lse = reinterpret_cast<float*>(static_cast<char*>(a->workspace) + align256((size_t)s.n_splits * rows * p.D * sizeof(float)));
        }
    }
    // a bias that does not depend on the query row and whose keys fit the kernel's LDS row
    if (a->bias && p.bias_dtype >= FA_BIAS_BOOL && p.bias_dtype <= FA_BIAS_F32 && (p.M == 1 || a->bias_strides[2] == 0) &&
        (k.n_splits > 1 ? k.keys_per_split : p.N) <= fa::kRowBiasKeys)
        k.row_bias_kind = p.bias_dtype;
    hipError_t e = fa::launch_fwd(k, p.D, p.dtype, p.bias_dtype, p.causal != 0, static_cast<hipStream_t>(stream));
    if (e == hipErrorNotSupported) return FA_ERR_UNSUPPORTED;
    return e == hipSuccess ? FA_OK : FA_ERR_LAUNCH;
}

size_t fa_bwd_workspace_bytes(const fa_problem* p) {
    if (!p || check_problem(*p) != FA_OK) return 0;
    return align256(delta_floats(*p) * sizeof(float)) + align256(partial_floats(*p) * sizeof(float)) + dq_share_bytes(*p);
}

}  // extern "C"

namespace {

// `delta` NULL: the scratch is the caller's workspace; else the workspace fields are ignored
int bwd_enqueue(const fa_bwd_args* a, void* stream, int stages, float* delta) {
    if (!a) return FA_ERR_NULL;
    if (stages <= 0 || (stages & ~(FA_STAGE_ALL | FA_STAGE_DQ_FROM_DBIAS))) return FA_ERR_UNSUPPORTED;
    if ((stages & FA_STAGE_DQ_FROM_DBIAS) && !(stages & FA_STAGE_DQ)) return FA_ERR_UNSUPPORTED;
    const fa_problem& p = a->p;
    int st = check_problem(p);
    if (st != FA_OK) return st;
    if (!a->q || !a->k || !a->v || !a->o || !a->dout || !a->lse) return FA_ERR_NULL;
    // outputs of stages that do not run may be NULL
    const bool need_dq = (stages & FA_STAGE_DQ) != 0, need_dkv = (stages & FA_STAGE_MAIN) != 0;
    if ((need_dq && !a->dq) || (need_dkv && (!a->dk || !a->dv))) return FA_ERR_NULL;
    if ((p.bias_dtype != FA_BIAS_NONE) != (a->bias != nullptr)) return FA_ERR_NULL;
    if (a->dbias && (p.bias_dtype == FA_BIAS_NONE || p.bias_dtype == FA_BIAS_BOOL)) return FA_ERR_DTYPE;
    const int db_mode = dbias_mode(a);
    if (db_mode < 0) return FA_ERR_LAYOUT;
    st = first_bad({qkv_layout(a->q, a->q_strides, p.B, p.M, p.H), qkv_layout(a->k, a->k_strides, p.B, p.N, p.H),
                    qkv_layout(a->v, a->v_strides, p.B, p.N, p.H), qkv_layout(a->o, a->o_strides, p.B, p.M, p.H),
                    qkv_layout(a->dout, a->do_strides, p.B, p.M, p.H),
                    need_dq ? qkv_layout(a->dq, a->dq_strides, p.B, p.M, p.H) : FA_OK,
                    need_dkv ? qkv_layout(a->dk, a->dk_strides, p.B, p.N, p.H) : FA_OK,
                    need_dkv ? qkv_layout(a->dv, a->dv_strides, p.B, p.N, p.H) : FA_OK});
    if (st != FA_OK) return st;
    float* partials = nullptr;
    int dq_splits = 1, dq_keys = 0;  // (the entry point without allocations does not split: its scratch is small)
    void* part_dq = nullptr;
    if (!delta) {
        size_t need = fa_bwd_workspace_bytes(&p);
        if (!a->workspace || a->workspace_bytes < need || reinterpret_cast<uintptr_t>(a->workspace) % 256 != 0)
            return FA_ERR_WORKSPACE;
        delta = static_cast<float*>(a->workspace);
        partials = reinterpret_cast<float*>(static_cast<char*>(a->workspace) + align256(delta_floats(p) * sizeof(float)));
        if (dq_share_bytes(p) > 0) {
            const FwdSplit s = fwd_split(p);
            dq_splits = s.n_splits;
            dq_keys = s.keys_per_split;
            part_dq = reinterpret_cast<char*>(partials) + align256(partial_floats(p) * sizeof(float));
        }
    } else {
        partials = delta + FA_NOALLOC_MAX_ROWS;
    }

    fa::BwdParams k{};
    k.q = a->q; k.k = a->k; k.v = a->v; k.o = a->o; k.dout = a->dout; k.bias = a->bias; k.lse = a->lse;
    k.dq = a->dq; k.dk = a->dk; k.dv = a->dv; k.dbias = a->dbias;
    k.delta = delta;
    k.partials = partials;
    k.dq_splits = dq_splits; k.dq_keys_per_split = dq_keys; k.part_dq = part_dq;
    k.sq = s3(a->q_strides); k.sk = s3(a->k_strides); k.sv = s3(a->v_strides); k.so = s3(a->o_strides);
    k.sdo = s3(a->do_strides); k.sdq = s3(a->dq_strides); k.sdk = s3(a->dk_strides); k.sdv = s3(a->dv_strides);
    if (a->bias && p.bias_dtype != FA_BIAS_ALIBI) {
        k.sbias = s4(a->bias_strides);
        k.bias_vec = bias_vec_ok(a->bias, a->bias_strides, p) ? 1 : 0;
    }
    // a bias that does not depend on the query row: the dK/dV kernel keeps it in one register per key
    if (a->bias && p.bias_dtype >= FA_BIAS_BOOL && p.bias_dtype <= FA_BIAS_F32 && (p.M == 1 || a->bias_strides[2] == 0))
        k.row_bias_kind = p.bias_dtype;
    if (a->dbias && p.bias_dtype != FA_BIAS_ALIBI) {
        k.sdbias = s4(a->dbias_strides);
        k.dbias_vec = db_mode == 1 && bias_vec_ok(a->dbias, a->dbias_strides, p) ? 1 : 0;
        if (db_mode == 1 && !k.dbias_vec) note_slow_bias("dbias", a->dbias, a->dbias_strides, p);
    }
    k.B = p.B; k.H = p.H; k.M = p.M; k.N = p.N;
    k.sm_scale = p.sm_scale;
    int bn = fa::bwd_block_n(p.D);
    if (bn <= 0) return FA_ERR_UNSUPPORTED;
    k.n_ntiles = (p.N + bn - 1) / bn;
    k.waves_per_role = bn / 32;
    k.n_mtiles = (p.M + fa::fwd_block_m() - 1) / fa::fwd_block_m();
    hipError_t e = fa::launch_bwd(k, p.D, p.dtype, p.bias_dtype, p.causal != 0, db_mode, stages,
                                  static_cast<hipStream_t>(stream));
    if (e == hipErrorNotSupported) return FA_ERR_UNSUPPORTED;
    return e == hipSuccess ? FA_OK : FA_ERR_LAUNCH;
}

}  // namespace

extern "C" {

int fa_bwd_stages(const fa_bwd_args* a, void* stream, int stages) { return bwd_enqueue(a, stream, stages, nullptr); }

int fa_bwd(const fa_bwd_args* a, void* stream) { return bwd_enqueue(a, stream, FA_STAGE_ALL, nullptr); }

int fa_bwd_noalloc(const fa_bwd_args* a, void* stream) {
    if (!a) return FA_ERR_NULL;
    int st = check_problem(a->p);
    if (st != FA_OK) return st;
    if (delta_floats(a->p) > (size_t)FA_NOALLOC_MAX_ROWS || partial_floats(a->p) > (size_t)FA_NOALLOC_MAX_ROWS)
        return FA_ERR_TOO_LARGE;
    float* delta = fa::scratch_on_current_device();
    if (!delta) return FA_ERR_LAUNCH;
    return bwd_enqueue(a, stream, FA_STAGE_ALL, delta);
}

}  // extern "C"
