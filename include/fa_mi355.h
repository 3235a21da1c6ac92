/*
 * fa_mi355.h -- C ABI of libfa_mi355.so: flash attention forward/backward with an optional
 * materialized bias for AMD MI355X (gfx950).
 *
 * The two launch entry points replace the host launchers of the reference one for one:
 *   fa_fwd  <->  _flash_attn_fwd(q, k, v, bias, causal, sm_scale) -> (o, M)
 *                /root/reference/flash_attention.py:649-685
 *   fa_bwd  <->  _flash_attn_bwd(do, q, k, v, o, bias, causal, sm_scale, M, dq, dk, dv, dbias)
 *                /root/reference/flash_attention.py:688-763
 * Like them, the library owns no memory: every buffer (including the backward workspace) is
 * allocated by the caller, every call only enqueues work on the stream it is given and returns
 * without synchronizing.  All entry points are re-entrant and keep no mutable global state, with
 * one exception: fa_bwd_noalloc (at the end of this header) keeps its scratch in a static device
 * array of the library, 8 MiB on every GPU it runs on, and a per-device cache of that array's
 * address; calls of it that overlap on one GPU race on the array.
 *
 * Layouts (element strides, as the reference passes them, flash_attention.py:670-675):
 *   q, o, do, dq : (B, M, H, D)     k, v, dk, dv : (B, N, H, D)     the D stride must be 1
 *   bias, dbias  : (B, H, M, N)     any strides, 0 included (an expanded mask works as is)
 *   lse, delta   : (B, H, M) fp32, dense, in log2 units: lse = log2(sum_j 2^(s_ij))
 * Base pointers of q/k/v/o/do/dq/dk/dv and their B/seq/H strides must be multiples of 16 bytes
 * (FA_ERR_LAYOUT otherwise; FA_ERR_HEAD_STRIDE for a D stride other than 1); bias/dbias have no
 * alignment requirement, but only rows with unit N stride and 16-byte aligned row starts that are
 * whole 16-byte chunks, or whose row stride covers the last chunk (N * element size rounded up to 16
 * bytes: a padded row pitch or a column slice of a wider tensor), take the fast path.  On that path
 * the bytes behind the last key of EVERY row, up to the end of its 16-byte chunk, are read (never
 * written), the last row of the last (batch, head) slice included: the caller guarantees that the
 * chunk holding the last element of the tensor lies inside the allocation (a row-strided view whose
 * last row ends the allocation does not qualify and must be copied to a padded pitch first).  With FA_MI355_VERBOSE set in the
 * environment the library says on stderr, once per process, when a bias or dbias misses that path
 * and is read or written element by element (several times slower).
 */
#ifndef FA_MI355_H
#define FA_MI355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FA_ABI_VERSION 3

/* element type of q, k, v, o and their gradients */
enum fa_dtype { FA_F16 = 0, FA_BF16 = 1 };

/* element type of bias (and of dbias, which always has the type of bias);
 * FA_BIAS_BOOL is one byte per element, non-zero = keep (flash_attention.py:48-50).
 * FA_BIAS_ALIBI has no counterpart in the reference, which needs such a bias materialized
 * (README.md:9): `bias` points to H fp32 slopes and the kernels compute
 *   bias[b, h, i, j] = -slope[h] * |i * N / M - j|
 * from the indices; bias_strides are ignored, and dbias (when non-NULL) receives the H fp32 slope
 * gradients, dslope[h] = sum over b, i, j of dS[b, h, i, j] * -|i * N / M - j|. */
enum fa_bias_dtype {
    FA_BIAS_NONE = 0, FA_BIAS_BOOL = 1, FA_BIAS_F16 = 2, FA_BIAS_BF16 = 3, FA_BIAS_F32 = 4, FA_BIAS_ALIBI = 5
};

enum fa_status {
    FA_OK = 0,
    FA_ERR_NULL = -1,        /* a required pointer is NULL */
    FA_ERR_SHAPE = -2,       /* a dimension is < 1, or causal with M != N */
    FA_ERR_HEAD_DIM = -3,    /* D not in {16, 32, 64, 128, 256}  (flash_attention.py:776) */
    FA_ERR_DTYPE = -4,       /* unknown dtype / bias dtype, or dbias requested for a bool bias */
    FA_ERR_LAYOUT = -5,      /* alignment or stride rule above violated */
    FA_ERR_WORKSPACE = -6,   /* workspace NULL or smaller than fa_bwd_workspace_bytes() */
    FA_ERR_UNSUPPORTED = -7, /* combination not built into this library */
    FA_ERR_LAUNCH = -8,      /* the HIP runtime rejected a launch (hipGetLastError) */
    FA_ERR_TOO_LARGE = -9,   /* fa_bwd_noalloc: the problem exceeds FA_NOALLOC_MAX_ROWS */
    FA_ERR_HEAD_STRIDE = -10 /* the head-dim stride of a q/k/v/o/do/dq/dk/dv tensor is not 1.  The reference's
                                kernels take any (flash_attention.py:91-94, :117-118); these read rows in 16-byte
                                chunks, so the caller copies such a tensor to unit stride first (the Python
                                layer of this package does) */
};

/* Problem description shared by forward and backward.  Strides are in elements. */
typedef struct fa_problem {
    int32_t B, H, M, N, D;
    int32_t dtype;       /* enum fa_dtype */
    int32_t bias_dtype;  /* enum fa_bias_dtype */
    int32_t causal;      /* 0 / 1; top-left aligned, requires M == N (flash_attention.py:45,777) */
    float sm_scale;      /* scores = (q . k) * sm_scale + bias  (flash_attention.py:149-150) */
} fa_problem;

/* _flash_attn_fwd: flash_attention.py:649-685.  o and lse are outputs. */
typedef struct fa_fwd_args {
    fa_problem p;
    const void *q, *k, *v, *bias; /* bias may be NULL iff bias_dtype == FA_BIAS_NONE */
    void *o;
    float *lse;                   /* (B, H, M) */
    int64_t q_strides[4], k_strides[4], v_strides[4], o_strides[4]; /* (B, seq, H, D) */
    int64_t bias_strides[4];      /* (B, H, M, N) */
    void *workspace;              /* optional (may be NULL): fa_fwd_workspace_bytes() bytes, 256-byte aligned */
    size_t workspace_bytes;
} fa_fwd_args;

/* _flash_attn_bwd: flash_attention.py:688-763.  dq, dk, dv (and dbias when non-NULL, i.e. when
 * the bias is trainable, flash_attention.py:693,799) are outputs and are fully overwritten:
 * unlike the reference's dbias they need no zero fill by the caller.
 *
 * dbias of a float bias comes in two layouts, told apart by dbias_strides:
 *   dense    (B, H, M, N), every stride of a dimension larger than 1 non-zero: dbias = dS, as the
 *            reference stores it (flash_attention.py:307-308);
 *   reduced  the gradient of a bias that was broadcast over the query rows, (B or 1, H or 1, 1, N):
 *            dbias_strides[2] == 0, and dbias_strides[0] / [1] == 0 where the bias was broadcast over
 *            batches / heads too.  The kernels sum dS over the rows (and a second small kernel over
 *            the broadcast batches / heads), so no (B, H, M, N) gradient is ever written.  No
 *            counterpart in the reference, which leaves that reduction to autograd. */
typedef struct fa_bwd_args {
    fa_problem p;
    const void *q, *k, *v, *o, *dout, *bias;
    const float *lse;             /* as written by fa_fwd */
    void *dq, *dk, *dv, *dbias;   /* dbias NULL = bias not trainable */
    void *workspace;              /* fa_bwd_workspace_bytes() bytes, 256-byte aligned */
    size_t workspace_bytes;
    int64_t q_strides[4], k_strides[4], v_strides[4], o_strides[4], do_strides[4];
    int64_t dq_strides[4], dk_strides[4], dv_strides[4];
    int64_t bias_strides[4], dbias_strides[4];
} fa_bwd_args;

/* Version of this header the library was built against (== FA_ABI_VERSION). */
int fa_abi_version(void);

/* Static, NUL-terminated description of a status code. */
const char *fa_strerror(int status);

/* Enqueue the forward on `stream` (a hipStream_t passed as void*; NULL = the null stream).
 * Replaces _flash_attn_fwd, flash_attention.py:649-685 (bias pre-scale :660-663 included). */
int fa_fwd(const fa_fwd_args *args, void *stream);

/* Bytes of scratch the backward needs for this problem: delta, (B, H, M) fp32
 * (flash_attention.py:689), followed by the partial sums of the reduced dbias layouts. */
size_t fa_bwd_workspace_bytes(const fa_problem *p);

/* Scratch with which fa_fwd splits the keys of a query tile between several work-groups and merges
 * their softmaxes (the outputs of the shares in fp32, and their LSEs); 0 when the
 * problem has enough query tiles to fill the GPU, or is causal.  No counterpart in the reference (its grid is one program
 * per query tile, flash_attention.py:666).  The workspace is optional: without it fa_fwd runs one
 * work-group per query tile, with the same results up to fp32 rounding of the merge.  "Enough" is
 * measured against the compute units of the CURRENT device (as is the dq part of
 * fa_bwd_workspace_bytes): ask with the device current on which fa_fwd / fa_bwd will run. */
size_t fa_fwd_workspace_bytes(const fa_problem *p);

/* Enqueue the backward (delta, dK/dV/dBias/dQ) on `stream`.
 * Replaces _flash_attn_bwd, flash_attention.py:688-763 (K and bias pre-scale :699-704 included). */
int fa_bwd(const fa_bwd_args *args, void *stream);

/* The three stages of the backward.  fa_bwd(args, stream) is fa_bwd_stages(args, stream, FA_STAGE_ALL).
 * They are enqueued in this order, except that a dQ stage which does not read dbias (see below) is
 * enqueued first when FA_STAGE_PREP is asked for in the same call: its kernel then forms delta itself,
 * bit for bit as the delta pass would, and stores it for the dK/dV kernel, and no delta pass is launched. */
enum fa_bwd_stage {
    FA_STAGE_PREP = 1, /* delta = rowsum(o * do)          (flash_attention.py:197-233) */
    FA_STAGE_MAIN = 2, /* dK, dV, dBias over key tiles    (flash_attention.py:237-454) */
    FA_STAGE_DQ = 4,   /* dQ over query tiles              (flash_attention.py:458-646) */
    FA_STAGE_ALL = 7,
    /* modifier of FA_STAGE_DQ when it is enqueued WITHOUT FA_STAGE_MAIN in the same call: the
     * caller vouches that args->dbias still holds what FA_STAGE_MAIN wrote for these very
     * arguments, so that dQ may be formed from it (one matrix product instead of three) */
    FA_STAGE_DQ_FROM_DBIAS = 8
};

/* Enqueue only the selected stages of the backward (same arguments and checks as fa_bwd).
 * No counterpart in the reference: it exists so that a benchmark or profiler can bracket one
 * stage with events.  FA_STAGE_MAIN and FA_STAGE_DQ both need the delta of FA_STAGE_PREP.  When
 * FA_STAGE_MAIN and FA_STAGE_DQ run in one call and dbias is requested in fp32 or in the element
 * type of q, dQ is formed from the dbias just written (it is the dS of the dQ product); a call with
 * FA_STAGE_DQ alone recomputes dS from q, k, v and the bias and never reads dbias, unless
 * FA_STAGE_DQ_FROM_DBIAS is added.  Both routes agree within the rounding of dS to 16 bits. */
int fa_bwd_stages(const fa_bwd_args *args, void *stream, int stages);

/* fa_bwd for callers that cannot allocate device memory (HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference, whose launcher allocates
 * delta itself (flash_attention.py:689).  args->workspace and args->workspace_bytes are ignored:
 * the scratch (delta and the partial sums of a reduced dbias) lives in a static device array
 * of 2 * FA_NOALLOC_MAX_ROWS floats (8 MiB per GPU, held until the process ends), so neither
 * B * H * M nor B * H * max(N, 4) may exceed FA_NOALLOC_MAX_ROWS (FA_ERR_TOO_LARGE
 * otherwise).  The call allocates and frees nothing.  All calls on one GPU share the array:
 * calls that may overlap on one GPU (different streams, different threads) race on it; on one
 * stream they are ordered and safe.  Results are bit-identical to fa_bwd.
 * The first call on a device asks the runtime for the array's address on that device
 * (hipGetSymbolAddress, which may load the library's code object): make one call on every device
 * before any stream capture; later calls only read the cached address. */
#define FA_NOALLOC_MAX_ROWS (1 << 20)
int fa_bwd_noalloc(const fa_bwd_args *args, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FA_MI355_H */
