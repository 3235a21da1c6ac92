// Forward attention kernel for gfx950: O = softmax(Q K^T * sm_scale + bias) V, LSE saved.
//
// Replaces _attn_fwd / _attn_fwd_inner of the reference (/root/reference/flash_attention.py:12-194)
// together with the host-side bias pre-scale (flash_attention.py:660-663), which is folded into
// the kernel as an fp32 multiply.
//
// Work split.  One work-group (4 waves) owns 128 query rows of one (batch, head); each wave
// owns 32 of them for the whole kernel.  Keys/values are streamed through LDS in steps of 32
// (with a bias) or 64 keys, consumed 32 at a time.
// Scores are computed TRANSPOSED, S^T = K Q^T, so that in the MFMA accumulator a lane holds one
// query row (column l%32 of S^T) and 16 of the 32 keys: the row maximum and row sum of the online
// softmax are then per-lane loops plus a single exchange with lane l^32, the running maximum, the
// running sum and the rescale factor are one scalar per lane, and P^T is already laid out as the
// B operand of O^T += V^T P^T.  V^T is gathered from the row-major V rows with
// ds_read_b64_tr_b16.
//
// Memory -> LDS.  The K and V rows of a step (ring of 3 slots issued two steps ahead; double
// buffered and one step ahead without a bias) and the bias slice of each wave (32 rows x 32 keys,
// ring of 4 wave-private slots, issued three steps ahead) arrive through direct global -> LDS copies that the compiler does not see; their
// completion is counted by hand (copies complete in issue order and every step issues the same
// number).  The bias is a pure HBM stream: only a queue this deep keeps enough bytes in flight.
#include <type_traits>

#include "fa_common.hpp"
#include "fa_params.hpp"

namespace fa {

// The K/V stream of a row-broadcast bias (kinds 6, 7) is tiled like that of ALiBi, in steps of 32
// keys: the bias values of a block need the registers that 64-key steps spend on a second block of
// scores.
constexpr int fwd_stream_kind(int bias) { return bias >= 5 ? 6 : bias; }

template <typename T, int D, int BIAS, bool CAUSAL>
__global__ __launch_bounds__(256, (StreamCfg<D, fwd_stream_kind(BIAS)>::MIN_BLOCKS)) void fa_fwd_kernel(const FwdParams p) {
    constexpr int TB = tile_kind(BIAS);  // kind of bias tile that is streamed (none for ALiBi)
    typedef StreamCfg<D, fwd_stream_kind(BIAS)> C;
    typedef Swz<D> SW;
    typedef typename VecOf<T>::v8 T8;
    typedef typename VecOf<T>::v4 T4;
    typedef typename BiasElem<tile_kind(BIAS)>::type E;
    constexpr int BM = C::BM, BK = C::BK, OS = C::OS, CPR = C::CPR;

    constexpr bool ROWB = BIAS >= 6;     // the same bias for every query row, kept as an fp32 row in LDS
    constexpr bool BOOLROW = BIAS == 7;  // ... a bool mask: the row holds 0 or the mask term, in log2 units

    __shared__ __align__(1024) unsigned char smem[C::LDS_BYTES + (ROWB ? kRowBiasKeys * 4 : 0)];
    const float* row_lds = reinterpret_cast<const float*>(smem + C::LDS_BYTES);

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int r = lane & 31, g = lane >> 5;

    int mt, bh;
    decode_block<CAUSAL>(blockIdx.x, p.n_mtiles * p.n_splits, p.B * p.H, mt, bh);
    // With the keys split between work-groups (never when causal) this one sees keys key0 ..
    // key0 + N - 1 as if they were all there are; only ALiBi needs to know better.
    const int split = mt % p.n_splits;
    mt /= p.n_splits;
    const int key0 = split * p.keys_per_split;
    if (CAUSAL) mt = p.n_mtiles - 1 - mt;  // longest rows first
    const int b = bh / p.H, h = bh % p.H;
    const int M = p.M;
    const int N = p.n_splits > 1 ? (p.N - key0 < p.keys_per_split ? p.N - key0 : p.keys_per_split) : p.N;
    const int m0 = mt * BM;
    const int mw = m0 + wave * 32;  // first query row of this wave
    const int my_m = mw + r;

    const T* qp = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.sq.b + (int64_t)h * p.sq.h;
    const T* kp = reinterpret_cast<const T*>(p.k) + (int64_t)b * p.sk.b + (int64_t)h * p.sk.h + (int64_t)key0 * p.sk.s;
    const T* vp = reinterpret_cast<const T*>(p.v) + (int64_t)b * p.sv.b + (int64_t)h * p.sv.h + (int64_t)key0 * p.sv.s;
    const E* bp = nullptr;
    if (TB != 0) bp = reinterpret_cast<const E*>(p.bias) + (int64_t)b * p.sbias.b + (int64_t)h * p.sbias.h + (int64_t)key0 * p.sbias.n;
    // ALiBi: the slope of this head and the position of this lane's query row on the key axis
    float neg_slope = 0.f, ratio = 0.f;
    if (BIAS == 5) {
        neg_slope = -reinterpret_cast<const float*>(p.bias)[h];
        ratio = (float)p.N / (float)p.M;
    }

    if (ROWB)
        stage_row_bias(reinterpret_cast<float*>(smem + C::LDS_BYTES), p.bias, p.row_bias_kind,
                       (int64_t)b * p.sbias.b + (int64_t)h * p.sbias.h + (int64_t)key0 * p.sbias.n, p.sbias.n, N, tid);

    // Q^T as B operand: column my_m, k = d
    T8 qreg[C::KSTEPS];
#pragma unroll
    for (int ks = 0; ks < C::KSTEPS; ks++) {
        i32x4 raw = {0, 0, 0, 0};
        if (my_m < M) raw = gld16(qp + (int64_t)my_m * p.sq.s + ks * 16 + 8 * g);
        qreg[ks] = as_vec<T8>(raw);
    }

    int n_steps = (N + BK - 1) / BK;
    if (CAUSAL) {
        int last = (m0 + BM - 1) / BK + 1;  // steps holding keys <= last row of this work-group
        n_steps = n_steps < last ? n_steps : last;
    }

    const float qk_scale = p.sm_scale * kLog2e;
    float m_i = -INFINITY, l_i = 0.f;
    f32x16 o_acc[C::DB];
#pragma unroll
    for (int db = 0; db < C::DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) o_acc[db][i] = 0.f;

    const unsigned rows_l = SW::rows_lane(lane), cols_l = SW::cols_lane(lane);
    KeyStream<T, D, fwd_stream_kind(BIAS)> ks_;
    ks_.init(smem, kp, vp, bp, p.sk.s, p.sv.s, p.sbias.m, p.sbias.n, M, N, mw, wave, lane);

    // One step of the K/V stream.  Interior steps (every key in range and visible to every row of
    // the work-group) run with STEP_MASKED = false: no range checks, no mask arithmetic.  BV: the
    // bias slices come by copy (rows that allow aligned 16-byte chunks), else element by element.
    // LEAN: the copies of the step need no clamps (KeyStream::issue_ahead_lean).
    auto kv_step = [&](int k, auto step_tag, auto bv_tag, auto lean_tag) {
        constexpr bool STEP_MASKED = decltype(step_tag)::value;
        constexpr bool BV = decltype(bv_tag)::value;
        constexpr bool LEAN = decltype(lean_tag)::value;
        auto issue_ahead = [&]() {
            if constexpr (LEAN) ks_.template issue_ahead_lean<BV>(k);
            else ks_.template issue_ahead<BV>(k);
        };
        const int n0 = k * BK;
        ks_.template begin_step<BV>(k);
        const unsigned k_rows = ks_.k_addr(k) + rows_l, v_cols = ks_.v_addr(k) + cols_l;  // operand reads by address
        const unsigned char* b_lds = ks_.b_lds(k);
        static_assert(TB == 0 || C::NH == 1, "a bias slot covers one 32-key block");
        // The step is consumed 32 keys at a time, each block with its own softmax step.  In interior
        // steps of more than one block all score products are issued up front: the MFMAs of the later
        // blocks then run while the vector pipeline works on the first.
        constexpr bool PRE = !STEP_MASKED && C::NH > 1;
        f32x16 s_pre[C::NH];
        if constexpr (PRE) {
#pragma unroll
            for (int nb = 0; nb < C::NH; nb++) {
#pragma unroll
                for (int i = 0; i < 16; i++) s_pre[nb][i] = 0.f;
#pragma unroll
                for (int ks = 0; ks < C::KSTEPS; ks++) {
                    T8 a = SW::template row8_at<T8>(k_rows, nb * 32, ks);
                    s_pre[nb] = mfma32(a, qreg[ks], s_pre[nb]);
                }
            }
            issue_ahead();  // in the shadow of the MFMAs just issued
        }
#pragma unroll
        for (int nb = 0; nb < C::NH; nb++) {
        const int nh = nb * 32;  // first key of this block inside the step
        __builtin_amdgcn_sched_barrier(0);  // keep the blocks apart
        // blocks entirely above this wave's diagonal or past the last key contribute nothing
        if (STEP_MASKED && ((CAUSAL && n0 + nh > mw + 31) || n0 + nh >= N)) {
            if (nb == 0) issue_ahead();  // every wave issues its copies in every step
            continue;
        }
        const bool need_mask = STEP_MASKED && ((n0 + nh + 32 > N) || (CAUSAL && n0 + nh + 31 > mw));

        // ---- S^T = K Q^T : s[i] is key n0 + nh + 8 (i/4) + 4 g + i%4, query my_m ----
        f32x16 s;
        if constexpr (PRE) {
            s = s_pre[nb];
        } else {
#pragma unroll
            for (int i = 0; i < 16; i++) s[i] = 0.f;
#pragma unroll
            for (int ks = 0; ks < C::KSTEPS; ks++) {
                T8 a = SW::template row8_at<T8>(k_rows, nh, ks);
                s = mfma32(a, qreg[ks], s);
            }
            if (nb == 0) issue_ahead();  // in the shadow of the MFMAs just issued
        }

        // ---- online softmax step.  `masked` steps (ragged edge, causal diagonal) and a
        // non-positive scale follow the reference's arithmetic term by term: scaled score,
        // plus additive -1e6 terms in log2 units, plus bias (flash_attention.py:39-53).  Interior
        // steps skip the mask terms and fold the scale into the exponent.
        // The running maximum m_i is only raised when a step exceeds it by more than 2^8: the
        // reference point of the exponentials is arbitrary (out = acc / l and LSE = m + log2 l
        // do not depend on it), so a stale one costs nothing but saves rescaling O every step.
        T8 pb[2];
        auto softmax_step = [&](auto masked_tag) {
            constexpr bool MASKED = decltype(masked_tag)::value;
            float mx = -INFINITY;
            const float mf = (float)my_m, nf0 = (float)(key0 + n0 + nh + 4 * g);  // ALiBi: row and first key as floats
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                const int nl = 8 * q4 + 4 * g;            // first of 4 consecutive keys
                float bv[4] = {0.f, 0.f, 0.f, 0.f};       // bias in natural units
                bool keep[4] = {true, true, true, true};
                if constexpr (BIAS == 1) {
                    unsigned int w = *reinterpret_cast<const unsigned int*>(b_lds + ks_.b_off(r, nl));
#pragma unroll
                    for (int e = 0; e < 4; e++) keep[e] = ((w >> (8 * e)) & 0xffu) != 0;
                } else if constexpr (BIAS == 2 || BIAS == 3) {
                    typedef typename VecOf<E>::v4 B4;
                    B4 hv = *reinterpret_cast<const B4*>(b_lds + ks_.b_off(r, nl));
#pragma unroll
                    for (int e = 0; e < 4; e++) bv[e] = (float)hv[e];
                } else if constexpr (BIAS == 4) {
                    f32x4 w = *reinterpret_cast<const f32x4*>(b_lds + ks_.b_off(r, nl));
#pragma unroll
                    for (int e = 0; e < 4; e++) bv[e] = w[e];
                } else if constexpr (BIAS == 5) {
#pragma unroll
                    for (int e = 0; e < 4; e++) bv[e] = alibi_bias(neg_slope, ratio, mf, nf0 + (float)(8 * q4 + e));
                } else if constexpr (ROWB) {
                    f32x4 w = *reinterpret_cast<const f32x4*>(row_lds + n0 + nh + nl);
#pragma unroll
                    for (int e = 0; e < 4; e++) bv[e] = w[e];
                }
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int i = q4 * 4 + e;
                    float x;
                    if constexpr (MASKED) {
                        x = __fmul_rn(s[i], qk_scale);
                        const int n = n0 + nh + nl + e;
                        float t = (n >= N) ? kMask : 0.f;
                        if (CAUSAL) t += (my_m < n) ? kMask : 0.f;
                        float add = 0.f;
                        if (BIAS == 1) add = keep[e] ? 0.f : kMask;
                        if (BOOLROW) add = bv[e];
                        if (BIAS >= 2 && !BOOLROW) add = __fmul_rn(bv[e], kLog2e);
                        if (BIAS != 0) add = (n >= N) ? kMask : add;  // out-of-range bias reads as masked
                        x = __fadd_rn(x, __fadd_rn(t, add));
                    } else if constexpr (BIAS == 0) {
                        x = s[i];                                    // raw score, scale folded below
                    } else if constexpr (BIAS == 1) {
                        x = keep[e] ? s[i] * qk_scale : s[i] * qk_scale + kMask;
                    } else if constexpr (BOOLROW) {
                        x = s[i] * qk_scale + bv[e];
                    } else {
                        x = s[i] * p.sm_scale + bv[e];               // natural units
                    }
                    s[i] = x;
                    mx = fmaxf(mx, x);
                }
            }
            // units of x: log2 (MASKED, bool bias), raw dot product (no bias), natural (float bias)
            constexpr bool RAW = !MASKED && BIAS == 0;
            constexpr bool NAT = !MASKED && BIAS >= 2 && !BOOLROW;
            const float to_log2 = RAW ? qk_scale : (NAT ? kLog2e : 1.f);
            mx = pair_max(mx) * to_log2;
            const bool raise = mx > m_i + 8.f;
            if (__builtin_amdgcn_ballot_w64(raise) != 0) {
                const float m_new = raise ? mx : m_i;
                const float alpha = fast_exp2(m_i - m_new);
                m_i = m_new;
                l_i *= alpha;
#pragma unroll
                for (int db = 0; db < C::DB; db++)
#pragma unroll
                    for (int i = 0; i < 16; i++) o_acc[db][i] *= alpha;
            }
            // ---- P and O^T += V^T P^T (A = V^T gathered down the columns of the V rows), 16 keys
            // at a time: the MFMAs of the first 16 keys run while the exponentials of the second 16
            // are computed ----
            float rs = 0.f;
#pragma unroll
            for (int kk = 0; kk < 2; kk++) {
#pragma unroll
                for (int i = kk * 8; i < kk * 8 + 8; i++) {
                    float pv;
                    if constexpr (RAW || NAT) pv = fast_exp2(__builtin_fmaf(s[i], to_log2, -m_i));
                    else pv = fast_exp2(s[i] - m_i);
                    rs += pv;
                    pb[kk][i & 7] = (T)pv;
                }
#pragma unroll
                for (int db = 0; db < C::DB; db++) {
                    T8 a = SW::template col8_at<T8>(v_cols, nh + kk * 16, db);
                    o_acc[db] = mfma32(a, pb[kk], o_acc[db]);
                }
            }
            l_i += rs;  // per-lane partial sum; the two halves of a row are added at the end
        };
        if constexpr (STEP_MASKED && D > 128) {
            // (head dim 256: one form of the softmax step in the edge loop; a second copy of the
            // 32 matrix products of a block there costs the registers that the interior loops need)
            softmax_step(std::true_type{});
        } else if constexpr (STEP_MASKED) {
            if (need_mask || !(qk_scale > 0.f)) softmax_step(std::true_type{});
            else softmax_step(std::false_type{});
        } else {
            softmax_step(std::false_type{});
        }
        }
    };

    int n_fast = N / BK;  // leading steps that need no masks
    if (CAUSAL) n_fast = n_fast < (m0 + 1) / BK ? n_fast : (m0 + 1) / BK;
    if (n_fast > n_steps) n_fast = n_steps;
    if (!(qk_scale > 0.f)) n_fast = 0;

    auto run = [&](auto bv_tag) {
        constexpr bool BV = decltype(bv_tag)::value;
        // The loads of this lane's rows issued above are the compiler's own.  Left in flight, they would
        // make it wait for "all vector-memory operations" at their first use inside EVERY step of the
        // loops (it cannot know that they land once), and that wait drains the queue of copies issued
        // steps ahead.  Waiting for them here, before the first copy, keeps the loops free of it.
        wait_vmcnt<0>();
        ks_.template prologue<BV>();
        // the leading fast steps whose copies stay inside the tensors issue them without clamps
        const int n_lean = (BV || TB == 0) ? ks_.lean_steps(n_fast, m0 + BM) : 0;
        int k = 0;
        if (n_lean > 0) {
            ks_.run_start(C::LA, C::NBS - 1);
#pragma unroll 1
            for (; k < n_lean; k++) kv_step(k, std::false_type{}, bv_tag, std::true_type{});
        }
#pragma unroll 1
        for (; k < n_fast; k++) kv_step(k, std::false_type{}, bv_tag, std::false_type{});
#pragma unroll 1
        for (; k < n_steps; k++) kv_step(k, std::true_type{}, bv_tag, std::false_type{});
    };
    if (TB != 0 && p.bias_vec) run(std::true_type{});
    else run(std::false_type{});

    // ---- epilogue (flash_attention.py:188-194) ----
    const float l_tot = pair_sum(l_i);
    const float inv_l = 1.f / l_tot;
    // one of several shares of the keys: output and LSE go to this share's slice of the scratch
    const bool shared = p.n_splits > 1;
    float* lse_out = shared ? p.part_lse + ((int64_t)split * p.B * p.H + bh) * M : p.lse + ((int64_t)b * p.H + h) * M;
    // (the row index passes through an empty asm so that the store address is formed here and not
    // kept in two registers across the loops)
    int my_m_late = my_m;
    asm volatile("" : "+v"(my_m_late));
    if (g == 0 && my_m_late < M) lse_out[my_m_late] = m_i + fast_log2(l_tot);

    ks_.drain();  // K/V slots are dead and no copy is in flight: reuse their LDS for the output tile
    if (shared) {
        // a share stays in fp32 (the merge rounds once, like an unsplit run): 16 bytes per lane straight
        // from the accumulators (only problems with few query tiles come here)
        float* pf = reinterpret_cast<float*>(p.part_o) + (((int64_t)split * p.B * p.H + bh) * M + my_m_late) * D;
        if (my_m_late < M) {
#pragma unroll
            for (int db = 0; db < C::DB; db++) {
#pragma unroll
                for (int q4 = 0; q4 < 4; q4++) {
                    const int d = db * 32 + 8 * q4 + 4 * g;
                    if (d < D) {
                        f32x4 w;
#pragma unroll
                        for (int e = 0; e < 4; e++) w[e] = o_acc[db][q4 * 4 + e] * inv_l;
                        *reinterpret_cast<f32x4*>(pf + d) = w;
                    }
                }
            }
        }
        return;
    }
    T* o_lds = reinterpret_cast<T*>(smem) + wave * 32 * OS;
#pragma unroll
    for (int db = 0; db < C::DB; db++) {
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
            T4 pk;
#pragma unroll
            for (int e = 0; e < 4; e++) pk[e] = (T)(o_acc[db][q4 * 4 + e] * inv_l);
            *reinterpret_cast<T4*>(o_lds + r * OS + db * 32 + 8 * q4 + 4 * g) = pk;
        }
    }
    __syncthreads();
    T* op = reinterpret_cast<T*>(p.o) + (int64_t)b * p.so.b + (int64_t)h * p.so.h;
    for (int c = lane; c < 32 * CPR; c += 64) {
        int row = c / CPR, ch = c % CPR;
        if (mw + row < M) gst16(op + (int64_t)(mw + row) * p.so.s + ch * 8, lds_read16(o_lds + row * OS + ch * 8));
    }
}

// out = sum over the shares of 2^(lse_s - lse) out_s with lse = log2 sum 2^lse_s: the softmax over
// all keys from the softmaxes over the shares.  One thread per 8 head-dim elements of a row.
template <typename T, int D> __global__ __launch_bounds__(256) void fa_fwd_merge_kernel(const FwdParams p) {
    typedef typename VecOf<T>::v8 T8;
    constexpr int TPR = D / 8;
    const int64_t rows = (int64_t)p.B * p.H * p.M;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t row = idx / TPR;
    const int c = (int)(idx % TPR);
    if (row >= rows) return;
    float mx = -INFINITY;
    for (int s = 0; s < p.n_splits; s++) mx = fmaxf(mx, p.part_lse[s * rows + row]);
    float sum = 0.f;
    for (int s = 0; s < p.n_splits; s++) sum += fast_exp2(p.part_lse[s * rows + row] - mx);
    const float lse = mx + fast_log2(sum);
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < p.n_splits; s++) {
        const float w = fast_exp2(p.part_lse[s * rows + row] - lse);
        const float* src = reinterpret_cast<const float*>(p.part_o) + (s * rows + row) * D + c * 8;
        const f32x4 lo = *reinterpret_cast<const f32x4*>(src), hi = *reinterpret_cast<const f32x4*>(src + 4);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            acc[e] += w * lo[e];
            acc[4 + e] += w * hi[e];
        }
    }
    const int m = (int)(row % p.M);
    const int64_t bh = row / p.M;
    const int b = (int)(bh / p.H), h = (int)(bh % p.H);
    T8 o8;
#pragma unroll
    for (int e = 0; e < 8; e++) o8[e] = (T)acc[e];
    gst16(reinterpret_cast<T*>(p.o) + (int64_t)b * p.so.b + (int64_t)h * p.so.h + (int64_t)m * p.so.s + c * 8, as_raw(o8));
    if (c == 0) p.lse[row] = lse;
}

template <typename T, int D, int BIAS, bool CAUSAL> static hipError_t launch_one(const FwdParams& p, hipStream_t st) {
    dim3 grid((unsigned)(p.n_mtiles * p.n_splits * p.B * p.H));
    hipLaunchKernelGGL((fa_fwd_kernel<T, D, BIAS, CAUSAL>), grid, dim3(256), 0, st, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || p.n_splits == 1) return e;
    const int64_t threads = (int64_t)p.B * p.H * p.M * (D / 8);
    hipLaunchKernelGGL((fa_fwd_merge_kernel<T, D>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, p);
    return hipGetLastError();
}

template <typename T, int D> static hipError_t launch_bias(const FwdParams& p, int bias, bool causal, hipStream_t st) {
#define FA_CASE(BK)                                                        \
    case BK:                                                               \
        return causal ? launch_one<T, D, BK, true>(p, st) : launch_one<T, D, BK, false>(p, st);
    // a bias without a row dimension is staged once per work-group instead of streamed
    if (p.row_bias_kind != 0) bias = p.row_bias_kind == 1 ? 7 : 6;
    switch (bias) {
        FA_CASE(0)
        FA_CASE(1)
        FA_CASE(2)
        FA_CASE(3)
        FA_CASE(4)
        FA_CASE(5)
        FA_CASE(6)
        FA_CASE(7)
    }
#undef FA_CASE
    return hipErrorInvalidValue;
}

// This file is compiled once per head dimension (-DFA_HEAD_DIM=16 ... 256); each object exports
// launch_fwd_d<FA_HEAD_DIM>.  dtype: 0 = fp16, 1 = bf16.  The caller has validated every argument.
#ifndef FA_HEAD_DIM
#error "compile with -DFA_HEAD_DIM=<16|32|64|128|256>"
#endif
template <int D> hipError_t launch_fwd_d(const FwdParams& p, int dtype, int bias, bool causal, hipStream_t st);
template <> hipError_t launch_fwd_d<FA_HEAD_DIM>(const FwdParams& p, int dtype, int bias, bool causal, hipStream_t st) {
    if (dtype == 0) return launch_bias<_Float16, FA_HEAD_DIM>(p, bias, causal, st);
    return launch_bias<__bf16, FA_HEAD_DIM>(p, bias, causal, st);
}

}  // namespace fa
