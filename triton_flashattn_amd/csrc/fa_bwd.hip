// Backward attention kernels for gfx950: dK, dV, dBias in one kernel over key tiles, dQ in a
// second kernel over query tiles.  Every output element has exactly one writer, so results are
// reproducible run to run, like the reference's (no atomics).
//
// Replaces _attn_bwd_preprocess, _attn_bwd_dkdv and _attn_bwd_dq of the reference
// (/root/reference/flash_attention.py:197-646) and the host-side K / bias pre-scales
// (flash_attention.py:699-704), which become fp32 multiplies inside the kernels.
//
//   fa_bwd_prep_kernel   delta[b,h,m] = sum_d o * do                  (flash_attention.py:215-227)
//   fa_bwd_kernel        dK, dV, dBias of 128 keys per work-group     (flash_attention.py:237-454)
//   fa_bwd_dq_kernel     dQ of 128 query rows per work-group          (flash_attention.py:458-646)
#include <type_traits>

#include "fa_common.hpp"
#include "fa_params.hpp"

namespace fa {

// ---------------------------------------------------------------------------------------------
// delta of one row: every 16-byte chunk c of the row is summed element by element with fused
// multiply-adds, then the D / 8 chunk sums are added pairwise, c with c ^ w for w = D / 16, ..., 2, 1.
// (fa_bwd_dq_kernel forms the same sums in the same order when it stands in for this kernel.)
template <typename T, int D>
__global__ __launch_bounds__(256) void fa_bwd_prep_kernel(const BwdParams p) {
    constexpr int LPR = D / 8;         // lanes per row (16 bytes each)
    constexpr int RPB = 256 / LPR;     // rows per block
    typedef typename VecOf<T>::v8 T8;
    const int64_t rows = (int64_t)p.B * p.H * p.M;
    const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / LPR;
    const int c = threadIdx.x % LPR;
    float acc = 0.f;
    if (row < rows) {
        const int m = (int)(row % p.M);
        const int bh = (int)(row / p.M);
        const int b = bh / p.H, h = bh % p.H;
        const T* op = reinterpret_cast<const T*>(p.o) + (int64_t)b * p.so.b + (int64_t)m * p.so.s + (int64_t)h * p.so.h;
        const T* dp = reinterpret_cast<const T*>(p.dout) + (int64_t)b * p.sdo.b + (int64_t)m * p.sdo.s + (int64_t)h * p.sdo.h;
        T8 ov = as_vec<T8>(gld16(op + c * 8));
        T8 dv = as_vec<T8>(gld16(dp + c * 8));
#pragma unroll
        for (int e = 0; e < 8; e++) acc = __builtin_fmaf((float)ov[e], (float)dv[e], acc);
    }
#pragma unroll
    for (int w = LPR / 2; w >= 1; w >>= 1) acc += __shfl_xor(acc, w, 64);
    if (row < rows && c == 0) p.delta[row] = acc;
}

// ---------------------------------------------------------------------------------------------
// dQ kernel: a work-group owns 128 query rows (Q^T and dO^T in registers), streams K / V rows
// and recomputes S^T = K Q^T and dP^T = V dO^T, so that dS^T sits in the accumulator layout that
// dQ^T += K^T dS^T wants as its B operand.  K, V and the bias slices arrive through the same
// counted direct-to-LDS copy rings as in the forward kernel.  Replaces _attn_bwd_dq
// (flash_attention.py:458-646).
//
// FROM_DS: when the key-tile kernel has just written dBias in the element type of q, that tensor IS
// dS rounded exactly as the reference rounds it before this product (flash_attention.py:516-520);
// an fp32 dBias is dS itself and is rounded here.  The kernel then reads the dBias slices through
// the bias ring instead of the bias, skips both recomputed products, the exponentials and the V
// rows, and is one product instead of three.
template <typename T, int D, int BIAS, bool CAUSAL, bool FROM_DS = false>
__global__ __launch_bounds__(256, (StreamCfg<D, stream_kind(BIAS)>::MIN_BLOCKS)) void fa_bwd_dq_kernel(const BwdParams p) {
    static_assert(!FROM_DS || BIAS == 4 || (BIAS == 2 && __is_same(T, _Float16)) || (BIAS == 3 && __is_same(T, __bf16)),
                  "dS can stand in for the recomputation only in fp32 or in the element type of q");
    constexpr int TB = tile_kind(BIAS);  // kind of bias tile that is streamed (none for ALiBi)
    typedef StreamCfg<D, stream_kind(BIAS)> C;
    typedef Swz<D> SW;
    typedef typename VecOf<T>::v8 T8;
    typedef typename VecOf<T>::v4 T4;
    typedef typename BiasElem<tile_kind(BIAS)>::type E;
    constexpr int BM = C::BM, BK = C::BK, OS = C::OS, CPR = C::CPR;
    constexpr bool ROWB = BIAS >= 6;     // the same bias for every query row, kept as an fp32 row in LDS
    constexpr bool BOOLROW = BIAS == 7;  // ... a bool mask: the row holds 0 or the mask term, in log2 units
    static_assert(!(FROM_DS && ROWB), "a row-broadcast bias has no dense dS");

    __shared__ __align__(1024) unsigned char smem[C::LDS_BYTES + (ROWB ? kRowBiasKeys * 4 : 0)];
    const float* row_lds = reinterpret_cast<const float*>(smem + C::LDS_BYTES);

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int r = lane & 31, g = lane >> 5;

    int mt, bh;
    decode_block<CAUSAL>(blockIdx.x, p.n_mtiles * p.dq_splits, p.B * p.H, mt, bh);
    // With the keys split between work-groups (never when causal) this one sees keys key0 ..
    // key0 + N - 1 as if they were all there are (its dq is a share, summed afterwards); only ALiBi
    // needs to know better.
    const int split = mt % p.dq_splits;
    mt /= p.dq_splits;
    const int key0 = split * p.dq_keys_per_split;
    if (CAUSAL) mt = p.n_mtiles - 1 - mt;  // longest rows first
    const int b = bh / p.H, h = bh % p.H;
    const int M = p.M;
    const int N = p.dq_splits > 1 ? (p.N - key0 < p.dq_keys_per_split ? p.N - key0 : p.dq_keys_per_split) : p.N;
    const int m0 = mt * BM;
    const int mw = m0 + wave * 32;  // first query row of this wave
    const int my_m = mw + r;

    const T* qp = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.sq.b + (int64_t)h * p.sq.h;
    const T* kp = reinterpret_cast<const T*>(p.k) + (int64_t)b * p.sk.b + (int64_t)h * p.sk.h + (int64_t)key0 * p.sk.s;
    const T* vp = reinterpret_cast<const T*>(p.v) + (int64_t)b * p.sv.b + (int64_t)h * p.sv.h + (int64_t)key0 * p.sv.s;
    const E* bp = nullptr;
    if (TB != 0) bp = reinterpret_cast<const E*>(p.bias) + (int64_t)b * p.sbias.b + (int64_t)h * p.sbias.h + (int64_t)key0 * p.sbias.n;
    float neg_slope = 0.f, ratio = 0.f;  // ALiBi: slope of this head, key positions per query row
    if (BIAS == 5) {
        neg_slope = -reinterpret_cast<const float*>(p.bias)[h];
        ratio = (float)p.N / (float)p.M;
    }
    if (FROM_DS) bp = reinterpret_cast<const E*>(p.dbias) + (int64_t)b * p.sdbias.b + (int64_t)h * p.sdbias.h + (int64_t)key0 * p.sdbias.n;

    if (ROWB)
        stage_row_bias(reinterpret_cast<float*>(smem + C::LDS_BYTES), p.bias, p.row_bias_kind,
                       (int64_t)b * p.sbias.b + (int64_t)h * p.sbias.h + (int64_t)key0 * p.sbias.n, p.sbias.n, N, tid);

    // Q^T and dO^T as B operands: column my_m, k = d
    const T* dop = reinterpret_cast<const T*>(p.dout) + (int64_t)b * p.sdo.b + (int64_t)h * p.sdo.h;
    T8 qreg[C::KSTEPS], doreg[C::KSTEPS];
#pragma unroll
    for (int ks = 0; ks < C::KSTEPS; ks++) {
        i32x4 rq = {0, 0, 0, 0}, rd = {0, 0, 0, 0};
        if (!FROM_DS && my_m < M) {
            rq = gld16(qp + (int64_t)my_m * p.sq.s + ks * 16 + 8 * g);
            rd = gld16(dop + (int64_t)my_m * p.sdo.s + ks * 16 + 8 * g);
        }
        qreg[ks] = as_vec<T8>(rq);
        doreg[ks] = as_vec<T8>(rd);
    }
    // LSE (log2 units) and delta of this lane's query row
    float lse_i = 0.f, delta_i = 0.f;
    if (!FROM_DS && my_m < M) {
        lse_i = p.lse[((int64_t)b * p.H + h) * M + my_m];
        if (!p.dq_makes_delta) delta_i = p.delta[((int64_t)b * p.H + h) * M + my_m];
    }
    if (!FROM_DS && p.dq_makes_delta) {
        // This kernel runs first and forms delta = sum_d o * do itself (flash_attention.py:215-227), in the
        // order of fa_bwd_prep_kernel: this lane holds the chunks 2 ks + g of its row (dO^T above), sums
        // each with fused multiply-adds, adds chunk c to chunk c ^ w for w = D / 16, ..., 2 (both in this
        // lane) and last to chunk c ^ 1 (in the lane of the other g).  The dK/dV kernel reads what is stored.
        const T* op = reinterpret_cast<const T*>(p.o) + (int64_t)b * p.so.b + (int64_t)h * p.so.h;
        float part[C::KSTEPS];
#pragma unroll
        for (int ks = 0; ks < C::KSTEPS; ks++) {
            i32x4 ro = {0, 0, 0, 0};
            if (my_m < M) ro = gld16(op + (int64_t)my_m * p.so.s + ks * 16 + 8 * g);
            const T8 ov = as_vec<T8>(ro);
            float a = 0.f;
#pragma unroll
            for (int e = 0; e < 8; e++) a = __builtin_fmaf((float)ov[e], (float)doreg[ks][e], a);
            part[ks] = a;
        }
#pragma unroll
        for (int hs = C::KSTEPS / 2; hs >= 1; hs >>= 1)
#pragma unroll
            for (int ks = 0; ks < hs; ks++) part[ks] = part[ks] + part[ks + hs];
        delta_i = part[0] + __shfl_xor(part[0], 32, 64);
        if (g == 0 && my_m < M && split == 0) p.delta[((int64_t)b * p.H + h) * M + my_m] = delta_i;
    }

    int n_steps = (N + BK - 1) / BK;
    if (CAUSAL) {
        int last = (m0 + BM - 1) / BK + 1;  // steps holding keys <= last row of this work-group
        n_steps = n_steps < last ? n_steps : last;
    }

    const float qk_scale = p.sm_scale * kLog2e;
    // bool mask, unmasked steps: the two values that the offset of a score's exponent can take (the lane
    // is one query row), so that an element costs a select and not a select and a subtraction
    const float neg_lse = 0.f - lse_i, mask_lse = kMask - lse_i;
    f32x16 dq_acc[C::DB];  // dQ^T: rows = head dim, column = my_m
#pragma unroll
    for (int db = 0; db < C::DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) dq_acc[db][i] = 0.f;

    const unsigned rows_l = SW::rows_lane(lane), cols_l = SW::cols_lane(lane);
    KeyStream<T, D, stream_kind(BIAS), !FROM_DS> ks_;
    ks_.init(smem, kp, vp, bp, p.sk.s, p.sv.s, FROM_DS ? p.sdbias.m : p.sbias.m, FROM_DS ? p.sdbias.n : p.sbias.n, M, N,
             mw, wave, lane);

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
        const unsigned k_tile = ks_.k_addr(k), v_tile = ks_.v_addr(k);  // operand reads by address
        const unsigned char* b_lds = ks_.b_lds(k);
        static_assert(TB == 0 || C::NH == 1, "a bias slot covers one 32-key block");
        // The step is consumed 32 keys at a time, so that only one 32 x 32 score block is live.
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
            T8 dsb[2];
            if constexpr (FROM_DS) {
                // dS^T of the block straight from the dBias slice: 4 consecutive keys per read, in
                // accumulator order; keys past N hold whatever column 0 holds and count as zero
#pragma unroll
                for (int q4 = 0; q4 < 4; q4++) {
                    const int nl = 8 * q4 + 4 * g;
                    T4 hv;
                    if constexpr (BIAS == 4) {
                        const f32x4 w = *reinterpret_cast<const f32x4*>(b_lds + ks_.b_off(r, nl));
#pragma unroll
                        for (int e = 0; e < 4; e++) hv[e] = (T)w[e];
                    } else {
                        hv = *reinterpret_cast<const T4*>(b_lds + ks_.b_off(r, nl));
                    }
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int i = q4 * 4 + e;
                        T val = hv[e];
                        if (STEP_MASKED && n0 + nh + nl + e >= N) val = (T)0.f;
                        dsb[i >> 3][i & 7] = val;
                    }
                }
            } else {

            // ---- S^T = K Q^T : s[i] is key n0 + nh + 8 (i/4) + 4 g + i%4, query my_m ----
            f32x16 s;
#pragma unroll
            for (int i = 0; i < 16; i++) s[i] = 0.f;
#pragma unroll
            for (int ks = 0; ks < C::KSTEPS; ks++) {
                T8 a = SW::template row8_at<T8>(k_tile + rows_l, nh, ks);
                s = mfma32(a, qreg[ks], s);
            }

            // ---- dP^T = V dO^T ----
            f32x16 dp;
#pragma unroll
            for (int i = 0; i < 16; i++) dp[i] = 0.f;
#pragma unroll
            for (int ks = 0; ks < C::KSTEPS; ks++) {
                T8 a = SW::template row8_at<T8>(v_tile + rows_l, nh, ks);
                dp = mfma32(a, doreg[ks], dp);
            }
            if (nb == 0) issue_ahead();  // in the shadow of the MFMAs just issued

            // ---- P = 2^(S*scale + bias - LSE), dS = P (dP - delta) (flash_attention.py:497-517).
            // Masked tiles follow the reference's additive -1e6 arithmetic term by term.
            auto ds_step = [&](auto masked_tag) {
                constexpr bool MASKED = decltype(masked_tag)::value;
#pragma unroll
                for (int q4 = 0; q4 < 4; q4++) {
                    const int nl = 8 * q4 + 4 * g;  // first of 4 consecutive keys of the block
                    float bv[4] = {0.f, 0.f, 0.f, 0.f};  // bias in natural units
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
                        for (int e = 0; e < 4; e++)
                            bv[e] = alibi_bias(neg_slope, ratio, (float)my_m, (float)(key0 + n0 + nh + 4 * g) + (float)(8 * q4 + e));
                    } else if constexpr (ROWB) {
                        f32x4 w = *reinterpret_cast<const f32x4*>(row_lds + n0 + nh + nl);
#pragma unroll
                        for (int e = 0; e < 4; e++) bv[e] = w[e];
                    }
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int i = q4 * 4 + e;
                        float pv;
                        if constexpr (MASKED) {
                            float x = __fmul_rn(s[i], qk_scale);
                            const int n = n0 + nh + nl + e;
                            const bool oob = (n >= N) || (my_m >= M);
                            float t = oob ? kMask : 0.f;
                            if (CAUSAL) t += (my_m < n) ? kMask : 0.f;
                            float add = 0.f;
                            if (BIAS == 1) add = keep[e] ? 0.f : kMask;
                            if (BOOLROW) add = bv[e];
                            if (BIAS >= 2 && !BOOLROW) add = __fmul_rn(bv[e], kLog2e);
                            if (BIAS != 0) add = oob ? kMask : add;  // out-of-range bias reads as masked
                            x = __fadd_rn(x, __fadd_rn(t, add));
                            pv = fast_exp2(x - lse_i);
                        } else if constexpr (BIAS == 0) {
                            pv = fast_exp2(__builtin_fmaf(s[i], qk_scale, -lse_i));
                        } else if constexpr (BIAS == 1) {
                            pv = fast_exp2(__builtin_fmaf(s[i], qk_scale, keep[e] ? neg_lse : mask_lse));
                        } else if constexpr (BOOLROW) {
                            pv = fast_exp2(__builtin_fmaf(s[i], qk_scale, bv[e] - lse_i));
                        } else {
                            pv = fast_exp2(__builtin_fmaf(bv[e], kLog2e, __builtin_fmaf(s[i], qk_scale, -lse_i)));
                        }
                        dsb[i >> 3][i & 7] = (T)(pv * (dp[i] - delta_i));
                    }
                }
            };
            if constexpr (STEP_MASKED) {
                if (need_mask || m0 + BM > M) ds_step(std::true_type{});
                else ds_step(std::false_type{});
            } else {
                ds_step(std::false_type{});
            }
            }

            // ---- dQ^T += K^T dS^T : A = K^T gathered down the columns of the K tile ----
#pragma unroll
            for (int kk = 0; kk < 2; kk++) {
#pragma unroll
                for (int db = 0; db < C::DB; db++) {
                    T8 a = SW::template col8_at<T8>(k_tile + cols_l, nh + kk * 16, db);
                    dq_acc[db] = mfma32(a, dsb[kk], dq_acc[db]);
                }
            }
            if (FROM_DS && nb == 0) issue_ahead();  // in the shadow of the MFMAs just issued
        }
    };

    int n_fast = N / BK;  // leading steps that need no masks
    if (CAUSAL) n_fast = n_fast < (m0 + 1) / BK ? n_fast : (m0 + 1) / BK;
    if (n_fast > n_steps) n_fast = n_steps;
    if (!(qk_scale > 0.f) || m0 + BM > M) n_fast = 0;
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
    if (FROM_DS || (TB != 0 && p.bias_vec)) run(std::true_type{});
    else run(std::false_type{});

    // ---- epilogue: dq = dQ * sm_scale (flash_attention.py:644-646) ----
    ks_.drain();  // K/V slots are dead and no copy is in flight: reuse their LDS for the output tile
    if (p.dq_splits > 1) {
        // one of several shares of the keys: into this share's slice of the scratch, in fp32 (the sum
        // rounds once, like an unsplit run), 16 bytes per lane straight from the accumulators
        float* pf = reinterpret_cast<float*>(p.part_dq) + (((int64_t)split * p.B * p.H + bh) * M + my_m) * D;
        if (my_m < M) {
#pragma unroll
            for (int db = 0; db < C::DB; db++) {
#pragma unroll
                for (int q4 = 0; q4 < 4; q4++) {
                    const int d = db * 32 + 8 * q4 + 4 * g;
                    if (d < D) {
                        f32x4 w;
#pragma unroll
                        for (int e = 0; e < 4; e++) w[e] = dq_acc[db][q4 * 4 + e] * p.sm_scale;
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
            for (int e = 0; e < 4; e++) pk[e] = (T)(dq_acc[db][q4 * 4 + e] * p.sm_scale);
            *reinterpret_cast<T4*>(o_lds + r * OS + db * 32 + 8 * q4 + 4 * g) = pk;
        }
    }
    __syncthreads();
    T* op = reinterpret_cast<T*>(p.dq) + (int64_t)b * p.sdq.b + (int64_t)h * p.sdq.h;
    for (int c = lane; c < 32 * CPR; c += 64) {
        int row = c / CPR, ch = c % CPR;
        if (mw + row < M) gst16(op + (int64_t)(mw + row) * p.sdq.s + ch * 8, lds_read16(o_lds + row * OS + ch * 8));
    }
}

// dq = sum of the shares that the work-groups of a split dQ kernel left in part_dq, added in fp32 in
// a fixed order.  One thread per 8 head-dim elements of a row.
template <typename T, int D> __global__ __launch_bounds__(256) void fa_bwd_dq_sum_kernel(const BwdParams p) {
    typedef typename VecOf<T>::v8 T8;
    constexpr int TPR = D / 8;
    const int64_t rows = (int64_t)p.B * p.H * p.M;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t row = idx / TPR;
    const int c = (int)(idx % TPR);
    if (row >= rows) return;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < p.dq_splits; s++) {
        const float* src = reinterpret_cast<const float*>(p.part_dq) + (s * rows + row) * D + c * 8;
        const f32x4 lo = *reinterpret_cast<const f32x4*>(src), hi = *reinterpret_cast<const f32x4*>(src + 4);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            acc[e] += lo[e];
            acc[4 + e] += hi[e];
        }
    }
    const int m = (int)(row % p.M);
    const int64_t bh = row / p.M;
    const int b = (int)(bh / p.H), h = (int)(bh % p.H);
    T8 o8;
#pragma unroll
    for (int e = 0; e < 8; e++) o8[e] = (T)acc[e];
    gst16(reinterpret_cast<T*>(p.dq) + (int64_t)b * p.sdq.b + (int64_t)h * p.sdq.h + (int64_t)m * p.sdq.s + c * 8, as_raw(o8));
}


// ---------------------------------------------------------------------------------------------
// The bias of 4 consecutive query rows at one key, as the dK/dV kernel reads it from a row-major
// slice (32 keys per row) in LDS; get(e) is the additive term of row e: natural units for a float
// bias, log2 units (0 or the mask value) for a bool mask.
template <int BIAS> struct BiasQuad;
template <> struct BiasQuad<0> {
    __device__ __forceinline__ void load(const unsigned char*, int, int, int) {}
    __device__ __forceinline__ float get(int) const { return 0.f; }
};
template <> struct BiasQuad<1> {
    unsigned char v[4];
    __device__ __forceinline__ void load(const unsigned char* slice, int row0, int key, int) {
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = slice[(row0 + e) * 32 + key];
    }
    __device__ __forceinline__ float get(int e) const { return v[e] ? 0.f : kMask; }
};
template <> struct BiasQuad<2> {
    i16x4 raw;  // 4 rows of one key column in one transposing read
    __device__ __forceinline__ void load(const unsigned char* slice, int row0, int, int lane) {
        raw = lds_read_tr4(reinterpret_cast<const _Float16*>(slice) + tr_offset(lane, row0, 0, 32));
    }
    __device__ __forceinline__ float get(int e) const { return (float)__builtin_bit_cast(f16x4, raw)[e]; }
};
template <> struct BiasQuad<3> {
    i16x4 raw;
    __device__ __forceinline__ void load(const unsigned char* slice, int row0, int, int lane) {
        raw = lds_read_tr4(reinterpret_cast<const __bf16*>(slice) + tr_offset(lane, row0, 0, 32));
    }
    __device__ __forceinline__ float get(int e) const { return (float)__builtin_bit_cast(bf16x4, raw)[e]; }
};
template <> struct BiasQuad<5> {  // ALiBi: nothing to read, the kernel computes the term from the indices
    __device__ __forceinline__ void load(const unsigned char*, int, int, int) {}
    __device__ __forceinline__ float get(int) const { return 0.f; }
};
template <> struct BiasQuad<6> : BiasQuad<5> {};  // row-broadcast bias: one value per key, held by the kernel
template <> struct BiasQuad<7> : BiasQuad<5> {};
template <> struct BiasQuad<4> {
    float v[4];
    __device__ __forceinline__ void load(const unsigned char* slice, int row0, int key, int) {
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = reinterpret_cast<const float*>(slice)[(row0 + e) * 32 + key];
    }
    __device__ __forceinline__ float get(int e) const { return v[e]; }
};

// ---------------------------------------------------------------------------------------------
// OCC2: two work-groups per CU (four waves per SIMD, 128 registers each, half of the LDS): the
// configuration of the small head dims without a bias tile (no bias, or one kept in a register per
// key), whose blocks are small enough.
constexpr bool bwd_occ2(int D, int bias) { return D <= 64 && (bias == 0 || bias == 6 || bias == 7); }
template <int D, int BIAS, bool OCC2 = false> struct BwdCfg {
    // waves per role: four pairs of waves on a 128-key tile, two on a 64-key tile for head dim 256,
    // where a wave needs the whole register file of its SIMD (128 accumulator registers and 64 of the
    // resident operand before anything streams)
    static constexpr int WPR = D > 128 ? 2 : 4;
    static constexpr int BN = 32 * WPR, NT = 128 * WPR;
    static constexpr int LDS_LIMIT = OCC2 ? 81920 : 163840;
    static constexpr int NSUB = (D <= 64 && BIAS == 0 && !OCC2) ? 2 : 1;  // 32-row sub-blocks of a query block
    static constexpr int BMI = 32 * NSUB;
    static constexpr int DP = D < 32 ? 32 : D;
    static constexpr int DB = DP / 32;
    static constexpr int KSTEPS = D / 16;
    static constexpr int CPR = D / 8;
    static constexpr int DSS = BMI + 4;                    // dS^T tile: elements between two keys
    static constexpr int ES = BIAS == 0 ? 0 : (BIAS == 1 ? 1 : (BIAS == 4 ? 4 : 2));
    static constexpr int EPC = ES > 0 ? 16 / ES : 8;       // bias elements per 16-byte chunk
    static constexpr int BCPR = 2 * ES;                    // 16-byte chunks per 32-key bias row
    static constexpr int BCH = (BMI * BCPR + 63) / 64;     // bias copies per S-wave per block
    static constexpr int Q_BYTES = BMI * D * 2;
    static constexpr int NQD = Q_BYTES / 1024;             // 1 KB copies per Q (or dO) block
    static constexpr int QD = NQD >= WPR ? NQD / WPR : 1;  // of which each wave of a role issues this many
    // Q, dO, LSE, delta and the bias slices reach LDS through direct global -> LDS copies issued
    // LA blocks ahead of their use (Q, LSE and bias by the S-waves, dO and delta by the dP-waves);
    // a copy has LA - 1 whole steps and the rest of its own to land before the barrier that
    // publishes it.
    static constexpr int DS_BYTES = (BIAS == 2 || BIAS == 3) ? BN * DSS * 2 : 0;  // dS^T tiles (dBias)
    // The LSE (delta) values of a block: a copy is 64 lanes wide, so a slot is 64 floats; with 32-row
    // blocks the upper lanes copy the same 32 values again (no lane mask, no branch around the copy).
    static constexpr int STAT_BYTES = 64 * 4;
    static constexpr int P_BYTES = 4 * NSUB * 64 * 16 * WPR;  // P hand-off: 16 floats per lane per sub-block
    static constexpr int BT_BYTES = BMI * 32 * ES;         // bias slice of one S-wave
    // LDS bytes with copies la blocks ahead: la + 1 dO buffers and bias slots, la + 2 Q buffers and
    // one more if the dK product of a block is deferred by a step (so that it does not wait for
    // the dS of the same step)
    static constexpr int lds_total(int la, int defer) {
        return (2 * la + 3 + defer) * (Q_BYTES + STAT_BYTES) + DS_BYTES + 2 * P_BYTES + WPR * (la + 1) * BT_BYTES;
    }
    static constexpr int LA = D > 128 ? 1 : (lds_total(3, 1) <= LDS_LIMIT ? 3 : 2);
    static constexpr bool DEFER_DK = D <= 128 && lds_total(LA, 1) <= LDS_LIMIT;
    static constexpr int NDOB = LA + 1;                    // dO (+delta) buffers
    static constexpr int RING = LA + 1;                    // bias slots per S-wave
    static constexpr int NQB = LA + 2 + (DEFER_DK ? 1 : 0);  // Q (+LSE) buffers
    static constexpr int OFF_DO = NQB * Q_BYTES;
    static constexpr int OFF_DS = OFF_DO + NDOB * Q_BYTES;
    static constexpr int OFF_P = OFF_DS + DS_BYTES;        // two hand-off buffers
    static constexpr int OFF_LSE = OFF_P + 2 * P_BYTES;
    static constexpr int OFF_DELTA = OFF_LSE + NQB * STAT_BYTES;
    static constexpr int OFF_BIAS = OFF_DELTA + NDOB * STAT_BYTES;
    static constexpr int LOOP_BYTES = OFF_BIAS + WPR * RING * BT_BYTES;
    static constexpr int LDS_BYTES = LOOP_BYTES;
    static_assert(LDS_BYTES <= LDS_LIMIT, "LDS budget of the configuration");
    static constexpr int WAVES_PER_SIMD = OCC2 ? 4 : (WPR == 2 ? 1 : 2);
};

// Work split inside a work-group of 8 waves.  Waves 0-3 ("S-waves") and waves 4-7 ("dP-waves")
// pair up on the four 32-key blocks of the tile (waves w and w + 4 run on the same SIMD; for head
// dim 256 a work-group is two such pairs on a 64-key tile, one wave per SIMD):
//   S-wave : S = Q K^T, P = 2^(S*scale + bias - LSE)  -> hands P to its partner through LDS,
//            dV^T += dO^T P, and the global -> LDS copies of the Q / LSE / bias blocks
//   dP-wave: dP = dO V^T, dS = P (dP - delta) (+ dBias through an LDS tile), dK^T += Q^T dS,
//            and the global -> LDS copies of the dO / delta blocks
// The roles are skewed by one query block so that a step needs a single barrier and nothing a
// wave does inside a step depends on what its partner does in the same step:
//   step t : S-wave : P(t+1) from Q(t+1), then dV += dO(t)^T P(t)        (P(t) kept in registers)
//            dP-wave: dS(t) from dO(t) and the P(t) handed over in step t-1, dK += Q(t-1)^T dS(t-1)
// While one wave of a SIMD runs exponentials or products the other issues MFMAs.
// DBIAS: 0 = the bias is not trainable; 1 = dBias is written densely, (B, H, M, N) in the bias dtype
// (flash_attention.py:307-308); 2 = reduced in the kernel: for a float bias the sums of dS over the
// query rows, one fp32 per (batch, head, key), for ALiBi the gradient of the slope, one fp32 per
// (batch, head, key tile, wave); a second small kernel sums those over the broadcast dimensions.
template <typename T, int D, int BIAS, bool CAUSAL, int DBIAS>
__global__ __launch_bounds__((BwdCfg<D, tile_kind(BIAS), bwd_occ2(D, BIAS)>::NT), (BwdCfg<D, tile_kind(BIAS), bwd_occ2(D, BIAS)>::WAVES_PER_SIMD)) void fa_bwd_kernel(const BwdParams p) {
    constexpr int TB = tile_kind(BIAS);  // kind of bias tile that is streamed (none for ALiBi)
    typedef BwdCfg<D, TB, bwd_occ2(D, BIAS)> C;
    typedef Swz<D> SW;
    typedef typename VecOf<T>::v8 T8;
    typedef typename VecOf<T>::v4 T4;
    typedef typename BiasElem<tile_kind(BIAS)>::type E;
    constexpr int BN = C::BN, BMI = C::BMI, CPR = C::CPR, DSS = C::DSS, NSUB = C::NSUB;
    // dBias leaves through the dS tile (16-byte row stores) when it has the element type of dS
    constexpr bool DB_VIA_LDS = DBIAS == 1 && ((BIAS == 2 && __is_same(T, _Float16)) || (BIAS == 3 && __is_same(T, __bf16)));
    // an fp32 dBias leaves through LDS too, as fp32: the dP-wave turns its part of the P hand-off buffer,
    // which it has just read and which is not written again before the next step, into a row-major
    // 32 x 32 tile (4-byte stores, one per element) and stores 16 bytes per lane from there
    constexpr bool DB_VIA_LDS32 = DBIAS == 1 && BIAS == 4 && BMI == 32;

    __shared__ __align__(16) unsigned char smem[C::LDS_BYTES];

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int r = lane & 31, g = lane >> 5;
    const bool s_wave = wave < C::WPR;  // role
    const int kb = __builtin_amdgcn_readfirstlane(wave % C::WPR);  // 32-key block of this wave (scalar)
    const unsigned lds_base = lds_addr_of(smem);

    int nt, bh;
    decode_block<CAUSAL>(blockIdx.x, p.n_ntiles, p.B * p.H, nt, bh);
    const int b = bh / p.H, h = bh % p.H;
    const int M = p.M, N = p.N;
    const int n0 = nt * BN;
    const int nw = n0 + kb * 32;
    const int my_n = nw + r;

    const T* qp = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.sq.b + (int64_t)h * p.sq.h;
    const T* kp = reinterpret_cast<const T*>(p.k) + (int64_t)b * p.sk.b + (int64_t)h * p.sk.h;
    const T* vp = reinterpret_cast<const T*>(p.v) + (int64_t)b * p.sv.b + (int64_t)h * p.sv.h;
    const T* dop = reinterpret_cast<const T*>(p.dout) + (int64_t)b * p.sdo.b + (int64_t)h * p.sdo.h;
    const float* lsep = p.lse + ((int64_t)b * p.H + h) * M;
    const float* deltap = p.delta + ((int64_t)b * p.H + h) * M;
    const E* bp = nullptr;
    E* dbp = nullptr;
    if (TB != 0) bp = reinterpret_cast<const E*>(p.bias) + (int64_t)b * p.sbias.b + (int64_t)h * p.sbias.h;
    if (DBIAS == 1) dbp = reinterpret_cast<E*>(p.dbias) + (int64_t)b * p.sdbias.b + (int64_t)h * p.sdbias.h;
    float neg_slope = 0.f, ratio = 0.f;  // ALiBi: slope of this head, key positions per query row
    if (BIAS == 5) {
        neg_slope = -reinterpret_cast<const float*>(p.bias)[h];
        ratio = (float)p.N / (float)p.M;
    }
    // row-broadcast bias: the term of this lane's key, natural units (6) or 0 / mask value in log2 units (7)
    float row_bv = 0.f;
    if (BIAS == 6 || BIAS == 7) {
        if (my_n < N) {
            const int64_t idx = (int64_t)b * p.sbias.b + (int64_t)h * p.sbias.h + (int64_t)my_n * p.sbias.n;
            switch (p.row_bias_kind) {
                case 1: row_bv = reinterpret_cast<const unsigned char*>(p.bias)[idx] ? 0.f : kMask; break;
                case 2: row_bv = (float)reinterpret_cast<const _Float16*>(p.bias)[idx]; break;
                case 3: row_bv = (float)reinterpret_cast<const __bf16*>(p.bias)[idx]; break;
                default: row_bv = reinterpret_cast<const float*>(p.bias)[idx]; break;
            }
        }
    }
    constexpr bool NATURAL = BIAS >= 2 && BIAS != 7;  // the bias term is in natural units (else log2 units)
    unsigned char* ring_lds = smem + C::OFF_BIAS + kb * C::RING * C::BT_BYTES;
    float* p_lds = reinterpret_cast<float*>(smem + C::OFF_P) + kb * NSUB * 64 * 16;  // + buffer * P_BYTES / 4

    // ---- this wave's 32 keys as B operand (column my_n, k = d): K for an S-wave, V for a dP-wave
    T8 opreg[C::KSTEPS];
    {
        const T* src = s_wave ? kp + (int64_t)my_n * p.sk.s : vp + (int64_t)my_n * p.sv.s;
#pragma unroll
        for (int ks = 0; ks < C::KSTEPS; ks++) {
            i32x4 v = {0, 0, 0, 0};
            if (my_n < N) v = gld16(src + ks * 16 + 8 * g);
            opreg[ks] = as_vec<T8>(v);
        }
    }

    // dV^T (S-wave) or dK^T (dP-wave) of this wave's 32 keys: rows = head dim, columns = keys
    f32x16 acc[C::DB];
#pragma unroll
    for (int db = 0; db < C::DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[db][i] = 0.f;

    const float qk_scale = p.sm_scale * kLog2e;
    const int n_mblocks = (M + BMI - 1) / BMI;
    // causal: query blocks that end above the first key of this tile see none of its keys
    const int mb_first = CAUSAL ? (n0 / BMI) : 0;
    const bool bias_vec = TB != 0 && p.bias_vec;
    const bool dbias_vec = DBIAS == 1 && p.dbias_vec;

    // blocks skipped by the causal schedule still owe zeros to dBias
    if (DBIAS == 1 && CAUSAL && !s_wave) {
        const int rows_skipped = mb_first * BMI < M ? mb_first * BMI : M;
        for (int c = lane; c < rows_skipped * C::BCPR; c += 64) {
            const int m = c / C::BCPR, nn = nw + (c % C::BCPR) * C::EPC;
            E* dst = dbp + (int64_t)m * p.sdbias.m + (int64_t)nn * p.sdbias.n;
            if (dbias_vec && nn + C::EPC <= N) {
                i32x4 z = {0, 0, 0, 0};
                gst16(dst, z);
            } else {
                for (int e = 0; e < C::EPC; e++)
                    if (nn + e < N) dst[(int64_t)e * p.sdbias.n] = (E)0.f;
            }
        }
    }

    // ---- global -> LDS copies of Q (+LSE), dO (+delta) and bias blocks ----
    // A block is NQD copies of 1 KB; copy ci fills bytes [1024 ci, 1024 ci + 1024) of the swizzled
    // tile, so lane l of it fetches the 16-byte chunk that lives at tile position 64 ci + l.  Each
    // wave of the issuing role issues QD of them (more than once where a block has fewer than four), every step the
    // same number: completion is counted (s_waitcnt vmcnt) and copies complete in issue order.
    // Rows past M re-read the last row: their P and dS are exactly zero.
    unsigned cq_off[C::QD], cdo_off[C::QD];
    int c_idx[C::QD];
#pragma unroll
    for (int i = 0; i < C::QD; i++) {
        c_idx[i] = (kb * C::QD + i) % C::NQD;
        const int c = c_idx[i] * 64 + lane;
        const int row = c / CPR, src = (c % CPR) ^ SW::f(row);
        cq_off[i] = (unsigned)(row * (int)p.sq.s * 2 + src * 16);
        cdo_off[i] = (unsigned)(row * (int)p.sdo.s * 2 + src * 16);
    }
    auto issue_rows = [&](const T* base, int64_t row_stride, const unsigned (&off)[C::QD], int mb, unsigned dst) {
        // a block past the end is the last row over and over: offsets never go negative
        const int m0 = mb * BMI < M ? mb * BMI : M - 1;
        const uint64_t blk = uniform_ptr(base + (int64_t)m0 * row_stride);
        const bool full = m0 + BMI <= M;
#pragma unroll
        for (int i = 0; i < C::QD; i++) {
            unsigned o = off[i];
            if (!full) {
                // (rare: the lane index passes through an empty asm so that these per-lane values are
                // formed here and not kept in registers across the loops)
                int lane_here = lane;
                asm volatile("" : "+v"(lane_here));
                const int c = c_idx[i] * 64 + lane_here;
                int row = c / CPR;
                const int src = (c % CPR) ^ SW::f(row);
                row = row < M - m0 ? row : M - 1 - m0;
                o = (unsigned)(row * (int)row_stride * 2 + src * 16);
            }
            lds_copy16(blk, o, dst + c_idx[i] * 1024);
        }
    };
    // one float per row
    auto issue_stat = [&](const float* src, int mb, unsigned dst) {
        int m = mb * BMI + lane % BMI;
        m = m < M ? m : M - 1;
        lds_copy4(uniform_ptr(src), (unsigned)m * 4u, dst);
    };
    // bias slice (BMI rows x 32 keys) of query block mb -> ring slot.  Chunk c = 64 it + lane of the
    // slice (row c / BCPR, 16-byte chunk c % BCPR) lands at byte 16 c of the slot, i.e. the slot
    // is the row-major slice.  Rows past M re-read row M - 1 and chunks that start past N re-read
    // column 0: both are masked where they are used.
    auto issue_bias = [&](int mb) {
        if constexpr (TB != 0) {
            const unsigned dst = lds_base + C::OFF_BIAS + (kb * C::RING + (mb - mb_first) % C::RING) * C::BT_BYTES;
            const uint64_t base = uniform_ptr(bp);
#pragma unroll
            for (int it = 0; it < C::BCH; it++) {
                const int c = it * 64 + lane;
                int m = mb * BMI + c / C::BCPR;
                int nn = nw + (c % C::BCPR) * C::EPC;
                m = m < M ? m : M - 1;
                nn = nn < N ? nn : 0;
                // a (batch, head) slice that takes this path is smaller than 2 GiB
                lds_copy16(base, (unsigned)(((int64_t)m * p.sbias.m + nn) * C::ES), dst + it * 1024);
            }
        }
    };
    // block mb of Q with its LSE (QD + 1 copies) / block mb of dO with its delta (QD + 1 copies);
    // all four waves of a role copy the 32 or 64 floats, which keeps their counts alike
    auto issue_q = [&](int mb) {
        issue_rows(qp, p.sq.s, cq_off, mb, lds_base + (mb % C::NQB) * C::Q_BYTES);
        issue_stat(lsep, mb, lds_base + C::OFF_LSE + (mb % C::NQB) * C::STAT_BYTES);
    };
    auto issue_do = [&](int mb) {
        issue_rows(dop, p.sdo.s, cdo_off, mb, lds_base + C::OFF_DO + (mb % C::NDOB) * C::Q_BYTES);
        issue_stat(deltap, mb, lds_base + C::OFF_DELTA + (mb % C::NDOB) * C::STAT_BYTES);
    };
    // Issuing a copy stalls the wave while the memory pipeline of the CU is backed up, so the
    // copies are dealt out between the roles: Q and the bias go with the S-waves, dO with the
    // dP-waves.
    constexpr bool Q_BY_S = true, DO_BY_S = false;
    static_assert(Q_BY_S && !DO_BY_S, "the running pointers of the interior steps are laid out for this deal");
    // Interior steps (every block they touch is whole, in range and unmasked: all but the first and
    // the last few of a tile) walk the query blocks in order, so their copies keep running block
    // pointers in scalar registers, one 64-bit add per block, and need no clamps; run_start() points
    // them at the first blocks an interior loop issues.
    // (The kernels that run two work-groups per CU have 128 registers per wave and no room for the
    // second copy of the loop: they run every step in its general form.  With their operand reads
    // left to the compiler they fit, and gain 2 % on the causal D = 64 shape: not worth a second form.)
    constexpr bool IN_LOOPS = !bwd_occ2(D, BIAS);
    const int n_full = M / BMI;  // blocks whose rows all exist
    uint64_t run_rows = 0, run_stat = 0, run_bias = 0;  // Q and LSE (role that issues Q) or dO and delta; bias slices
    unsigned bias_off0 = 0;  // this lane's byte offset in the first bias copy of a block, from the block's first row
    if constexpr (TB != 0) {
        int nn = nw + (lane % C::BCPR) * C::EPC;
        nn = nn < N ? nn : 0;
        bias_off0 = (unsigned)(((int64_t)(lane / C::BCPR) * p.sbias.m + nn) * C::ES);
    }
    auto run_start = [&](const T* rows, int64_t row_stride, const float* stat, int mb, int mb_bias) {
        run_rows = uniform_ptr(rows + (int64_t)mb * BMI * row_stride);
        run_stat = uniform_ptr(stat + (int64_t)mb * BMI);
        if constexpr (TB != 0) run_bias = uniform_ptr(bp + (int64_t)mb_bias * BMI * p.sbias.m);
    };
    // the next block of Q (or dO) with its LSE (or delta): QD + 1 copies, like issue_q / issue_do
    // (the caller has passed the running pointers through settle_ptrs() since they were last advanced)
    auto issue_next_rows = [&](int64_t row_stride, const unsigned (&off)[C::QD], unsigned dst, unsigned stat_dst) {
#pragma unroll
        for (int i = 0; i < C::QD; i++) lds_copy16(run_rows, off[i], dst + c_idx[i] * 1024);
        run_rows += (uint64_t)(BMI * 2) * (uint64_t)row_stride;
        // (the lane index passes through an empty asm so that the offset is formed here, two
        // instructions, and does not hold a register across the loop)
        unsigned lane_here = (unsigned)lane;
        asm volatile("" : "+v"(lane_here));
        lds_copy4(run_stat, (lane_here % BMI) * 4u, stat_dst);
        run_stat += BMI * 4;
    };
    auto issue_next_q = [&](int mb) {
        const unsigned slot = (unsigned)mb % C::NQB;
        issue_next_rows(p.sq.s, cq_off, lds_base + slot * C::Q_BYTES, lds_base + C::OFF_LSE + slot * C::STAT_BYTES);
    };
    auto issue_next_do = [&](int mb) {
        const unsigned slot = (unsigned)mb % C::NDOB;
        issue_next_rows(p.sdo.s, cdo_off, lds_base + C::OFF_DO + slot * C::Q_BYTES, lds_base + C::OFF_DELTA + slot * C::STAT_BYTES);
    };
    auto issue_next_bias = [&](int mb) {
        if constexpr (TB != 0) {
            const unsigned dst = lds_base + C::OFF_BIAS + (kb * C::RING + (unsigned)(mb - mb_first) % C::RING) * C::BT_BYTES;
            const unsigned rows_step = (unsigned)((64 / C::BCPR) * (int)p.sbias.m * C::ES);  // the rows one copy covers
#pragma unroll
            for (int it = 0; it < C::BCH; it++) lds_copy16(run_bias, bias_off0 + it * rows_step, dst + it * 1024);
            run_bias += (uint64_t)(BMI * C::ES) * (uint64_t)p.sbias.m;
        }
    };
    // per-element path for bias rows that cannot be copied in aligned 16-byte chunks
    auto load_bias_scalar = [&](int mb, unsigned char* dst) {
        if constexpr (TB != 0) {
            // all loads of a 32-row sub-block in flight together (clamped addresses instead of
            // branches; what lies outside the bias is masked where it is used)
            const int m0 = mb * BMI;
            const int nn = my_n < N ? my_n : N - 1;
#pragma unroll 1
            for (int sb = 0; sb < NSUB; sb++) {
                E vals[16];
#pragma unroll
                for (int j = 0; j < 16; j++) {
                    int m = m0 + sb * 32 + 2 * j + g;
                    m = m < M ? m : M - 1;
                    vals[j] = bp[(int64_t)m * p.sbias.m + (int64_t)nn * p.sbias.n];
                }
#pragma unroll
                for (int j = 0; j < 16; j++) reinterpret_cast<E*>(dst)[(sb * 32 + 2 * j + g) * 32 + r] = vals[j];
            }
        }
    };

    // ---- prologue: the first LA blocks of Q and LA - 1 blocks of dO ----
    {
        const unsigned saved_m0 = lds_copy_begin();
#pragma unroll 1
        for (int i = 0; i < C::LA; i++) {
            if (s_wave == Q_BY_S) issue_q(mb_first + i);
            if (s_wave && TB != 0 && bias_vec) issue_bias(mb_first + i);
            if (s_wave == DO_BY_S && i < C::LA - 1) issue_do(mb_first + i);
        }
        lds_copy_end(saved_m0);
    }
    wait_vmcnt<0>();
    __syncthreads();

    T8 op_cur[NSUB][2];  // P^T (S-wave) or dS^T (dP-wave) of the block whose accumulation is still due
#pragma unroll
    for (int sb = 0; sb < NSUB; sb++)
#pragma unroll
        for (int kk = 0; kk < 2; kk++) op_cur[sb][kk] = as_vec<T8>(i32x4{0, 0, 0, 0});

    // A wave issues its instructions in order and only two waves share a SIMD, so every LDS round
    // trip that sits between two dependent pieces of a step is dead time.  A step therefore
    // fetches what it needs from LDS into registers at its top (PRELOAD): the A operands of both
    // products and the inputs of the element-wise work, each ahead of work that hides the trip.
    // With D = 256 there is no register room for that and the compiler places the reads.
    constexpr bool PRELOAD = D <= 128;
    constexpr int NR = NSUB * C::KSTEPS;  // A operands of a row product: 32 rows x 16 of the head dim each
    constexpr int NA = NSUB * 2 * C::DB;  // A operands of a column product: 32 of the head dim x 16 rows each
    // tiles are named by their LDS byte address (scalar); the two per-lane address constants of
    // Swz cover every operand read of the loop
    const unsigned rows_l = SW::rows_lane(lane), cols_l = SW::cols_lane(lane);
    auto load_rows = [&](unsigned tile, T8 (&a)[NR]) {
        const unsigned base = tile + rows_l;
#pragma unroll
        for (int sb = 0; sb < NSUB; sb++)
#pragma unroll
            for (int ks = 0; ks < C::KSTEPS; ks++) a[sb * C::KSTEPS + ks] = SW::template row8_at<T8>(base, sb * 32, ks);
    };
    // sacc = rows(tile) x opreg: S = Q K^T (S-wave) or dP = dO V^T (dP-wave)
    auto mma_rows = [&](const T8 (&a)[NR], f32x16 (&sacc)[NSUB]) {
#pragma unroll
        for (int sb = 0; sb < NSUB; sb++) {
#pragma unroll
            for (int i = 0; i < 16; i++) sacc[sb][i] = 0.f;
#pragma unroll
            for (int ks = 0; ks < C::KSTEPS; ks++) sacc[sb] = mfma32(a[sb * C::KSTEPS + ks], opreg[ks], sacc[sb]);
        }
    };
    // the A operands of acc^T += tile^T op are columns of the tile, gathered with ds_read_b64_tr_b16
    auto load_cols = [&](unsigned tile, T8 (&a)[NA]) {
        const unsigned base = tile + cols_l;
#pragma unroll
        for (int sb = 0; sb < NSUB; sb++)
#pragma unroll
            for (int kk = 0; kk < 2; kk++)
#pragma unroll
                for (int db = 0; db < C::DB; db++)
                    a[(sb * 2 + kk) * C::DB + db] = SW::template col8_at<T8>(base, sb * 32 + kk * 16, db);
    };
    // acc^T += tile^T op: dV^T += dO^T P (S-wave) or dK^T += Q^T dS (dP-wave)
    auto mma_cols = [&](const T8 (&a)[NA], const T8 (&op)[NSUB][2]) {
#pragma unroll
        for (int sb = 0; sb < NSUB; sb++)
#pragma unroll
            for (int kk = 0; kk < 2; kk++)
#pragma unroll
                for (int db = 0; db < C::DB; db++) acc[db] = mfma32(a[(sb * 2 + kk) * C::DB + db], op[sb][kk], acc[db]);
    };
    // ring slots of a block index that may run one or two blocks below zero at the first steps
    auto q_tile = [&](int mb) { return lds_base + (unsigned)(((mb < 0 ? 0 : mb) % C::NQB) * C::Q_BYTES); };
    auto do_tile = [&](int mb) { return lds_base + (unsigned)(C::OFF_DO + ((mb < 0 ? 0 : mb) % C::NDOB) * C::Q_BYTES); };
    // the same for the interior steps, whose block indices are never negative
    auto q_tile_in = [&](int mb) { return lds_base + ((unsigned)mb % C::NQB) * C::Q_BYTES; };
    auto do_tile_in = [&](int mb) { return lds_base + C::OFF_DO + ((unsigned)mb % C::NDOB) * C::Q_BYTES; };

    if (s_wave) {
        // ================================ S-wave ================================
        auto s_loop = [&](auto bv_tag) {
        constexpr bool BV = decltype(bv_tag)::value;                    // bias slices come by copy
        constexpr int OPS = (BV ? C::BCH : 0) + ((Q_BY_S ? 1 : 0) + (DO_BY_S ? 1 : 0)) * (C::QD + 1);  // copies per step
        // S_AHEAD: the scores of a block are formed at the END of the step before the one that turns
        // them into P, so that a step of this role opens with vector work (exponentials) while the
        // partner wave on the same SIMD opens with matrix products, and closes with matrix products
        // while the partner does its vector work.  It needs the Q block one step earlier, i.e. a copy
        // look-ahead of at least three blocks.  Measured: 3 % on the kernel that writes dBias (whose
        // dP-wave has the most vector work), a loss of 5 % with a bias that is only read and of 4 %
        // without one, which keep the plain order.
        constexpr bool S_AHEAD = TB != 0 && C::LA >= 3 && DBIAS == 1;
        f32x16 sacc[NSUB];
        if constexpr (S_AHEAD) {
            T8 a_rows[NR];
            load_rows(q_tile(mb_first), a_rows);
            mma_rows(a_rows, sacc);
        }
        auto s_step = [&](int t, auto in_tag) {
            // IN: an interior step: blocks t .. t + 2 + LA are whole and in range, block t + 1 needs no mask
            constexpr bool IN = decltype(in_tag)::value;
            const int nb = t + 1;  // the block whose P is produced in this step
            T8 op_next[NSUB][2];
            // Copies for the steps to come (their buffers were last read one step ago).  With a bias
            // they are issued behind the LDS reads of the step, whose round trip they cover; without
            // one right after the barrier: measured, each way is a few per cent better in its case.
            auto issue_copies = [&]() {
                const unsigned saved_m0 = lds_copy_begin();
                if constexpr (IN) {
                    settle_ptrs(run_rows, run_stat, run_bias);
                    if constexpr (Q_BY_S) issue_next_q(nb + C::LA);
                    if constexpr (BV) issue_next_bias(nb + C::LA);
                    if constexpr (DO_BY_S) issue_next_do(t + C::LA);
                } else {
                    if constexpr (Q_BY_S) issue_q(nb + C::LA);
                    if constexpr (BV) issue_bias(nb + C::LA);
                    if constexpr (DO_BY_S) issue_do(t + C::LA);
                }
                lds_copy_end(saved_m0);
            };
            const unsigned char* bt_lds = ring_lds + ((nb - mb_first) % C::RING) * C::BT_BYTES;
            const float* lse_lds = reinterpret_cast<const float*>(smem + C::OFF_LSE) + (IN ? (unsigned)nb % C::NQB : nb % C::NQB) * (C::STAT_BYTES / 4);
            // inputs of P: LSE of 4 consecutive rows and the bias of those rows at this lane's key
            f32x4 lse_in[NSUB][4];
            BiasQuad<BIAS> bias_in[NSUB][4];
            auto load_p_inputs = [&]() {
#pragma unroll
                for (int sb = 0; sb < NSUB; sb++)
#pragma unroll
                    for (int q4 = 0; q4 < 4; q4++) {
                        const int ml0 = sb * 32 + 8 * q4 + 4 * g;  // first of 4 consecutive rows
                        lse_in[sb][q4] = *reinterpret_cast<const f32x4*>(lse_lds + ml0);
                        bias_in[sb][q4].load(bt_lds, ml0, r, lane);
                    }
            };
            // ---- P (flash_attention.py:281-294) of block nb from its scores; register i of sub-block
            // sb is row m0 + 32 sb + 8 (i/4) + 4 g + i%4, the lane is key my_n.  Blocks that touch a
            // ragged edge or the causal diagonal follow the reference's additive -1e6 arithmetic term
            // by term; interior blocks fold everything into one exponent. ----
            auto make_p = [&](auto&& after_pair) {
                const int m0 = nb * BMI;
                const bool need_mask = !IN && ((m0 + BMI > M) || (n0 + BN > N) || (CAUSAL && m0 < n0 + BN - 1));
                const float mf0 = (float)(m0 + 4 * g);  // ALiBi: first row of this lane's registers, as a float
                float* p_out = p_lds + (nb & 1) * (C::P_BYTES / 4);
                auto p_step = [&](auto masked_tag) {
                    constexpr bool MASKED = decltype(masked_tag)::value;
#pragma unroll
                    for (int sb = 0; sb < NSUB; sb++) {
#pragma unroll
                        for (int q4 = 0; q4 < 4; q4++) {
                            const int ml0 = sb * 32 + 8 * q4 + 4 * g;
                            const f32x4 lse4 = lse_in[sb][q4];
                            f32x4 p4;
#pragma unroll
                            for (int e = 0; e < 4; e++) {
                                const int i = q4 * 4 + e;
                                // bool mask: the additive term in log2 units; float bias: natural units
                                float bv = bias_in[sb][q4].get(e);
                                if constexpr (BIAS == 5) bv = alibi_bias(neg_slope, ratio, mf0 + (float)(ml0 - 4 * g + e), (float)my_n);
                                if constexpr (BIAS == 6 || BIAS == 7) bv = row_bv;
                                float pv;
                                if constexpr (MASKED) {
                                    const int m = m0 + ml0 + e;
                                    float x = __fmul_rn(sacc[sb][i], qk_scale);
                                    const bool oob = (m >= M) || (my_n >= N);
                                    float tmask = oob ? kMask : 0.f;
                                    if (CAUSAL) tmask += (m < my_n) ? kMask : 0.f;
                                    float add = NATURAL ? __fmul_rn(bv, kLog2e) : bv;
                                    if (BIAS != 0) add = oob ? kMask : add;  // out-of-range bias reads as masked
                                    x = __fadd_rn(x, __fadd_rn(tmask, add));
                                    pv = fast_exp2(x - lse4[e]);
                                } else {
                                    // (without a bias the offset is the negated LSE itself: written as 0 - lse it
                                    // would cost a subtraction per element, +0 - x not being -x)
                                    const float off = BIAS == 0 ? -lse4[e] : (NATURAL ? __builtin_fmaf(bv, kLog2e, -lse4[e]) : bv - lse4[e]);
                                    pv = fast_exp2(__builtin_fmaf(sacc[sb][i], qk_scale, off));
                                }
                                p4[e] = pv;
                                op_next[sb][i >> 3][i & 7] = (T)pv;
                                if (e & 1) after_pair(sb * 8 + (i >> 1));
                            }
                            // hand P to the dP-wave of the same keys: same lane, same register order
                            *reinterpret_cast<f32x4*>(p_out + ((sb * 4 + q4) * 64 + lane) * 4) = p4;
                        }
                    }
                };
                if constexpr (IN) {
                    p_step(std::false_type{});
                } else {
                    if (need_mask) p_step(std::true_type{});
                    else p_step(std::false_type{});
                }
            };
            if constexpr (TB != 0 && !BV) {
                if (nb < n_mblocks) load_bias_scalar(nb, ring_lds + ((nb - mb_first) % C::RING) * C::BT_BYTES);
            }
            if constexpr (S_AHEAD) {
                // vector work first: P(nb) from the scores formed at the end of the last step
                T8 a_cols[NA], a_rows[NR];
                if constexpr (PRELOAD) {
                    load_p_inputs();
                    __builtin_amdgcn_sched_barrier(0);
                }
                issue_copies();  // behind the reads, whose round trip they cover
                if constexpr (!PRELOAD) load_p_inputs();
                if (IN || nb < n_mblocks) make_p([](int) {});
                if constexpr (PRELOAD) __builtin_amdgcn_sched_barrier(0);
                load_cols((IN ? do_tile_in(t) : do_tile(t)), a_cols);
                load_rows((IN ? q_tile_in(nb + 1) : q_tile(nb + 1)), a_rows);  // lands while the first product runs
                if constexpr (PRELOAD) __builtin_amdgcn_sched_barrier(0);
                // dV^T += dO(t)^T P(t), then the scores of block nb + 1 for the next step
                if (IN || (t >= mb_first && t < n_mblocks)) mma_cols(a_cols, op_cur);
                if (IN || nb + 1 < n_mblocks) mma_rows(a_rows, sacc);
            } else {
                T8 a_cols[NA], a_rows[NR];
                if constexpr (TB == 0) issue_copies();
                load_cols((IN ? do_tile_in(t) : do_tile(t)), a_cols);
                load_rows((IN ? q_tile_in(nb) : q_tile(nb)), a_rows);
                if constexpr (PRELOAD) {
                    load_p_inputs();
                    __builtin_amdgcn_sched_barrier(0);
                }
                if constexpr (TB != 0) issue_copies();
                // Interior steps: the scores first, then the dV product (its operands do not depend on this
                // step) one MFMA at a time between the exponentials of two score elements, so that the wave
                // has vector work to issue while its matrix instructions execute (measured 2-3 % on the
                // kernels of head dim 128 without a bias and with a bias that is only read, a loss of 5 % at
                // head dim 64 with a bool mask; the same interleaving of the dK product into the dS
                // arithmetic of the dP-wave costs 1-4 %).
                constexpr bool FUSE = IN && NSUB == 1 && D == 128;
                if constexpr (FUSE) {
                    mma_rows(a_rows, sacc);
                    __builtin_amdgcn_sched_barrier(0);
                    make_p([&](int j) {
                        __builtin_amdgcn_sched_barrier(0);
                        acc[j % C::DB] = mfma32(a_cols[j], op_cur[0][j / C::DB], acc[j % C::DB]);
                        __builtin_amdgcn_sched_barrier(0);
                    });
                } else {
                // dV^T += dO(t)^T P(t) first: its operands do not depend on this step
                if (IN || (t >= mb_first && t < n_mblocks)) mma_cols(a_cols, op_cur);
                if (IN || nb < n_mblocks) {
                    mma_rows(a_rows, sacc);
                    if constexpr (!PRELOAD) load_p_inputs();
                    make_p([](int) {});
                }
                }
            }
#pragma unroll
            for (int sb = 0; sb < NSUB; sb++)
#pragma unroll
                for (int kk = 0; kk < 2; kk++) op_cur[sb][kk] = op_next[sb][kk];
            // The barrier publishes the copies that the next step reads.  Copies complete in issue
            // order (Q rows, then the bias slice of the same step).  S_AHEAD: the next step reads the
            // Q rows issued one step ago, so only the bias slice issued behind them and this step's
            // copies may still be in flight; else everything but the last LA - 1 steps has landed.
            // Without a bias the compiler is kept from moving work of the step across its closing
            // barrier (it sinks matrix instructions below it where it can): measured 3 % faster at head
            // dim 128 without a bias, slower or equal everywhere else, so only there.
            if constexpr (BIAS == 0 && D == 128) __builtin_amdgcn_sched_barrier(0);
            if constexpr (S_AHEAD) wait_vmcnt<(BV ? C::BCH : 0) + OPS*(C::LA - 2)>();
            else wait_vmcnt<OPS*(C::LA - 1)>();
            lds_barrier();
        };
        // interior steps: t >= mb_first (block t is accumulated), the copied blocks up to t + 1 + LA are
        // whole, and block t + 1 lies below the causal diagonal of every key of the tile
        // Both roles run steps mb_first - 1 .. n_mblocks, whatever part of them is interior.
        const int t_end = n_mblocks + 1;
        int t_in = mb_first, t_out = n_full - C::LA - 1;
        if (CAUSAL) t_in = (n0 + BN - 1 + BMI - 1) / BMI - 1 > t_in ? (n0 + BN - 1 + BMI - 1) / BMI - 1 : t_in;
        if (n0 + BN > N || (TB != 0 && !BV)) t_out = t_in;  // a ragged key tile, bias element by element: no interior
        t_in = t_in < t_end ? t_in : t_end;
        t_out = t_out < t_in ? t_in : (t_out < t_end ? t_out : t_end);
        if (!IN_LOOPS) t_in = t_out = t_end;  // one general loop
        // (two passes over ONE copy of the general loop, the interior loop between them)
        int t = mb_first - 1, stop = t_in;
#pragma unroll 1
        for (int pass = 0; pass < (IN_LOOPS ? 2 : 1); pass++) {
#pragma unroll 1
            for (; t < stop; t++) s_step(t, std::false_type{});
            if constexpr (IN_LOOPS) {
                if (pass == 0 && t_in < t_out) {
                    run_start(qp, p.sq.s, lsep, t_in + 1 + C::LA, t_in + 1 + C::LA);
#pragma unroll 1
                    for (; t < t_out; t++) s_step(t, std::true_type{});
                }
            }
            stop = t_end;
        }
        };
        if (TB != 0 && bias_vec) s_loop(std::true_type{});
        else s_loop(std::false_type{});
    } else {
        // ================================ dP-wave ================================
        // dS^T tile of this wave: 32 keys x BMI rows.  A lane writes its 4 consecutive rows of one key
        // with one 8-byte store, and ds_read_b64_tr_b16 hands a lane 4 consecutive keys of one row.
        T* ds_lds = reinterpret_cast<T*>(smem + C::OFF_DS) + kb * 32 * DSS;
        static_assert(!DB_VIA_LDS || BMI == 32, "the dBias path is laid out for 32-row blocks");
        // lane -> row 16 ((lane/16)%2) + lane%16, keys 8 (lane/32 + 2 it) .. + 7 of the slice
        const int db_row = 16 * ((lane >> 4) & 1) + (lane & 15);
        const int db_src = (8 * (lane >> 5) + ((lane & 15) >> 2)) * DSS + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
        // dBias rows that are whole aligned 16-byte chunks leave through unconditional buffer
        // stores (chunks outside the tensor get an offset outside the view): a loop without
        // branches around its stores lets the loads of the next blocks stay in flight across them.
        const bool db_fast = (DB_VIA_LDS && dbias_vec && (N % 8 == 0)) || (DB_VIA_LDS32 && dbias_vec && (N % 4 == 0));
        __amdgpu_buffer_rsrc_t db_rsrc = make_buffer(nullptr, 0);
        int db_off[2];
        const int db_row_bytes = (DB_VIA_LDS || DB_VIA_LDS32) ? (int)p.sdbias.m * C::ES : 0;
        // fp32: lane -> row 8 it + lane / 8, keys 4 (lane % 8) .. + 3 of the slice, it = 0 .. 3
        const int db32_row = lane >> 3, db32_key = 4 * (lane & 7);
        if (db_fast) {
            db_rsrc = make_buffer(dbp, ((int64_t)(M - 1) * p.sdbias.m + N) * C::ES);
            if constexpr (DB_VIA_LDS32) {
                db_off[0] = nw + db32_key < N ? db32_row * db_row_bytes + (nw + db32_key) * 4 : (int)0x80000000;
                db_off[1] = 0;
            } else {
#pragma unroll
                for (int it = 0; it < 2; it++) {
                    const int nn = nw + 8 * ((lane >> 5) + 2 * it);
                    db_off[it] = nn < N ? db_row * db_row_bytes + nn * 2 : (int)0x80000000;
                }
            }
        }
        float red_acc = 0.f;  // DBIAS == 2: this lane's share of the reduced gradient
        auto dp_loop = [&](auto fast_tag) {
        constexpr bool DB_FAST = decltype(fast_tag)::value;
        // copies per step; the dBias stores that may sit between them in the queue are not
        // counted, which only makes the wait at the end of a step stricter
        constexpr int COPIES = ((Q_BY_S ? 0 : 1) + (DO_BY_S ? 0 : 1)) * (C::QD + 1);
        auto dp_step = [&](int t, auto in_tag) {
            // IN: an interior step: blocks t - 1 .. t + LA are whole and in range
            constexpr bool IN = decltype(in_tag)::value;
            auto issue_copies = [&]() {
                if constexpr (COPIES > 0) {
                    const unsigned saved_m0 = lds_copy_begin();
                    if constexpr (IN) {
                        settle_ptrs(run_rows, run_stat, run_bias);
                        issue_next_do(t + C::LA);
                    } else {
                        if constexpr (!Q_BY_S) issue_q(t + 1 + C::LA);
                        if constexpr (!DO_BY_S) issue_do(t + C::LA);
                    }
                    lds_copy_end(saved_m0);
                }
            };
            const bool live = IN || (t >= mb_first && t < n_mblocks);
            const int m0 = t * BMI;
            const float* delta_lds = reinterpret_cast<const float*>(smem + C::OFF_DELTA) + (IN ? (unsigned)t % C::NDOB : (t < 0 ? 0 : t) % C::NDOB) * (C::STAT_BYTES / 4);
            const float* p_in = p_lds + (t & 1) * (C::P_BYTES / 4);
            T8 a_cols[NA], a_rows[NR];
            f32x4 del_in[NSUB][4], p_vals[NSUB][4];
            auto load_ds_inputs = [&]() {
#pragma unroll
                for (int sb = 0; sb < NSUB; sb++)
#pragma unroll
                    for (int q4 = 0; q4 < 4; q4++) {
                        del_in[sb][q4] = *reinterpret_cast<const f32x4*>(delta_lds + sb * 32 + 8 * q4 + 4 * g);
                        p_vals[sb][q4] = *reinterpret_cast<const f32x4*>(p_in + ((sb * 4 + q4) * 64 + lane) * 4);
                    }
            };
            if constexpr (TB == 0) issue_copies();
            // operands of both products up front: Q(t-1)^T for dK, the rows of dO(t) for dP
            if constexpr (C::DEFER_DK) load_cols((IN ? q_tile_in(t - 1) : q_tile(t - 1)), a_cols);
            load_rows((IN ? do_tile_in(t) : do_tile(t)), a_rows);
            if constexpr (PRELOAD && TB == 0) __builtin_amdgcn_sched_barrier(0);
            if constexpr (TB != 0) issue_copies();  // behind the reads, whose round trip they cover
            if (C::DEFER_DK && (IN || t - 1 >= mb_first)) mma_cols(a_cols, op_cur);  // dK^T += Q(t-1)^T dS(t-1)
            if (live) {
                f32x16 sacc[NSUB];
                if constexpr (PRELOAD) {
                    load_ds_inputs();  // land while the products run
                    __builtin_amdgcn_sched_barrier(0);
                }
                mma_rows(a_rows, sacc);
                if constexpr (!PRELOAD) load_ds_inputs();
                // ---- dS = P (dP - delta) (flash_attention.py:303-308) ----
#pragma unroll
                for (int sb = 0; sb < NSUB; sb++) {
                    i32x2 pk_even = {0, 0};
#pragma unroll
                    for (int q4 = 0; q4 < 4; q4++) {
                        const int ml0 = sb * 32 + 8 * q4 + 4 * g;
                        const f32x4 del4 = del_in[sb][q4];
                        const f32x4 p4 = p_vals[sb][q4];
                        T4 d4;
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const int i = q4 * 4 + e;
                            const float dsv = p4[e] * (sacc[sb][i] - del4[e]);
                            d4[e] = (T)dsv;
                            if constexpr (DBIAS == 2) {
                                // rows past M and keys past N have P = 0 exactly, hence dS = 0
                                if constexpr (BIAS == 5)  // d bias / d slope = -|i N / M - j|
                                    red_acc -= dsv * __builtin_fabsf(__builtin_fmaf((float)(m0 + 4 * g) + (float)(ml0 - 4 * g + e), ratio, -(float)my_n));
                                else red_acc += dsv;
                            }
                            if constexpr (DBIAS == 1 && !DB_VIA_LDS && !DB_VIA_LDS32) {
                                const int m = m0 + ml0 + e;
                                if (m < M && my_n < N) dbp[(int64_t)m * p.sdbias.m + (int64_t)my_n * p.sdbias.n] = (E)dsv;
                            }
                            // (p_in is this wave's part of the hand-off buffer read at the top of the step)
                            if constexpr (DB_VIA_LDS32) const_cast<float*>(p_in)[(ml0 + e) * 32 + r] = dsv;
                        }
                        // the operand of the dK product is made of the same packed words that go to the dS
                        // tile (assembled as integers: element-wise inserts made the compiler convert
                        // every value a second time, one by one, and merge the halves with permutes)
                        const i32x2 pk = __builtin_bit_cast(i32x2, d4);
                        if (q4 & 1) op_cur[sb][q4 >> 1] = __builtin_bit_cast(T8, (i32x4){pk_even[0], pk_even[1], pk[0], pk[1]});
                        else pk_even = pk;
                        if constexpr (DB_VIA_LDS) *reinterpret_cast<T4*>(ds_lds + r * DSS + ml0) = d4;
                    }
                }
                // ---- dBias rows of this wave's 32 keys, 16 bytes per lane, out of the dS^T tile ----
                if constexpr (DB_VIA_LDS) {
#pragma unroll
                    for (int it = 0; it < 2; it++) {
                        const i16x4 lo = lds_read_tr4(ds_lds + db_src + it * 16 * DSS);
                        const i16x4 hi = lds_read_tr4(ds_lds + db_src + it * 16 * DSS + 4 * DSS);
                        typedef short i16x8 __attribute__((ext_vector_type(8)));
                        const i32x4 v = __builtin_bit_cast(i32x4, (i16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                        const int m = m0 + db_row, nn = nw + 8 * ((lane >> 5) + 2 * it);
                        if constexpr (DB_FAST) {
                            // rows past M: m0 * row bytes alone is past the view only if the view is
                            // tight, so the row test is explicit
                            const int off = (IN || m < M) ? db_off[it] + m0 * db_row_bytes : (int)0x80000000;
                            buf_store16(db_rsrc, v, off);
                        } else if (m < M && nn < N) {
                            E* dst = dbp + (int64_t)m * p.sdbias.m + (int64_t)nn * p.sdbias.n;
                            if (dbias_vec && nn + 8 <= N) {
                                gst16(dst, v);
                            } else {
                                const T8 v8 = as_vec<T8>(v);
#pragma unroll
                                for (int e = 0; e < 8; e++)
                                    if (nn + e < N) dst[(int64_t)e * p.sdbias.n] = __builtin_bit_cast(E, (T)v8[e]);
                            }
                        }
                    }
                }
                if constexpr (DB_VIA_LDS32) {
#pragma unroll
                    for (int it = 0; it < 4; it++) {
                        const int row = 8 * it + db32_row;
                        const f32x4 w = *reinterpret_cast<const f32x4*>(p_in + row * 32 + db32_key);
                        const i32x4 v = __builtin_bit_cast(i32x4, w);
                        const int m = m0 + row, nn = nw + db32_key;
                        if constexpr (DB_FAST) {
                            const int off = (IN || m < M) ? db_off[0] + (m0 + 8 * it) * db_row_bytes : (int)0x80000000;
                            buf_store16(db_rsrc, v, off);
                        } else if (m < M && nn < N) {
                            float* dst = reinterpret_cast<float*>(dbp) + (int64_t)m * p.sdbias.m + (int64_t)nn * p.sdbias.n;
                            if (dbias_vec && nn + 4 <= N) {
                                gst16(dst, v);
                            } else {
#pragma unroll
                                for (int e = 0; e < 4; e++)
                                    if (nn + e < N) dst[(int64_t)e * p.sdbias.n] = w[e];
                            }
                        }
                    }
                }
                if constexpr (!C::DEFER_DK) {  // dK^T += Q(t)^T dS(t)
                    load_cols((IN ? q_tile_in(t) : q_tile(t)), a_cols);
                    mma_cols(a_cols, op_cur);
                }
            }
            if constexpr (COPIES > 0) wait_vmcnt<COPIES*(C::LA - 1)>();
            lds_barrier();
        };
        // interior steps: block t - 1 was accumulated into dS (t - 1 >= mb_first) and the copied block t + LA is whole
        const int t_end = n_mblocks + 1;
        int t_in = mb_first + 1, t_out = n_full - C::LA;
        t_in = t_in < t_end ? t_in : t_end;
        t_out = t_out < t_in ? t_in : (t_out < t_end ? t_out : t_end);
        if (!IN_LOOPS) t_in = t_out = t_end;  // one general loop
        // (two passes over ONE copy of the general loop, the interior loop between them)
        int t = mb_first - 1, stop = t_in;
#pragma unroll 1
        for (int pass = 0; pass < (IN_LOOPS ? 2 : 1); pass++) {
#pragma unroll 1
            for (; t < stop; t++) dp_step(t, std::false_type{});
            if constexpr (IN_LOOPS) {
                if (pass == 0 && t_in < t_out) {
                    run_start(dop, p.sdo.s, deltap, t_in + C::LA, 0);
#pragma unroll 1
                    for (; t < t_out; t++) dp_step(t, std::true_type{});
                }
            }
            stop = t_end;
        }
        };
        if constexpr (DB_VIA_LDS || DB_VIA_LDS32) {
            if (db_fast) dp_loop(std::true_type{});
            else dp_loop(std::false_type{});
        } else {
            dp_loop(std::false_type{});
        }
        if constexpr (DBIAS == 2) {
            if constexpr (BIAS == 5) {
                // slope gradient of this wave's 32 keys: one float per (batch, head, key tile, wave), summed
                // over the lanes in a fixed order
                float s = red_acc;
#pragma unroll
                for (int w = 32; w >= 1; w >>= 1) s += __shfl_xor(s, w, 64);
                if (lane == 0) p.partials[((int64_t)bh * p.n_ntiles + nt) * C::WPR + kb] = s;
            } else {
                // column sums: lanes l and l + 32 hold different rows of the same key
                const float s = pair_sum(red_acc);
                if (g == 0 && my_n < N) p.partials[(int64_t)bh * N + my_n] = s;
            }
        }
    }
    // ---- dV (S-wave) or dK (dP-wave) of this wave's 32 keys (flash_attention.py:449-454) ----
    if (my_n < N) {
        T* dst = s_wave ? reinterpret_cast<T*>(p.dv) + (int64_t)b * p.sdv.b + (int64_t)h * p.sdv.h + (int64_t)my_n * p.sdv.s
                        : reinterpret_cast<T*>(p.dk) + (int64_t)b * p.sdk.b + (int64_t)h * p.sdk.h + (int64_t)my_n * p.sdk.s;
        const float out_scale = s_wave ? 1.f : p.sm_scale;
#pragma unroll
        for (int db = 0; db < C::DB; db++) {
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                const int d = db * 32 + 8 * q4 + 4 * g;
                if (d < D) {
                    T4 o4;
#pragma unroll
                    for (int e = 0; e < 4; e++) o4[e] = (T)(acc[db][q4 * 4 + e] * out_scale);
                    *reinterpret_cast<T4*>(dst + d) = o4;
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
template <typename T, int D, int BIAS, bool CAUSAL, int DBIAS>
static hipError_t launch_main(const BwdParams& p, hipStream_t st) {
    dim3 grid((unsigned)(p.n_ntiles * p.B * p.H));
    hipLaunchKernelGGL((fa_bwd_kernel<T, D, BIAS, CAUSAL, DBIAS>), grid, dim3((BwdCfg<D, tile_kind(BIAS), bwd_occ2(D, BIAS)>::NT)), 0, st, p);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------
// Second pass of the reduced dBias modes (DBIAS == 2), one thread per output element, sums in a
// fixed order: every output has one writer and the result is reproducible run to run.
//   float bias: dbias[b', h', 0, n] = sum over the broadcast batches / heads of colsum[b, h, n]
template <typename E>
__global__ __launch_bounds__(256) void fa_bwd_colsum_reduce_kernel(const BwdParams p) {
    const int nb_out = p.sdbias.b == 0 ? 1 : p.B, nh_out = p.sdbias.h == 0 ? 1 : p.H;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)nb_out * nh_out * p.N) return;
    const int n = (int)(idx % p.N);
    const int ho = (int)((idx / p.N) % nh_out), bo = (int)(idx / ((int64_t)p.N * nh_out));
    float s = 0.f;
    for (int b = (nb_out == 1 ? 0 : bo); b < (nb_out == 1 ? p.B : bo + 1); b++)
        for (int h = (nh_out == 1 ? 0 : ho); h < (nh_out == 1 ? p.H : ho + 1); h++)
            s += p.partials[((int64_t)b * p.H + h) * p.N + n];
    reinterpret_cast<E*>(p.dbias)[(int64_t)bo * p.sdbias.b + (int64_t)ho * p.sdbias.h + (int64_t)n * p.sdbias.n] = (E)s;
}
//   ALiBi: dslope[h] = sum over batches, key tiles and waves of the partial slope gradients
// (a template so that the per-head-dim compile units may each hold a copy)
template <int LANES>
__global__ __launch_bounds__(LANES) void fa_bwd_slope_reduce_kernel(const BwdParams p) {
    static_assert(LANES == 64, "one wave");
    const int h = blockIdx.x, lane = threadIdx.x;
    const int per_bh = p.n_ntiles * p.waves_per_role;
    float s = 0.f;
    for (int b = 0; b < p.B; b++)
        for (int i = lane; i < per_bh; i += 64) s += p.partials[((int64_t)b * p.H + h) * per_bh + i];
#pragma unroll
    for (int w = 32; w >= 1; w >>= 1) s += __shfl_xor(s, w, 64);
    if (lane == 0) reinterpret_cast<float*>(p.dbias)[h] = s;
}

// dbias: 0 = none, 1 = dense, 2 = reduced in the kernels (see fa_bwd_kernel)
template <typename T, int D> static hipError_t launch_all(const BwdParams& p, int bias, bool causal, int dbias, int stages, hipStream_t st) {
    constexpr int RPB = 256 / (D / 8);
    const int64_t rows = (int64_t)p.B * p.H * p.M;
    dim3 rgrid((unsigned)((rows + RPB - 1) / RPB));
    hipError_t e = hipSuccess;
    // dBias in fp32 or in the element type of q, written densely a moment ago by the key-tile kernel
    // in rows of whole 16-byte chunks, is the dS the dQ product needs.  Only when that kernel ran in
    // this very call (or the caller vouches for the contents of dbias, bit 8) is it read.
    constexpr int DS_BIAS = __is_same(T, _Float16) ? 2 : 3;
    const bool ds_valid = dbias == 1 && ((stages & 2) || (stages & 8));
    const bool from_ds = (stages & 4) && ds_valid && (bias == DS_BIAS || bias == 4) && p.dbias_vec;
    // A dQ kernel that recomputes dS depends on nothing but delta.  When delta and dQ are asked for in one
    // call it runs FIRST and forms delta itself, bit for bit as fa_bwd_prep_kernel would, which saves a
    // launch and a pass over o and do; the dK/dV kernel then reads the delta it has stored.
    const bool dq_first = (stages & 5) == 5 && !from_ds;
    auto launch_dq = [&](bool makes_delta) -> hipError_t {
        // the one-product form runs at the rate of the dS stream and gains nothing from more work-groups
        BwdParams pq = p;
        pq.dq_makes_delta = makes_delta ? 1 : 0;
        if (from_ds) pq.dq_splits = 1;
        dim3 qgrid((unsigned)(pq.n_mtiles * pq.dq_splits * pq.B * pq.H));
        if (from_ds && bias == DS_BIAS) {
            if (causal) hipLaunchKernelGGL((fa_bwd_dq_kernel<T, D, DS_BIAS, true, true>), qgrid, dim3(256), 0, st, pq);
            else hipLaunchKernelGGL((fa_bwd_dq_kernel<T, D, DS_BIAS, false, true>), qgrid, dim3(256), 0, st, pq);
        } else if (from_ds && bias == 4) {
            if (causal) hipLaunchKernelGGL((fa_bwd_dq_kernel<T, D, 4, true, true>), qgrid, dim3(256), 0, st, pq);
            else hipLaunchKernelGGL((fa_bwd_dq_kernel<T, D, 4, false, true>), qgrid, dim3(256), 0, st, pq);
        } else {
#define FA_CASE(BK)                                                                                               \
    case BK:                                                                                                      \
        if (causal) hipLaunchKernelGGL((fa_bwd_dq_kernel<T, D, BK, true>), qgrid, dim3(256), 0, st, pq);           \
        else hipLaunchKernelGGL((fa_bwd_dq_kernel<T, D, BK, false>), qgrid, dim3(256), 0, st, pq);                 \
        break;
            // a bias without a row dimension whose keys (of one share) fit the LDS row is staged once per
            // work-group instead of streamed
            const int keys_per_wg = pq.dq_splits > 1 ? pq.dq_keys_per_split : pq.N;
            const int qbias = (p.row_bias_kind != 0 && keys_per_wg <= kRowBiasKeys) ? (p.row_bias_kind == 1 ? 7 : 6) : bias;
            switch (qbias) {
                FA_CASE(0)
                FA_CASE(1)
                FA_CASE(2)
                FA_CASE(3)
                FA_CASE(4)
                FA_CASE(5)
                FA_CASE(6)
                FA_CASE(7)
                default: return hipErrorInvalidValue;
            }
#undef FA_CASE
        }
        hipError_t eq = hipGetLastError();
        if (eq == hipSuccess && pq.dq_splits > 1) {
            const int64_t threads = (int64_t)p.B * p.H * p.M * (D / 8);
            hipLaunchKernelGGL((fa_bwd_dq_sum_kernel<T, D>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, pq);
            eq = hipGetLastError();
        }
        return eq;
    };
    if ((stages & 1) && !dq_first) {
        hipLaunchKernelGGL((fa_bwd_prep_kernel<T, D>), rgrid, dim3(256), 0, st, p);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    if (dq_first) {
        e = launch_dq(true);
        if (e != hipSuccess) return e;
    }
    if (stages & 2) {
#define FA_CASE(BK, DBK)                                                                                      \
    if (kbias == BK && dbias == DBK)                                                                          \
        e = causal ? launch_main<T, D, BK, true, DBK>(p, st) : launch_main<T, D, BK, false, DBK>(p, st);
    // a bias that is the same for every query row is one register per key for this kernel
    const int kbias = (p.row_bias_kind != 0 && dbias != 1) ? (p.row_bias_kind == 1 ? 7 : 6) : bias;
    FA_CASE(0, 0)
    else FA_CASE(6, 0)
    else FA_CASE(6, 2)
    else FA_CASE(7, 0)
    else FA_CASE(1, 0)
    else FA_CASE(2, 0)
    else FA_CASE(2, 1)
    else FA_CASE(2, 2)
    else FA_CASE(3, 0)
    else FA_CASE(3, 1)
    else FA_CASE(3, 2)
    else FA_CASE(4, 0)
    else FA_CASE(4, 1)
    else FA_CASE(4, 2)
    else FA_CASE(5, 0)
    else FA_CASE(5, 2)
    else return hipErrorInvalidValue;
#undef FA_CASE
        if (e != hipSuccess) return e;
        if (dbias == 2) {
            if (bias == 5) {
                hipLaunchKernelGGL((fa_bwd_slope_reduce_kernel<64>), dim3((unsigned)p.H), dim3(64), 0, st, p);
            } else {
                const int64_t outs = (int64_t)(p.sdbias.b == 0 ? 1 : p.B) * (p.sdbias.h == 0 ? 1 : p.H) * p.N;
                dim3 g((unsigned)((outs + 255) / 256));
                if (bias == 2) hipLaunchKernelGGL((fa_bwd_colsum_reduce_kernel<_Float16>), g, dim3(256), 0, st, p);
                else if (bias == 3) hipLaunchKernelGGL((fa_bwd_colsum_reduce_kernel<__bf16>), g, dim3(256), 0, st, p);
                else hipLaunchKernelGGL((fa_bwd_colsum_reduce_kernel<float>), g, dim3(256), 0, st, p);
            }
            e = hipGetLastError();
            if (e != hipSuccess) return e;
        }
    }
    if ((stages & 4) && !dq_first) e = launch_dq(false);
    return e;
}

// This file is compiled once per head dimension (-DFA_HEAD_DIM=16 ... 256); each object exports
// launch_bwd_d<FA_HEAD_DIM>.
#ifndef FA_HEAD_DIM
#error "compile with -DFA_HEAD_DIM=<16|32|64|128|256>"
#endif
template <int D> hipError_t launch_bwd_d(const BwdParams& p, int dtype, int bias, bool causal, int dbias, int stages, hipStream_t st);
template <> hipError_t launch_bwd_d<FA_HEAD_DIM>(const BwdParams& p, int dtype, int bias, bool causal, int dbias, int stages, hipStream_t st) {
    if (dtype == 0) return launch_all<_Float16, FA_HEAD_DIM>(p, bias, causal, dbias, stages, st);
    return launch_all<__bf16, FA_HEAD_DIM>(p, bias, causal, dbias, stages, st);
}

}  // namespace fa

