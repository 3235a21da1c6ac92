// Forward attention kernel for gfx950: O = softmax(Q K^T * sm_scale + bias) V, LSE saved.
//
// Replaces _attn_fwd / _attn_fwd_inner of the reference (/root/reference/flash_attention.py:12-194)
// together with the host-side bias pre-scale (flash_attention.py:660-663), which is folded into
// the kernel as an fp32 multiply.
//
// Work split.  One work-group (4 waves) owns 128 query rows of one (batch, head); each wave
// owns 32 of them for the whole kernel.  Keys/values are streamed in tiles of 64 through LDS.
// Scores are computed TRANSPOSED, S^T = K Q^T, so that in the MFMA accumulator a lane holds one
// query row (column l%32 of S^T) and 32 of the 64 keys: the row maximum and row sum of the online
// softmax are then per-lane loops plus a single exchange with lane l^32, the running maximum, the
// running sum and the rescale factor are one scalar per lane, and P^T is already laid out as the
// B operand of O^T += V^T P^T.  V^T is gathered from the row-major V tile with
// ds_read_b64_tr_b16.  The bias tile of a wave (32 rows x 64 keys) is staged through a
// wave-private LDS region with 16-byte coalesced global loads and read back in accumulator
// layout (4 consecutive keys per read).
#include "fa_common.hpp"
#include "fa_params.hpp"

namespace fa {

template <int D, int BIAS> struct FwdCfg {
    static constexpr int BM = 128, BN = 64, NT = 256;
    static constexpr int DP = D < 32 ? 32 : D;       // head dim padded to one 32-wide MFMA block
    static constexpr int KS = D + 8;                 // K tile row stride (elements): 16 B skew
    static constexpr int VS = DP + 32;               // V tile row stride: 64 B skew (transposed reads)
    static constexpr int OS = DP + 8;                // O staging row stride
    static constexpr int CPR = D / 8;                // 16-byte chunks per row
    static constexpr int NCH = (BN * CPR + NT - 1) / NT;  // chunks per thread per K (or V) tile
    static constexpr int KSTEPS = D / 16;            // MFMA k-steps of Q K^T
    static constexpr int DB = DP / 32;               // 32-wide blocks of the head dim
    static constexpr int ES = BIAS == 0 ? 0 : (BIAS == 1 ? 1 : (BIAS == 4 ? 4 : 2));
    static constexpr int BROW = BIAS == 0 ? 0 : (ES == 1 ? 72 : (ES == 2 ? 136 : 272));  // bytes
    static constexpr int BCH = 2 * ES;               // 16-byte bias chunks per lane per tile
    static constexpr int K_BYTES = BN * KS * 2;
    static constexpr int V_BYTES = BN * VS * 2;
    static constexpr int O_BYTES = BM * OS * 2;
    static constexpr int KV_BYTES = (K_BYTES + V_BYTES) > O_BYTES ? (K_BYTES + V_BYTES) : O_BYTES;
    static constexpr int BIAS_BYTES = 4 * 32 * BROW;
    static constexpr int LDS_BYTES = KV_BYTES + BIAS_BYTES;
    // two work-groups per CU whenever registers allow it
    static constexpr int MIN_BLOCKS = D <= 128 ? 2 : 1;
};

template <typename T, int D, int BIAS, bool CAUSAL>
__global__ __launch_bounds__(256, (FwdCfg<D, BIAS>::MIN_BLOCKS)) void fa_fwd_kernel(const FwdParams p) {
    typedef FwdCfg<D, BIAS> C;
    typedef typename VecOf<T>::v8 T8;
    typedef typename VecOf<T>::v4 T4;
    typedef typename BiasElem<BIAS>::type E;
    constexpr int BM = C::BM, BN = C::BN, KS = C::KS, VS = C::VS, OS = C::OS, CPR = C::CPR;

    __shared__ __align__(16) unsigned char smem[C::LDS_BYTES];
    T* k_lds = reinterpret_cast<T*>(smem);
    T* v_lds = reinterpret_cast<T*>(smem + C::K_BYTES);

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int r = lane & 31, g = lane >> 5;

    int mt, bh;
    decode_block(blockIdx.x, p.n_mtiles, p.B * p.H, mt, bh);
    if (CAUSAL) mt = p.n_mtiles - 1 - mt;  // longest rows first
    const int b = bh / p.H, h = bh % p.H;
    const int M = p.M, N = p.N;
    const int m0 = mt * BM;
    const int mw = m0 + wave * 32;  // first query row of this wave
    const int my_m = mw + r;

    const T* qp = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.sq.b + (int64_t)h * p.sq.h;
    const T* kp = reinterpret_cast<const T*>(p.k) + (int64_t)b * p.sk.b + (int64_t)h * p.sk.h;
    const T* vp = reinterpret_cast<const T*>(p.v) + (int64_t)b * p.sv.b + (int64_t)h * p.sv.h;
    const E* bp = nullptr;
    unsigned char* bias_lds = nullptr;
    if (BIAS != 0) {
        bp = reinterpret_cast<const E*>(p.bias) + (int64_t)b * p.sbias.b + (int64_t)h * p.sbias.h;
        bias_lds = smem + C::KV_BYTES + wave * 32 * C::BROW;
    }

    // V columns D..DP-1 (only when D < 32) are never loaded: keep them zero
    if (D < C::DP) {
        for (int i = tid; i < BN * VS; i += C::NT) v_lds[i] = (T)0.f;
    }

    // Q^T as B operand: column my_m, k = d
    T8 qreg[C::KSTEPS];
#pragma unroll
    for (int ks = 0; ks < C::KSTEPS; ks++) {
        i32x4 raw = {0, 0, 0, 0};
        if (my_m < M) raw = gld16(qp + (int64_t)my_m * p.sq.s + ks * 16 + 8 * g);
        qreg[ks] = as_vec<T8>(raw);
    }

    int n_tiles = (N + BN - 1) / BN;
    if (CAUSAL) {
        int last = (m0 + BM - 1) / BN + 1;  // tiles holding keys <= last row of this work-group
        n_tiles = n_tiles < last ? n_tiles : last;
    }

    const float qk_scale = p.sm_scale * kLog2e;
    float m_i = -INFINITY, l_i = 0.f;
    f32x16 o_acc[C::DB];
#pragma unroll
    for (int db = 0; db < C::DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) o_acc[db][i] = 0.f;

    i32x4 kreg[C::NCH], vreg[C::NCH];
    i32x4 breg[C::BCH > 0 ? C::BCH : 1];

    auto prefetch = [&](int j) {
        const int n0 = j * BN;
#pragma unroll
        for (int it = 0; it < C::NCH; it++) {
            int c = it * C::NT + tid;
            int row = c / CPR, ch = c % CPR;
            bool ok = (c < BN * CPR) && (n0 + row < N);
            i32x4 z = {0, 0, 0, 0};
            kreg[it] = ok ? gld16(kp + (int64_t)(n0 + row) * p.sk.s + ch * 8) : z;
            vreg[it] = ok ? gld16(vp + (int64_t)(n0 + row) * p.sv.s + ch * 8) : z;
        }
        if (BIAS != 0) {
            if (p.bias_vec && n0 + BN <= N) {
                constexpr int CH_ROW = 4 * C::ES;  // 16-byte chunks per 64-key row
#pragma unroll
                for (int it = 0; it < C::BCH; it++) {
                    int c = it * 64 + lane;
                    int row = c / CH_ROW, ch = c % CH_ROW;
                    i32x4 z = {0, 0, 0, 0};
                    const unsigned char* src = reinterpret_cast<const unsigned char*>(
                        bp + (int64_t)(mw + row) * p.sbias.m + n0) + ch * 16;
                    breg[it] = (mw + row < M) ? gld16(src) : z;
                }
            }
        }
    };

    if (n_tiles > 0) prefetch(0);

    for (int j = 0; j < n_tiles; j++) {
        const int n0 = j * BN;
        __syncthreads();  // every wave is done reading the previous tile
#pragma unroll
        for (int it = 0; it < C::NCH; it++) {
            int c = it * C::NT + tid;
            int row = c / CPR, ch = c % CPR;
            if (c < BN * CPR) {
                lds_write16(k_lds + row * KS + ch * 8, kreg[it]);
                lds_write16(v_lds + row * VS + ch * 8, vreg[it]);
            }
        }
        if (BIAS != 0) {
            if (p.bias_vec && n0 + BN <= N) {
                constexpr int CH_ROW = 4 * C::ES;
#pragma unroll
                for (int it = 0; it < C::BCH; it++) {
                    int c = it * 64 + lane;
                    int row = c / CH_ROW, ch = c % CH_ROW;
                    i32x2* dst = reinterpret_cast<i32x2*>(bias_lds + row * C::BROW + ch * 16);
                    i32x2 lo = {breg[it][0], breg[it][1]}, hi = {breg[it][2], breg[it][3]};
                    dst[0] = lo;
                    dst[1] = hi;
                }
            } else {
                // ragged or unaligned bias: one element per lane per row, any strides
#pragma unroll 1
                for (int row = 0; row < 32; row++) {
                    int n = n0 + lane;
                    E val = (E)0.f;
                    if (mw + row < M && n < N)
                        val = bp[(int64_t)(mw + row) * p.sbias.m + (int64_t)n * p.sbias.n];
                    *reinterpret_cast<E*>(bias_lds + row * C::BROW + lane * C::ES) = val;
                }
            }
        }
        __syncthreads();
        if (j + 1 < n_tiles) prefetch(j + 1);

        // tiles entirely above this wave's diagonal contribute nothing
        if (CAUSAL && n0 > mw + 31) continue;
        const bool need_mask = (n0 + BN > N) || (CAUSAL && n0 + BN - 1 > mw);

        // ---- S^T = K Q^T : s[nb][i] is key n0 + 32 nb + 8 (i/4) + 4 g + i%4, query my_m ----
        f32x16 s[2];
#pragma unroll
        for (int nb = 0; nb < 2; nb++) {
#pragma unroll
            for (int i = 0; i < 16; i++) s[nb][i] = 0.f;
#pragma unroll
            for (int ks = 0; ks < C::KSTEPS; ks++) {
                T8 a = as_vec<T8>(lds_read16(k_lds + (nb * 32 + r) * KS + ks * 16 + 8 * g));
                s[nb] = mfma32(a, qreg[ks], s[nb]);
            }
        }

        // ---- scale, bias, masks (additive -1e6 in log2 units, flash_attention.py:39-53) ----
        float mx = -INFINITY;
#pragma unroll
        for (int nb = 0; nb < 2; nb++) {
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                const int nl = nb * 32 + 8 * q4 + 4 * g;  // first of 4 consecutive keys
                float bv[4] = {0.f, 0.f, 0.f, 0.f};
                if constexpr (BIAS == 1) {
                    unsigned int w = *reinterpret_cast<const unsigned int*>(bias_lds + r * C::BROW + nl);
#pragma unroll
                    for (int e = 0; e < 4; e++) bv[e] = ((w >> (8 * e)) & 0xffu) ? 0.f : kMask;
                } else if constexpr (BIAS == 2 || BIAS == 3) {
                    typedef typename VecOf<E>::v4 B4;
                    B4 hv = *reinterpret_cast<const B4*>(bias_lds + r * C::BROW + nl * 2);
#pragma unroll
                    for (int e = 0; e < 4; e++) bv[e] = (float)hv[e] * kLog2e;
                } else if constexpr (BIAS == 4) {
                    f32x4 w = *reinterpret_cast<const f32x4*>(bias_lds + r * C::BROW + nl * 4);
#pragma unroll
                    for (int e = 0; e < 4; e++) bv[e] = w[e] * kLog2e;
                }
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int i = q4 * 4 + e;
                    float x = __fmul_rn(s[nb][i], qk_scale);
                    float add = bv[e];
                    if (need_mask) {
                        const int n = n0 + nl + e;
                        float t = 0.f;
                        if (n >= N) t = kMask;
                        if (CAUSAL && my_m < n) t += kMask;
                        if (BIAS != 0 && n >= N) add = kMask;  // out-of-range bias reads as masked
                        add = t + add;
                    }
                    x = __fadd_rn(x, add);
                    s[nb][i] = x;
                    mx = fmaxf(mx, x);
                }
            }
        }
        mx = pair_max(mx);
        const float m_new = fmaxf(m_i, mx);
        const float alpha = fast_exp2(m_i - m_new);
        m_i = m_new;
        float rs = 0.f;
        T8 pb[2][2];
#pragma unroll
        for (int nb = 0; nb < 2; nb++) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                float pv = fast_exp2(s[nb][i] - m_new);
                rs += pv;
                pb[nb][i >> 3][i & 7] = (T)pv;
            }
        }
        l_i = l_i * alpha + rs;  // per-lane partial sum; the two halves are added at the end
#pragma unroll
        for (int db = 0; db < C::DB; db++)
#pragma unroll
            for (int i = 0; i < 16; i++) o_acc[db][i] *= alpha;

        // ---- O^T += V^T P^T : A = V^T gathered down the columns of the V tile ----
#pragma unroll
        for (int nb = 0; nb < 2; nb++) {
#pragma unroll
            for (int kk = 0; kk < 2; kk++) {
#pragma unroll
                for (int db = 0; db < C::DB; db++) {
                    T8 a = lds_read_col8<T8>(v_lds, lane, nb * 32 + kk * 16, db * 32, VS);
                    o_acc[db] = mfma32(a, pb[nb][kk], o_acc[db]);
                }
            }
        }
    }

    // ---- epilogue (flash_attention.py:188-194) ----
    const float l_tot = pair_sum(l_i);
    const float inv_l = 1.f / l_tot;
    if (g == 0 && my_m < M) p.lse[((int64_t)b * p.H + h) * M + my_m] = m_i + fast_log2(l_tot);

    __syncthreads();  // K/V tiles are dead: reuse their LDS for the output tile
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

template <typename T, int D, int BIAS, bool CAUSAL> static hipError_t launch_one(const FwdParams& p, hipStream_t st) {
    dim3 grid((unsigned)(p.n_mtiles * p.B * p.H));
    hipLaunchKernelGGL((fa_fwd_kernel<T, D, BIAS, CAUSAL>), grid, dim3(256), 0, st, p);
    return hipGetLastError();
}

template <typename T, int D> static hipError_t launch_bias(const FwdParams& p, int bias, bool causal, hipStream_t st) {
#define FA_CASE(BK)                                                        \
    case BK:                                                               \
        return causal ? launch_one<T, D, BK, true>(p, st) : launch_one<T, D, BK, false>(p, st);
    switch (bias) {
        FA_CASE(0)
        FA_CASE(1)
        FA_CASE(2)
        FA_CASE(3)
        FA_CASE(4)
    }
#undef FA_CASE
    return hipErrorInvalidValue;
}

template <typename T> static hipError_t launch_d(const FwdParams& p, int D, int bias, bool causal, hipStream_t st) {
    switch (D) {
        case 16: return launch_bias<T, 16>(p, bias, causal, st);
        case 32: return launch_bias<T, 32>(p, bias, causal, st);
        case 64: return launch_bias<T, 64>(p, bias, causal, st);
        case 128: return launch_bias<T, 128>(p, bias, causal, st);
        case 256: return launch_bias<T, 256>(p, bias, causal, st);
    }
    return hipErrorInvalidValue;
}

// dtype: 0 = fp16, 1 = bf16.  The caller has validated every argument.
hipError_t launch_fwd(const FwdParams& p, int D, int dtype, int bias, bool causal, hipStream_t st) {
    if (dtype == 0) return launch_d<_Float16>(p, D, bias, causal, st);
    return launch_d<__bf16>(p, D, bias, causal, st);
}

int fwd_block_m() { return 128; }

}  // namespace fa
