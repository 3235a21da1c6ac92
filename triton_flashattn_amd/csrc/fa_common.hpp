// Device-side building blocks shared by the gfx950 attention kernels.
//
// Wave = 64 lanes.  All matrix products use v_mfma_f32_32x32x16_{bf16,f16}:
//   A (32 x 16): lane l holds row l%32, k = 8*(l/32) .. 8*(l/32)+7
//   B (16 x 32): lane l holds col l%32, k = 8*(l/32) .. 8*(l/32)+7
//   C (32 x 32): lane l holds col l%32; register i holds row 8*(i/4) + 4*(l/32) + i%4
// Only the pairing of A's and B's k slots matters to the product, so operands taken from a C
// fragment (registers 8j..8j+7 = rows {16j + 4g + 0..3, 16j + 8 + 4g + 0..3}, g = l/32) are
// matched by loading the other operand with the same k order.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fa {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kMask = -1.0e6f;  // additive mask term, in log2 units

template <typename T> struct VecOf;
template <> struct VecOf<__bf16> { typedef bf16x8 v8; typedef bf16x4 v4; };
template <> struct VecOf<_Float16> { typedef f16x8 v8; typedef f16x4 v4; };

__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x16 mfma32(f16x8 a, f16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

template <typename V> __device__ __forceinline__ V as_vec(i32x4 x) { return __builtin_bit_cast(V, x); }
template <typename V> __device__ __forceinline__ i32x4 as_raw(V x) { return __builtin_bit_cast(i32x4, x); }

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// Value of `x` held by lane l ^ 32.
__device__ __forceinline__ float partner32(float x) {
    int xi = __builtin_bit_cast(int, x);
    auto r = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
    int other = (threadIdx.x & 32) ? r[0] : r[1];
    return __builtin_bit_cast(float, other);
}
// max / sum over the lane pair {l, l ^ 32}
__device__ __forceinline__ float pair_max(float x) {
    int xi = __builtin_bit_cast(int, x);
    auto r = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
    return fmaxf(__builtin_bit_cast(float, (int)r[0]), __builtin_bit_cast(float, (int)r[1]));
}
__device__ __forceinline__ float pair_sum(float x) {
    int xi = __builtin_bit_cast(int, x);
    auto r = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
    return __builtin_bit_cast(float, (int)r[0]) + __builtin_bit_cast(float, (int)r[1]);
}

// Work-group barrier that orders LDS traffic only.  Unlike __syncthreads() it does not wait for
// outstanding global loads, stores or direct-to-LDS copies, so prefetches issued before it stay in
// flight across it (a consumer of such a copy waits on vmcnt itself).
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// ---- LDS access ---------------------------------------------------------------------------
__device__ __forceinline__ i32x4 lds_read16(const void* p) { return *reinterpret_cast<const i32x4*>(p); }

// ds_read_b64_tr_b16.  Within each group of 16 lanes, lane s supplies the address of four
// consecutive 16-bit elements: row s/4, columns 4*(s%4) .. 4*(s%4)+3 of a 4 x 16 matrix.  Lane i
// of the group receives column i of that matrix (4 values, rows 0..3).
__device__ __forceinline__ i16x4 lds_read_tr4(const void* p) {
    typedef i16x4 __attribute__((address_space(3))) * lds_ptr;
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p));
}
// Address a lane must supply so that a 32-lane half of the wave reads a 4-row x 32-column
// block (16-bit elements, `stride` elements between rows) and lane l ends up with column l%32:
// returns the element offset of (row0 + (l%16)/4, col0 + 16*((l/16)%2) + 4*(l%4)).
__device__ __forceinline__ int tr_offset(int lane, int row0, int col0, int stride) {
    int s = lane & 15;
    return (row0 + (s >> 2)) * stride + col0 + ((lane >> 4) & 1) * 16 + (s & 3) * 4;
}
// The same two reads by LDS byte address (a 32-bit integer) instead of by pointer
__device__ __forceinline__ i32x4 lds_read16_at(unsigned addr) {
    typedef const i32x4 __attribute__((address_space(3))) * lds_ptr;
    return *(lds_ptr)(uintptr_t)addr;
}
__device__ __forceinline__ i16x4 lds_read_tr4_at(unsigned addr) {
    typedef i16x4 __attribute__((address_space(3))) * lds_ptr;
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(uintptr_t)addr);
}
// Row-major LDS tile of 16-bit elements, D per row, no padding; the 16-byte chunks of a row are
// XOR-swizzled by a function of the row so that both 16-byte row reads (lane = row) and 4-row
// column gathers (ds_read_b64_tr_b16) are free of bank conflicts.
//
// Operand fetches by address.  A tile starts at a multiple of its row length in bytes, so the
// XOR of the swizzle and the step along the head dim only touch address bits below the row
// stride: the address of a lane's chunk is (tile + L) ^ step + rows, with ONE per-lane constant
// L per access pattern (rows_lane for row operands, cols_lane for column gathers), a
// compile-time `step`, and a compile-time row term that goes into the offset field of the read.
// A kernel so keeps two address constants per lane instead of one per read.
template <int D> struct Swz {
    static constexpr int CPR = D / 8;  // chunks per row
    static constexpr int RB = 2 * D;   // bytes per row
    __device__ static __forceinline__ int f(int row) {
        if (CPR >= 16) return ((row & 3) << 2) | ((row >> 2) & 3);
        if (CPR == 8) return (((row >> 1) & 1) << 2) | ((row >> 2) & 3);
        if (CPR == 4) return (row >> 2) & 3;
        return (row >> 3) & 1;
    }
    __device__ static __forceinline__ int off(int row, int col) {
        return row * D + ((((col >> 3) ^ f(row)) << 3) | (col & 7));
    }
    // 8 k-slots gathered down column col0 + lane%32: rows row0 + 4g + {0..3}, row0 + 8 + 4g + {0..3}
    template <typename V8, typename T>
    __device__ static __forceinline__ V8 col8(const T* tile, int lane, int row0, int col0) {
        const int g = lane >> 5, s = lane & 15;
        const int row = row0 + 4 * g + (s >> 2);
        const int col = (col0 + ((lane >> 4) & 1) * 16 + (s & 3) * 4) & (D - 1);
        i16x4 lo = lds_read_tr4(tile + off(row, col));
        i16x4 hi = lds_read_tr4(tile + off(row + 8, col));
        typedef short i16x8 __attribute__((ext_vector_type(8)));
        return __builtin_bit_cast(V8, (i16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    }
    // Row operand: lane l reads row (rows + l%32), head-dim elements 16 ks + 8 (l/32) .. + 7.
    // rows_lane(lane) is L; `rows` is a multiple of 32 known at compile time.
    __device__ static __forceinline__ unsigned rows_lane(int lane) {
        const int r = lane & 31, g = lane >> 5;
        return (unsigned)(r * RB + 16 * (g ^ f(r)));
    }
    template <typename V8> __device__ static __forceinline__ V8 row8_at(unsigned tile_plus_l, int rows, int ks) {
        return __builtin_bit_cast(V8, lds_read16_at((tile_plus_l ^ (unsigned)(32 * ks)) + (unsigned)(rows * RB)));
    }
    // Column operand (what col8 returns) for head-dim block db (32 wide) and rows row0 .. row0 + 15,
    // row0 a multiple of 16 known at compile time.  The second gather sits 8 rows further down,
    // where the swizzle differs by one fixed bit.
    __device__ static __forceinline__ unsigned cols_lane(int lane) {
        const int g = lane >> 5, s = lane & 15;
        const int rl = 4 * g + (s >> 2);
        const int col = (((lane >> 4) & 1) * 16 + (s & 3) * 4) & (D - 1);
        return (unsigned)(rl * RB + 16 * ((col >> 3) ^ f(rl)) + 2 * (col & 7));
    }
    template <typename V8> __device__ static __forceinline__ V8 col8_at(unsigned tile_plus_l, int row0, int db) {
        constexpr unsigned H = CPR == 2 ? 16u : 32u;  // f(row + 8) ^ f(row), as a byte offset
        const unsigned x = (unsigned)((64 * db) & (RB - 1));
        i16x4 lo = lds_read_tr4_at((tile_plus_l ^ x) + (unsigned)(row0 * RB));
        i16x4 hi = lds_read_tr4_at((tile_plus_l ^ x ^ H) + (unsigned)((row0 + 8) * RB));
        typedef short i16x8 __attribute__((ext_vector_type(8)));
        return __builtin_bit_cast(V8, (i16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    }
};

// ---- global access ------------------------------------------------------------------------
// Direct global -> LDS copies, issued behind the compiler's back.
//
// global_load_lds_dwordx4: lane l copies the 16 bytes at base + voff (voff per lane) to LDS address
// M0 + 16 l, without passing through registers; completion counts on vmcnt.  Issued through the
// compiler's builtin, every later LDS read that might alias the copy would wait for ALL
// outstanding vector-memory operations, which empties a queue of copies issued several steps
// ahead.  Issued from inline assembly the compiler sees neither the LDS write nor the vmcnt
// increment: the consumer waits with an explicit s_waitcnt vmcnt(n) (copies complete in issue
// order) before it reads the destination, and a wave that uses this must not mix it with loads
// whose completion the compiler counts.
//
// A copy costs the issuing wave about 20 clocks when everything it needs is in scalar registers
// (57 with M0 saved and restored around each one and the addresses moved over from vector
// registers), so copies are issued in batches: M0 saved once, restored once, LDS addresses and
// base pointers scalar.
__device__ __forceinline__ unsigned lds_copy_begin() {
    unsigned saved_m0;
    asm volatile("s_mov_b32 %0, m0" : "=s"(saved_m0) : : "memory");
    return saved_m0;
}
__device__ __forceinline__ void lds_copy_end(unsigned saved_m0) {
    asm volatile("s_mov_b32 m0, %0" : : "s"(saved_m0) : "memory");
}
// the LDS address (scalar) of a generic pointer into LDS that is the same in every lane: the low
// half of the generic pointer
__device__ __forceinline__ unsigned lds_addr_of(const void* p) {
    return __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)p);
}
// A wave-uniform pointer, forced into scalar registers (the compiler may have computed it with
// vector instructions, and an inline-asm scalar operand is not moved there by itself).
// A vector-memory instruction that reads an SGPR written by a VALU instruction (v_readfirstlane
// here) needs five wait states in between.  The compiler inserts them for its own instructions
// but cannot see into inline assembly, so they are added here, tied to the two registers so that
// they sit between the write and every use.
__device__ __forceinline__ uint64_t uniform_ptr(const void* p) {
    const uint64_t b = (uint64_t)(uintptr_t)p;
    unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)b);
    unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(b >> 32));
    asm volatile("s_nop 4" : "+s"(lo), "+s"(hi));
    return ((uint64_t)hi << 32) | lo;
}
// The same for up to three addresses that a loop keeps and advances in scalar registers: one wait
// for all of them, in place, so that no copy of an address is made per use.
__device__ __forceinline__ void settle_ptrs(uint64_t& a, uint64_t& b, uint64_t& c) {
    unsigned r[6] = {(unsigned)a, (unsigned)(a >> 32), (unsigned)b, (unsigned)(b >> 32), (unsigned)c, (unsigned)(c >> 32)};
#pragma unroll
    for (int i = 0; i < 6; i++) r[i] = __builtin_amdgcn_readfirstlane(r[i]);
    asm volatile("s_nop 4" : "+s"(r[0]), "+s"(r[1]), "+s"(r[2]), "+s"(r[3]), "+s"(r[4]), "+s"(r[5]));
    a = ((uint64_t)r[1] << 32) | r[0];
    b = ((uint64_t)r[3] << 32) | r[2];
    c = ((uint64_t)r[5] << 32) | r[4];
}
// between lds_copy_begin() and lds_copy_end(): 16 bytes per lane from base + voff to lds_addr + 16 l
__device__ __forceinline__ void lds_copy16(uint64_t base, unsigned voff, unsigned lds_addr) {
    asm volatile(
        "s_mov_b32 m0, %2\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %0, %1"
        :
        : "v"(voff), "s"(base), "s"(lds_addr)
        : "memory");
}
// the same for 4 bytes per lane, to lds_addr + 4 l
__device__ __forceinline__ void lds_copy4(uint64_t base, unsigned voff, unsigned lds_addr) {
    asm volatile(
        "s_mov_b32 m0, %2\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dword %0, %1"
        :
        : "v"(voff), "s"(base), "s"(lds_addr)
        : "memory");
}
// s_waitcnt vmcnt(n) alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14, the other counters maxed)
template <int N> __device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// Raw buffer view of `bytes` bytes at `base` (16-byte aligned): stores beyond the end are dropped
// (and loads beyond it would return 0).  The range check works on whole dwords, so the length is
// rounded up to the dword that holds the last byte (still inside the aligned allocation); a
// caller that stores through the view must not address the rounding slack.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_buffer(const void* base, int64_t bytes) {
    const int64_t cap = 0xfffffffcll;
    bytes = (bytes + 3) & ~(int64_t)3;
    const unsigned n = bytes < 0 ? 0u : (unsigned)(bytes > cap ? cap : bytes);
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)n, 0x00020000);
}
// 16-byte store through a buffer view; an offset outside the view drops the store
__device__ __forceinline__ void buf_store16(__amdgpu_buffer_rsrc_t r, i32x4 v, int voff) {
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(__attribute__((__vector_size__(4 * sizeof(unsigned int)))) unsigned int, v), r, voff, 0, 0);
}
__device__ __forceinline__ i32x4 gld16(const void* p) { return *reinterpret_cast<const i32x4*>(p); }
__device__ __forceinline__ void gst16(void* p, i32x4 v) { *reinterpret_cast<i32x4*>(p) = v; }

// bias element -> fp32 (natural units); E is the storage type selected by the bias kind
template <int BIAS> struct BiasElem;
template <> struct BiasElem<0> { typedef unsigned char type; };
template <> struct BiasElem<1> { typedef unsigned char type; };
template <> struct BiasElem<2> { typedef _Float16 type; };
template <> struct BiasElem<3> { typedef __bf16 type; };
template <> struct BiasElem<4> { typedef float type; };
template <> struct BiasElem<5> { typedef float type; };  // ALiBi: one fp32 slope per head, no tile
template <> struct BiasElem<6> { typedef unsigned char type; };  // the stream kind of ALiBi (below)
template <> struct BiasElem<7> { typedef unsigned char type; };

// Bias kind 5 (ALiBi): bias[b,h,i,j] = -slope[h] * |i * N / M - j| is computed from the indices, so no
// bias tile exists and the K/V stream is tiled as without a bias.  TILE_KIND maps a bias kind to
// the kind of tile that StreamCfg / KeyStream handle.
// Kinds 6 and 7: a float bias / a bool mask that is the same for every query row (stride 0 along M).
// In the dK/dV kernel the lane is the key, so the whole bias of a wave is ONE register per lane, read
// once, and nothing is streamed.  In the forward and dQ kernels the lane is the row: the work-group
// converts the row to fp32 once into an LDS region behind the K/V slots (at most kRowBiasKeys keys,
// longer rows take the dense path through their zero stride) and every lane reads the values of its
// keys from there; the K/V stream is tiled as without a bias.
constexpr int tile_kind(int bias) { return bias >= 5 ? 0 : bias; }
// ... and to the kind that StreamCfg / KeyStream tile the K/V stream for: 6 = no bias tile, but steps of
// 32 keys like the kernels with one (the element-wise work of ALiBi needs the registers that the
// 64-key steps of the bias-free kernels spend on a second block of scores)
constexpr int stream_kind(int bias) { return bias == 5 ? 6 : (bias >= 6 ? 0 : bias); }
// -slope * |m * ratio - n| for query row m and key n (both exact as floats), natural units
__device__ __forceinline__ float alibi_bias(float neg_slope, float ratio, float mf, float nf) {
    return neg_slope * __builtin_fabsf(__builtin_fmaf(mf, ratio, -nf));
}

// Kinds 6 / 7 of the forward and dQ kernels: the 256 threads of a work-group write the bias row of
// keys 0 .. N-1 (element kind 1 bool, 2 fp16, 3 bf16, 4 fp32, n-th element at bias[at0 + n stride_n])
// to row_lds as fp32, a float bias in natural units, a bool mask as the additive term of the
// reference in log2 units (0 or -1e6, flash_attention.py:49-53); zeros up to the next multiple of 64.
__device__ __forceinline__ void stage_row_bias(float* row_lds, const void* bias, int kind, int64_t at0, int64_t stride_n,
                                               int N, int tid) {
    const int n_stage = (N + 63) & ~63;
    for (int n = tid; n < n_stage; n += 256) {
        float v = 0.f;
        if (n < N) {
            const int64_t at = at0 + (int64_t)n * stride_n;
            switch (kind) {
                case 1: v = reinterpret_cast<const unsigned char*>(bias)[at] != 0 ? 0.f : kMask; break;
                case 2: v = (float)reinterpret_cast<const _Float16*>(bias)[at]; break;
                case 3: v = (float)reinterpret_cast<const __bf16*>(bias)[at]; break;
                default: v = reinterpret_cast<const float*>(bias)[at]; break;
            }
        }
        row_lds[n] = v;
    }
    __syncthreads();
}

// Tiling of the forward and the dQ kernel: a work-group owns 128 query rows (4 waves x 32 rows) and streams
// keys in steps of NH blocks of 32.  K and V rows of a step and the bias slice of each wave reach
// LDS through direct global -> LDS copies issued ahead of their use.  With a bias: steps of 32
// keys, K/V in a ring of 3 slots (two steps ahead), the bias in a ring of 4 slots per wave (three
// steps ahead).  Without: steps of 64 keys, K/V double buffered (one step ahead), which halves the
// number of barriers.
template <int D, int BIAS> struct StreamCfg {
    static constexpr int NH = BIAS == 0 ? 2 : 1;     // 32-key blocks per step
    // steps the K/V copies run ahead (an fp32 bias: shallower rings, so that two work-groups fit a
    // CU: measured 27 % faster in the forward than one work-group with the deeper rings)
    static constexpr int LA = (BIAS == 0 || BIAS == 4) ? 1 : 2;
    static constexpr int BM = 128, BK = 32 * NH, NT = 256;
    static constexpr int DP = D < 32 ? 32 : D;       // head dim padded to one 32-wide MFMA block
    static constexpr int OS = DP + 8;                // O staging row stride (elements)
    static constexpr int CPR = D / 8;                // 16-byte chunks per row
    static constexpr int KSTEPS = D / 16;            // MFMA k-steps of Q K^T
    static constexpr int DB = DP / 32;               // 32-wide blocks of the head dim
    static constexpr int ES = (BIAS == 0 || BIAS == 6) ? 0 : (BIAS == 1 ? 1 : (BIAS == 4 ? 4 : 2));
    static constexpr int EPC = ES > 0 ? 16 / ES : 8; // bias elements per 16-byte chunk
    static constexpr int STEP_BYTES = BK * D * 2;    // K (or V) rows of one step, unpadded, swizzled
    static constexpr int NKD = STEP_BYTES / 1024;    // 1 KB copies per K (or V) step
    static constexpr int KD = NKD >= 4 ? NKD / 4 : 1;  // of which each wave issues this many
    static constexpr int NKV = LA + 1;               // K/V ring slots
    static constexpr int O_BYTES = BM * OS * 2;
    static constexpr int KV_BYTES = 2 * NKV * STEP_BYTES;
    static constexpr int BCPR = 2 * ES;              // 16-byte chunks per bias row of 32 keys
    static constexpr int BROW = 32 * ES;             // bytes per bias row of a slot
    static constexpr int BSLOT = 32 * BROW;          // one wave's bias slice of one step
    static constexpr int BCH = BSLOT / 1024;         // 1 KB copies per bias slice
    static constexpr int NBS = BIAS == 4 ? 3 : 4;    // bias ring slots per wave
    static constexpr int BIAS_BYTES = 4 * NBS * BSLOT;
    // (the output tile is staged over the K/V slots and, where it is larger, into the bias rings
    // behind them: all of them are dead by then)
    static constexpr int LDS_BYTES = KV_BYTES + BIAS_BYTES > O_BYTES ? KV_BYTES + BIAS_BYTES : O_BYTES;
    // 16-byte chunk c of bias row `row` is stored at chunk c ^ bswz(row): rows that share LDS banks
    // get different chunk orders
    __device__ static __forceinline__ int bswz(int row) {
        return ES == 4 ? ((row >> 1) & 7) : (ES == 2 ? ((row >> 2) & 3) : ((row >> 3) & 1));
    }
    // two work-groups per CU whenever registers and LDS allow it
    static constexpr int MIN_BLOCKS = (D <= 128 && LDS_BYTES <= 81920) ? 2 : 1;
};

// The copy machinery of the kernels tiled by StreamCfg (forward, dQ): one object per thread.
// Completion of the copies is counted by hand: they complete in issue order and every wave issues
// the same number every step, also past the last step (clamped rows, never used).
// WITH_V = false leaves the V rows out (a kernel that only needs K).
template <typename T, int D, int BIAS, bool WITH_V = true> struct KeyStream {
    typedef StreamCfg<D, BIAS> C;
    typedef Swz<D> SW;
    typedef typename BiasElem<BIAS>::type E;
    unsigned char* smem;      // K slots, then V slots, then the bias rings of the four waves
    unsigned char* bias_lds;  // this wave's ring of bias slots
    const T* kp;
    const T* vp;
    const E* bp;              // (batch, head) slices
    int64_t sk, sv, sbm, sbn; // row strides of K and V, row and key stride of the bias (elements)
    int M, N, mw, lane;
    // LEAN (rows of LEAN_CPR chunks): the per-lane offsets of the KD copies are formed from three
    // per-lane constants when a copy is issued, instead of being held in 3 KD registers that such a
    // kernel does not have: a copy of chunk c = 64 ci + l reads row r0 + q (r0 = (64 / CPR) ci, q =
    // l / CPR), chunk (l % CPR) ^ f(r0 + q), and f(r0 + q) = (q << 2) ^ f(r0) with f(r0) the same for
    // every lane (holds for rows of 16 and of 32 chunks).
    // Used at head dim 256; at 128 the kernels have the registers and the extra address arithmetic per
    // copy buys nothing.
    static constexpr bool LEAN = C::CPR == 32;
    unsigned k_off[LEAN ? 1 : C::KD], v_off[LEAN ? 1 : C::KD];
    int c_idx[LEAN ? 1 : C::KD];
    unsigned lean_x16, lean_rk, lean_rv;  // ((l % 32) ^ (g << 2)) * 16, byte offsets of row g of K and of V
    int wave_s;                           // wave index (scalar)
    unsigned lds_kv, lds_bias;  // LDS addresses (scalar) of the K slots and of this wave's bias ring
    // Lean steps (issue_ahead_lean): every row they copy exists, so the copies need no clamps and walk
    // the keys with running 64-bit addresses in scalar registers, one add per step: the K and V rows
    // of the next step to copy, and this wave's bias rows at the first key of the next slice to copy.
    uint64_t run_k, run_v, run_b;
    // byte offset of this lane's chunk in bias copy `it`: with 1- and 2-byte elements the copies of a
    // slice are whole groups of rows apart with the same chunk order, so one offset and a stride do
    static constexpr int NBOFF = C::ES == 4 ? C::BCH : 1;
    unsigned lean_boff[NBOFF];
    // chunk index of copy i of this wave (scalar)
    __device__ __forceinline__ int copy_idx(int i) const { return LEAN ? (wave_s * C::KD + i) % C::NKD : c_idx[i]; }

    // K / V rows of a step: NKD copies of 1 KB each; copy ci fills bytes [1024 ci, 1024 ci + 1024) of
    // the swizzled slot, so lane l of it fetches the chunk that lives at slot position 64 ci + l
    // (row c / CPR, LDS chunk c % CPR holds global chunk (c % CPR) ^ f(row)).  Each wave issues KD
    // of them (more than once where a step has fewer than four).
    __device__ __forceinline__ void init(unsigned char* smem_, const T* kp_, const T* vp_, const E* bp_, int64_t sk_,
                                         int64_t sv_, int64_t sbm_, int64_t sbn_, int M_, int N_, int mw_, int wave, int lane_) {
        smem = smem_; kp = kp_; vp = vp_; bp = bp_; sk = sk_; sv = sv_; sbm = sbm_; sbn = sbn_;
        M = M_; N = N_; mw = mw_; lane = lane_;
        wave = __builtin_amdgcn_readfirstlane(wave);  // the same in every lane: keep it scalar
        bias_lds = smem + C::KV_BYTES + wave * C::NBS * C::BSLOT;
        lds_kv = lds_addr_of(smem);
        lds_bias = lds_kv + C::KV_BYTES + wave * C::NBS * C::BSLOT;
        wave_s = wave;
        if constexpr (LEAN) {
            static_assert(C::CPR == 16 || C::CPR == 32, "rows of 16 or 32 chunks");
            const int q = lane / C::CPR;
            lean_x16 = (unsigned)(((lane % C::CPR) ^ (q << 2)) << 4);
            lean_rk = (unsigned)(q * (int)sk * 2);
            lean_rv = (unsigned)(q * (int)sv * 2);
        } else {
#pragma unroll
            for (int i = 0; i < C::KD; i++) {
                c_idx[i] = (wave * C::KD + i) % C::NKD;
                const int c = c_idx[i] * 64 + lane;
                const int row = c / C::CPR, src = (c % C::CPR) ^ SW::f(row);
                k_off[i] = (unsigned)(row * (int)sk * 2 + src * 16);
                v_off[i] = (unsigned)(row * (int)sv * 2 + src * 16);
            }
        }
    }
    __device__ __forceinline__ const T* k_lds(int k) const { return reinterpret_cast<const T*>(smem + (k % C::NKV) * C::STEP_BYTES); }
    __device__ __forceinline__ const T* v_lds(int k) const { return reinterpret_cast<const T*>(smem + (C::NKV + k % C::NKV) * C::STEP_BYTES); }
    __device__ __forceinline__ unsigned char* b_lds(int k) const { return bias_lds + (k % C::NBS) * C::BSLOT; }
    // the K and V slots by LDS byte address (scalar), for the operand reads by address of Swz
    __device__ __forceinline__ unsigned k_addr(int k) const { return lds_kv + (unsigned)((k % C::NKV) * C::STEP_BYTES); }
    __device__ __forceinline__ unsigned v_addr(int k) const { return lds_kv + (unsigned)((C::NKV + k % C::NKV) * C::STEP_BYTES); }
    // byte offset of bias (row, key .. key + 3) inside a slot
    __device__ static __forceinline__ int b_off(int row, int key) {
        const int byte = key * C::ES;
        return row * C::BROW + (((byte >> 4) ^ C::bswz(row)) << 4) + (byte & 15);
    }

    // Rows past N re-read row N - 1 (their scores are masked); a step past the end is that row
    // over and over, so that offsets never go negative.
    __device__ __forceinline__ void issue_kv(int k) {
        const int n0 = k * C::BK < N ? k * C::BK : N - 1;
        const uint64_t kt = uniform_ptr(kp + (int64_t)n0 * sk);
        const uint64_t vt = uniform_ptr(vp + (int64_t)n0 * sv);
        const unsigned k_dst = lds_kv + (k % C::NKV) * C::STEP_BYTES;
        const unsigned v_dst = lds_kv + (C::NKV + k % C::NKV) * C::STEP_BYTES;
        const bool full = n0 + C::BK <= N;
#pragma unroll
        for (int i = 0; i < C::KD; i++) {
            const int ci = copy_idx(i);
            unsigned ko, vo;
            if constexpr (LEAN) {
                const int r0 = (64 / C::CPR) * ci;  // first of the rows of this copy
                const unsigned x = lean_x16 ^ (unsigned)((((r0 & 3) << 2) | ((r0 >> 2) & 3)) << 4);
                ko = x + lean_rk + (unsigned)(r0 * (int)sk * 2);
                vo = x + lean_rv + (unsigned)(r0 * (int)sv * 2);
            } else {
                ko = k_off[i];
                vo = v_off[i];
            }
            if (!full) {
                // (rare: the lane index passes through an empty asm so that these per-lane values are
                // formed here and not kept in registers across the loops)
                int lane_here = lane;
                asm volatile("" : "+v"(lane_here));
                const int c = ci * 64 + lane_here;
                int row = c / C::CPR;
                const int src = (c % C::CPR) ^ SW::f(row);
                row = row < N - n0 ? row : N - 1 - n0;
                ko = (unsigned)(row * (int)sk * 2 + src * 16);
                vo = (unsigned)(row * (int)sv * 2 + src * 16);
            }
            lds_copy16(kt, ko, k_dst + ci * 1024);
            if constexpr (WITH_V) lds_copy16(vt, vo, v_dst + ci * 1024);
        }
    }
    // Bias slice of this wave for step k (32 rows x 32 keys) -> ring slot k % NBS.  Position c =
    // 64 it + lane of the slot (row c / BCPR, LDS chunk c % BCPR) holds chunk (c % BCPR) ^ bswz(row)
    // of the row.  Rows past M re-read row M - 1 (never stored) and chunks that start past N
    // re-read column 0 (masked).
    __device__ __forceinline__ void issue_bias(int k) {
        if constexpr (C::ES != 0) {
            const unsigned dst = lds_bias + (k % C::NBS) * C::BSLOT;
            const uint64_t base = uniform_ptr(bp);
#pragma unroll
            for (int it = 0; it < C::BCH; it++) {
                const int c = it * 64 + lane;
                const int row = c / C::BCPR;
                int m = mw + row;
                int n = k * C::BK + ((c % C::BCPR) ^ C::bswz(row)) * C::EPC;
                m = m < M ? m : M - 1;
                n = n < N ? n : 0;
                // a (batch, head) slice that takes this path is smaller than 2 GiB
                lds_copy16(base, (unsigned)(((int64_t)m * sbm + n) * C::ES), dst + it * 1024);
            }
        }
    }
    // Points the running addresses at K/V step `k_kv` and bias slice `k_b` (the next ones a lean step issues).
    __device__ __forceinline__ void run_start(int k_kv, int k_b) {
        run_k = uniform_ptr(kp + (int64_t)k_kv * C::BK * sk);
        run_v = uniform_ptr(vp + (int64_t)k_kv * C::BK * sv);
        run_b = 0;
        if constexpr (C::ES != 0) {
            run_b = uniform_ptr(reinterpret_cast<const unsigned char*>(bp) + ((int64_t)mw * sbm + (int64_t)k_b * C::BK) * C::ES);
            // (2-byte elements: a copy covers 16 rows and the chunk order depends on (row / 4) % 4;
            // 1-byte elements: one copy per slice)
            static_assert(C::ES == 4 || C::ES == 2 || C::BCH == 1, "chunk order repeats from copy to copy");
#pragma unroll
            for (int it = 0; it < NBOFF; it++) {
                const int c = it * 64 + lane;
                const int row = c / C::BCPR;
                lean_boff[it] = (unsigned)(((int64_t)row * sbm + ((c % C::BCPR) ^ C::bswz(row)) * C::EPC) * C::ES);
            }
        }
    }
    // issue_ahead for a step whose copies (K/V rows of step k + LA, bias slice of step k + NBS - 1, all
    // 32 rows of this wave) lie wholly inside the tensors; run_start() was called for the first such step
    template <bool BV> __device__ __forceinline__ void issue_ahead_lean(int k) {
        const unsigned saved_m0 = lds_copy_begin();
        settle_ptrs(run_k, run_v, run_b);
        const unsigned k_dst = lds_kv + (unsigned)((k + C::LA) % C::NKV) * C::STEP_BYTES;
        const unsigned v_dst = k_dst + C::NKV * C::STEP_BYTES;
#pragma unroll
        for (int i = 0; i < C::KD; i++) {
            const int ci = copy_idx(i);
            unsigned ko, vo;
            if constexpr (LEAN) {
                const int r0 = (64 / C::CPR) * ci;
                const unsigned x = lean_x16 ^ (unsigned)((((r0 & 3) << 2) | ((r0 >> 2) & 3)) << 4);
                ko = x + lean_rk + (unsigned)(r0 * (int)sk * 2);
                vo = x + lean_rv + (unsigned)(r0 * (int)sv * 2);
            } else {
                ko = k_off[i];
                vo = v_off[i];
            }
            lds_copy16(run_k, ko, k_dst + ci * 1024);
            if constexpr (WITH_V) lds_copy16(run_v, vo, v_dst + ci * 1024);
        }
        run_k += (uint64_t)(C::BK * 2) * (uint64_t)sk;
        run_v += (uint64_t)(C::BK * 2) * (uint64_t)sv;
        if constexpr (BV && C::ES != 0) {
            const unsigned dst = lds_bias + (unsigned)((k + C::NBS - 1) % C::NBS) * C::BSLOT;
#pragma unroll
            for (int it = 0; it < C::BCH; it++) {
                const unsigned off = C::ES == 4 ? lean_boff[it < NBOFF ? it : 0]
                                                : lean_boff[0] + (unsigned)(it * (64 / C::BCPR) * (int)sbm * C::ES);
                lds_copy16(run_b, off, dst + it * 1024);
            }
            run_b += C::BK * C::ES;
        }
        lds_copy_end(saved_m0);
    }
    // lean steps a kernel may run from step 0: those whose copies stay inside N keys (and, with a bias, whose
    // work-group has all of its rows), at most `limit`
    __device__ __forceinline__ int lean_steps(int limit, int wg_rows_end) const {
        constexpr int AHEAD = (C::ES != 0 && C::NBS - 1 > C::LA) ? C::NBS - 1 : C::LA;
        int n = N / C::BK - AHEAD;
        if (C::ES != 0 && wg_rows_end > M) n = 0;
        n = n < limit ? n : limit;
        return n < 0 ? 0 : n;
    }
    // Before the first step, in the order the steps assume: the first bias slices, then K/V of a
    // step followed by the bias slice issued in the same step.  BV: the bias slices come by copy.
    // k0: the first step of the stream (0 unless the keys are split between work-groups)
    template <bool BV> __device__ __forceinline__ void prologue(int k0 = 0) {
        const unsigned saved_m0 = lds_copy_begin();
        if constexpr (BV) {
#pragma unroll
            for (int i = 0; i < C::NBS - 1 - C::LA; i++) issue_bias(k0 + i);
        }
#pragma unroll
        for (int i = 0; i < C::LA; i++) {
            issue_kv(k0 + i);
            if constexpr (BV) issue_bias(k0 + C::NBS - 1 - C::LA + i);
        }
        lds_copy_end(saved_m0);
    }
    // Top of step k: wait for its K/V rows (and with them its bias slice, issued earlier) and
    // publish them.  The slots that step k - 1 read are free from here on.
    template <bool BV> __device__ __forceinline__ void begin_step(int k) {
        static_assert(BIAS == 0 || C::LA < C::NBS - 1, "the bias slice of a step must be issued before its K/V rows");
        constexpr int OPS = (WITH_V ? 2 : 1) * C::KD + (BV ? C::BCH : 0);  // copies per wave per step
        // K/V of this step were issued LA steps ago; the bias copies issued right after them and
        // the copies of the steps since may still be in flight
        wait_vmcnt<(BV ? C::BCH : 0) + OPS*(C::LA - 1)>();
        lds_barrier();
        if constexpr (C::ES != 0 && !BV) {
            // unaligned bias rows or non-unit key stride: one element per lane, 16 rows per lane,
            // RB loads in flight together (clamped addresses instead of branches; what lies outside
            // the bias is masked where it is used)
            if constexpr (D >= 128 && C::ES == 4) {
                // (no register to spare in this variant: one row at a time)
                if (lane < 32) {
#pragma unroll 1
                    for (int row = 0; row < 32; row++) {
                        const int n = k * C::BK + lane;
                        E val = (E)0.f;
                        if (mw + row < M && n < N) val = bp[(int64_t)(mw + row) * sbm + (int64_t)n * sbn];
                        *reinterpret_cast<E*>(b_lds(k) + b_off(row, lane)) = val;
                    }
                }
            } else {
                constexpr int RB = D >= 128 ? 4 : 16;  // as many as the registers of the kernel allow
                const int key = lane & 31;
                int n = k * C::BK + key;
                n = n < N ? n : N - 1;
#pragma unroll 1
                for (int j0 = 0; j0 < 16; j0 += RB) {
                    E vals[RB];
#pragma unroll
                    for (int j = 0; j < RB; j++) {
                        int m = mw + 2 * (j0 + j) + (lane >> 5);
                        m = m < M ? m : M - 1;
                        vals[j] = bp[(int64_t)m * sbm + (int64_t)n * sbn];
                    }
#pragma unroll
                    for (int j = 0; j < RB; j++)
                        *reinterpret_cast<E*>(b_lds(k) + b_off(2 * (j0 + j) + (lane >> 5), key)) = vals[j];
                }
            }
        }
    }
    // Once per step, anywhere after begin_step(k): the copies that go into the slots step k - 1 has
    // left.  Issuing a copy holds the wave while the copies of the other waves drain through the
    // CU's 64 bytes/clock copy path, so the best place is right behind a batch of MFMAs, whose
    // execution then hides it; right after the barrier all waves would queue up at once.
    template <bool BV> __device__ __forceinline__ void issue_ahead(int k) {
        const unsigned saved_m0 = lds_copy_begin();
        issue_kv(k + C::LA);
        if constexpr (BV) issue_bias(k + C::NBS - 1);
        lds_copy_end(saved_m0);
    }
    // After the last step: nothing may land in LDS that is about to be reused.
    __device__ __forceinline__ void drain() {
        wait_vmcnt<0>();
        __syncthreads();
    }
};

// Work-group id -> (tile, batch*head).  Work-groups are dealt round-robin to the 8 XCDs; when
// the number of (batch, head) pairs is a multiple of 8 every tile of one pair is sent to the same
// XCD so that its K/V (or Q/dO) stay in that XCD's L2.
// TILE_MAJOR = false: all tiles of a pair are consecutive (one pair at a time per XCD: the
// streams of a kernel that reads a bias stay together).  TILE_MAJOR = true: tile t of every pair
// comes before tile t + 1 of any; the causal kernels, whose tiles are numbered longest first,
// so start all long tiles before any short one (a greedy schedule with the longest jobs first
// ends near the average load, one that mixes them ends up to one long tile later).
template <bool TILE_MAJOR = false>
__device__ __forceinline__ void decode_block(int id, int n_tiles, int BH, int& tile, int& bh) {
    if ((BH & 7) == 0) {
        const int xcd = id & 7, slot = id >> 3, per_xcd = BH >> 3;
        if (TILE_MAJOR) {
            tile = slot / per_xcd;
            bh = (slot % per_xcd) * 8 + xcd;
        } else {
            bh = (slot / n_tiles) * 8 + xcd;
            tile = slot % n_tiles;
        }
    } else if (TILE_MAJOR) {
        tile = id / BH;
        bh = id % BH;
    } else {
        bh = id / n_tiles;
        tile = id % n_tiles;
    }
}

}  // namespace fa
