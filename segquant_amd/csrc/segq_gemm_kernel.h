// Segmented GEMM on CDNA4 MFMA with fused de-quantisation and bias.
//
// One workgroup computes a BM x BN tile of the output.  The contraction walks a
// list of "ranges" (runs of K that share one pair of scales) in steps of 128
// code bytes.  Each step's activation and weight tiles are staged through LDS,
// double-buffered, 16-byte chunks XOR-swizzled so that both the staging writes
// and the MFMA fragment reads are free of bank conflicts.  Operands are handed
// to the MFMA in swapped roles (weights as the first operand, activations as
// the second) so that each lane's four accumulator registers are four
// CONSECUTIVE output columns of one output row: the epilogue then scales,
// adds bias, rounds once and stores 8 bytes (bf16) per lane.
//
//   int8 x int8    v_mfma_i32_16x16x64_i8          int32 accumulators
//   e4m3 x e4m3    v_mfma_f32_16x16x128_f8f6f4     fp32 accumulators
//   int8 x int4    weights unpacked to int8 (times 16) while they are staged
//                  into LDS; the factor 16 is exact and is shifted out again
//
// With more than one range the accumulator of a finished range is folded into
// an fp32 accumulator, multiplied by 1 / (sx * sw) of that range.
#pragma once
#include "segq_common.h"

namespace segq {

struct KRange {
    int32_t k0, k1;
    int32_t a_sel;
    int32_t sx_rs;
    int32_t sw_cs;
    int32_t pad;
    const float* sx;
    const float* sw;
};

struct GemmParams {
    const uint8_t* A;
    const uint8_t* A2;
    const uint8_t* B;
    void* C;
    const void* bias;
    int32_t M, N;
    int64_t lda, ldb, ldc;
    int64_t bsA, bsB, bsC, bsSx, bsSw;
    int32_t out_dtype, bias_dtype;
    int32_t nr;
    int32_t tiles_m, tiles_n, group_m;
    int32_t vec_store;    // output rows allow 4-element vector stores
    int32_t vec_store16;  // 16-bit output rows allow 16-byte stores
    const void* addend;   // (M, N) tensor of the output's dtype added before the one rounding, or null
    int64_t ldadd;
    int32_t vec_add;      // its rows allow 4-element vector loads
    int32_t pad2_;
    int32_t splits;       // > 1: grid.y workgroups share the K steps of a tile (gemm_pipe_kernel only)
    int32_t rot;          // several ranges, no K split: XCD x starts its walk at range x mod nr (gemm_pipe_kernel only)
    float* park;          // fp32 workspace, one tile-sized slot per workgroup, for finished ranges (or null)
    float* part;          // splits == 2 finished in the launch: two tile-sized fp32 shares per tile (or null)
    unsigned int* arrived;  // ... and one word per tile: the first of the two workgroups leaves `stamp` there
    unsigned int stamp;     // differs from launch to launch
    unsigned int pad4_;
    const float* grw;     // group-wise de-quantisation factors [K / 128][grw_gs], or null
    int64_t grw_gs;
    const uint16_t* lr_t;   // low-rank branch: T (M x lr_rank) and L2^T (N x lr_rank) in the output's 16-bit dtype, or null
    const uint16_t* lr_l2;
    int64_t lr_ldt, lr_ldl;  // their row strides in elements
    int32_t lr_rank;         // multiple of 32; 0: no low-rank branch
    void* oc;                // codes instead of floats: the (M, N) code tensor, or null
    void* oc_neg;            // DualScale: the second code tensor (Xn), or null
    int64_t ldoc;            // their row stride in bytes
    const float* oc_scale;   // one multiplicative scale (x >= 0, or everything when oc_neg is null)
    const float* oc_scale_neg;
    int32_t oc_fmt, oc_pre;  // segq_code (I8 / E4M3), segq_pre_op
    int32_t oc_vec;          // rows allow 8-byte stores
    int32_t pad3_;
    int32_t dry;             // host only: walk the dispatch down to the kernel instance, launch nothing (segq_gemm_plan)
    KRange r[SEGQ_MAX_RANGES];
};

enum { GEMM_I8 = 0, GEMM_F8 = 1 };

// o[0..3] += addend[z][m][n .. n + 3] (columns beyond N skipped)
__device__ __forceinline__ void add_addend4(const GemmParams& p, int64_t z, int m, int n, float (&o)[4]) {
    if (!p.addend) return;
    const int64_t e = z * p.bsC + (int64_t)m * p.ldadd + n;
    if (p.out_dtype == SEGQ_F32) {
        const float* q = static_cast<const float*>(p.addend) + e;
        if (p.vec_add && n + 3 < p.N) {
            const float4 t = *reinterpret_cast<const float4*>(q);
            o[0] += t.x; o[1] += t.y; o[2] += t.z; o[3] += t.w;
        } else {
#pragma unroll
            for (int v = 0; v < 4; ++v)
                if (n + v < p.N) o[v] += q[v];
        }
    } else {
        const uint16_t* q = static_cast<const uint16_t*>(p.addend) + e;
        uint32_t h[4] = {0, 0, 0, 0};
        if (p.vec_add && n + 3 < p.N) {
            const uint2 t = *reinterpret_cast<const uint2*>(q);
            h[0] = t.x & 0xffffu; h[1] = t.x >> 16; h[2] = t.y & 0xffffu; h[3] = t.y >> 16;
        } else {
#pragma unroll
            for (int v = 0; v < 4; ++v)
                if (n + v < p.N) h[v] = q[v];
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) o[v] += (p.out_dtype == SEGQ_BF16) ? bf16_bits_to_f32(h[v]) : f16_bits_to_f32(h[v]);
    }
}
// acc / (sx sw) + bias as the epilogues evaluate it: the row factor first, then one fused
// multiply-add with the column factor and the bias.  One definition, no contraction left to the
// compiler: the epilogue that stores floats and the one that stores codes must round alike.
__device__ __forceinline__ float dequant_bias(float acc, float rx, float rw, float bias) {
#pragma clang fp contract(off)
    return __builtin_fmaf(acc * rx, rw, bias);
}

constexpr int BK = 128;  // code bytes of K per step

// Chunk swizzle.  The LDS of gfx950 has 64 banks of 4 bytes (a 256-byte span),
// so a 128-byte row covers half of them and rows 2j and 2j+1 cover different
// halves.  XOR-ing the 16-byte chunk index with (row >> 1) & 7 makes the MFMA
// fragment reads (16 or 32 consecutive rows at one logical chunk) and the
// staging writes (8 lanes across one row) free of bank conflicts; measured with
// a four-wave ds_read_b128 loop: 18 clocks per instruction against 32 for
// row & 7 on 32-row fragments and 64 without a swizzle.
__device__ __forceinline__ int swz(int row) { return (row >> 1) & 7; }

// 0xFF in every byte of x whose top bit is set.
__device__ __forceinline__ uint32_t neg_byte_mask(uint32_t x) { return ((x >> 7) & 0x01010101u) * 0xFFu; }

__device__ __forceinline__ uint4 select_sign(uint4 v, int a_sel) {
    if (a_sel == 2) {
        v.x &= ~neg_byte_mask(v.x); v.y &= ~neg_byte_mask(v.y);
        v.z &= ~neg_byte_mask(v.z); v.w &= ~neg_byte_mask(v.w);
    } else if (a_sel == 3) {
        v.x &= neg_byte_mask(v.x); v.y &= neg_byte_mask(v.y);
        v.z &= neg_byte_mask(v.z); v.w &= neg_byte_mask(v.w);
    }
    return v;
}

// Eight packed nibbles (element 0 lowest) -> eight bytes holding value * 16.
__device__ __forceinline__ void unpack8_i4x16(uint32_t w, uint32_t& o0, uint32_t& o1) {
    const uint32_t ev = (w << 4) & 0xF0F0F0F0u;  // elements 0,2,4,6
    const uint32_t od = w & 0xF0F0F0F0u;         // elements 1,3,5,7
    o0 = (ev & 0xFFu) | ((od & 0xFFu) << 8) | ((ev & 0xFF00u) << 8) | ((od & 0xFF00u) << 16);
    o1 = ((ev >> 16) & 0xFFu) | (((od >> 16) & 0xFFu) << 8) | (((ev >> 16) & 0xFF00u) << 8) | (((od >> 16) & 0xFF00u) << 16);
}

template <int FMT> struct AccT;
template <> struct AccT<GEMM_I8> { typedef v4i type; typedef int32_t elem; };
template <> struct AccT<GEMM_F8> { typedef v4f type; typedef float elem; };

template <int BM, int BN, int WGM, int WGN, int FMT, bool B4, bool FOLD>
__global__ void __launch_bounds__(WGM* WGN * 64) gemm_kernel(const GemmParams p) {
    constexpr int NT = WGM * WGN * 64;
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int TM = WM / 16, TN = WN / 16;
    constexpr int A_IT = BM * 8 / NT;
    constexpr int B_IT = (B4 ? BN * 4 : BN * 8) / NT;
    static_assert(BM * 8 % NT == 0 && BN * 4 % NT == 0, "tile does not divide over the threads");
    static_assert((NT / 8) % 16 == 0, "row swizzle must not depend on the load iteration");
    static_assert(!B4 || FMT == GEMM_I8, "int4 weights pair with int8 activations");
    typedef typename AccT<FMT>::type acc_t;
    typedef typename AccT<FMT>::elem acc_e;
    const acc_t acc_zero = {0, 0, 0, 0};

    extern __shared__ __align__(16) uint8_t smem[];
    uint8_t* const As = smem;                 // [2][BM][128]
    uint8_t* const Bs = smem + 2 * BM * BK;   // [2][BN][128]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave % WGM, wn = wave / WGM;
    const int lrow = lane & 15, lgrp = lane >> 4;

    // ---- which output tile: spread consecutive tiles of a group over one XCD
    int bid = blockIdx.x;
    {
        const int nb = p.tiles_m * p.tiles_n;
        if ((nb & 7) == 0) bid = (bid & 7) * (nb >> 3) + (bid >> 3);
    }
    int tile_m, tile_n;
    {
        const int gsz = p.group_m * p.tiles_n;
        const int g = bid / gsz;
        const int first_m = g * p.group_m;
        const int rows_in_group = min(p.tiles_m - first_m, p.group_m);
        const int in_g = bid - g * gsz;
        tile_m = first_m + in_g % rows_in_group;
        tile_n = in_g / rows_in_group;
    }
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int64_t z = blockIdx.y;

    const uint8_t* const Ab = p.A + z * p.bsA;
    const uint8_t* const A2b = p.A2 ? p.A2 + z * p.bsA : nullptr;
    const uint8_t* const Bb = p.B + z * p.bsB;

    // ---- staging assignment: 8 consecutive lanes cover one 128-byte row
    const int a_ch = tid & 7;
    const int a_r0 = tid >> 3;
    const int a_lds = a_r0 * BK + ((a_ch ^ swz(a_r0)) << 4);
    int64_t a_goff[A_IT];
#pragma unroll
    for (int i = 0; i < A_IT; ++i) a_goff[i] = (int64_t)min(m0 + a_r0 + i * (NT / 8), p.M - 1) * p.lda + a_ch * 16;

    const int b_ch = B4 ? (tid & 3) : (tid & 7);
    const int b_r0 = B4 ? (tid >> 2) : (tid >> 3);
    constexpr int B_RSTEP = B4 ? NT / 4 : NT / 8;
    int64_t b_goff[B_IT];
#pragma unroll
    for (int i = 0; i < B_IT; ++i) b_goff[i] = (int64_t)min(n0 + b_r0 + i * B_RSTEP, p.N - 1) * p.ldb + b_ch * 16;
    const int b_sw = swz(b_r0);

    uint4 ra[A_IT], rb[B_IT];

    auto load_tile = [&](int r, int k) {
        const int k1 = p.r[r].k1;
        const uint8_t* ap = (p.r[r].a_sel == 1) ? A2b : Ab;
        const bool a_ok = (k + a_ch * 16) < k1;
#pragma unroll
        for (int i = 0; i < A_IT; ++i)
            ra[i] = a_ok ? *reinterpret_cast<const uint4*>(ap + a_goff[i] + k) : make_uint4(0, 0, 0, 0);
        if constexpr (B4) {
            const bool b_ok = (k + b_ch * 32) < k1;
#pragma unroll
            for (int i = 0; i < B_IT; ++i)
                rb[i] = b_ok ? *reinterpret_cast<const uint4*>(Bb + b_goff[i] + (k >> 1)) : make_uint4(0, 0, 0, 0);
        } else {
            const bool b_ok = (k + b_ch * 16) < k1;
#pragma unroll
            for (int i = 0; i < B_IT; ++i)
                rb[i] = b_ok ? *reinterpret_cast<const uint4*>(Bb + b_goff[i] + k) : make_uint4(0, 0, 0, 0);
        }
    };

    auto store_tile = [&](int buf, int a_sel) {
        uint8_t* as = As + buf * BM * BK + a_lds;
#pragma unroll
        for (int i = 0; i < A_IT; ++i)
            *reinterpret_cast<uint4*>(as + i * (NT / 8) * BK) = select_sign(ra[i], a_sel);
        uint8_t* bs = Bs + buf * BN * BK + b_r0 * BK;
        if constexpr (B4) {
#pragma unroll
            for (int i = 0; i < B_IT; ++i) {
                uint4 lo, hi;
                unpack8_i4x16(rb[i].x, lo.x, lo.y);
                unpack8_i4x16(rb[i].y, lo.z, lo.w);
                unpack8_i4x16(rb[i].z, hi.x, hi.y);
                unpack8_i4x16(rb[i].w, hi.z, hi.w);
                uint8_t* row = bs + i * B_RSTEP * BK;
                *reinterpret_cast<uint4*>(row + (((2 * b_ch) ^ b_sw) << 4)) = lo;
                *reinterpret_cast<uint4*>(row + (((2 * b_ch + 1) ^ b_sw) << 4)) = hi;
            }
        } else {
#pragma unroll
            for (int i = 0; i < B_IT; ++i)
                *reinterpret_cast<uint4*>(bs + i * B_RSTEP * BK + ((b_ch ^ b_sw) << 4)) = rb[i];
        }
    };

    // ---- accumulators
    acc_t acc[TN][TM];
    v4f accf[FOLD ? TN : 1][FOLD ? TM : 1];
#pragma unroll
    for (int a = 0; a < TN; ++a)
#pragma unroll
        for (int b = 0; b < TM; ++b) acc[a][b] = acc_zero;
    if constexpr (FOLD) {
#pragma unroll
        for (int a = 0; a < TN; ++a)
#pragma unroll
            for (int b = 0; b < TM; ++b) accf[a][b] = v4f{0.f, 0.f, 0.f, 0.f};
    }

    const int f_sw = swz(lrow);
    const int a_frag = (wm * WM + lrow) * BK;  // + tm * 16 * BK
    const int b_frag = (wn * WN + lrow) * BK;  // + tn * 16 * BK

    auto compute = [&](int buf) {
        const uint8_t* as = As + buf * BM * BK + a_frag;
        const uint8_t* bs = Bs + buf * BN * BK + b_frag;
        if constexpr (FMT == GEMM_I8) {
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const int off = ((ks * 4 + lgrp) ^ f_sw) << 4;
                v4i fa[TM], fb[TN];
#pragma unroll
                for (int t = 0; t < TM; ++t) fa[t] = *reinterpret_cast<const v4i*>(as + t * 16 * BK + off);
#pragma unroll
                for (int t = 0; t < TN; ++t) fb[t] = *reinterpret_cast<const v4i*>(bs + t * 16 * BK + off);
#pragma unroll
                for (int a = 0; a < TN; ++a)
#pragma unroll
                    for (int b = 0; b < TM; ++b)
                        acc[a][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb[a], fa[b], acc[a][b], 0, 0, 0);
            }
        } else {
            // (K slot g of the MFMA gets 16-byte pieces g and 4 + g of the step, for both operands:
            // the int8 path's conflict-free read pattern)
            const int off0 = (lgrp ^ f_sw) << 4;
            const int off1 = ((4 + lgrp) ^ f_sw) << 4;
            v8i fa[TM], fb[TN];
#pragma unroll
            for (int t = 0; t < TM; ++t) {
                const v4i lo = *reinterpret_cast<const v4i*>(as + t * 16 * BK + off0);
                const v4i hi = *reinterpret_cast<const v4i*>(as + t * 16 * BK + off1);
                fa[t] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            }
#pragma unroll
            for (int t = 0; t < TN; ++t) {
                const v4i lo = *reinterpret_cast<const v4i*>(bs + t * 16 * BK + off0);
                const v4i hi = *reinterpret_cast<const v4i*>(bs + t * 16 * BK + off1);
                fb[t] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            }
#pragma unroll
            for (int a = 0; a < TN; ++a)
#pragma unroll
                for (int b = 0; b < TM; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[a], fa[b], acc[a][b], 0, 0, 0, 0, 0, 0);
        }
    };

    // Output coordinates of this lane: row m_of(tm), columns n_of(tn) .. +3.
    const int m_base = m0 + wm * WM + lrow;
    const int n_base = n0 + wn * WN + 4 * lgrp;

    // 1 / (sx * sw) factors of range r for this lane's rows and columns.
    auto range_rx = [&](int r, float (&rx)[TM]) {
        const float* sx = p.r[r].sx + z * p.bsSx;
        const int rs = p.r[r].sx_rs;
#pragma unroll
        for (int b = 0; b < TM; ++b) rx[b] = 1.0f / sx[(int64_t)min(m_base + b * 16, p.M - 1) * rs];
    };
    auto range_rw = [&](int r, int a, float (&rw)[4]) {
        const float* sw = p.r[r].sw + z * p.bsSw;
        const int cs = p.r[r].sw_cs;
        // the factor 16 of the staged int4 weights is exact and removed here
        const float unscale = B4 ? 0.0625f : 1.0f;
#pragma unroll
        for (int v = 0; v < 4; ++v) rw[v] = unscale / sw[(int64_t)min(n_base + a * 16 + v, p.N - 1) * cs];
    };

    auto fold = [&](int r) {
        if constexpr (FOLD) {
            float rx[TM];
            range_rx(r, rx);
#pragma unroll
            for (int a = 0; a < TN; ++a) {
                float rw[4];
                range_rw(r, a, rw);
#pragma unroll
                for (int b = 0; b < TM; ++b) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) accf[a][b][v] += (float)acc[a][b][v] * rx[b] * rw[v];
                    acc[a][b] = acc_zero;
                }
            }
        }
    };

    // ---- main loop over (range, k) steps
    int r = 0, k = p.r[0].k0;
    load_tile(r, k);
    store_tile(0, p.r[0].a_sel);
    __syncthreads();
    int buf = 0;
    while (true) {
        int rn = r, kn = k + BK;
        const bool range_done = kn >= p.r[r].k1;
        if (range_done) {
            rn = r + 1;
            kn = (rn < p.nr) ? p.r[rn].k0 : 0;
        }
        const bool more = rn < p.nr;
        if (more) load_tile(rn, kn);
        compute(buf);
        if (FOLD && range_done) fold(r);
        if (!more) break;
        store_tile(buf ^ 1, p.r[rn].a_sel);
        __syncthreads();
        buf ^= 1;
        r = rn;
        k = kn;
    }

    // ---- epilogue
    const int64_t c_off = z * p.bsC;
    if (p.out_dtype == SEGQ_ACC) {
        // raw accumulators of the single range
#pragma unroll
        for (int a = 0; a < TN; ++a)
#pragma unroll
            for (int b = 0; b < TM; ++b) {
                const int m = m_base + b * 16, n = n_base + a * 16;
                if (m >= p.M) continue;
                acc_t t = acc[a][b];
                if constexpr (B4) { t[0] >>= 4; t[1] >>= 4; t[2] >>= 4; t[3] >>= 4; }
                acc_e* dst = static_cast<acc_e*>(p.C) + c_off + (int64_t)m * p.ldc + n;
                if (p.vec_store && n + 3 < p.N) {
                    *reinterpret_cast<acc_t*>(dst) = t;
                } else {
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        if (n + v < p.N) dst[v] = t[v];
                }
            }
        return;
    }

    float rx[TM];
    if constexpr (!FOLD) range_rx(0, rx);
#pragma unroll
    for (int a = 0; a < TN; ++a) {
        float rw[4];
        if constexpr (!FOLD) range_rw(0, a, rw);
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
        if (p.bias) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int n = min(n_base + a * 16 + v, p.N - 1);
                if (p.bias_dtype == SEGQ_F32) bv[v] = static_cast<const float*>(p.bias)[n];
                else if (p.bias_dtype == SEGQ_BF16) bv[v] = bf16_bits_to_f32(static_cast<const uint16_t*>(p.bias)[n]);
                else bv[v] = f16_bits_to_f32(static_cast<const uint16_t*>(p.bias)[n]);
            }
        }
#pragma unroll
        for (int b = 0; b < TM; ++b) {
            const int m = m_base + b * 16, n = n_base + a * 16;
            if (m >= p.M || n >= p.N) continue;
            float o[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                if constexpr (FOLD) o[v] = accf[a][b][v] + bv[v];
                else o[v] = dequant_bias((float)acc[a][b][v], rx[b], rw[v], bv[v]);
            }
            add_addend4(p, z, m, n, o);
            const int64_t e = c_off + (int64_t)m * p.ldc + n;
            const bool vec = p.vec_store && (n + 3 < p.N);
            if (p.out_dtype == SEGQ_F32) {
                float* dst = static_cast<float*>(p.C) + e;
                if (vec) *reinterpret_cast<float4*>(dst) = make_float4(o[0], o[1], o[2], o[3]);
                else
#pragma unroll
                    for (int v = 0; v < 4; ++v) if (n + v < p.N) dst[v] = o[v];
            } else {
                uint32_t h[4];
#pragma unroll
                for (int v = 0; v < 4; ++v) h[v] = (p.out_dtype == SEGQ_BF16) ? f32_to_bf16_bits(o[v]) : f32_to_f16_bits(o[v]);
                uint16_t* dst = static_cast<uint16_t*>(p.C) + e;
                if (vec) *reinterpret_cast<uint2*>(dst) = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
                else
#pragma unroll
                    for (int v = 0; v < 4; ++v) if (n + v < p.N) dst[v] = (uint16_t)h[v];
            }
        }
    }
}

// ---- host-side launch of one (format, tile, fold) instance -------------------
struct TileCfg { int bm, bn, wgm, wgn; };
constexpr int NUM_TILE_CFG = 21;
constexpr int FIRST_BIG_CFG = 8;    // two retired ids (a 4-wave 256 x 256 kernel that no shape profited from)
constexpr int FIRST_WIDE_CFG = 10;  // the 8-wave kernels from here on (segq_gemm_wide.h)
constexpr TileCfg TILE_CFGS[NUM_TILE_CFG] = {
    {256, 256, 2, 2}, {256, 128, 2, 2}, {128, 128, 2, 2}, {64, 128, 2, 2}, {128, 256, 2, 2},
    {256, 256, 2, 4}, {256, 256, 4, 2}, {256, 128, 4, 2}, {256, 256, 2, 2}, {256, 256, 2, 2},
    {256, 256, 4, 2}, {256, 128, 4, 2}, {128, 256, 2, 4}, {128, 128, 2, 4}, {192, 288, 4, 2}, {288, 192, 2, 4},
    {256, 192, 4, 2}, {192, 256, 2, 4}, {128, 128, 2, 4}, {384, 192, 4, 2}, {128, 96, 4, 2},
};

template <int BM, int BN, int WGM, int WGN, int FMT, bool B4, bool FOLD>
int launch_instance(const GemmParams& p, int64_t batch, hipStream_t st) {
    auto kern = gemm_kernel<BM, BN, WGM, WGN, FMT, B4, FOLD>;
    constexpr int lds = 2 * (BM + BN) * BK;
    if (p.dry) return SEGQ_OK;
    static unsigned long long attr_done = 0;
    if (const int rc = reserve_lds(reinterpret_cast<const void*>(kern), lds, &attr_done)) return rc;
    dim3 grid((unsigned)(p.tiles_m * p.tiles_n), (unsigned)batch);
    hipLaunchKernelGGL(kern, grid, dim3(WGM * WGN * 64), lds, st, p);
    return check_launch("segq_gemm");
}

template <int FMT, bool B4>
int launch_wide(const GemmParams& p, int wcfg, bool fold, bool asel, int64_t batch, hipStream_t st);

template <int FMT, bool B4>
int launch_format(const GemmParams& p, int cfg, bool fold, int64_t batch, hipStream_t st) {
    if (cfg >= FIRST_WIDE_CFG) {
        bool asel = false;
        for (int i = 0; i < p.nr; ++i) asel = asel || p.r[i].a_sel >= 2;
        return launch_wide<FMT, B4>(p, cfg - FIRST_WIDE_CFG, fold, asel, batch, st);
    }
    if (cfg == FIRST_BIG_CFG || cfg == FIRST_BIG_CFG + 1)
        return fail(SEGQ_ERR_UNSUPPORTED, "segq_gemm: tile ids %d and %d are retired", FIRST_BIG_CFG + 1, FIRST_BIG_CFG + 2);
    switch (cfg * 2 + (fold ? 1 : 0)) {
        case 0: return launch_instance<256, 256, 2, 2, FMT, B4, false>(p, batch, st);
        case 2: return launch_instance<256, 128, 2, 2, FMT, B4, false>(p, batch, st);
        case 3: return launch_instance<256, 128, 2, 2, FMT, B4, true>(p, batch, st);
        case 4: return launch_instance<128, 128, 2, 2, FMT, B4, false>(p, batch, st);
        case 5: return launch_instance<128, 128, 2, 2, FMT, B4, true>(p, batch, st);
        case 6: return launch_instance<64, 128, 2, 2, FMT, B4, false>(p, batch, st);
        case 7: return launch_instance<64, 128, 2, 2, FMT, B4, true>(p, batch, st);
        case 8: return launch_instance<128, 256, 2, 2, FMT, B4, false>(p, batch, st);
        case 9: return launch_instance<128, 256, 2, 2, FMT, B4, true>(p, batch, st);
        case 10: return launch_instance<256, 256, 2, 4, FMT, B4, false>(p, batch, st);
        case 12: return launch_instance<256, 256, 4, 2, FMT, B4, false>(p, batch, st);
        case 14: return launch_instance<256, 128, 4, 2, FMT, B4, false>(p, batch, st);
        case 15: return launch_instance<256, 128, 4, 2, FMT, B4, true>(p, batch, st);
    }
    return fail(SEGQ_ERR_UNSUPPORTED, "segq_gemm: no kernel for tile %d%s", cfg + 1, fold ? " with several ranges" : "");
}

// one translation unit per operand format
int launch_gemm_i8(const GemmParams& p, int cfg, bool fold, int64_t batch, hipStream_t st);
int launch_gemm_f8(const GemmParams& p, int cfg, bool fold, int64_t batch, hipStream_t st);
int launch_gemm_w4(const GemmParams& p, int cfg, bool fold, int64_t batch, hipStream_t st);

}  // namespace segq
