// Segmented GEMM, main kernel: eight waves per workgroup, K walked in whole
// 128-byte steps, operands streamed global -> LDS without passing through
// registers wherever no per-byte transform is needed.
//
// Design points, each backed by a measurement on MI355X:
//  * Two waves per SIMD.  The 4-pass v_mfma_i32_16x16x64_i8 issued back to back
//    from ONE wave reaches 56 % of the matrix pipe's rate, from two waves 90 %.
//  * global_load_lds_dwordx4 for plain operands: no staging VGPRs, no ds_write
//    instructions (ds_write_b128 moves ~80 B/clk/CU, a third of what reads do),
//    and nothing in the loop consumes a loaded value, so the loads of step k+1
//    really overlap the MFMAs of step k.  The LDS side of such a load is
//    lane-linear, so the bank swizzle is applied to the global address instead.
//  * Activations that need sign selection (merged DualScale codes) and int4
//    weights go through registers; their transform is branch-free.
//  * Epilogue through LDS for 16-bit outputs: each lane owns 4 consecutive
//    columns of 16 different rows, which as direct stores are 32-byte pieces of
//    16 lines per instruction (measured 1.7 TB/s); transposed through a private
//    LDS patch every store instruction writes four full 256-byte row pieces.
#pragma once
#include "segq_gemm_kernel.h"
#include "segq_encode.h"
#include <type_traits>

namespace segq {

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* glb_ptr_t;

// One lane's 16 bytes from global memory to LDS at lds_base + lane * 16.
__device__ __forceinline__ void load16_to_lds(const uint8_t* g, uint8_t* lds_base) {
    __builtin_amdgcn_global_load_lds((glb_ptr_t)g, (lds_ptr_t)lds_base, 16, 0, 0);
}

// Four consecutive outputs of one row, rounded once to the output type.
template <int OUT>
__device__ __forceinline__ void store4(void* C, int64_t e, const float (&o)[4], bool vec, int n_left) {
    if constexpr (OUT == SEGQ_F32) {
        float* dst = static_cast<float*>(C) + e;
        if (vec) {
            *reinterpret_cast<float4*>(dst) = make_float4(o[0], o[1], o[2], o[3]);
        } else {
#pragma unroll
            for (int v = 0; v < 4; ++v)
                if (v < n_left) dst[v] = o[v];
        }
    } else {
        const uint32_t lo = (OUT == SEGQ_BF16) ? pack2_bf16(o[0], o[1]) : pack2_f16(o[0], o[1]);
        const uint32_t hi = (OUT == SEGQ_BF16) ? pack2_bf16(o[2], o[3]) : pack2_f16(o[2], o[3]);
        uint16_t* dst = static_cast<uint16_t*>(C) + e;
        if (vec) {
            *reinterpret_cast<uint2*>(dst) = make_uint2(lo, hi);
        } else {
            const uint32_t h[4] = {lo & 0xffffu, lo >> 16, hi & 0xffffu, hi >> 16};
#pragma unroll
            for (int v = 0; v < 4; ++v)
                if (v < n_left) dst[v] = (uint16_t)h[v];
        }
    }
}


// Four codes of fmt from four values (already scaled), low byte first.
__device__ __forceinline__ uint32_t pack4_codes(int fmt, float a, float b, float c, float d) {
    return fmt == SEGQ_CODE_I8 ? pack4_i8(a, b, c, d) : pack4_e4m3(a, b, c, d);
}

// The epilogue that writes CODES: what a quantise launch with a static per-tensor scale (or a
// DualScale pair, two code tensors) and a fused activation function would have made of this
// GEMM's 16-bit output, bit for bit: the de-quantised sum plus bias (and addend) is rounded to
// out_dtype, the activation function applied in fp32 and rounded to out_dtype again, then
// scaled and encoded.  The float output itself is never written to memory: every wave passes
// 16 rows at a time through its own LDS patch in out_dtype (which is also the transposition that
// gives each lane eight consecutive columns of one row), reads them back, and stores eight
// codes per lane.  epi: the tile's vectors parked in LDS, [1/sx BM | 1/sw BN | bias BN].
template <int BM, int BN, int WGM, int WGN, int FMT>
__device__ __forceinline__ void codes_epilogue(const GemmParams& p, typename AccT<FMT>::type (&acc)[BN / WGN / 16][BM / WGM / 16],
                                               uint8_t* smem, int m0, int n0, int wave, int lane, const float* epi) {
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int TM = WM / 16, TN = WN / 16;
    const int wm = wave % WGM, wn = wave / WGM;
    const int lrow = lane & 15, lgrp = lane >> 4;
    const int m_base = m0 + wm * WM + lrow;
    const int n_base = n0 + wn * WN + 4 * lgrp;
    const bool dual = p.oc_neg != nullptr;
    const float s_pos = p.oc_scale[0];
    const float s_neg = dual ? p.oc_scale_neg[0] : s_pos;
    const bool bf = p.out_dtype == SEGQ_BF16;
    const int dt = p.out_dtype, fmt = p.oc_fmt, op = p.oc_pre;
    constexpr int RS = WN * 2 + 16;  // patch row stride in bytes; the 16 spreads the rows over the banks
    constexpr int CH = WN / 8;       // 8-element pieces per patch row
    __syncthreads();                 // the operand tiles are dead from here on
    uint8_t* const patch = smem + wave * 16 * RS;
    uint8_t* const ocp = static_cast<uint8_t*>(p.oc);
    uint8_t* const ocn = static_cast<uint8_t*>(p.oc_neg);
    // the 16 rows in the patch -> codes.  A real loop over b would have to index the accumulators, so
    // the blocks below are unrolled, each followed by this loop
    auto encode_rows = [&](int b) __attribute__((always_inline)) {
        for (int j = 0; j < (16 * CH + 63) / 64; ++j) {
            const int c = j * 64 + lane;
            const int row = c / CH, col = c % CH;
            if ((16 * CH) % 64 != 0 && c >= 16 * CH) continue;
            const uint4 raw = *reinterpret_cast<const uint4*>(patch + row * RS + col * 16);
            const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
            float cp[8], cn[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t h = (i & 1) ? (w[i >> 1] >> 16) : (w[i >> 1] & 0xffffu);
                float t = bf ? bf16_bits_to_f32(h) : f16_bits_to_f32(h);
                if (op != SEGQ_PRE_NONE) t = round_to(dt, act_value(op, t));
                // x >= 0 takes the positive scale; the branch not taken holds code(0)
                // (segquant/src/real_quant/quantizer.cuh:193-203).  One tensor: one scale for both signs.
                cp[i] = dual ? (t >= 0.0f ? t * s_pos : 0.0f) : t * s_pos;
                cn[i] = (t >= 0.0f) ? 0.0f : t * s_neg;
            }
            const int mm = m0 + wm * WM + b * 16 + row;
            const int n = n0 + wn * WN + col * 8;
            if (mm >= p.M || n >= p.N) continue;
            const int64_t e = (int64_t)mm * p.ldoc + n;
            const uint2 vp = make_uint2(pack4_codes(fmt, cp[0], cp[1], cp[2], cp[3]), pack4_codes(fmt, cp[4], cp[5], cp[6], cp[7]));
            uint2 vn = make_uint2(0u, 0u);
            if (dual) vn = make_uint2(pack4_codes(fmt, cn[0], cn[1], cn[2], cn[3]), pack4_codes(fmt, cn[4], cn[5], cn[6], cn[7]));
            if (p.oc_vec && n + 7 < p.N) {
                *reinterpret_cast<uint2*>(ocp + e) = vp;
                if (dual) *reinterpret_cast<uint2*>(ocn + e) = vn;
            } else {
                const uint64_t bp = ((uint64_t)vp.y << 32) | vp.x, bn = ((uint64_t)vn.y << 32) | vn.x;
                for (int i = 0; i < 8 && n + i < p.N; ++i) {
                    ocp[e + i] = (uint8_t)(bp >> (8 * i));
                    if (dual) ocn[e + i] = (uint8_t)(bn >> (8 * i));
                }
            }
        }
    };
#pragma unroll
    for (int b = 0; b < TM; ++b) {
        const float rx = epi[wm * WM + b * 16 + lrow];
#pragma unroll
        for (int a = 0; a < TN; ++a) {
            const v4f rw = *reinterpret_cast<const v4f*>(epi + BM + wn * WN + a * 16 + 4 * lgrp);
            const v4f bias = *reinterpret_cast<const v4f*>(epi + BM + BN + wn * WN + a * 16 + 4 * lgrp);
            float o[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) o[v] = dequant_bias((float)acc[a][b][v], rx, rw[v], bias[v]);
            if (p.addend) add_addend4(p, 0, min(m_base + b * 16, p.M - 1), n_base + a * 16, o);
            *reinterpret_cast<uint2*>(patch + lrow * RS + (a * 16 + 4 * lgrp) * 2) =
                make_uint2(bf ? pack2_bf16(o[0], o[1]) : pack2_f16(o[0], o[1]), bf ? pack2_bf16(o[2], o[3]) : pack2_f16(o[2], o[3]));
        }
        __builtin_amdgcn_wave_barrier();
        encode_rows(b);
        __builtin_amdgcn_wave_barrier();
    }
}

// Scale, add bias, round once, store.  16-bit outputs of full tiles go through a
// per-wave LDS patch so that every store instruction writes whole row pieces.
template <int BM, int BN, int WGM, int WGN, int FMT, bool B4, bool FOLD>
__device__ __forceinline__ void wide_epilogue(const GemmParams& p, typename AccT<FMT>::type (&acc)[BN / WGN / 16][BM / WGM / 16],
                                              v4f (&accf)[FOLD ? BN / WGN / 16 : 1][FOLD ? BM / WGM / 16 : 1],
                                              uint8_t* smem, int64_t z, int m0, int n0, int wave, int lane, int r_epi = 0,
                                              const float* epi = nullptr) {
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int TM = WM / 16, TN = WN / 16;
    typedef typename AccT<FMT>::type acc_t;
    typedef typename AccT<FMT>::elem acc_e;
    const int wm = wave % WGM, wn = wave / WGM;
    const int lrow = lane & 15, lgrp = lane >> 4;
    const int m_base = m0 + wm * WM + lrow;
    const int n_base = n0 + wn * WN + 4 * lgrp;
    auto range_rx = [&](int r, float (&rx)[TM]) {
        const float* sx = p.r[r].sx + z * p.bsSx;
        const int rs = p.r[r].sx_rs;
#pragma unroll
        for (int b = 0; b < TM; ++b) rx[b] = __builtin_amdgcn_rcpf(sx[(int64_t)min(m_base + b * 16, p.M - 1) * rs]);
    };
    auto range_rw = [&](int r, int a, float (&rw)[4]) {
        const float* sw = p.r[r].sw + z * p.bsSw;
        const int cs = p.r[r].sw_cs;
        const float unscale = B4 ? 0.0625f : 1.0f;
#pragma unroll
        for (int v = 0; v < 4; ++v) rw[v] = unscale * __builtin_amdgcn_rcpf(sw[(int64_t)min(n_base + a * 16 + v, p.N - 1) * cs]);
    };
    const int64_t c_off = z * p.bsC;
    if (p.out_dtype == SEGQ_ACC) {
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
    const bool is16 = p.out_dtype != SEGQ_F32;
    const bool via_lds = is16 && p.vec_store16 && (n0 + BN <= p.N);
    float rx[TM];
    // epi: the tile's vectors parked in LDS by the caller, [1/sx BM | 1/sw BN | bias BN]
    if constexpr (!FOLD) {
        if (via_lds && epi) {
#pragma unroll
            for (int b = 0; b < TM; ++b) rx[b] = epi[wm * WM + b * 16 + lrow];
        } else {
            range_rx(r_epi, rx);  // the range whose scales the accumulators are in units of
        }
    }
    if (via_lds) {
        // every wave transposes 16 rows at a time through its own patch of LDS
        constexpr int RS = WN * 2 + 16;  // row stride in bytes; the 16 spreads rows over the banks
        __syncthreads();                 // the operand tiles are dead from here on
        uint8_t* patch = smem + wave * 16 * RS;
        constexpr int CH = WN / 8;  // 16-byte pieces per patch row
        float rwv[TN][4], bvv[TN][4];
        if (epi) {
#pragma unroll
            for (int a = 0; a < TN; ++a) {
                const v4f w = *reinterpret_cast<const v4f*>(epi + BM + wn * WN + a * 16 + 4 * lgrp);
                const v4f bb = *reinterpret_cast<const v4f*>(epi + BM + BN + wn * WN + a * 16 + 4 * lgrp);
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    rwv[a][v] = w[v];
                    bvv[a][v] = bb[v];
                }
            }
        } else {
#pragma unroll
            for (int a = 0; a < TN; ++a) {
                if constexpr (!FOLD) range_rw(r_epi, a, rwv[a]);
#pragma unroll
                for (int v = 0; v < 4; ++v) bvv[a][v] = p.bias ? load_bias(p.bias, p.bias_dtype, n_base + a * 16 + v) : 0.0f;
            }
        }
        // (two instances, so that launches without an addend carry no trace of it)
        auto blocks = [&](auto add_c) __attribute__((always_inline)) {
            constexpr bool ADD = decltype(add_c)::value;
#pragma unroll
            for (int b = 0; b < TM; ++b) {
#pragma unroll
                for (int a = 0; a < TN; ++a) {
                    float o[4];
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        o[v] = FOLD ? accf[a][b][v] + bvv[a][v] : dequant_bias((float)acc[a][b][v], rx[b], rwv[a][v], bvv[a][v]);
                    if constexpr (ADD) add_addend4(p, z, min(m_base + b * 16, p.M - 1), n_base + a * 16, o);
                    const bool bf = p.out_dtype == SEGQ_BF16;
                    *reinterpret_cast<uint2*>(patch + lrow * RS + (a * 16 + 4 * lgrp) * 2) =
                        make_uint2(bf ? pack2_bf16(o[0], o[1]) : pack2_f16(o[0], o[1]),
                                   bf ? pack2_bf16(o[2], o[3]) : pack2_f16(o[2], o[3]));
                }
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int j = 0; j < (16 * CH + 63) / 64; ++j) {
                    const int c = j * 64 + lane;
                    const int row = c / CH, col = c % CH;
                    if ((16 * CH) % 64 != 0 && c >= 16 * CH) continue;
                    const uint4 v = *reinterpret_cast<const uint4*>(patch + row * RS + col * 16);
                    const int m = m0 + wm * WM + b * 16 + row;
                    if (m < p.M) {
                        *reinterpret_cast<uint4*>(static_cast<uint16_t*>(p.C) + c_off + (int64_t)m * p.ldc + n0 + wn * WN + col * 8) = v;
                    }
                }
                __builtin_amdgcn_wave_barrier();
            }
        };
        if (p.addend) blocks(std::true_type{});
        else blocks(std::false_type{});
        return;
    }
#pragma unroll
    for (int a = 0; a < TN; ++a) {
        float rw[4];
        if constexpr (!FOLD) range_rw(r_epi, a, rw);
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
        if (p.bias) {
#pragma unroll
            for (int v = 0; v < 4; ++v) bv[v] = load_bias(p.bias, p.bias_dtype, min(n_base + a * 16 + v, p.N - 1));
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
            if (p.out_dtype == SEGQ_F32) store4<SEGQ_F32>(p.C, e, o, vec, p.N - n);
            else if (p.out_dtype == SEGQ_BF16) store4<SEGQ_BF16>(p.C, e, o, vec, p.N - n);
            else store4<SEGQ_F16>(p.C, e, o, vec, p.N - n);
        }
    }
}

template <int BM, int BN, int WGM, int WGN, int FMT, bool B4, bool FOLD, bool ASEL>
__global__ void __launch_bounds__(WGM* WGN * 64) gemm_wide_kernel(const GemmParams p) {
    constexpr int NW = WGM * WGN, NT = NW * 64;
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int TM = WM / 16, TN = WN / 16;
    constexpr int A_IT = BM * 8 / NT;                 // 16-byte chunks per thread, activations
    constexpr int B_IT = (B4 ? BN * 4 : BN * 8) / NT;  // same, weights (packed chunks when int4)
    constexpr int RPI = NT / 8;                        // rows covered by one pass of all threads
    constexpr int RPI4 = NT / 4;
    static_assert(BM * 8 % NT == 0 && BN * 4 % NT == 0 && RPI % 16 == 0, "tile does not divide over the threads");
    static_assert(!B4 || FMT == GEMM_I8, "int4 weights pair with int8 activations");
    typedef typename AccT<FMT>::type acc_t;
    typedef typename AccT<FMT>::elem acc_e;
    const acc_t acc_zero = {0, 0, 0, 0};

    extern __shared__ __align__(16) uint8_t smem[];
    uint8_t* const As = smem;                // [2][BM][128]
    uint8_t* const Bs = smem + 2 * BM * BK;  // [2][BN][128]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WGM, wn = wave / WGM;
    const int lrow = lane & 15, lgrp = lane >> 4;

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

    // ---- staging.  Thread t, pass i: row i * RPI + t / 8, physical chunk t % 8,
    // which holds logical chunk (t % 8) ^ swz(row).
    const int s_row = tid >> 3;
    const int s_pc = tid & 7;
    const int s_lc = s_pc ^ swz(s_row);
    uint32_t a_goff[A_IT];
#pragma unroll
    for (int i = 0; i < A_IT; ++i) a_goff[i] = (uint32_t)min(m0 + s_row + i * RPI, p.M - 1) * (uint32_t)p.lda + s_lc * 16;
    // weights: same scheme, or 4 packed chunks per row when int4
    const int b_row = B4 ? (tid >> 2) : s_row;
    const int b_pk = tid & 3;  // int4: packed chunk = 32 k = logical chunks 2 b_pk, 2 b_pk + 1
    constexpr int B_RSTEP = B4 ? RPI4 : RPI;
    uint32_t b_goff[B_IT];
#pragma unroll
    for (int i = 0; i < B_IT; ++i)
        b_goff[i] = (uint32_t)min(n0 + b_row + i * B_RSTEP, p.N - 1) * (uint32_t)p.ldb + (B4 ? b_pk : s_lc) * 16;
    const int b_sw = swz(b_row);
    const int w_lds = wave * 8 * BK;  // direct loads: the 8 rows this wave fills per pass

    uint4 ra[ASEL ? A_IT : 1], rb[B4 ? B_IT : 1];

    auto issue_loads = [&](const uint8_t* ap, int k, int buf) {
        if constexpr (ASEL) {
#pragma unroll
            for (int i = 0; i < A_IT; ++i) ra[i] = *reinterpret_cast<const uint4*>(ap + k + a_goff[i]);
        } else {
            uint8_t* as = As + buf * BM * BK + w_lds;
#pragma unroll
            for (int i = 0; i < A_IT; ++i) load16_to_lds(ap + k + a_goff[i], as + i * RPI * BK);
        }
        if constexpr (B4) {
#pragma unroll
            for (int i = 0; i < B_IT; ++i) rb[i] = *reinterpret_cast<const uint4*>(Bb + (k >> 1) + b_goff[i]);
        } else {
            uint8_t* bs = Bs + buf * BN * BK + w_lds;
#pragma unroll
            for (int i = 0; i < B_IT; ++i) load16_to_lds(Bb + k + b_goff[i], bs + i * RPI * BK);
        }
    };
    // sel_or / sel_xor: branch-free sign selection, kept = x & ((negmask ^ sel_xor) | sel_or)
    auto commit_loads = [&](int buf, uint32_t sel_or, uint32_t sel_xor) {
        if constexpr (ASEL) {
            uint8_t* as = As + buf * BM * BK + s_row * BK + s_pc * 16;
#pragma unroll
            for (int i = 0; i < A_IT; ++i) {
                uint4 v = ra[i];
                v.x &= (neg_byte_mask(v.x) ^ sel_xor) | sel_or;
                v.y &= (neg_byte_mask(v.y) ^ sel_xor) | sel_or;
                v.z &= (neg_byte_mask(v.z) ^ sel_xor) | sel_or;
                v.w &= (neg_byte_mask(v.w) ^ sel_xor) | sel_or;
                *reinterpret_cast<uint4*>(as + i * RPI * BK) = v;
            }
        }
        if constexpr (B4) {
            uint8_t* bs = Bs + buf * BN * BK + b_row * BK;
#pragma unroll
            for (int i = 0; i < B_IT; ++i) {
                uint4 lo, hi;
                unpack8_i4x16(rb[i].x, lo.x, lo.y);
                unpack8_i4x16(rb[i].y, lo.z, lo.w);
                unpack8_i4x16(rb[i].z, hi.x, hi.y);
                unpack8_i4x16(rb[i].w, hi.z, hi.w);
                uint8_t* row = bs + i * B_RSTEP * BK;
                *reinterpret_cast<uint4*>(row + (((2 * b_pk) ^ b_sw) << 4)) = lo;
                *reinterpret_cast<uint4*>(row + (((2 * b_pk + 1) ^ b_sw) << 4)) = hi;
            }
        }
        if constexpr (!ASEL || !B4) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): direct loads have landed
    };

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
    const int a_frag = (wm * WM + lrow) * BK;
    const int b_frag = (wn * WN + lrow) * BK;

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

    // lane's output coordinates: row m_base + 16 b, columns n_base + 16 a + 0..3
    const int m_base = m0 + wm * WM + lrow;
    const int n_base = n0 + wn * WN + 4 * lgrp;

    auto range_rx = [&](int r, float (&rx)[TM]) {
        const float* sx = p.r[r].sx + z * p.bsSx;
        const int rs = p.r[r].sx_rs;
#pragma unroll
        for (int b = 0; b < TM; ++b) rx[b] = __builtin_amdgcn_rcpf(sx[(int64_t)min(m_base + b * 16, p.M - 1) * rs]);
    };
    auto range_rw = [&](int r, int a, float (&rw)[4]) {
        const float* sw = p.r[r].sw + z * p.bsSw;
        const int cs = p.r[r].sw_cs;
        const float unscale = B4 ? 0.0625f : 1.0f;  // the staged int4 weights carry an exact factor 16
#pragma unroll
        for (int v = 0; v < 4; ++v) rw[v] = unscale * __builtin_amdgcn_rcpf(sw[(int64_t)min(n_base + a * 16 + v, p.N - 1) * cs]);
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
    auto sel_masks = [&](int a_sel, uint32_t& so, uint32_t& sx) {
        so = (a_sel >= 2) ? 0u : 0xFFFFFFFFu;
        sx = (a_sel == 2) ? 0xFFFFFFFFu : 0u;
    };

    // ---- main loop over (range, k) steps; every range is whole 128-byte steps
    int r = 0, k = p.r[0].k0;
    uint32_t so, sxm;
    sel_masks(p.r[0].a_sel, so, sxm);
    issue_loads((p.r[0].a_sel == 1) ? A2b : Ab, k, 0);
    commit_loads(0, so, sxm);
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
        if (more) {
            const int sel = p.r[rn].a_sel;
            sel_masks(sel, so, sxm);
            issue_loads((sel == 1) ? A2b : Ab, kn, buf ^ 1);
        }
        compute(buf);
        if (FOLD && range_done) fold(r);
        if (!more) break;
        commit_loads(buf ^ 1, so, sxm);
        __syncthreads();
        buf ^= 1;
        r = rn;
        k = kn;
    }

    wide_epilogue<BM, BN, WGM, WGN, FMT, B4, FOLD>(p, acc, accf, smem, z, m0, n0, wave, lane);
}

// Low-rank branch of the epilogue: of[a][b] += sum_k L2T[n][k] T[m][k] over k < lr_rank, on the
// matrix cores (v_mfma_f32_16x16x32_bf16 / _f16, fp32 accumulation), for the wave's WM x WN
// patch at (m_row0, n_col0).  `of` holds the de-quantised sums in output units in the lane layout
// of the accumulators (four consecutive columns of one row per lane and block), which is also
// the result layout of these MFMAs with L2T as the first operand.  Both fragments are 16 rows of
// 32 contiguous 16-bit values: a lane reads the 16 bytes of its row at k + 8 lgrp straight from
// memory (T and L2T are small and stay in the L2).
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

template <int TM, int TN>
__device__ __forceinline__ void lowrank_accumulate(const GemmParams& p, v4f (&of)[TN][TM], int m_row0, int n_col0, int lane) {
    const int lrow = lane & 15, lgrp = lane >> 4;
    const bool bf = p.out_dtype == SEGQ_BF16;
    for (int kk = 0; kk < p.lr_rank; kk += 32) {
        uint4 tf[TM];
#pragma unroll
        for (int b = 0; b < TM; ++b) {
            const int64_t m = min(m_row0 + b * 16 + lrow, p.M - 1);
            tf[b] = *reinterpret_cast<const uint4*>(p.lr_t + m * p.lr_ldt + kk + lgrp * 8);
        }
#pragma unroll
        for (int a = 0; a < TN; ++a) {
            const int64_t n = min(n_col0 + a * 16 + lrow, p.N - 1);
            const uint4 lf = *reinterpret_cast<const uint4*>(p.lr_l2 + n * p.lr_ldl + kk + lgrp * 8);
#pragma unroll
            for (int b = 0; b < TM; ++b) {
                if (bf)
                    of[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, lf), __builtin_bit_cast(v8bf, tf[b]), of[a][b], 0, 0, 0);
                else
                    of[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, lf), __builtin_bit_cast(v8h, tf[b]), of[a][b], 0, 0, 0);
            }
        }
    }
}

// Software-pipelined variant for plain int8 operands (both straight to LDS) with
// NS LDS stages.  Two stages are what is instantiated: on FLUX shapes three and
// four stages measured slower (they cost a co-resident workgroup or buy nothing,
// the global -> LDS path being throughput- rather than latency-bound: ~31 of a
// measured ~55 B/clk/CU).  The K step is split at its one barrier:
//
//   barrier (tile s landed, tile s-1 fully in registers)
//     DMA tile s+1 into the buffer of tile s-1      <- a whole step of latency cover
//     LDS -> fragments F0 of tile s
//     MFMAs on fragments F1 of tile s-1             <- hides the F0 reads
//     LDS -> fragments F1 of tile s
//     MFMAs on F0 of tile s                         <- hides the F1 reads
//   wait own DMA and LDS reads, barrier
//
// so fragment reads never stand between an MFMA group and the one before it.
// s_waitcnt immediate for "vmcnt(n) lgkmcnt(0)" on gfx9-family encodings
constexpr int waitcnt_vm_lgkm0(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4); }

template <int BM, int BN, int WGM, int WGN, int FMT, bool FOLD, int NS, bool GRP = false, bool PARK = false, bool FINISH = false,
          bool CODES = false>  // CODES: the epilogue writes the next linear's codes instead of floats (one range)
__global__ void __launch_bounds__(WGM* WGN * 64) gemm_pipe_kernel(const GemmParams p) {
    static_assert(!CODES || (!FOLD && !GRP && !PARK && !FINISH), "codes out: plain operands, one range");
    constexpr int NW = WGM * WGN, NT = NW * 64;
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int TM = WM / 16, TN = WN / 16;
    constexpr int RPI = NT / 8;                                  // rows one pass of all threads covers
    constexpr int A_IT = (BM + RPI - 1) / RPI, B_IT = (BN + RPI - 1) / RPI;
    constexpr int A_TAIL = BM % RPI, B_TAIL = BN % RPI;          // rows of a last, partial pass (0: none)
    static_assert(A_TAIL % 8 == 0 && B_TAIL % 8 == 0 && WM % 16 == 0 && WN % 16 == 0, "tile does not divide over the waves");
    typedef typename AccT<FMT>::type acc_t;
    constexpr bool F8 = FMT == GEMM_F8;
    // Several ranges: int32 accumulators are folded into a second, fp32 set at the
    // end of each range.  fp32 accumulators (e4m3) need no second set: at a range
    // boundary they are rescaled from the finished range's scales to the next
    // one's (acc *= sx' sw' / (sx sw), one fp32 rounding), so the sum stays in
    // units of the current range and the epilogue divides by the last range's.
    //
    // GRP (int8): every K step of 128 is a group with its own de-quantisation
    // factor per output column (group-wise weight scales).  The step's int32
    // sums are multiplied by the factors and added to an fp32 set, which from
    // there on is treated like e4m3's fp32 accumulators: in units of the current
    // range, rescaled at range boundaries, scaled by 1/(sx sw) in the epilogue.
    // The group kernel runs the e4m3 schedule (whole-step fragments of 32 bytes,
    // refilled as the step lets go of them): both 64-byte K halves of an output
    // block are multiplied back to back into a handful of int32 temporaries,
    // which are converted at once, so no int32 accumulator set lives across
    // steps and the 64 x 64 wave tile fits.
    static_assert(!GRP || (!F8 && NS == 2), "group factors: int8, two stages");
    // int8 tiles above 256 x 256 run the whole-step schedule too: one set of 32-byte fragments
    // instead of two sets of 16-byte ones leaves room for their accumulators
    constexpr bool WS = !F8 && !GRP && BM * BN > 256 * 256;
    constexpr bool S8 = F8 || GRP || WS;  // whole-step fragments
    //
    // PARK (int8, several ranges): no second register set at all.  When a range
    // ends, its int32 sums are converted to the LAST range's units
    // (x sx_L sw_L / (sx sw)) and added to this tile's fp32 slot of a workspace
    // the caller lends; the accumulators restart from zero.  The epilogue adds the
    // slot to the last range's sums and scales once.  Each thread only ever reads
    // back what it wrote itself.  This keeps the big tiles for int8 with K
    // segments or DualScale: a few hundred KB of traffic per tile and range
    // boundary against ~14 MB of operands.
    static_assert(!PARK || (FOLD && !F8 && !GRP), "parking: int8 with several ranges");
    static_assert(!WS || (!FOLD && !PARK), "int8 above 256 x 256: one range");
    constexpr bool ACCF = FOLD && !F8 && !GRP && !PARK;
    constexpr bool HASF = ACCF || GRP;
    const acc_t acc_zero = {0, 0, 0, 0};
    // Split K (p.splits > 1): workgroup (tile, y) multiplies the y-th share of the K steps,
    // counted through the ranges, and writes an fp32 partial result that a second kernel
    // sums.  r_last is the range its last step lies in: the one whose units its
    // accumulators end up in (without a split: the last range).
    int r_last = p.nr - 1, r_begin = 0;  // (r_begin: the range its first step lies in)

    static_assert(NS >= 2 && (NS - 1) * (A_IT + B_IT) < 64, "vmcnt holds 6 bits");
    static_assert(!S8 || (NS == 2 && TN >= 3), "the e4m3 schedule reads two weight fragments ahead in a two-stage ring");
    extern __shared__ __align__(16) uint8_t smem[];
    uint8_t* const As = smem;                  // [NS][BM][128]
    uint8_t* const Bs = smem + NS * BM * BK;   // [NS][BN][128]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WGM, wn = wave / WGM;
    const int lrow = lane & 15, lgrp = lane >> 4;

    // Workgroups are dealt to the eight XCDs in turn, each with an L2 of its own.  Every XCD gets a
    // run of consecutive tiles (with a K split: of consecutive (share, tile) pairs), so that its
    // workgroups stream few distinct operand panels and its L2 serves most of their requests.
    int bid = blockIdx.x, zy = blockIdx.y;
    {
        const int nb = p.tiles_m * p.tiles_n;
        if (p.splits > 1) {
            const int total = nb * p.splits, lin = zy * nb + bid, q = total >> 3, r = total & 7, x = lin & 7;
            const int v = x * q + min(x, r) + (lin >> 3);
            zy = v / nb;
            bid = v - zy * nb;
        } else if ((nb & 7) == 0) {
            bid = (bid & 7) * (nb >> 3) + (bid >> 3);
        }
    }
    const int tile_id = bid;  // names this tile's room in the workspaces
    // Several ranges, no K split: the workgroups of XCD x walk the ranges starting from range
    // x mod nr (and wrap), so that at any K step only part of the chip is at a range boundary, where
    // int8 tiles store their sums to the workspace.  All workgroups of an XCD keep the same order:
    // they share operand panels through its L2.  The order of a tile's fp32 additions depends on
    // its XCD only, so a launch gives the same bits every time.  ph(j): the range walked j-th.
    const int r_off = (FOLD && p.rot) ? (int)(blockIdx.x & 7) % p.nr : 0;
    auto ph = [&](int j) { const int t = j + r_off; return t >= p.nr ? t - p.nr : t; };
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
    const int64_t z = zy;
    const uint8_t* const Ab = p.A + z * p.bsA;
    const uint8_t* const A2b = p.A2 ? p.A2 + z * p.bsA : nullptr;
    const uint8_t* const Bb = p.B + z * p.bsB;

    const int s_row = tid >> 3;
    const int s_lc = (tid & 7) ^ swz(s_row);
    uint32_t a_goff[A_IT], b_goff[B_IT];
#pragma unroll
    for (int i = 0; i < A_IT; ++i) a_goff[i] = (uint32_t)min(m0 + s_row + i * RPI, p.M - 1) * (uint32_t)p.lda + s_lc * 16;
#pragma unroll
    for (int i = 0; i < B_IT; ++i) b_goff[i] = (uint32_t)min(n0 + s_row + i * RPI, p.N - 1) * (uint32_t)p.ldb + s_lc * 16;
    const int w_lds = wave * 8 * BK;

    // a wave covers 8 rows of a pass, so whether it takes part in a partial last pass is wave-uniform
    const bool a_skip = A_TAIL != 0 && wave * 8 >= A_TAIL;
    const bool b_skip = B_TAIL != 0 && wave * 8 >= B_TAIL;
    auto dma1 = [&](const uint8_t* ap, const uint8_t* bp, int buf, int i) {
        if (i < A_IT) {
            if (i == A_IT - 1 && a_skip) return;
            load16_to_lds(ap + a_goff[i], As + buf * BM * BK + w_lds + i * RPI * BK);
        } else {
            if (i == A_IT + B_IT - 1 && b_skip) return;
            load16_to_lds(bp + b_goff[i - A_IT], Bs + buf * BN * BK + w_lds + (i - A_IT) * RPI * BK);
        }
    };
    // "all but the newest nt tiles of this wave's DMA have landed, and all its LDS reads"
    auto wait_dma = [&](auto nt_c) {
        constexpr int nt = decltype(nt_c)::value;
        constexpr int full = A_IT + B_IT;
        if constexpr (nt == 0 || (A_TAIL == 0 && B_TAIL == 0)) {
            __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(nt * full));
        } else {
            const int miss = (a_skip ? 1 : 0) + (b_skip ? 1 : 0);
            if (miss == 0) __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(nt * full));
            else if (miss == 1) __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(nt * (full - 1)));
            else __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(nt * (full - 2)));
        }
    };
    auto dma = [&](const uint8_t* ap, const uint8_t* bp, int buf) {
#pragma unroll
        for (int i = 0; i < A_IT + B_IT; ++i) dma1(ap, bp, buf, i);
    };

    acc_t acc[TN][TM];
    v4f accf[HASF ? TN : 1][HASF ? TM : 1];
#pragma unroll
    for (int a = 0; a < TN; ++a)
#pragma unroll
        for (int b = 0; b < TM; ++b) acc[a][b] = acc_zero;
    if constexpr (HASF) {
#pragma unroll
        for (int a = 0; a < TN; ++a)
#pragma unroll
            for (int b = 0; b < TM; ++b) accf[a][b] = v4f{0.f, 0.f, 0.f, 0.f};
    }


    const int f_sw = swz(lrow);
    const int a_frag = (wm * WM + lrow) * BK;
    const int b_frag = (wn * WN + lrow) * BK;
    // int8: two fragment sets, one per 64-byte K half of a step.  e4m3: one set of
    // 32-byte fragments (the 16 x 16 x 128 MFMA eats a whole step), whose registers
    // are refilled for the next step as the current one lets go of them.
    v4i fa[S8 ? 1 : 2][S8 ? 1 : TM], fb[S8 ? 1 : 2][S8 ? 1 : TN];
    v8i fa8[S8 ? TM : 1], fb8[S8 ? TN : 1];
    auto frag8 = [&](int buf, int i) {  // fragment i of the step in buffer buf: 0 .. TM-1 activations, then weights
      if constexpr (S8) {
        // Lane group g feeds K slot [32 g, 32 g + 32) of the MFMA with bytes [16 g, 16 g + 16) and
        // [64 + 16 g, 64 + 16 g + 16) of the step: activations and weights are permuted alike, so the
        // sum is the same, and each of the two reads has the int8 kernels' conflict-free pattern (the
        // four groups of a row read four neighbouring 16-byte pieces; reading pieces 2 g and 2 g + 1
        // instead costs a two-way bank conflict on every read).
        const int off0 = (lgrp ^ f_sw) << 4;
        const int off1 = ((4 + lgrp) ^ f_sw) << 4;
        const uint8_t* src = (i < TM) ? As + buf * BM * BK + a_frag + i * 16 * BK : Bs + buf * BN * BK + b_frag + (i - TM) * 16 * BK;
        const v4i lo = *reinterpret_cast<const v4i*>(src + off0);
        const v4i hi = *reinterpret_cast<const v4i*>(src + off1);
        const v8i f = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        if (i < TM) fa8[i] = f;
        else fb8[i - TM] = f;
      }
    };

    // K half h of the tile in buffer buf -> fragment slot h, one 16-byte read at a
    // time: reads 0 .. TM-1 are the activation fragments, TM .. TM+TN-1 the weights
    auto frag1 = [&](int buf, int h, int i) {
        if constexpr (!S8) {
            const int off = ((h * 4 + lgrp) ^ f_sw) << 4;
            if (i < TM) fa[h][i] = *reinterpret_cast<const v4i*>(As + buf * BM * BK + a_frag + i * 16 * BK + off);
            else fb[h][i - TM] = *reinterpret_cast<const v4i*>(Bs + buf * BN * BK + b_frag + (i - TM) * 16 * BK + off);
        }
    };
    auto frags = [&](int buf, int h) {
#pragma unroll
        for (int i = 0; i < TM + TN; ++i) frag1(buf, h, i);
    };
    const int m_base = m0 + wm * WM + lrow;
    const int n_base = n0 + wn * WN + 4 * lgrp;
    v4f* const slot = PARK ? reinterpret_cast<v4f*>(p.park) + ((int64_t)zy * gridDim.x + tile_id) * (BM * BN / 4) + tid : nullptr;
    auto park = [&](int r) __attribute__((always_inline)) {
        if constexpr (PARK) {
            if (r < r_last) {
                const int rl = r_last;
                const float* sx = p.r[ph(r)].sx;
                const float* sw = p.r[ph(r)].sw;
                const float* sx2 = p.r[ph(rl)].sx;
                const float* sw2 = p.r[ph(rl)].sw;
                const int rs = p.r[ph(r)].sx_rs, cs = p.r[ph(r)].sw_cs, rs2 = p.r[ph(rl)].sx_rs, cs2 = p.r[ph(rl)].sw_cs;
                float fx[TM];
#pragma unroll
                for (int b = 0; b < TM; ++b) {
                    const int64_t m = min(m_base + b * 16, p.M - 1);
                    fx[b] = sx2[m * rs2] * __builtin_amdgcn_rcpf(sx[m * rs]);
                }
#pragma unroll
                for (int a = 0; a < TN; ++a) {
                    v4f fw;
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int64_t n = min(n_base + a * 16 + v, p.N - 1);
                        fw[v] = sw2[n * cs2] * __builtin_amdgcn_rcpf(sw[n * cs]);
                    }
                    v4f old[TM];
                    if (r > r_begin) {
#pragma unroll
                        for (int b = 0; b < TM; ++b) old[b] = slot[(a * TM + b) * NT];
                    }
#pragma unroll
                    for (int b = 0; b < TM; ++b) {
                        v4f t = __builtin_convertvector(acc[a][b], v4f) * (fw * fx[b]);
                        if (r > r_begin) t += old[b];
                        slot[(a * TM + b) * NT] = t;
                        acc[a][b] = acc_zero;
                    }
                }
            }
        }
    };
    auto fold = [&](int r) __attribute__((always_inline)) {
        if constexpr (FOLD && (F8 || GRP)) {
            auto& facc = [&]() -> auto& { if constexpr (GRP) return accf; else return acc; }();
            if (r < r_last) {  // rescale to the next range's units
                const float* sx = p.r[ph(r)].sx + z * p.bsSx;
                const float* sw = p.r[ph(r)].sw + z * p.bsSw;
                const float* sx2 = p.r[ph(r + 1)].sx + z * p.bsSx;
                const float* sw2 = p.r[ph(r + 1)].sw + z * p.bsSw;
                const int rs = p.r[ph(r)].sx_rs, cs = p.r[ph(r)].sw_cs, rs2 = p.r[ph(r + 1)].sx_rs, cs2 = p.r[ph(r + 1)].sw_cs;
                float fx[TM];
#pragma unroll
                for (int b = 0; b < TM; ++b) {
                    const int64_t m = min(m_base + b * 16, p.M - 1);
                    fx[b] = sx2[m * rs2] * __builtin_amdgcn_rcpf(sx[m * rs]);
                }
#pragma unroll
                for (int a = 0; a < TN; ++a) {
                    v4f fw;
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int64_t n = min(n_base + a * 16 + v, p.N - 1);
                        fw[v] = sw2[n * cs2] * __builtin_amdgcn_rcpf(sw[n * cs]);
                    }
#pragma unroll
                    for (int b = 0; b < TM; ++b) facc[a][b] = facc[a][b] * (fw * fx[b]);
                }
            }
        }
        if constexpr (ACCF) {
            const float* sx = p.r[ph(r)].sx + z * p.bsSx;
            const float* sw = p.r[ph(r)].sw + z * p.bsSw;
            const int rs = p.r[ph(r)].sx_rs, cs = p.r[ph(r)].sw_cs;
            float rx[TM];
#pragma unroll
            for (int b = 0; b < TM; ++b) rx[b] = __builtin_amdgcn_rcpf(sx[(int64_t)min(m_base + b * 16, p.M - 1) * rs]);
#pragma unroll
            for (int a = 0; a < TN; ++a) {
                float rw[4];
#pragma unroll
                for (int v = 0; v < 4; ++v) rw[v] = __builtin_amdgcn_rcpf(sw[(int64_t)min(n_base + a * 16 + v, p.N - 1) * cs]);
#pragma unroll
                for (int b = 0; b < TM; ++b) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) accf[a][b][v] += (float)acc[a][b][v] * rx[b] * rw[v];
                    acc[a][b] = acc_zero;
                }
            }
        }
    };

    // Two cursors walk the ranges: (lr, lk) is the tile loaded NS steps ahead,
    // (cr, ck) the tile being multiplied.  The end of the current range and the
    // source of its activations stay in registers, so the range table is read
    // only when a cursor crosses into the next range.
    int steps = 0;
    for (int i = 0; i < p.nr; ++i) steps += (p.r[i].k1 - p.r[i].k0) / BK;
    int lr = 0, skip = 0;  // this workgroup's first step: `skip` steps into range lr
    if (p.splits > 1) {
        skip = (int)((int64_t)steps * zy / p.splits);
        steps = (int)((int64_t)steps * (zy + 1) / p.splits) - skip;
        while (lr + 1 < p.nr && skip >= (p.r[ph(lr)].k1 - p.r[ph(lr)].k0) / BK) {
            skip -= (p.r[ph(lr)].k1 - p.r[ph(lr)].k0) / BK;
            ++lr;
        }
        r_last = r_begin = lr;
        for (int left = skip + steps; r_last + 1 < p.nr && left > (p.r[ph(r_last)].k1 - p.r[ph(r_last)].k0) / BK; ++r_last)
            left -= (p.r[ph(r_last)].k1 - p.r[ph(r_last)].k0) / BK;
    }
    const int r_first = lr, k_first = p.r[ph(lr)].k0 + skip * BK;
    int lk = k_first, lk1 = p.r[ph(lr)].k1;
    const uint8_t* la = (p.r[ph(lr)].a_sel == 1) ? A2b : Ab;
    auto advance_load = [&]() {
        lk += BK;
        if (lk >= lk1) {
            ++lr;
            const int rr = min(lr, p.nr - 1);  // past the last range nothing more is loaded
            lk = p.r[ph(rr)].k0;
            lk1 = (lr < p.nr) ? p.r[ph(rr)].k1 : 0x7fffffff;
            la = (p.r[ph(rr)].a_sel == 1) ? A2b : Ab;
        }
    };

    // The epilogue's vectors (1/sx per row, 1/sw and bias per column of this tile)
    // are fetched first of all, so that the wait for the first DMA covers them, and
    // parked in LDS behind the stages: the epilogue then starts without a round
    // trip to memory, and without the ~70 small loads per wave it would take there.
    constexpr int EPI_FLOATS = BM + 2 * BN, EPI_IT = (EPI_FLOATS + NT - 1) / NT;
    float* const epi = reinterpret_cast<float*>(smem + NS * (BM + BN) * BK);
    // group factors: a ring of four rows of BN floats behind the epilogue's vectors.  The row of
    // step s arrives with the step's operands and is read all through step s, at whose end the
    // row of step s + 2 is already on its way
    float* const grw = epi + EPI_FLOATS;
    int lslot = 0, cslot = 0;  // slots of the step being loaded / multiplied
    auto dma_g = [&]() {
        if constexpr (GRP) {
            if (wave < BN / 64) {
                const int n = min(n0 + wave * 64 + lane, p.N - 1);
                __builtin_amdgcn_global_load_lds((glb_ptr_t)(p.grw + (int64_t)(lk >> 7) * p.grw_gs + n),
                                                 (lds_ptr_t)(grw + lslot * BN + wave * 64), 4, 0, 0);
            }
            lslot = (lslot + 1) & 3;
        }
    };
    const int r_epi = ACCF ? 0 : ph(r_last);  // the range (as the caller numbers them) whose units the accumulators end up in
    float epi_val[EPI_IT];
    const bool want_epi = p.out_dtype != SEGQ_ACC;  // raw accumulators come with no scales at all (null pointers)
#pragma unroll
    for (int i = 0; i < EPI_IT; ++i) {
        const int e = i * NT + tid;
        float v = 0.0f;
        if (!want_epi) {
        } else if (e < BM) {
            if constexpr (!ACCF) v = (p.r[r_epi].sx + z * p.bsSx)[(int64_t)min(m0 + e, p.M - 1) * p.r[r_epi].sx_rs];
        } else if (e < BM + BN) {
            if constexpr (!ACCF) v = (p.r[r_epi].sw + z * p.bsSw)[(int64_t)min(n0 + e - BM, p.N - 1) * p.r[r_epi].sw_cs];
        } else if (e < EPI_FLOATS) {
            if (p.bias) v = load_bias(p.bias, p.bias_dtype, min(n0 + e - BM - BN, p.N - 1));
        }
        epi_val[i] = v;
    }

    // prologue: tiles 0 .. NS-1 on their way into buffers 0 .. NS-1; wait for tile 0
    int issued = 0;
#pragma unroll
    for (int t = 0; t < NS; ++t) {
        if (t < steps) {
            dma(la + lk, Bb + lk, t);
            dma_g();
            advance_load();
            ++issued;
        }
    }
    if (issued == NS && !GRP) wait_dma(std::integral_constant<int, NS - 1>{});
    else wait_dma(std::integral_constant<int, 0>{});  // (with group factors the waves' DMA counts differ)
#pragma unroll
    for (int i = 0; i < EPI_IT; ++i) {
        const int e = i * NT + tid;
        if (e < EPI_FLOATS) epi[e] = (e < BM + BN && !ACCF) ? __builtin_amdgcn_rcpf(epi_val[i]) : epi_val[i];
    }
    __syncthreads();
    if constexpr (S8) {
#pragma unroll
        for (int i = 0; i <= TM; ++i) frag8(0, i);  // activations and the first weight fragment
    } else {
        frags(0, 0);
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the loop head must see them as landed on every path

    // One K step.  Fragment reads and DMA instructions are spread between the
    // MFMAs: a wave issues in order, and an LDS or DMA instruction that has to
    // queue holds up the MFMAs behind it, so a burst of them drains the matrix
    // pipe of the whole SIMD (both its waves are in the same phase).  Issued one
    // at a time they never queue.  DMA_ and MORE_ are compile-time so that the
    // steady-state loop body has no branches.
    int cr = r_first, ck = k_first, ck1 = p.r[ph(r_first)].k1;  // the tile being multiplied
    bool dirty = false;  // int32 sums not yet folded into the fp32 set (a split can end inside a range)
    int buf = 0;                                   // its buffer, s % NS
    constexpr int NMF = TM * TN, NRD = TM + TN, NDM = A_IT + B_IT;
    constexpr int RD_EVERY = (NMF >= 2 * NRD + 4) ? 2 : 1;
    constexpr int DM_EVERY = (NMF / NDM > 1) ? NMF / NDM : 1;
    static_assert(NRD * RD_EVERY <= NMF && NDM * DM_EVERY <= NMF, "more reads than MFMA slots");
    // e4m3 schedule of one step.  On entry the activation fragments and weight
    // fragment 0 are in registers.  Column block a reads weight fragment a + 2
    // (block 0 also fragment 1), so after block TN - 3 every read of this step is
    // issued; there the step has its barrier.  The last two blocks refill the
    // registers this step is done with: next weight fragment 0, then each
    // activation fragment right behind the last MFMA that reads it, with the DMA
    // of step s + 2 spread over the same MFMAs.
    auto step8 = [&](auto dma_c, auto more_c) __attribute__((always_inline)) {
        constexpr bool DMA_ = decltype(dma_c)::value;
        constexpr bool MORE_ = decltype(more_c)::value;
        constexpr int NDM8 = A_IT + B_IT, TAIL = 2 * TM;  // DMA instructions over the tail's MFMAs
        const int nbuf = buf ^ 1;
        // group mode: an output block is both K halves of the step into an int32 temporary
        // (first MFMA with a zero C operand), converted and scaled by this step's factors at once
        auto lo4 = [](const v8i& f) __attribute__((always_inline)) { return v4i{f[0], f[1], f[2], f[3]}; };
        auto hi4 = [](const v8i& f) __attribute__((always_inline)) { return v4i{f[4], f[5], f[6], f[7]}; };
        const float* const gsrc = grw + cslot * BN + wn * WN + 4 * lgrp;
#pragma unroll
        for (int a = 0; a < TN - 2; ++a) {
            if constexpr (GRP) {
                v4i t[TM];
                const v4f g = *reinterpret_cast<const v4f*>(gsrc + a * 16);
#pragma unroll
                for (int b = 0; b < TM; ++b) {
                    if (b == 0 && a == 0) frag8(buf, TM + 1);
                    if (b == (TM > 1 ? 1 : 0)) frag8(buf, TM + a + 2);
                    t[b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(lo4(fb8[a]), lo4(fa8[b]), acc_zero, 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int b = 0; b < TM; ++b) {
                    t[b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(hi4(fb8[a]), hi4(fa8[b]), t[b], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int b = 0; b < TM; ++b) accf[a][b] += __builtin_convertvector(t[b], v4f) * g;
            } else if constexpr (WS) {
                // int8: the two 64-byte K halves of a block, TM MFMAs apart
#pragma unroll
                for (int b = 0; b < TM; ++b) {
                    if (b == 0 && a == 0) frag8(buf, TM + 1);
                    if (b == (TM > 1 ? 1 : 0)) frag8(buf, TM + a + 2);
                    if constexpr (!F8) acc[a][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(lo4(fb8[a]), lo4(fa8[b]), acc[a][b], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int b = 0; b < TM; ++b) {
                    if constexpr (!F8) acc[a][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(hi4(fb8[a]), hi4(fa8[b]), acc[a][b], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
#pragma unroll
                for (int b = 0; b < TM; ++b) {
                    if (b == 0 && a == 0) frag8(buf, TM + 1);
                    if (b == (TM > 1 ? 1 : 0)) frag8(buf, TM + a + 2);
                    if constexpr (F8)
                        acc[a][b] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb8[a], fa8[b], acc[a][b], 0, 0, 0, 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        wait_dma(std::integral_constant<int, 0>{});
        __syncthreads();
        const uint8_t* const ap = la + lk;
        const uint8_t* const bp = Bb + lk;
#pragma unroll
        for (int a = TN - 2; a < TN; ++a) {
            if constexpr (GRP) {
                v4i t[TM];
                const v4f g = *reinterpret_cast<const v4f*>(gsrc + a * 16);
#pragma unroll
                for (int b = 0; b < TM; ++b) {
                    t[b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(lo4(fb8[a]), lo4(fa8[b]), acc_zero, 0, 0, 0);
                    const int j = (a - (TN - 2)) * TM + b;
                    if constexpr (DMA_) {
#pragma unroll
                        for (int i = j * NDM8 / TAIL; i < (j + 1) * NDM8 / TAIL; ++i) dma1(ap, bp, buf, i);
                        if (j == TAIL - 1) dma_g();
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int b = 0; b < TM; ++b) {
                    t[b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(hi4(fb8[a]), hi4(fa8[b]), t[b], 0, 0, 0);
                    if constexpr (MORE_) {
                        if (a == TN - 2 && b == 0) frag8(nbuf, TM);  // next weight fragment 0: free since block 0
                        if (a == TN - 1) frag8(nbuf, b);              // next activation fragment b: this was its last reader
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int b = 0; b < TM; ++b) accf[a][b] += __builtin_convertvector(t[b], v4f) * g;
            } else if constexpr (WS) {
#pragma unroll
                for (int b = 0; b < TM; ++b) {
                    if constexpr (!F8) acc[a][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(lo4(fb8[a]), lo4(fa8[b]), acc[a][b], 0, 0, 0);
                    const int j = (a - (TN - 2)) * TM + b;
                    if constexpr (DMA_) {
#pragma unroll
                        for (int i = j * NDM8 / TAIL; i < (j + 1) * NDM8 / TAIL; ++i) dma1(ap, bp, buf, i);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int b = 0; b < TM; ++b) {
                    if constexpr (!F8) acc[a][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(hi4(fb8[a]), hi4(fa8[b]), acc[a][b], 0, 0, 0);
                    if constexpr (MORE_) {
                        if (a == TN - 2 && b == 0) frag8(nbuf, TM);  // next weight fragment 0: free since block 0
                        if (a == TN - 1) frag8(nbuf, b);              // next activation fragment b: this was its last reader
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
#pragma unroll
                for (int b = 0; b < TM; ++b) {
                    if constexpr (F8)
                        acc[a][b] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb8[a], fa8[b], acc[a][b], 0, 0, 0, 0, 0, 0);
                    const int j = (a - (TN - 2)) * TM + b;
                    if constexpr (DMA_) {
#pragma unroll
                        for (int i = j * NDM8 / TAIL; i < (j + 1) * NDM8 / TAIL; ++i) dma1(ap, bp, buf, i);
                    }
                    if constexpr (MORE_) {
                        if (a == TN - 2 && b == 0) frag8(nbuf, TM);  // next weight fragment 0: its registers were free since block 0
                        if (a == TN - 1) frag8(nbuf, b);              // next activation fragment b: this was its last reader
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        // A full LDS wait: the last activation fragments were read a few MFMAs ago
        // and this exposes part of their latency, but with reads still in flight
        // over the loop's back edge the compiler puts the same wait in front of the
        // next step's second MFMA, behind that step's first reads.
        __builtin_amdgcn_s_waitcnt(0xC07F);
        if constexpr (DMA_) advance_load();
        ck += BK;
        cslot = (cslot + 1) & 3;
        if (ck >= ck1) {
            if constexpr (FOLD) fold(cr);
            ++cr;
            const int rr = min(cr, p.nr - 1);
            ck = p.r[ph(rr)].k0;
            ck1 = p.r[ph(rr)].k1;
        }
        buf = nbuf;
    };
    // Measurement hooks (off in the library that ships: `make variant`, see the Makefile): the int8 K loop
    // with its MFMAs, its fragment reads or its DMA compiled out, barriers and waits in place.  The
    // results are wrong; the durations say what each of the three costs alone and in pairs.
#ifdef SEGQ_ABLATE_MFMA
    constexpr bool abl_mfma = true;
#else
    constexpr bool abl_mfma = false;
#endif
#ifdef SEGQ_ABLATE_LDS
    constexpr bool abl_lds = true;
#else
    constexpr bool abl_lds = false;
#endif
#ifdef SEGQ_ABLATE_DMA
    constexpr bool abl_dma = true;
#else
    constexpr bool abl_dma = false;
#endif
    auto step_i8 = [&](auto dma_c, auto more_c) __attribute__((always_inline)) {
        constexpr bool DMA_ = decltype(dma_c)::value;
        constexpr bool MORE_ = decltype(more_c)::value;
        const int nbuf = (buf + 1 == NS) ? 0 : buf + 1;
#pragma unroll
        for (int a = 0; a < TN; ++a)
#pragma unroll
            for (int b = 0; b < TM; ++b) {
                const int i = a * TM + b;
                if (i % RD_EVERY == 0 && i / RD_EVERY < NRD && !abl_lds) frag1(buf, 1, i / RD_EVERY);
                if constexpr (!abl_mfma) acc[a][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb[0][a], fa[0][b], acc[a][b], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        // Tile s+1 must have landed (the NS-2 tiles issued after it may still be in
        // flight) and this wave's reads of tile s must be done, before anyone reads
        // tile s+1 or overwrites the buffer of tile s.
        wait_dma(std::integral_constant<int, DMA_ ? NS - 2 : 0>{});
        __syncthreads();
        // tile s+NS goes where tile s was: both its halves are in registers
        const uint8_t* const ap = la + lk;
        const uint8_t* const bp = Bb + lk;
#pragma unroll
        for (int a = 0; a < TN; ++a)
#pragma unroll
            for (int b = 0; b < TM; ++b) {
                const int i = a * TM + b;
                if constexpr (DMA_) {
                    if (i % DM_EVERY == DM_EVERY - 1 && i / DM_EVERY < NDM && !abl_dma) dma1(ap, bp, buf, i / DM_EVERY);
                }
                if constexpr (MORE_) {
                    if (i % RD_EVERY == 0 && i / RD_EVERY < NRD && !abl_lds) frag1(nbuf, 0, i / RD_EVERY);
                }
                if constexpr (!abl_mfma) acc[a][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb[1][a], fa[1][b], acc[a][b], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        // The reads of the next tile's first half have had most of an MFMA group to
        // land.  Waiting for them here, explicitly, keeps the compiler from putting
        // a full LDS wait in front of the first MFMA at the loop head (it cannot
        // count reads across the back edge).
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0), vmcnt untouched
        if constexpr (DMA_) advance_load();
        ck += BK;
        dirty = true;
        if (ck >= ck1) {  // the range is complete: fold it, move to the next one
            if constexpr (PARK) park(cr);
            else if constexpr (FOLD) fold(cr);
            dirty = false;
            ++cr;
            const int rr = min(cr, p.nr - 1);
            ck = p.r[ph(rr)].k0;
            ck1 = p.r[ph(rr)].k1;
        }
        buf = nbuf;
    };
    auto step = [&](auto dma_c, auto more_c) __attribute__((always_inline)) {
        if constexpr (S8) step8(dma_c, more_c);
        else step_i8(dma_c, more_c);
    };
    int s = 0;
    for (; s + NS < steps; ++s) step(std::true_type{}, std::true_type{});
    for (; s + 1 < steps; ++s) step(std::false_type{}, std::true_type{});
    if (s < steps) step(std::false_type{}, std::false_type{});
    if constexpr (ACCF) {
        if (dirty) fold(cr);
    }
    if constexpr (FINISH) {
        // FINISH instances serve the launches that finish in output units (the others do not pay for
        // the registers of it): the low-rank branch and a tile split in two along K.  The sums are
        // scaled first (1 / (sx sw) of the range they are in units of, from the vectors parked in LDS); then
        //  * a tile split in two along K: the two workgroups meet in the workspace (below);
        //  * low-rank branch (out += T L2): the product joins in fp32 on the matrix cores;
        // and the epilogue only adds the bias and the addend and rounds once.
        v4f of[TN][TM];
        [[maybe_unused]] const bool parked = r_begin < r_last;
        constexpr int CH = 8;  // blocks whose loads are in flight at once (registers: the sums are still live)
#pragma unroll
        for (int c0 = 0; c0 < TN * TM; c0 += CH) {
            [[maybe_unused]] v4f old[CH];
            if constexpr (PARK) {
#pragma unroll
                for (int i = 0; i < CH; ++i)
                    if (c0 + i < TN * TM) old[i] = parked ? slot[(c0 + i) * NT] : v4f{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int i = 0; i < CH; ++i) {
                if (c0 + i < TN * TM) {
                    const int a = (c0 + i) / TM, b = (c0 + i) % TM;
                    v4f t;
                    if constexpr (HASF) t = accf[a][b];
                    else t = __builtin_convertvector(acc[a][b], v4f);
                    if constexpr (PARK) t += old[i];
                    if constexpr (!ACCF)
                        t = t * (*reinterpret_cast<const v4f*>(epi + BM + wn * WN + a * 16 + 4 * lgrp) * epi[wm * WM + b * 16 + lrow]);
                    of[a][b] = t;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (p.part) {
            // Two workgroups share a tile.  Each leaves its share in the workspace and counts itself in;
            // the one that finds the other counted adds that share to its own (a + b = b + a: the result
            // does not depend on who came last) and finishes the tile.  The two can sit on different
            // XCDs, whose L2 caches do not see each other's lines, so the shares are written through
            // and read past the caches (agent scope: what the compiler emits for a relaxed agent-scope
            // atomic, but 16 bytes per lane: 1 KB contiguous per wave and instruction).
            using v4u = __attribute__((ext_vector_type(4))) unsigned int;
            constexpr int AGENT = 16;  // the cache-policy bit for agent scope
            constexpr int SHARE = BM * BN * 4;
            const int my = zy;
            const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
                reinterpret_cast<uint8_t*>(p.part) + (int64_t)tile_id * 2 * SHARE, 0, 2 * SHARE, 0x00020000);
#pragma unroll
            for (int i = 0; i < TN * TM; ++i)
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, of[i / TM][i % TM]), rs, tid * 16, my * SHARE + i * NT * 16, AGENT);
            __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));  // this wave's stores have reached memory
            __syncthreads();                                  // ... and so have the other waves'
            int* const flag = reinterpret_cast<int*>(epi);    // (1 / sx of row 0: no longer needed)
            if (tid == 0) {
                // the launch's own stamp instead of a count: whatever the word held before (an earlier
                // launch's stamp, or anything at all in a fresh workspace) reads as "nobody yet"
                const unsigned before = __hip_atomic_exchange(p.arrived + tile_id, p.stamp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                *flag = before == p.stamp;
                // the second one clears the word: a replay of this very launch (a captured graph keeps
                // the stamp it was recorded with) must find "nobody yet" again
                if (before == p.stamp) __hip_atomic_store(p.arrived + tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            __syncthreads();
            if (!*flag) return;
#pragma unroll
            for (int c0 = 0; c0 < TN * TM; c0 += CH) {
                v4u other[CH];
#pragma unroll
                for (int i = 0; i < CH; ++i)
                    if (c0 + i < TN * TM)
                        other[i] = __builtin_amdgcn_raw_buffer_load_b128(rs, tid * 16, (1 - my) * SHARE + (c0 + i) * NT * 16, AGENT);
#pragma unroll
                for (int i = 0; i < CH; ++i)
                    if (c0 + i < TN * TM) of[(c0 + i) / TM][(c0 + i) % TM] += __builtin_bit_cast(v4f, other[i]);
            }
        }
        if (p.lr_rank > 0) lowrank_accumulate<TM, TN>(p, of, m0 + wm * WM, n0 + wn * WN, lane);
        wide_epilogue<BM, BN, WGM, WGN, GEMM_F8, false, true>(p, of, of, smem, z, m0, n0, wave, lane, r_epi, epi);
        return;
    }
    if constexpr (GRP) {
        v4f none[1][1];
        wide_epilogue<BM, BN, WGM, WGN, GEMM_F8, false, false>(p, accf, none, smem, z, m0, n0, wave, lane, r_epi, epi);
    } else if constexpr (PARK) {
        // the earlier ranges' sums come back in two halves, each with all its loads in flight at once
        v4f accp[TN][TM];
        constexpr int H = (TN + 1) / 2;
        const bool parked = r_begin < r_last;  // (a split's share can lie inside one range)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            v4f old[H][TM];
#pragma unroll
            for (int a = h * H; a < min(TN, (h + 1) * H); ++a)
#pragma unroll
                for (int b = 0; b < TM; ++b) old[a - h * H][b] = parked ? slot[(a * TM + b) * NT] : v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int a = h * H; a < min(TN, (h + 1) * H); ++a)
#pragma unroll
                for (int b = 0; b < TM; ++b) accp[a][b] = __builtin_convertvector(acc[a][b], v4f) + old[a - h * H][b];
        }
        v4f none[1][1];
        wide_epilogue<BM, BN, WGM, WGN, GEMM_F8, false, false>(p, accp, none, smem, z, m0, n0, wave, lane, r_epi, epi);
    } else if constexpr (CODES) {
        codes_epilogue<BM, BN, WGM, WGN, FMT>(p, acc, smem, m0, n0, wave, lane, epi);
    } else {
        wide_epilogue<BM, BN, WGM, WGN, FMT, false, ACCF>(p, acc, accf, smem, z, m0, n0, wave, lane, r_epi, epi);
    }
}

template <int BM, int BN, int WGM, int WGN, int FMT, bool B4, bool FOLD, bool ASEL>
int launch_wide_instance(const GemmParams& p, int64_t batch, hipStream_t st) {
    auto kern = gemm_wide_kernel<BM, BN, WGM, WGN, FMT, B4, FOLD, ASEL>;
    constexpr int lds = 2 * (BM + BN) * BK;
    if (p.dry) return SEGQ_OK;
    static unsigned long long attr_done = 0;
    if (const int rc = reserve_lds(reinterpret_cast<const void*>(kern), lds, &attr_done)) return rc;
    dim3 grid((unsigned)(p.tiles_m * p.tiles_n), (unsigned)batch);
    hipLaunchKernelGGL(kern, grid, dim3(WGM * WGN * 64), lds, st, p);
    return check_launch("segq_gemm");
}

// wide tile ids (after the generic ones): 256x256 | 256x128 | 128x256 | 128x128, eight waves each
template <int BM, int BN, int WGM, int WGN, int FMT, bool FOLD, int NS, bool GRP = false, bool PARK = false, bool FINISH = false,
          bool CODES = false>
int launch_pipe_instance(const GemmParams& p, int64_t batch, hipStream_t st) {
    auto kern = gemm_pipe_kernel<BM, BN, WGM, WGN, FMT, FOLD, NS, GRP, PARK, FINISH, CODES>;
    // the stages, the epilogue's vectors, and the ring of group factors
    constexpr int lds = NS * (BM + BN) * BK + (BM + 2 * BN) * 4 + (GRP ? 4 * BN * 4 : 0);
    if (p.dry) return SEGQ_OK;
    static unsigned long long attr_done = 0;
    if (const int rc = reserve_lds(reinterpret_cast<const void*>(kern), lds, &attr_done)) return rc;
    dim3 grid((unsigned)(p.tiles_m * p.tiles_n), (unsigned)batch);
    hipLaunchKernelGGL(kern, grid, dim3(WGM * WGN * 64), lds, st, p);
    return check_launch("segq_gemm");
}

template <int FMT, bool B4>
int launch_wide(const GemmParams& p, int wcfg, bool fold, bool asel, int64_t batch, hipStream_t st) {
    const bool tail = p.lr_rank > 0 || p.part;  // finishes in output units: the FINISH instances (tail_tile() says which exist)
    if constexpr (!B4 && FMT == GEMM_I8) {
        if (p.grw) {  // group-wise factors (the host has checked: plain codes, K ranges in whole steps)
            if (asel || tail) return fail(SEGQ_ERR_UNSUPPORTED, "segq_gemm: group factors need plain codes, and serve no low-rank branch");
            switch (wcfg) {
                case 0: case 1:
                    return fold ? launch_pipe_instance<256, 128, 4, 2, FMT, true, 2, true>(p, batch, st)
                                : launch_pipe_instance<256, 128, 4, 2, FMT, false, 2, true>(p, batch, st);
                case 2:
                    return fold ? launch_pipe_instance<128, 256, 2, 4, FMT, true, 2, true>(p, batch, st)
                                : launch_pipe_instance<128, 256, 2, 4, FMT, false, 2, true>(p, batch, st);
                case 3:
                    return fold ? launch_pipe_instance<128, 128, 4, 2, FMT, true, 2, true>(p, batch, st)
                                : launch_pipe_instance<128, 128, 4, 2, FMT, false, 2, true>(p, batch, st);
            }
            return fail(SEGQ_ERR_UNSUPPORTED, "segq_gemm: group factors run on the 256x128, 128x256 and 128x128 tiles of eight waves");
        }
    }
// a tile that exists with and without the tail / without only
#define SEGQ_PIPE2(BM_, BN_, WGM_, WGN_, FOLD_, PARK_)                                                               \
    return tail ? launch_pipe_instance<BM_, BN_, WGM_, WGN_, FMT, FOLD_, 2, false, PARK_, true>(p, batch, st)        \
                : launch_pipe_instance<BM_, BN_, WGM_, WGN_, FMT, FOLD_, 2, false, PARK_, false>(p, batch, st)
#define SEGQ_PIPE1(BM_, BN_, WGM_, WGN_, FOLD_, PARK_)                                                               \
    if (tail) break;                                                                                                 \
    return launch_pipe_instance<BM_, BN_, WGM_, WGN_, FMT, FOLD_, 2, false, PARK_, false>(p, batch, st)
    if (p.oc) {  // the epilogue writes codes: instances of their own, so that the others carry no trace of it
        if constexpr (!B4) {
            if (!asel && !fold && !tail && !p.park) {
                switch (wcfg) {
                    case 0: return launch_pipe_instance<256, 256, 4, 2, FMT, false, 2, false, false, false, true>(p, batch, st);
                    case 3: return launch_pipe_instance<128, 128, (FMT == GEMM_F8 ? 4 : 2), (FMT == GEMM_F8 ? 2 : 4), FMT, false, 2, false, false, false, true>(p, batch, st);
                }
            }
        }
        return fail(SEGQ_ERR_UNSUPPORTED, "segq_gemm: out_codes runs on tiles %d and %d with plain 8-bit codes on both sides and one range",
                    FIRST_WIDE_CFG + 1, FIRST_WIDE_CFG + 4);
    }
    if constexpr (!B4) {
        constexpr bool F8W = FMT == GEMM_F8;  // the e4m3 schedule wants three or more column blocks per wave
        if (!asel) {  // plain 8-bit operands, both straight to LDS: the software-pipelined kernel
            if (!fold) {
                switch (wcfg) {
                    case 0: SEGQ_PIPE2(256, 256, 4, 2, false, false);
                    case 1: SEGQ_PIPE2(256, 128, 4, 2, false, false);
                    case 2: SEGQ_PIPE1(128, 256, 2, 4, false, false);
                    case 3: SEGQ_PIPE2(128, 128, (F8W ? 4 : 2), (F8W ? 2 : 4), false, false);
                    case 4: SEGQ_PIPE1(192, 288, 4, 2, false, false);
                    case 5: SEGQ_PIPE1(288, 192, 2, 4, false, false);
                    case 6: SEGQ_PIPE2(256, 192, 4, 2, false, false);
                    case 7: SEGQ_PIPE2(192, 256, 2, 4, false, false);
                    case 8:  // four LDS stages: three K steps in flight per CU, for shapes that wait on HBM latency
                        if constexpr (!F8W) {
                            if (tail) break;
                            return launch_pipe_instance<128, 128, 2, 4, FMT, false, 4, false, false, false>(p, batch, st);
                        }
                        break;
                    case 9:  // wave tiles of 96 x 96
                        if (tail) break;
                        return launch_pipe_instance<384, 192, 4, 2, FMT, false, 2, false, false, false>(p, batch, st);
                    case 10:  // 128 x 96, five LDS stages: few tokens, more workgroups with four K steps in flight each
                        if constexpr (!F8W) {
                            if (tail) break;
                            return launch_pipe_instance<128, 96, 4, 2, FMT, false, 5, false, false, false>(p, batch, st);
                        }
                        break;
                }
            } else if constexpr (F8W) {  // fp32 accumulators are rescaled in place: every tile serves several ranges
                switch (wcfg) {
                    case 0: SEGQ_PIPE2(256, 256, 4, 2, true, false);
                    case 1: SEGQ_PIPE2(256, 128, 4, 2, true, false);
                    case 2: SEGQ_PIPE1(128, 256, 2, 4, true, false);
                    case 3: SEGQ_PIPE2(128, 128, 4, 2, true, false);
                    case 4: SEGQ_PIPE1(192, 288, 4, 2, true, false);
                    case 5: SEGQ_PIPE1(288, 192, 2, 4, true, false);
                    case 6: SEGQ_PIPE2(256, 192, 4, 2, true, false);
                    case 7: SEGQ_PIPE2(192, 256, 2, 4, true, false);
                    case 9: SEGQ_PIPE1(384, 192, 4, 2, true, false);
                }
            } else if (p.park) {  // int8, several ranges, a workspace to park finished ranges in: every tile
                if constexpr (!F8W) {
                    switch (wcfg) {
                        case 0: SEGQ_PIPE2(256, 256, 4, 2, true, true);
                        case 1: SEGQ_PIPE2(256, 128, 4, 2, true, true);
                        case 2: SEGQ_PIPE1(128, 256, 2, 4, true, true);
                        case 3: SEGQ_PIPE2(128, 128, 2, 4, true, true);
                        case 4: SEGQ_PIPE1(192, 288, 4, 2, true, true);
                        case 5: SEGQ_PIPE1(288, 192, 2, 4, true, true);
                        case 6: SEGQ_PIPE2(256, 192, 4, 2, true, true);
                        case 7: SEGQ_PIPE2(192, 256, 2, 4, true, true);
                    }
                }
            } else {
                switch (wcfg) {
                    case 0: case 1: SEGQ_PIPE2(256, 128, 4, 2, true, false);
                    case 2: SEGQ_PIPE1(128, 256, 2, 4, true, false);
                    case 3: SEGQ_PIPE2(128, 128, (F8W ? 4 : 2), (F8W ? 2 : 4), true, false);
                }
            }
        }
    }
#undef SEGQ_PIPE1
#undef SEGQ_PIPE2
    if (tail)
        return fail(SEGQ_ERR_UNSUPPORTED, "segq_gemm: tile %d finishes neither a low-rank branch nor a two-way K split", wcfg + FIRST_WIDE_CFG + 1);
#define SEGQ_WIDE(BM_, BN_, WGM_, WGN_, FOLD_)                                                          \
    return asel ? launch_wide_instance<BM_, BN_, WGM_, WGN_, FMT, B4, FOLD_, true>(p, batch, st)       \
                : launch_wide_instance<BM_, BN_, WGM_, WGN_, FMT, B4, FOLD_, false>(p, batch, st)
    if (!fold) {
        switch (wcfg) {
            case 0: SEGQ_WIDE(256, 256, 4, 2, false);
            case 1: SEGQ_WIDE(256, 128, 4, 2, false);
            case 2: SEGQ_WIDE(128, 256, 2, 4, false);
            case 3: SEGQ_WIDE(128, 128, 2, 4, false);
        }
    } else {
        switch (wcfg) {  // a second accumulator set: halve the wave tile
            case 0: case 1: SEGQ_WIDE(256, 128, 4, 2, true);
            case 2: SEGQ_WIDE(128, 256, 2, 4, true);
            case 3: SEGQ_WIDE(128, 128, 2, 4, true);
        }
    }
#undef SEGQ_WIDE
    return fail(SEGQ_ERR_UNSUPPORTED,
                "segq_gemm: tile %d is not built for this launch (its code format, several ranges, a sign selection, a low-rank "
                "branch or a K split); tile 0 lets the library choose",
                FIRST_WIDE_CFG + wcfg + 1);
}

}  // namespace segq
