// 256 x 256 output tile, four waves, each owning a 128 x 128 quadrant built from
// 32 x 32 MFMA tiles whose sixteen accumulator registers per tile live in AGPRs.
//
// Why this shape: with 8-bit operands the LDS, not the matrix pipe, is the first
// limit.  A wave reads (wave_m + wave_n) * 128 bytes of fragments per 128-byte K
// step and does wave_m * wave_n * 128 MACs with them, so the bytes read per MAC
// fall with the wave tile; 128 x 128 halves the LDS traffic of 64 x 64.  The
// 32 x 32 x 32 (int8) and 32 x 32 x 64 (e4m3) instructions run 8 and 16 passes,
// long enough for ONE wave per SIMD to keep the matrix pipe busy, which the
// 4-pass 16 x 16 x 64 int8 instruction does not do.
//
// Global -> LDS goes either through registers (needed when the activations are
// sign-selected or the weights are int4) or straight into LDS with
// global_load_lds_dwordx4; there the 16-byte chunk swizzle is applied on the
// SOURCE side, because the LDS side of such a load is lane-linear.
#pragma once
#include "segq_gemm_kernel.h"
#include <type_traits>

namespace segq {

typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

template <int FMT> struct BigAcc;
template <> struct BigAcc<GEMM_I8> { typedef v16i type; typedef int32_t elem; };
template <> struct BigAcc<GEMM_F8> { typedef v16f type; typedef float elem; };

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

template <int FMT, bool DIRECT>
__global__ void __launch_bounds__(256) gemm_big_kernel(const GemmParams p) {
    constexpr int BM = 256, BN = 256, NT = 256;
    constexpr int TM = 4, TN = 4;         // 32 x 32 tiles per wave quadrant
    constexpr int IT = BM * 8 / NT;       // 16-byte chunks per thread and operand
    typedef typename BigAcc<FMT>::type acc_t;
    typedef typename BigAcc<FMT>::elem acc_e;

    extern __shared__ __align__(16) uint8_t smem[];
    uint8_t* const As = smem;                // [2][256][128]
    uint8_t* const Bs = smem + 2 * BM * BK;  // [2][256][128]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 1, wn = wave >> 1;
    const int l32 = lane & 31, lhalf = lane >> 5;

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

    // staging: thread t, pass i covers row i * 32 + t / 8; physical chunk t % 8
    // of that row holds logical chunk (t % 8) ^ swz(row)
    const int s_row = tid >> 3;
    const int s_pc = tid & 7;
    const int s_lc = s_pc ^ swz(s_row);
    uint32_t a_goff[IT], b_goff[IT];
#pragma unroll
    for (int i = 0; i < IT; ++i) {
        a_goff[i] = (uint32_t)min(m0 + s_row + i * 32, p.M - 1) * (uint32_t)p.lda + s_lc * 16;
        b_goff[i] = (uint32_t)min(n0 + s_row + i * 32, p.N - 1) * (uint32_t)p.ldb + s_lc * 16;
    }
    const int s_lds = s_row * BK + s_pc * 16;           // register path: this thread's slot
    const int w_lds = wave * 8 * BK;                      // direct path: this wave's 8 rows

    uint4 ra[DIRECT ? 1 : IT], rb[DIRECT ? 1 : IT];

    // this kernel serves exactly one range: everything about it is loop invariant
    const int a_sel = p.r[0].a_sel;
    const int k_begin = p.r[0].k0, k_end = p.r[0].k1;
    const uint8_t* const Asel = (a_sel == 1) ? A2b : Ab;

    auto issue_loads = [&](int k, int buf) {
        const uint8_t* ap = Asel + k;
        const uint8_t* bp = Bb + k;
        if constexpr (DIRECT) {
            uint8_t* as = As + buf * BM * BK + w_lds;
            uint8_t* bs = Bs + buf * BN * BK + w_lds;
#pragma unroll
            for (int i = 0; i < IT; ++i) {
                load16_to_lds(ap + a_goff[i], as + i * 32 * BK);
                load16_to_lds(bp + b_goff[i], bs + i * 32 * BK);
            }
        } else {
#pragma unroll
            for (int i = 0; i < IT; ++i) {
                ra[i] = *reinterpret_cast<const uint4*>(ap + a_goff[i]);
                rb[i] = *reinterpret_cast<const uint4*>(bp + b_goff[i]);
            }
        }
    };
    auto commit_loads = [&](int buf) {
        if constexpr (DIRECT) {
            __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the LDS writes of this wave have landed
        } else {
            uint8_t* as = As + buf * BM * BK + s_lds;
            uint8_t* bs = Bs + buf * BN * BK + s_lds;
#pragma unroll
            for (int i = 0; i < IT; ++i) {
                *reinterpret_cast<uint4*>(as + i * 32 * BK) = select_sign(ra[i], a_sel);
                *reinterpret_cast<uint4*>(bs + i * 32 * BK) = rb[i];
            }
        }
    };

    acc_t acc[TN][TM];
    {
        const acc_t zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int a = 0; a < TN; ++a)
#pragma unroll
            for (int b = 0; b < TM; ++b) acc[a][b] = zero;
    }

    const int f_sw = swz(l32);
    const int a_frag = (wm * 128 + l32) * BK;
    const int b_frag = (wn * 128 + l32) * BK;

    auto compute = [&](int buf) {
        const uint8_t* as = As + buf * BM * BK + a_frag;
        const uint8_t* bs = Bs + buf * BN * BK + b_frag;
        if constexpr (FMT == GEMM_I8) {
            v4i fa[2][TM], fb[2][TN];
            auto frags = [&](int ks, int slot) {
                const int off = ((ks * 2 + lhalf) ^ f_sw) << 4;
#pragma unroll
                for (int t = 0; t < TM; ++t) fa[slot][t] = *reinterpret_cast<const v4i*>(as + t * 32 * BK + off);
#pragma unroll
                for (int t = 0; t < TN; ++t) fb[slot][t] = *reinterpret_cast<const v4i*>(bs + t * 32 * BK + off);
            };
            frags(0, 0);
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                if (ks < 3) frags(ks + 1, (ks + 1) & 1);
#pragma unroll
                for (int a = 0; a < TN; ++a)
#pragma unroll
                    for (int b = 0; b < TM; ++b)
                        acc[a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[ks & 1][a], fa[ks & 1][b], acc[a][b], 0, 0, 0);
            }
        } else {
            v8i fa[2][TM], fb[2][TN];
            auto frags = [&](int ks, int slot) {
                const int off0 = ((ks * 4 + 2 * lhalf) ^ f_sw) << 4;
                const int off1 = ((ks * 4 + 2 * lhalf + 1) ^ f_sw) << 4;
#pragma unroll
                for (int t = 0; t < TM; ++t) {
                    const v4i lo = *reinterpret_cast<const v4i*>(as + t * 32 * BK + off0);
                    const v4i hi = *reinterpret_cast<const v4i*>(as + t * 32 * BK + off1);
                    fa[slot][t] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
                }
#pragma unroll
                for (int t = 0; t < TN; ++t) {
                    const v4i lo = *reinterpret_cast<const v4i*>(bs + t * 32 * BK + off0);
                    const v4i hi = *reinterpret_cast<const v4i*>(bs + t * 32 * BK + off1);
                    fb[slot][t] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
                }
            };
            frags(0, 0);
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                if (ks < 1) frags(ks + 1, (ks + 1) & 1);
#pragma unroll
                for (int a = 0; a < TN; ++a)
#pragma unroll
                    for (int b = 0; b < TM; ++b)
                        acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[ks & 1][a], fa[ks & 1][b], acc[a][b], 0, 0, 0, 0, 0, 0);
            }
        }
    };

    // ---- main loop: K in whole 128-byte steps, LDS double-buffered
    issue_loads(k_begin, 0);
    commit_loads(0);
    __syncthreads();
    int buf = 0;
    for (int k = k_begin; k < k_end; k += BK) {
        const bool more = k + BK < k_end;
        if (more) issue_loads(k + BK, buf ^ 1);
        compute(buf);
        if (more) {
            commit_loads(buf ^ 1);
            __syncthreads();
            buf ^= 1;
        }
    }

    // ---- epilogue.  Lane holds row m = .. + lane % 32 and, per tile, columns
    // n = 8 * (v / 4) + 4 * (lane / 32) + v % 4: four runs of four consecutive columns.
    const int m_base = m0 + wm * 128 + l32;
    const int n_base = n0 + wn * 128 + 4 * lhalf;
    const int64_t c_off = z * p.bsC;
    float rx[TM];
    if (p.out_dtype != SEGQ_ACC) {
        const float* sxp = p.r[0].sx + z * p.bsSx;
#pragma unroll
        for (int b = 0; b < TM; ++b) rx[b] = 1.0f / sxp[(int64_t)min(m_base + b * 32, p.M - 1) * p.r[0].sx_rs];
    }
    // one instance per output type keeps each unrolled loop nest small enough
    // for the accumulators to stay in registers
    auto epilogue = [&](auto out_tag) {
        constexpr int OUT = decltype(out_tag)::value;
#pragma unroll
        for (int a = 0; a < TN; ++a) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = n_base + a * 32 + q * 8;
                float rw[4], bv[4];
                if constexpr (OUT != SEGQ_ACC) {
                    const float* swp = p.r[0].sw + z * p.bsSw;
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int nn = min(n + v, p.N - 1);
                        rw[v] = 1.0f / swp[(int64_t)nn * p.r[0].sw_cs];
                        bv[v] = p.bias ? load_bias(p.bias, p.bias_dtype, nn) : 0.0f;
                    }
                }
                const bool vec = p.vec_store && (n + 3 < p.N);
#pragma unroll
                for (int b = 0; b < TM; ++b) {
                    const int m = m_base + b * 32;
                    if (m < p.M && n < p.N) {
                        const int64_t e = c_off + (int64_t)m * p.ldc + n;
                        if constexpr (OUT == SEGQ_ACC) {
                            acc_e* dst = static_cast<acc_e*>(p.C) + e;
#pragma unroll
                            for (int v = 0; v < 4; ++v)
                                if (n + v < p.N) dst[v] = acc[a][b][q * 4 + v];
                        } else {
                            float o[4];
#pragma unroll
                            for (int v = 0; v < 4; ++v) o[v] = (float)acc[a][b][q * 4 + v] * rx[b] * rw[v] + bv[v];
                            add_addend4(p, z, m, n, o);
                            store4<OUT>(p.C, e, o, vec, p.N - n);
                        }
                    }
                }
            }
        }
    };
    switch (p.out_dtype) {
        case SEGQ_ACC: epilogue(std::integral_constant<int, SEGQ_ACC>{}); break;
        case SEGQ_F32: epilogue(std::integral_constant<int, SEGQ_F32>{}); break;
        case SEGQ_F16: epilogue(std::integral_constant<int, SEGQ_F16>{}); break;
        default: epilogue(std::integral_constant<int, SEGQ_BF16>{}); break;
    }
}

template <int FMT, bool DIRECT>
int launch_big(const GemmParams& p, int64_t batch, hipStream_t st) {
    auto kern = gemm_big_kernel<FMT, DIRECT>;
    constexpr int lds = 2 * (256 + 256) * BK;
    static bool attr_set = false;
    if (!attr_set) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
            return fail(SEGQ_ERR_LAUNCH, "segq_gemm: cannot reserve %d bytes of LDS", lds);
        attr_set = true;
    }
    dim3 grid((unsigned)(p.tiles_m * p.tiles_n), (unsigned)batch);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, st, p);
    return check_launch("segq_gemm");
}

}  // namespace segq
