// Quantise kernels of libsegq: float matrix -> int8 / e4m3 / packed-int4 codes.
//
// One pass over HBM: every thread converts runs of 16 consecutive elements of a
// row (two or four 16-byte loads, one 16-byte or 8-byte store).  The static
// kernel is a flat grid over such runs; the dynamic kernel gives a row to a
// block, keeps the row in registers while it reduces the absolute maximum, and
// quantises from registers.
#include "segq_common.h"
#include "segq_encode.h"

namespace segq {

struct QuantParams {
    const void* x;
    void* codes;
    void* codes_neg;
    float* scale;
    float* scale_neg;
    int64_t rows, cols, ldx, ldc;
    int64_t seg_rows, seg_stride, row_stride, kseg_stride;
    int32_t x_dtype, fmt;
    int32_t n_kseg, dual, dynamic;
    uint32_t dual_mask;
    float scale_imm;  // used when scale == nullptr (one scale passed by value)
    int32_t pre_op;   // segq_pre_op applied to the input before it is quantised
    const void* gate; // with a pre_op: x is multiplied by op(gate) instead of being replaced by op(x)
    int64_t ldg;
    const float* col_div;  // per-column divisors (SmoothQuant's s), applied after the pre_op, or null
    int32_t group;         // > 0: column segments are runs of this many columns (any number of them), kb unused
    int32_t kb[SEGQ_MAX_KSEG + 1];
};

// ---- element conversion --------------------------------------------------

// 16 consecutive elements of dtype DT starting at p (16-byte aligned) -> fp32.
template <int DT>
__device__ __forceinline__ void load16(const void* p, float (&v)[16]) {
    if constexpr (DT == SEGQ_F32) {
        const float4* q = reinterpret_cast<const float4*>(p);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float4 t = q[i];
            v[4 * i + 0] = t.x; v[4 * i + 1] = t.y; v[4 * i + 2] = t.z; v[4 * i + 3] = t.w;
        }
    } else {
        const uint4* q = reinterpret_cast<const uint4*>(p);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            uint4 t = q[i];
            uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if constexpr (DT == SEGQ_BF16) {
                    v[8 * i + 2 * j + 0] = __uint_as_float(w[j] << 16);
                    v[8 * i + 2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
                } else {
                    v[8 * i + 2 * j + 0] = f16_bits_to_f32(w[j] & 0xffffu);
                    v[8 * i + 2 * j + 1] = f16_bits_to_f32(w[j] >> 16);
                }
            }
        }
    }
}

// 8 values -> 8 nibbles, element 0 in the lowest nibble.
__device__ __forceinline__ uint32_t pack8_i4(const float* v) {
    uint32_t r = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) r |= (uint32_t)(q_i4(v[i]) & 0xf) << (4 * i);
    return r;
}

// Encodes 16 scaled values and stores them at row-relative element offset col.
template <int FMT>
__device__ __forceinline__ void store16(void* row_base, int64_t col, const float (&v)[16]) {
    if constexpr (FMT == SEGQ_CODE_I4) {
        uint2 o;
        o.x = pack8_i4(v);
        o.y = pack8_i4(v + 8);
        *reinterpret_cast<uint2*>(static_cast<uint8_t*>(row_base) + (col >> 1)) = o;
    } else {
        uint4 o;
        if constexpr (FMT == SEGQ_CODE_I8) {
            o.x = pack4_i8(v[0], v[1], v[2], v[3]);
            o.y = pack4_i8(v[4], v[5], v[6], v[7]);
            o.z = pack4_i8(v[8], v[9], v[10], v[11]);
            o.w = pack4_i8(v[12], v[13], v[14], v[15]);
        } else {
            o.x = pack4_e4m3(v[0], v[1], v[2], v[3]);
            o.y = pack4_e4m3(v[4], v[5], v[6], v[7]);
            o.z = pack4_e4m3(v[8], v[9], v[10], v[11]);
            o.w = pack4_e4m3(v[12], v[13], v[14], v[15]);
        }
        *reinterpret_cast<uint4*>(static_cast<uint8_t*>(row_base) + col) = o;
    }
}

// Scales 16 raw values and writes the merged tensor, or Xp and Xn.
template <int FMT>
__device__ __forceinline__ void encode16(const QuantParams& p, int64_t row, int64_t col, const float (&x)[16],
                                         float s_pos, float s_neg, bool two_tensors) {
    const int64_t cstride = p.ldc;
    uint8_t* base = static_cast<uint8_t*>(p.codes) + row * cstride;
    float v[16];
    if (!two_tensors) {
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] = x[i] * ((x[i] >= 0.0f) ? s_pos : s_neg);
        store16<FMT>(base, col, v);
    } else {
        // The branch that was not taken holds code(0) (quantizer.cuh:193-203).
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] = (x[i] >= 0.0f) ? x[i] * s_pos : 0.0f;
        store16<FMT>(base, col, v);
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] = (x[i] >= 0.0f) ? 0.0f : x[i] * s_neg;
        store16<FMT>(static_cast<uint8_t*>(p.codes_neg) + row * cstride, col, v);
    }
}

__device__ __forceinline__ int64_t row_scale_index(const QuantParams& p, int64_t row) {
    if (p.seg_rows >= p.rows) return row * p.row_stride;
    const int64_t seg = row / p.seg_rows;
    return seg * p.seg_stride + (row - seg * p.seg_rows) * p.row_stride;
}

__device__ __forceinline__ int kseg_of(const QuantParams& p, int col) {
    if (p.group > 0) return col / p.group;
    int s = 0;
    for (int i = 1; i < p.n_kseg; ++i) s += (col >= p.kb[i]) ? 1 : 0;
    return s;
}

// ---- dynamic per-row scales ------------------------------------------------
template <int FMT>
__device__ __forceinline__ float qmax_pos() {
    return FMT == SEGQ_CODE_I8 ? 127.0f : (FMT == SEGQ_CODE_I4 ? 7.0f : 448.0f);
}
template <int FMT>
__device__ __forceinline__ float qmax_neg() {
    return FMT == SEGQ_CODE_I8 ? 128.0f : (FMT == SEGQ_CODE_I4 ? 8.0f : 448.0f);
}

template <int DT>
struct RawRun {  // 16 consecutive elements as they sit in memory
    uint4 q[DT == SEGQ_F32 ? 4 : 2];
};

template <int DT>
__device__ __forceinline__ void load_raw(const void* p, RawRun<DT>& r) {
    const uint4* q = reinterpret_cast<const uint4*>(p);
#pragma unroll
    for (int i = 0; i < (DT == SEGQ_F32 ? 4 : 2); ++i) r.q[i] = q[i];
}

template <int DT>
__device__ __forceinline__ void raw_to_f32(const RawRun<DT>& r, float (&v)[16]) {
    if constexpr (DT == SEGQ_F32) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[4 * i + 0] = __uint_as_float(r.q[i].x); v[4 * i + 1] = __uint_as_float(r.q[i].y);
            v[4 * i + 2] = __uint_as_float(r.q[i].z); v[4 * i + 3] = __uint_as_float(r.q[i].w);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint32_t w[4] = {r.q[i].x, r.q[i].y, r.q[i].z, r.q[i].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if constexpr (DT == SEGQ_BF16) {
                    v[8 * i + 2 * j + 0] = __uint_as_float(w[j] << 16);
                    v[8 * i + 2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
                } else {
                    v[8 * i + 2 * j + 0] = f16_bits_to_f32(w[j] & 0xffffu);
                    v[8 * i + 2 * j + 1] = f16_bits_to_f32(w[j] >> 16);
                }
            }
        }
    }
}

// 16 fp32 values -> a run in the tensor's dtype, rounded to nearest even
template <int DT>
__device__ __forceinline__ void f32_to_raw(const float (&v)[16], RawRun<DT>& r) {
    if constexpr (DT == SEGQ_F32) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            r.q[i] = make_uint4(__float_as_uint(v[4 * i]), __float_as_uint(v[4 * i + 1]), __float_as_uint(v[4 * i + 2]),
                                __float_as_uint(v[4 * i + 3]));
    } else {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            uint32_t w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                w[j] = (DT == SEGQ_BF16) ? pack2_bf16(v[8 * i + 2 * j], v[8 * i + 2 * j + 1])
                                         : pack2_f16(v[8 * i + 2 * j], v[8 * i + 2 * j + 1]);
            r.q[i] = make_uint4(w[0], w[1], w[2], w[3]);
        }
    }
}

// r holds 16 elements of x at (row, col); on return it holds what is quantised:
// op(x), or x * op(gate), each operator's result rounded to the tensor's dtype
template <int DT>
__device__ __forceinline__ void pre_run(const QuantParams& p, int64_t row, int64_t col, RawRun<DT>& r) {
    float v[16];
    raw_to_f32<DT>(r, v);
    if (p.pre_op != SEGQ_PRE_NONE) {
        if (p.gate) {
            const size_t esz = (DT == SEGQ_F32) ? 4 : 2;
            RawRun<DT> gr;
            load_raw<DT>(static_cast<const uint8_t*>(p.gate) + (row * p.ldg + col) * esz, gr);
            float g[16];
            raw_to_f32<DT>(gr, g);
#pragma unroll
            for (int i = 0; i < 16; ++i) g[i] = act_value(p.pre_op, g[i]);
            f32_to_raw<DT>(g, gr);
            raw_to_f32<DT>(gr, g);
#pragma unroll
            for (int i = 0; i < 16; ++i) v[i] *= g[i];
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i) v[i] = act_value(p.pre_op, v[i]);
        }
        if (p.col_div) {  // the activation's result is rounded to the dtype before it is divided
            f32_to_raw<DT>(v, r);
            raw_to_f32<DT>(r, v);
        }
    }
    if (p.col_div) {
        // x / s as torch's in-place div_ in the tensor's dtype: an IEEE fp32 division, rounded to the dtype
        const float4* q = reinterpret_cast<const float4*>(p.col_div + col);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float4 t = q[i];
            v[4 * i + 0] = v[4 * i + 0] / t.x; v[4 * i + 1] = v[4 * i + 1] / t.y;
            v[4 * i + 2] = v[4 * i + 2] / t.z; v[4 * i + 3] = v[4 * i + 3] / t.w;
        }
    }
    f32_to_raw<DT>(v, r);
}

// With a fused activation the run kept in registers is the activation's output
// (already in the tensor's dtype, so repacking it loses nothing).
template <int DT, bool PRE>
__device__ __forceinline__ void load_run(const QuantParams& p, const uint8_t* xrow, int64_t row, int c, RawRun<DT>& r) {
    const size_t esz = (DT == SEGQ_F32) ? 4 : 2;
    load_raw<DT>(xrow + (size_t)c * 16 * esz, r);
    if constexpr (PRE) pre_run<DT>(p, row, (int64_t)c << 4, r);
}

// Maximum of two non-negative floats, taken on their encodings: non-negative floats are ordered
// like their bit patterns and every NaN pattern lies above infinity's, so a NaN wins and travels
// on (fmaxf would drop it), as it does through torch's amax (segquant/quantizers/quantizer.py:212).
__device__ __forceinline__ float max_nn(float a, float b) {
    const uint32_t ua = __float_as_uint(a), ub = __float_as_uint(b);
    return __uint_as_float(ua > ub ? ua : ub);
}

// DualScale segments: running maxima of the positive and of the negative side (strict masks
// x > 0 and x < 0, segquant/quantizers/quantizer.py:172-189; a NaN is on neither side).  Other
// segments: the maximum of |x| in amax_p, NaN if the segment holds one.
template <bool DUAL>
__device__ __forceinline__ void track_amax(const float (&v)[16], float& amax_p, float& amax_n, const bool dual = DUAL) {
    if (DUAL && dual) {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            amax_p = fmaxf(amax_p, v[j]);    // starts at 0, so negatives never win
            amax_n = fmaxf(amax_n, -v[j]);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 16; ++j) amax_p = max_nn(amax_p, fabsf(v[j]));
    }
}

__device__ __forceinline__ float wave_max(float v) {  // of non-negative values or NaN
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = max_nn(v, __shfl_xor(v, o, 64));
    return v;
}

// One workgroup per row, for rows longer than a wave can hold.  All loads of
// the row are issued before anything is computed; up to CACHE runs per thread
// stay in registers in packed form between the reduction and the encode, longer
// rows are read again (they hit in L2).
template <int DT, int FMT, bool DUAL, bool PRE>
__global__ void __launch_bounds__(256) quant_dynamic_kernel(const QuantParams p) {
    constexpr int CACHE = 4;
    __shared__ float red[2][4];
    const int64_t row = blockIdx.x;
    const size_t esz = (DT == SEGQ_F32) ? 4 : 2;
    const uint8_t* xrow = static_cast<const uint8_t*>(p.x) + row * p.ldx * esz;
    const float eps = 5.9604644775390625e-08f;  // 2^-24
    for (int ks = 0; ks < p.n_kseg; ++ks) {
        const int c0 = p.kb[ks] >> 4, c1 = p.kb[ks + 1] >> 4;
        const bool dual = DUAL && ((p.dual_mask >> ks) & 1u);
        const bool two = dual && p.codes_neg != nullptr;  // the second tensor exists only for DualScale segments
        RawRun<DT> raw[CACHE];
#pragma unroll
        for (int i = 0; i < CACHE; ++i) {
            const int c = c0 + threadIdx.x + i * 256;
            if (c < c1) load_run<DT, PRE>(p, xrow, row, c, raw[i]);
        }
        float amax_p = 0.0f, amax_n = 0.0f;
#pragma unroll
        for (int i = 0; i < CACHE; ++i) {
            const int c = c0 + threadIdx.x + i * 256;
            if (c < c1) {
                float v[16];
                raw_to_f32<DT>(raw[i], v);
                track_amax<DUAL>(v, amax_p, amax_n, dual);
            }
        }
        for (int c = c0 + threadIdx.x + CACHE * 256; c < c1; c += 256) {
            RawRun<DT> t;
            float v[16];
            load_run<DT, PRE>(p, xrow, row, c, t);
            raw_to_f32<DT>(t, v);
            track_amax<DUAL>(v, amax_p, amax_n, dual);
        }
        amax_p = wave_max(amax_p);
        if constexpr (DUAL) amax_n = wave_max(amax_n);
        __syncthreads();  // red may still be read from the previous column segment
        if ((threadIdx.x & 63) == 0) {
            red[0][threadIdx.x >> 6] = amax_p;
            red[1][threadIdx.x >> 6] = amax_n;
        }
        __syncthreads();
        amax_p = max_nn(max_nn(red[0][0], red[0][1]), max_nn(red[0][2], red[0][3]));
        amax_n = max_nn(max_nn(red[1][0], red[1][1]), max_nn(red[1][2], red[1][3]));
        float s_pos, s_neg;
        if (dual) {
            s_pos = qmax_pos<FMT>() / fmaxf(amax_p, eps);
            s_neg = qmax_neg<FMT>() / fmaxf(amax_n, eps);
        } else {
            s_pos = s_neg = qmax_pos<FMT>() / max_nn(amax_p, eps);
        }
        const int64_t si = row_scale_index(p, row) + (int64_t)ks * p.kseg_stride;
        if (threadIdx.x == 0) {
            p.scale[si] = s_pos;
            if (DUAL) p.scale_neg[si] = s_neg;
        }
#pragma unroll
        for (int i = 0; i < CACHE; ++i) {
            const int c = c0 + threadIdx.x + i * 256;
            if (c < c1) {
                float v[16];
                raw_to_f32<DT>(raw[i], v);
                encode16<FMT>(p, row, (int64_t)c << 4, v, s_pos, s_neg, two);
            }
        }
        for (int c = c0 + threadIdx.x + CACHE * 256; c < c1; c += 256) {
            RawRun<DT> t;
            float v[16];
            load_run<DT, PRE>(p, xrow, row, c, t);
            raw_to_f32<DT>(t, v);
            encode16<FMT>(p, row, (int64_t)c << 4, v, s_pos, s_neg, two);
        }
    }
}

// ---- dynamic per-row scales, one WAVE per row --------------------------------
// For rows of up to 64 * CPL runs: the whole row is in flight at once, the
// maximum is reduced with cross-lane shuffles only, and four rows share a
// workgroup without ever synchronising.
template <int DT, int FMT, int CPL, bool DUAL, bool PRE, bool KEEP = (CPL <= 4)>
__global__ void __launch_bounds__(256) quant_dynamic_wave_kernel(const QuantParams p) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= p.rows) return;
    const size_t esz = (DT == SEGQ_F32) ? 4 : 2;
    const uint8_t* xrow = static_cast<const uint8_t*>(p.x) + row * p.ldx * esz;
    const float eps = 5.9604644775390625e-08f;  // 2^-24
    for (int ks = 0; ks < p.n_kseg; ++ks) {
        const int c0 = p.kb[ks] >> 4, c1 = p.kb[ks + 1] >> 4;
        const bool dual = DUAL && ((p.dual_mask >> ks) & 1u);
        const bool two = dual && p.codes_neg != nullptr;  // the second tensor exists only for DualScale segments
        RawRun<DT> raw[CPL];
#pragma unroll
        for (int i = 0; i < CPL; ++i) {
            const int c = c0 + lane + i * 64;
            if (c < c1) load_run<DT, PRE>(p, xrow, row, c, raw[i]);
        }
        // short rows: unpack once and keep the floats (64 registers) instead of unpacking
        // again for the encode; longer rows stay packed
        float vf[KEEP ? CPL : 1][16];
        float amax_p = 0.0f, amax_n = 0.0f;
#pragma unroll
        for (int i = 0; i < CPL; ++i) {
            const int c = c0 + lane + i * 64;
            if (c < c1) {
                if constexpr (KEEP) {
                    raw_to_f32<DT>(raw[i], vf[i]);
                    track_amax<DUAL>(vf[i], amax_p, amax_n, dual);
                } else {
                    float v[16];
                    raw_to_f32<DT>(raw[i], v);
                    track_amax<DUAL>(v, amax_p, amax_n, dual);
                }
            }
        }
        amax_p = wave_max(amax_p);
        if constexpr (DUAL) amax_n = wave_max(amax_n);
        float s_pos, s_neg;
        if (dual) {
            s_pos = qmax_pos<FMT>() / fmaxf(amax_p, eps);
            s_neg = qmax_neg<FMT>() / fmaxf(amax_n, eps);
        } else {
            s_pos = s_neg = qmax_pos<FMT>() / max_nn(amax_p, eps);
        }
        const int64_t si = row_scale_index(p, row) + (int64_t)ks * p.kseg_stride;
        if (lane == 0) {
            p.scale[si] = s_pos;
            if (DUAL) p.scale_neg[si] = s_neg;
        }
#pragma unroll
        for (int i = 0; i < CPL; ++i) {
            const int c = c0 + lane + i * 64;
            if (c < c1) {
                if constexpr (KEEP) {
                    encode16<FMT>(p, row, (int64_t)c << 4, vf[i], s_pos, s_neg, two);
                } else {
                    float v[16];
                    raw_to_f32<DT>(raw[i], v);
                    encode16<FMT>(p, row, (int64_t)c << 4, v, s_pos, s_neg, two);
                }
            }
        }
    }
}

// ---- dynamic per-row scales, one wave per row, one column segment -------------
// The common case (no column segments, no fused producer) without the segment
// loop: every wave is a workgroup of its own, so consecutive rows spread over
// the compute units from the first moment of the launch.  Measured against the
// segment-aware kernel above, cache-cold, bf16 -> int8: 4608 x 3072 12.1 -> 10.3 us,
// 9216 x 3072 19.7 -> 17.7 us, 8192 x 1280 11.0 -> 9.1 us.  (A version whose waves
// walked several rows with the next row's loads in flight measured the same.)
template <int DT, int FMT, int CPL, bool DUAL>
__device__ __forceinline__ void quant_dynamic_row_body(const QuantParams& p, const int64_t row, const int lane) {
    const size_t esz = (DT == SEGQ_F32) ? 4 : 2;
    const int c1 = (int)(p.cols >> 4);
    const float eps = 5.9604644775390625e-08f;  // 2^-24
    const bool two = DUAL && p.codes_neg != nullptr;
    RawRun<DT> raw[CPL];
    {
        const uint8_t* xrow = static_cast<const uint8_t*>(p.x) + row * p.ldx * esz;
#pragma unroll
        for (int i = 0; i < CPL; ++i)
            if (lane + i * 64 < c1) load_raw<DT>(xrow + (size_t)(lane + i * 64) * 16 * esz, raw[i]);
    }
    {
        float amax_p = 0.0f, amax_n = 0.0f;
#pragma unroll
        for (int i = 0; i < CPL; ++i) {
            if (lane + i * 64 < c1) {
                float v[16];
                raw_to_f32<DT>(raw[i], v);
                track_amax<DUAL>(v, amax_p, amax_n);
            }
        }
        amax_p = wave_max(amax_p);
        if constexpr (DUAL) amax_n = wave_max(amax_n);
        float s_pos, s_neg;
        if constexpr (DUAL) {
            s_pos = qmax_pos<FMT>() / fmaxf(amax_p, eps);
            s_neg = qmax_neg<FMT>() / fmaxf(amax_n, eps);
        } else {
            s_pos = s_neg = qmax_pos<FMT>() / max_nn(amax_p, eps);
        }
        const int64_t si = row_scale_index(p, row);
        if (lane == 0) {
            p.scale[si] = s_pos;
            if (DUAL) p.scale_neg[si] = s_neg;
        }
#pragma unroll
        for (int i = 0; i < CPL; ++i) {
            if (lane + i * 64 < c1) {
                float v[16];
                raw_to_f32<DT>(raw[i], v);
                encode16<FMT>(p, row, (int64_t)(lane + i * 64) << 4, v, s_pos, s_neg, two);
            }
        }
    }
}

template <int DT, int FMT, int CPL, bool DUAL>
__global__ void __launch_bounds__(64) quant_dynamic_row_kernel(const QuantParams p) {
    quant_dynamic_row_body<DT, FMT, CPL, DUAL>(p, blockIdx.x, threadIdx.x);
}

// The same for up to SEGQ_QUANT_BATCH tensors in one grid: workgroup w serves row w - first[i] of tensor i.
constexpr int SEGQ_QUANT_BATCH = 4;
struct QuantBatch {
    int32_t n;
    int32_t first[SEGQ_QUANT_BATCH + 1];  // first workgroup of each tensor, then the grid size
    QuantParams p[SEGQ_QUANT_BATCH];
};

template <int DT, int FMT, int CPL, bool DUAL>
__global__ void __launch_bounds__(64) quant_dynamic_row_many_kernel(const QuantBatch b) {
    const int w = blockIdx.x;
    int i = 0;
    while (i + 1 < b.n && w >= b.first[i + 1]) ++i;
    quant_dynamic_row_body<DT, FMT, CPL, DUAL>(b.p[i], w - b.first[i], threadIdx.x);
}


// ---- static scales ---------------------------------------------------------
template <int DT, int FMT, bool PRE>
__global__ void __launch_bounds__(256) quant_static_kernel(const QuantParams p) {
    const int64_t cpr = p.cols >> 4;  // runs of 16 per row
    const int64_t run = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (run >= p.rows * cpr) return;
    const int64_t row = run / cpr;
    const int col = (int)(run - row * cpr) << 4;
    const int ks = kseg_of(p, col);
    const int64_t si = row_scale_index(p, row) + (int64_t)ks * p.kseg_stride;
    const bool dual = p.dual && ((p.dual_mask >> (ks & 31)) & 1u);
    const float s_pos = p.scale ? p.scale[si] : p.scale_imm;
    const float s_neg = dual ? p.scale_neg[si] : s_pos;
    const size_t esz = (DT == SEGQ_F32) ? 4 : 2;
    float x[16];
    if constexpr (PRE) {
        RawRun<DT> r;
        load_raw<DT>(static_cast<const uint8_t*>(p.x) + (row * p.ldx + col) * esz, r);
        pre_run<DT>(p, row, col, r);
        raw_to_f32<DT>(r, x);
    } else {
        load16<DT>(static_cast<const uint8_t*>(p.x) + (row * p.ldx + col) * esz, x);
    }
    // the second tensor exists only for DualScale column segments
    encode16<FMT>(p, row, col, x, s_pos, s_neg, dual && p.codes_neg != nullptr);
}

// ---- fake e4m3 round trip ----------------------------------------------------
__device__ __forceinline__ float e4m3_roundtrip(float v) {
    int r = __builtin_amdgcn_cvt_pk_fp8_f32(sat_e4m3(v), 0.0f, 0, false);
    return (v != v) ? v : __builtin_amdgcn_cvt_f32_fp8(r, 0);
}

template <int DT>
__global__ void __launch_bounds__(256) fake_e4m3_kernel(const void* x, void* out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    if constexpr (DT == SEGQ_F32) {
        static_cast<float*>(out)[i] = e4m3_roundtrip(static_cast<const float*>(x)[i]);
    } else if constexpr (DT == SEGQ_BF16) {
        const float v = bf16_bits_to_f32(static_cast<const uint16_t*>(x)[i]);
        static_cast<uint16_t*>(out)[i] = (uint16_t)f32_to_bf16_bits(e4m3_roundtrip(v));
    } else {
        const float v = f16_bits_to_f32(static_cast<const uint16_t*>(x)[i]);
        static_cast<uint16_t*>(out)[i] = (uint16_t)f32_to_f16_bits(e4m3_roundtrip(v));
    }
}

// ---- host side ---------------------------------------------------------------
template <int DT, int FMT, bool PRE>
static int launch_quant(const QuantParams& p, hipStream_t st) {
    if (p.dynamic) {
        int longest = 0;  // runs of 16 in the longest column segment
        for (int i = 0; i < p.n_kseg; ++i) longest = longest > (p.kb[i + 1] - p.kb[i]) / 16 ? longest : (p.kb[i + 1] - p.kb[i]) / 16;
        const dim3 wgrid((unsigned)((p.rows + 3) / 4)), bgrid((unsigned)p.rows);
        if constexpr (!PRE) {
            if (p.n_kseg == 1 && longest <= 64 * 8 && (!p.dual || (p.dual_mask & 1u))) {
                const dim3 rgrid((unsigned)p.rows), one_wave(64);
#define SEGQ_ROW(CPL_)                                                                                              \
    if (p.dual) hipLaunchKernelGGL((quant_dynamic_row_kernel<DT, FMT, CPL_, true>), rgrid, one_wave, 0, st, p);     \
    else hipLaunchKernelGGL((quant_dynamic_row_kernel<DT, FMT, CPL_, false>), rgrid, one_wave, 0, st, p)
                if (longest <= 64) { SEGQ_ROW(1); }
                else if (longest <= 128) { SEGQ_ROW(2); }
                else if (longest <= 192) { SEGQ_ROW(3); }
                else if (longest <= 256) { SEGQ_ROW(4); }
                else if (longest <= 384) { SEGQ_ROW(6); }
                else { SEGQ_ROW(8); }
#undef SEGQ_ROW
                return check_launch("segq_quantize");
            }
        }
        if (longest <= 64 * 4) {
            if (p.dual) hipLaunchKernelGGL((quant_dynamic_wave_kernel<DT, FMT, 4, true, PRE>), wgrid, dim3(256), 0, st, p);
            else hipLaunchKernelGGL((quant_dynamic_wave_kernel<DT, FMT, 4, false, PRE>), wgrid, dim3(256), 0, st, p);
        } else if (longest <= 64 * 8 && longest % 256 != 0) {
            // rows a workgroup's 256 threads would share unevenly (320 runs: a quarter of the threads
            // with two, the rest with one) stay with one wave per row
            if (p.dual) hipLaunchKernelGGL((quant_dynamic_wave_kernel<DT, FMT, 8, true, PRE>), wgrid, dim3(256), 0, st, p);
            else hipLaunchKernelGGL((quant_dynamic_wave_kernel<DT, FMT, 8, false, PRE>), wgrid, dim3(256), 0, st, p);
        } else {
            if (p.dual) hipLaunchKernelGGL((quant_dynamic_kernel<DT, FMT, true, PRE>), bgrid, dim3(256), 0, st, p);
            else hipLaunchKernelGGL((quant_dynamic_kernel<DT, FMT, false, PRE>), bgrid, dim3(256), 0, st, p);
        }
    } else {
        const int64_t runs = p.rows * (p.cols >> 4);
        hipLaunchKernelGGL((quant_static_kernel<DT, FMT, PRE>), dim3((unsigned)((runs + 255) / 256)), dim3(256), 0, st, p);
    }
    return check_launch("segq_quantize");
}

template <int DT>
static int launch_quant_fmt(const QuantParams& p, hipStream_t st) {
    switch (p.fmt) {
        case SEGQ_CODE_I8: return (p.pre_op || p.col_div) ? launch_quant<DT, SEGQ_CODE_I8, true>(p, st) : launch_quant<DT, SEGQ_CODE_I8, false>(p, st);
        case SEGQ_CODE_E4M3: return (p.pre_op || p.col_div) ? launch_quant<DT, SEGQ_CODE_E4M3, true>(p, st) : launch_quant<DT, SEGQ_CODE_E4M3, false>(p, st);
        case SEGQ_CODE_I4: return (p.pre_op || p.col_div) ? launch_quant<DT, SEGQ_CODE_I4, true>(p, st) : launch_quant<DT, SEGQ_CODE_I4, false>(p, st);
    }
    return fail(SEGQ_ERR_ARG, "segq_quantize: unknown code_fmt %d", p.fmt);
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Checks a descriptor and turns it into kernel parameters.  *empty: nothing to do (no rows or no columns).
static int quant_params(const segq_quant_desc* d, const float* scale_by_value, QuantParams& p, bool* empty) {
    *empty = false;
    if (!d) return fail(SEGQ_ERR_ARG, "segq_quantize: null descriptor");
    if (d->rows < 0 || d->cols < 0) return fail(SEGQ_ERR_ARG, "segq_quantize: negative size");
    if (d->rows == 0 || d->cols == 0) { *empty = true; return SEGQ_OK; }
    if (!d->x || !d->codes || (!d->scale && !scale_by_value))
        return fail(SEGQ_ERR_ARG, "segq_quantize: null x, codes or scale");
    if (scale_by_value && (d->dual || d->dynamic))
        return fail(SEGQ_ERR_ARG, "segq_quantize: a scale by value is static and single");
    if (d->cols % 16) return fail(SEGQ_ERR_ARG, "segq_quantize: cols (%lld) must be a multiple of 16", (long long)d->cols);
    if (d->x_dtype != SEGQ_F32 && d->x_dtype != SEGQ_F16 && d->x_dtype != SEGQ_BF16)
        return fail(SEGQ_ERR_ARG, "segq_quantize: x_dtype %d is not a float type", d->x_dtype);
    const int64_t esz = d->x_dtype == SEGQ_F32 ? 4 : 2;
    if (d->ldx < d->cols || (d->ldx * esz) % 16) return fail(SEGQ_ERR_ARG, "segq_quantize: ldx must be >= cols and 16-byte aligned");
    const int64_t min_ldc = d->code_fmt == SEGQ_CODE_I4 ? d->cols / 2 : d->cols;
    const int64_t ldc_align = d->code_fmt == SEGQ_CODE_I4 ? 8 : 16;
    if (d->ld_codes < min_ldc || d->ld_codes % ldc_align) return fail(SEGQ_ERR_ARG, "segq_quantize: bad ld_codes %lld", (long long)d->ld_codes);
    if (!aligned16(d->x) || (reinterpret_cast<uintptr_t>(d->codes) % ldc_align) ||
        (d->codes_neg && (reinterpret_cast<uintptr_t>(d->codes_neg) % ldc_align)))
        return fail(SEGQ_ERR_ARG, "segq_quantize: x and codes must be 16-byte aligned");
    if (d->dual && !d->scale_neg) return fail(SEGQ_ERR_ARG, "segq_quantize: dual needs scale_neg");
    if (d->n_kseg < 1 || d->n_kseg > SEGQ_MAX_KSEG) return fail(SEGQ_ERR_ARG, "segq_quantize: n_kseg %d out of range", d->n_kseg);
    if (d->rows * (d->cols / 16) > (int64_t)0x7fffffff * 256 || d->cols > 0x7fffffff || d->rows > 0x7fffffff)
        return fail(SEGQ_ERR_ARG, "segq_quantize: matrix too large");

    p = QuantParams{};
    p.x = d->x; p.codes = d->codes; p.codes_neg = d->codes_neg;
    p.scale = d->scale; p.scale_neg = d->scale_neg;
    p.rows = d->rows; p.cols = d->cols; p.ldx = d->ldx; p.ldc = d->ld_codes;
    p.seg_rows = d->seg_rows > 0 ? d->seg_rows : d->rows;
    p.seg_stride = d->seg_stride; p.row_stride = d->row_stride; p.kseg_stride = d->kseg_stride;
    p.x_dtype = d->x_dtype; p.fmt = d->code_fmt;
    p.n_kseg = d->n_kseg; p.dual = d->dual ? 1 : 0; p.dynamic = d->dynamic ? 1 : 0;
    p.dual_mask = d->dual_kseg_mask;
    p.scale_imm = scale_by_value ? *scale_by_value : 0.0f;
    if (d->pre_op < SEGQ_PRE_NONE || d->pre_op > SEGQ_PRE_SILU) return fail(SEGQ_ERR_ARG, "segq_quantize: unknown pre_op %d", d->pre_op);
    if (d->gate) {
        if (d->pre_op == SEGQ_PRE_NONE) return fail(SEGQ_ERR_ARG, "segq_quantize: a gate needs a pre_op");
        if (d->ld_gate < d->cols || (d->ld_gate * esz) % 16 || !aligned16(d->gate))
            return fail(SEGQ_ERR_ARG, "segq_quantize: gate must be 16-byte aligned with ld_gate >= cols");
    }
    p.pre_op = d->pre_op; p.gate = d->gate; p.ldg = d->ld_gate;
    if (d->col_div && !aligned16(d->col_div)) return fail(SEGQ_ERR_ARG, "segq_quantize: col_div must be 16-byte aligned");
    p.col_div = d->col_div;
    if (d->n_kseg == 1) {
        p.kb[0] = 0; p.kb[1] = (int32_t)d->cols;
    } else {
        if (d->kseg_bounds[0] != 0 || d->kseg_bounds[d->n_kseg] != d->cols)
            return fail(SEGQ_ERR_ARG, "segq_quantize: kseg_bounds must span [0, cols]");
        for (int i = 0; i <= d->n_kseg; ++i) {
            if (d->kseg_bounds[i] % 16 || (i && d->kseg_bounds[i] <= d->kseg_bounds[i - 1]))
                return fail(SEGQ_ERR_ARG, "segq_quantize: kseg_bounds must be increasing multiples of 16");
            p.kb[i] = (int32_t)d->kseg_bounds[i];
        }
    }
    if (p.dynamic && p.row_stride != 1 && p.rows != 1 && p.seg_rows != 1)
        return fail(SEGQ_ERR_ARG, "segq_quantize: dynamic scales are per row (row_stride must be 1)");
    return SEGQ_OK;
}

static int launch_params(const QuantParams& p, hipStream_t st) {
    switch (p.x_dtype) {
        case SEGQ_F32: return launch_quant_fmt<SEGQ_F32>(p, st);
        case SEGQ_F16: return launch_quant_fmt<SEGQ_F16>(p, st);
        default: return launch_quant_fmt<SEGQ_BF16>(p, st);
    }
}

int quantize_impl(const segq_quant_desc* d, hipStream_t st, const float* scale_by_value) {
    QuantParams p;
    bool empty;
    if (const int rc = quant_params(d, scale_by_value, p, &empty)) return rc;
    return empty ? SEGQ_OK : launch_params(p, st);
}

// Several tensors in one launch.  Two or more descriptors that the one-wave-per-row kernel serves
// in the same instance (dynamic scales, one column segment, no fused producer, 16-bit input, int8
// or e4m3 codes, rows of the same length class, the same DualScale setting) share a grid: a launch
// of a few tens of MB is a third ramp and tail, which they then pay once (two 4608 x 3072 bf16
// tensors: 2 x 10.8 us apart, ~16.5 us together).  Anything else is launched one by one.
template <int DT, int FMT, int CPL>
static int launch_row_batch(const QuantBatch& b, bool dual, hipStream_t st) {
    const dim3 grid((unsigned)b.first[b.n]), one_wave(64);
    if (dual) hipLaunchKernelGGL((quant_dynamic_row_many_kernel<DT, FMT, CPL, true>), grid, one_wave, 0, st, b);
    else hipLaunchKernelGGL((quant_dynamic_row_many_kernel<DT, FMT, CPL, false>), grid, one_wave, 0, st, b);
    return check_launch("segq_quantize_many");
}

template <int DT, int FMT>
static int launch_row_batch_cpl(const QuantBatch& b, int cpl, bool dual, hipStream_t st) {
    switch (cpl) {
        case 1: return launch_row_batch<DT, FMT, 1>(b, dual, st);
        case 2: return launch_row_batch<DT, FMT, 2>(b, dual, st);
        case 3: return launch_row_batch<DT, FMT, 3>(b, dual, st);
        case 4: return launch_row_batch<DT, FMT, 4>(b, dual, st);
        case 6: return launch_row_batch<DT, FMT, 6>(b, dual, st);
        default: return launch_row_batch<DT, FMT, 8>(b, dual, st);
    }
}

static int row_cpl(const QuantParams& p) {  // runs of 16 per lane in the row kernel; 0: not its case
    const int64_t runs = p.cols / 16;
    if (!p.dynamic || p.n_kseg != 1 || p.pre_op || p.col_div || p.group || runs > 64 * 8) return 0;
    if (p.x_dtype == SEGQ_F32 || (p.fmt != SEGQ_CODE_I8 && p.fmt != SEGQ_CODE_E4M3)) return 0;
    if (p.dual && !(p.dual_mask & 1u)) return 0;
    return runs <= 64 ? 1 : runs <= 128 ? 2 : runs <= 192 ? 3 : runs <= 256 ? 4 : runs <= 384 ? 6 : 8;
}

int quantize_many_impl(const segq_quant_desc* descs, int32_t n, hipStream_t st) {
    if (n < 0 || (n > 0 && !descs)) return fail(SEGQ_ERR_ARG, "segq_quantize_many: bad descriptor array");
    int i = 0;
    while (i < n) {
        QuantBatch b{};
        bool empty;
        if (const int rc = quant_params(&descs[i], nullptr, b.p[0], &empty)) return rc;
        if (empty) { ++i; continue; }
        const int cpl = row_cpl(b.p[0]);
        b.n = 1;
        b.first[0] = 0; b.first[1] = (int32_t)b.p[0].rows;
        int j = i + 1;
        while (cpl && j < n && b.n < SEGQ_QUANT_BATCH) {  // gather the descriptors that follow and fit the same instance
            QuantParams q;
            if (const int rc = quant_params(&descs[j], nullptr, q, &empty)) return rc;
            if (empty || row_cpl(q) != cpl || q.x_dtype != b.p[0].x_dtype || q.fmt != b.p[0].fmt || q.dual != b.p[0].dual ||
                (int64_t)b.first[b.n] + q.rows > 0x7fffffff)
                break;
            b.p[b.n] = q;
            b.first[b.n + 1] = b.first[b.n] + (int32_t)q.rows;
            ++b.n; ++j;
        }
        int rc;
        if (b.n == 1) {
            rc = launch_params(b.p[0], st);
        } else {
            const bool dual = b.p[0].dual != 0, f8 = b.p[0].fmt == SEGQ_CODE_E4M3;
            if (b.p[0].x_dtype == SEGQ_BF16)
                rc = f8 ? launch_row_batch_cpl<SEGQ_BF16, SEGQ_CODE_E4M3>(b, cpl, dual, st) : launch_row_batch_cpl<SEGQ_BF16, SEGQ_CODE_I8>(b, cpl, dual, st);
            else
                rc = f8 ? launch_row_batch_cpl<SEGQ_F16, SEGQ_CODE_E4M3>(b, cpl, dual, st) : launch_row_batch_cpl<SEGQ_F16, SEGQ_CODE_I8>(b, cpl, dual, st);
        }
        if (rc) return rc;
        i = j;
    }
    return SEGQ_OK;
}

// Weight codes with one scale per (row, group of `group` contraction columns): the static kernel
// with its column segments given by a stride instead of a bounds table.
int quantize_groups_impl(const void* w, int32_t w_dtype, int64_t n, int64_t k, void* codes, int32_t fmt, const float* scales,
                         int64_t group, hipStream_t st) {
    if (n < 0 || k < 0) return fail(SEGQ_ERR_ARG, "segq_quantize_weights_groups: negative size");
    if (n == 0 || k == 0) return SEGQ_OK;
    if (!w || !codes || !scales) return fail(SEGQ_ERR_ARG, "segq_quantize_weights_groups: null weights, codes or scales");
    if (group <= 0 || group % 16 || k % group || group > 0x7fffffff)
        return fail(SEGQ_ERR_ARG, "segq_quantize_weights_groups: the group size (%lld) must be a multiple of 16 that divides k (%lld)",
                    (long long)group, (long long)k);
    if (w_dtype != SEGQ_F32 && w_dtype != SEGQ_F16 && w_dtype != SEGQ_BF16)
        return fail(SEGQ_ERR_ARG, "segq_quantize_weights_groups: w_dtype %d is not a float type", w_dtype);
    if (fmt != SEGQ_CODE_I8 && fmt != SEGQ_CODE_E4M3 && fmt != SEGQ_CODE_I4)
        return fail(SEGQ_ERR_ARG, "segq_quantize_weights_groups: unknown code_fmt %d", fmt);
    const int64_t esz = w_dtype == SEGQ_F32 ? 4 : 2;
    if ((k * esz) % 16 || !aligned16(w) || (reinterpret_cast<uintptr_t>(codes) % (fmt == SEGQ_CODE_I4 ? 8 : 16)))
        return fail(SEGQ_ERR_ARG, "segq_quantize_weights_groups: weights and codes must be 16-byte aligned");
    if (n * (k / 16) > (int64_t)0x7fffffff * 256 || k > 0x7fffffff || n > 0x7fffffff)
        return fail(SEGQ_ERR_ARG, "segq_quantize_weights_groups: matrix too large");
    QuantParams p{};
    p.x = w; p.codes = codes; p.scale = const_cast<float*>(scales);
    p.rows = n; p.cols = k; p.ldx = k; p.ldc = fmt == SEGQ_CODE_I4 ? k / 2 : k;
    p.seg_rows = n; p.row_stride = 1; p.kseg_stride = n;
    p.x_dtype = w_dtype; p.fmt = fmt; p.n_kseg = 1; p.group = (int32_t)group;
    p.kb[0] = 0; p.kb[1] = (int32_t)k;
    switch (w_dtype) {
        case SEGQ_F32: return launch_quant_fmt<SEGQ_F32>(p, st);
        case SEGQ_F16: return launch_quant_fmt<SEGQ_F16>(p, st);
        default: return launch_quant_fmt<SEGQ_BF16>(p, st);
    }
}

// int4 codes packed down the columns (two output rows per byte, the layout the reference's GPTQ
// loop produces) -> packed along the rows (two input channels per byte, the layout the GEMM reads).
// A workgroup transposes a patch of 64 input channels x 128 output rows through LDS so that both
// its reads (along the rows of the source) and its writes (along the rows of the result) are
// contiguous.
__global__ void __launch_bounds__(256) repack_i4_kernel(const uint8_t* src, uint8_t* dst, int64_t out, int64_t cols) {
    __shared__ uint8_t tile[64][65];
    const int64_t half_out = out >> 1, half_cols = cols >> 1;
    const int64_t c0 = (int64_t)blockIdx.x * 64, j0 = (int64_t)blockIdx.y * 64;
    for (int idx = threadIdx.x; idx < 64 * 64; idx += 256) {
        const int c = idx >> 6, j = idx & 63;
        uint8_t v = 0;
        if (c0 + c < cols && j0 + j < half_out) v = src[(c0 + c) * half_out + j0 + j];
        tile[c][j] = v;
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < 128 * 32; idx += 256) {
        const int r = idx >> 5, m = idx & 31;  // output row 2 j0 + r, output byte c0 / 2 + m
        const int sh = (r & 1) * 4;
        const uint8_t lo = (tile[2 * m][r >> 1] >> sh) & 0xF, hi = (tile[2 * m + 1][r >> 1] >> sh) & 0xF;
        const int64_t row = 2 * j0 + r, byte = (c0 >> 1) + m;
        if (row < out && byte < half_cols) dst[row * half_cols + byte] = (uint8_t)(lo | (hi << 4));
    }
}

int repack_i4_impl(const void* colpacked, void* rowpacked, int64_t out, int64_t cols, hipStream_t st) {
    if (out < 0 || cols < 0) return fail(SEGQ_ERR_ARG, "segq_repack_int4: negative size");
    // the reference asserts both even (segquant/calibrator/calibrator.py:204)
    if ((out | cols) & 1) return fail(SEGQ_ERR_ARG, "segq_repack_int4: out (%lld) and cols (%lld) must be even", (long long)out, (long long)cols);
    if (out == 0 || cols == 0) return SEGQ_OK;
    if (!colpacked || !rowpacked || colpacked == rowpacked) return fail(SEGQ_ERR_ARG, "segq_repack_int4: null or aliased buffers");
    const int64_t gx = (cols + 63) / 64, gy = (out / 2 + 63) / 64;
    if (gx > 0x7fffffff || gy > 65535) return fail(SEGQ_ERR_ARG, "segq_repack_int4: matrix too large");
    hipLaunchKernelGGL(repack_i4_kernel, dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, st, static_cast<const uint8_t*>(colpacked),
                       static_cast<uint8_t*>(rowpacked), out, cols);
    return check_launch("segq_repack_int4");
}

int fake_e4m3_impl(const void* x, void* out, int32_t dtype, int64_t numel, hipStream_t st) {
    if (numel < 0) return fail(SEGQ_ERR_ARG, "segq_fake_e4m3: negative numel");
    if (numel == 0) return SEGQ_OK;
    if (!x || !out) return fail(SEGQ_ERR_ARG, "segq_fake_e4m3: null pointer");
    const dim3 grid((unsigned)((numel + 255) / 256)), block(256);
    switch (dtype) {
        case SEGQ_F32: hipLaunchKernelGGL(fake_e4m3_kernel<SEGQ_F32>, grid, block, 0, st, x, out, numel); break;
        case SEGQ_F16: hipLaunchKernelGGL(fake_e4m3_kernel<SEGQ_F16>, grid, block, 0, st, x, out, numel); break;
        case SEGQ_BF16: hipLaunchKernelGGL(fake_e4m3_kernel<SEGQ_BF16>, grid, block, 0, st, x, out, numel); break;
        default: return fail(SEGQ_ERR_ARG, "segq_fake_e4m3: dtype %d is not a float type", dtype);
    }
    return check_launch("segq_fake_e4m3");
}

}  // namespace segq
