/*
 * libsegq -- C ABI of the MI355X (gfx950) real-quantized segmented linear.
 *
 * Plain pointers and sizes only; no torch types.  Every pointer named "device"
 * is HIP device memory on the current device.  No entry point allocates,
 * frees, synchronises or throws: each enqueues its kernels on the stream it is
 * given and returns 0, or returns a non-zero segq_status and leaves a message
 * for segq_last_error().
 *
 * Scale convention (the reference's): a scale is multiplicative,
 * code = round(x * scale); de-quantisation divides by scale_x * scale_w
 * (segquant/src/real_quant/quantizer.cuh:65, dequantizer.cuh:48).
 */
#ifndef SEGQ_H
#define SEGQ_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* segq_stream_t; /* a hipStream_t; NULL is the default stream */

enum segq_status {
    SEGQ_OK = 0,
    SEGQ_ERR_ARG = 1,         /* bad pointer, size, alignment or enum */
    SEGQ_ERR_UNSUPPORTED = 2, /* a combination this build has no kernel for */
    SEGQ_ERR_LAUNCH = 3       /* the HIP runtime refused the launch */
};

/* float element types of inputs, outputs and bias.  Mirrors the dtypes the
 * reference dispatches over (segquant/src/real_quant/real_gemm.cu:22-28). */
enum segq_dtype {
    SEGQ_F32 = 0,
    SEGQ_F16 = 1,
    SEGQ_BF16 = 2,
    SEGQ_ACC = 3 /* GEMM output only: the raw accumulator, int32 (integer codes) or fp32 (e4m3) */
};

/* storage formats of codes.  Mirrors StoreType<> (segquant/src/real_quant/seg_utils.h:25-45):
 * int8 travels as int8, e4m3 as one byte, int4 as two values per byte with the
 * even element in the low nibble (segquant/src/real_quant/quantizer.cuh:37-50). */
enum segq_code {
    SEGQ_CODE_I8 = 0,
    SEGQ_CODE_E4M3 = 1,
    SEGQ_CODE_I4 = 2
};

#define SEGQ_MAX_KSEG 8
#define SEGQ_MAX_RANGES 64

int segq_version(void);

/* Message of the last failing call on this thread ("" if none). */
const char* segq_last_error(void);

/* ------------------------------------------------------------------------
 * Quantise a row-major float matrix to codes.
 *
 * Replaces the reference's quantise kernels and their launches:
 *   activations  real_quantize_scaled_kernel / real_quantize_dual_scaled_kernel,
 *                segment form (segquant/src/real_quant/quantizer.cuh:148-206),
 *                launched from real_gemm.cu:701-705 and :818-826;
 *   weights      the scalar and per-row forms (quantizer.cuh:55-68, :103-118)
 *                behind real_quantized_quantize_weights (real_gemm.cu:538-638).
 *
 * The scale of element (row, col) is
 *     scale[(row / seg_rows) * seg_stride + (row % seg_rows) * row_stride
 *           + kseg(col) * kseg_stride]
 * where kseg(col) is the index of the column segment that holds col.  With the
 * reference's (S, ..., M, K) activations flattened to rows = S*M, seg_rows = M:
 * a per-segment scale tensor is {seg_stride 1, row_stride 0}, a per-token one
 * is {seg_stride M, row_stride 1} (quantizer.cuh:148-157).
 *
 * dual != 0 selects DualScale (quantizer.cuh:178-206): x >= 0 uses scale[],
 * anything else uses scale_neg[] at the same index.  Bit i of dual_kseg_mask
 * says whether column segment i is dual; other segments use scale[] for both
 * signs.  With codes_neg == NULL one merged code tensor is written (the code of
 * the branch that was taken); with codes_neg != NULL the reference's two
 * tensors are written, Xp to codes and Xn to codes_neg (column segments that are
 * not dual write their one code to codes and leave codes_neg untouched).
 *
 * dynamic != 0: scale[] (and scale_neg[]) are OUTPUTS.  The kernel takes the
 * absolute maximum of every (row, column segment), writes
 * qmax / max(amax, 2^-24) there (segquant/quantizers/quantizer.py:211-219;
 * dual: :183-203; e4m3: 448) and quantises with it.  A NaN in the segment makes a
 * single scale NaN, as torch's amax does (and every code of the segment the NaN
 * code); the two DualScale maxima are taken over x > 0 and x < 0, where a NaN is on
 * neither side; an infinite maximum gives scale 0.  Needs row_stride == 1 or a
 * single row per scale; has no counterpart kernel in the reference, whose
 * dynamic mode calls a method that does not exist (optimum/optimizer.py:96-100).
 *
 * pre_op != SEGQ_PRE_NONE fuses the activation function of the layer in front:
 * what is quantised (and, when dynamic, what the maximum is taken of) is op(x),
 * or x * op(gate) when gate is given, each operator's result rounded to x_dtype
 * as that layer would have stored it.  These are the reference's GELU(tanh) MLP
 * (backend/torch/modules/transformer_flux.py:91), GELU / SiLU
 * (backend/torch/layers/activations.py:52-57) and the gated GEGLU / SwiGLU
 * (activations.py:77-80, :110-121), which there run as separate torch operators
 * writing a full-size tensor that the quantise kernel then reads back.
 * ---------------------------------------------------------------------- */
typedef enum segq_pre_op {
    SEGQ_PRE_NONE = 0,
    SEGQ_PRE_GELU_TANH = 1, /* 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))) */
    SEGQ_PRE_GELU = 2,      /* 0.5 x (1 + erf(x / sqrt(2))) */
    SEGQ_PRE_SILU = 3       /* x / (1 + exp(-x)) */
} segq_pre_op;

typedef struct segq_quant_desc {
    const void* x;      /* device, rows x cols, x_dtype, row stride ldx elements */
    int32_t x_dtype;    /* segq_dtype: F32 | F16 | BF16 */
    int32_t code_fmt;   /* segq_code */
    int64_t rows;
    int64_t cols;       /* multiple of 16 */
    int64_t ldx;        /* elements; multiple of 8 */
    void* codes;        /* device, rows x cols bytes (I8, E4M3) or rows x cols/2 bytes (I4) */
    void* codes_neg;    /* device or NULL, see above */
    int64_t ld_codes;   /* bytes; multiple of 16 (8 for I4) */
    float* scale;       /* device; input, or output when dynamic */
    float* scale_neg;   /* device or NULL (required when dual) */
    int64_t seg_rows;   /* rows per row segment; 0 means rows */
    int64_t seg_stride;
    int64_t row_stride;
    int64_t kseg_stride;
    int32_t n_kseg;     /* 1 .. SEGQ_MAX_KSEG */
    int32_t dual;
    uint32_t dual_kseg_mask;
    int32_t dynamic;
    int64_t kseg_bounds[SEGQ_MAX_KSEG + 1]; /* column segment i = [bounds[i], bounds[i+1]); multiples of 16 */
    int32_t pre_op;     /* segq_pre_op */
    const void* gate;   /* device or NULL: rows x cols of x_dtype, row stride ld_gate; needs a pre_op */
    int64_t ld_gate;
    const float* col_div; /* device or NULL: cols divisors, 16-byte aligned.  Every element (after the pre_op, if
                         * any) is divided by the divisor of its column and the quotient rounded to x_dtype: the
                         * SmoothQuant step x / s that the reference applies to a clone of the activation right
                         * before it quantises it (segquant/optimum/optimizer.py:467-470, :517).  Pass s as the
                         * reference uses it, i.e. already rounded to x_dtype. */
} segq_quant_desc;

int segq_quantize(const segq_quant_desc* d, segq_stream_t stream);

/* n descriptors in order, with the results of n segq_quantize calls.  Neighbouring descriptors
 * that one kernel instance serves (dynamic per-row scales, one column segment, no pre_op or
 * col_div, 16-bit input, int8 or e4m3 codes, rows of up to 8192 elements in the same length class,
 * the same `dual`) share one launch, up to four at a time: launches of a few tens of MB are a third
 * ramp and tail.  For inputs that exist at the same time (the image and text streams of a
 * double-stream block, whose projections the reference quantises one tensor at a time,
 * segquant/src/real_quant/real_gemm.cu:700-716).  The outputs must not overlap. */
int segq_quantize_many(const segq_quant_desc* descs, int32_t n, segq_stream_t stream);

/* The reference's two weight entry points under their own names
 * (segquant/src/real_quant/seg_utils.h:82-119): one scale by value, or one per
 * output row.  weights is (n, k) row-major contiguous; codes is (n, k) bytes,
 * or n*k/2 bytes for int4. */
int segq_quantize_weights_scalar(const void* weights, int32_t w_dtype, int64_t n, int64_t k,
                                 void* codes, int32_t code_fmt, float scale_w, segq_stream_t stream);
int segq_quantize_weights_rows(const void* weights, int32_t w_dtype, int64_t n, int64_t k,
                               void* codes, int32_t code_fmt, const float* scale_w_rows,
                               segq_stream_t stream);

/* Weight codes with one scale per (output row, group of `group` input channels):
 *     codes[r][c] = store(weights[r][c] * scales[(c / group) * n + r])
 * scales is a contiguous (k / group, n) matrix of multiplicative scales, the layout whose
 * reciprocals segq_gemm takes as group_dequant.  group: a multiple of 16 that divides k (32 for
 * int4 codes that the GEMM is to read).  One launch for any number of groups.  The reference has
 * per-tensor and per-row weight scales only (segquant/src/real_quant/real_gemm.cu:538-638); its
 * GPTQ calibrator quantises group by group on the host (segquant/calibrator/calibrator.py:262-330). */
int segq_quantize_weights_groups(const void* weights, int32_t w_dtype, int64_t n, int64_t k, void* codes,
                                 int32_t code_fmt, const float* scales, int64_t group, segq_stream_t stream);

/* int4 weight codes packed down the columns -> packed along the rows.
 * colpacked: cols * out / 2 bytes, viewed as (cols, out / 2): byte j of input channel c holds
 * output rows 2j (low nibble) and 2j + 1 (high nibble) -- what the reference's GPTQ loop emits.
 * rowpacked: out * cols / 2 bytes, (out, cols / 2): byte m of row r holds input channels 2m (low
 * nibble) and 2m + 1 (high nibble) -- the layout every int4 consumer reads
 * (segquant/src/real_quant/quantizer.cuh:37-50).  Replaces
 * GPTQCalibrator.colpacked1d_to_rowpacked1d (segquant/calibrator/calibrator.py:202-223), which
 * does it with seven torch operators on full-size temporaries.  out and cols even; the buffers
 * must not alias. */
int segq_repack_int4_cols_to_rows(const void* colpacked, void* rowpacked, int64_t out, int64_t cols,
                                  segq_stream_t stream);

/* ------------------------------------------------------------------------
 * Segmented GEMM with fused de-quantisation and bias.
 *
 * Replaces, in one launch, the reference's GEMM launches and the de-quantise
 * pass that follows them: launch_gemm_scaled / launch_batched_gemm_scaled /
 * launch_array_gemm_scaled (segquant/src/real_quant/real_gemm.cu:424-532) and
 * real_dequantize_scaled_kernel / real_dequantize_dual_scaled_kernel
 * (segquant/src/real_quant/dequantizer.cuh:35-74), plus the recombination and
 * bias add of SegmentLinear.forward (segquant/layers/SegmentLinear.py:233-241).
 *
 *   out[z][m][n] = sum over ranges r of
 *                    ( sum_{k in r} A_r[z][m][k] * B[z][n][k] ) / (sx_r[z][m] * sw_r[z][n])
 *                  + bias[n]
 *
 * A "range" is a run of contraction columns that shares one pair of scales:
 * an input-channel segment, or one sign half of a DualScale segment.  Output-
 * column segments need no range: they are a per-column sw vector.  A_r is
 * chosen by a_sel:
 *   0  the code tensor a
 *   1  the second code tensor a_neg (the reference's Xn)
 *   2  the non-negative codes of a, negatives read as zero  (merged DualScale)
 *   3  the negative codes of a, the rest read as zero       (merged DualScale)
 * Accumulation is int32 for integer codes and fp32 for e4m3; the partial sums
 * of different ranges are combined in fp32 and rounded once to out_dtype.
 * ---------------------------------------------------------------------- */
typedef struct segq_krange {
    int64_t k_begin;        /* first contraction column; multiple of 16 (32 with int4 weights) */
    int64_t k_len;          /* multiple of 16 (32 with int4 weights) */
    int32_t a_sel;
    int32_t sx_row_stride;  /* 0: sx[0] for every row; 1: sx[m] */
    int32_t sw_col_stride;  /* 0: sw[0] for every column; 1: sw[n] */
    int32_t reserved;
    const float* sx;        /* device */
    const float* sw;        /* device */
} segq_krange;

typedef struct segq_gemm_desc {
    int32_t a_fmt;      /* SEGQ_CODE_I8 | SEGQ_CODE_E4M3 */
    int32_t b_fmt;      /* same as a_fmt, or SEGQ_CODE_I4 with a_fmt == SEGQ_CODE_I8 */
    int32_t out_dtype;  /* segq_dtype; SEGQ_ACC needs n_ranges == 1 and ignores scales and bias */
    int32_t bias_dtype; /* F32 | F16 | BF16 */
    int64_t m, n;
    const void* a;      /* device, m x K codes, row stride lda bytes (multiple of 16) */
    const void* a_neg;  /* device or NULL */
    int64_t lda;
    const void* b;      /* device, n x K codes, row stride ldb bytes (multiple of 16); int4: K/2 bytes per row */
    int64_t ldb;
    void* out;          /* device, m x n, row stride ldo elements */
    int64_t ldo;
    const void* bias;   /* device, n entries, or NULL */
    int64_t batch;      /* >= 1 independent problems (the reference's leading S dimension) */
    int64_t batch_stride_a;   /* bytes */
    int64_t batch_stride_b;   /* bytes */
    int64_t batch_stride_out; /* elements */
    int64_t batch_stride_sx;  /* floats, applied to every range's sx */
    int64_t batch_stride_sw;  /* floats, applied to every range's sw */
    int32_t n_ranges;   /* 1 .. SEGQ_MAX_RANGES */
    int32_t tile;       /* 0 = choose; otherwise a tile configuration id, see segq_gemm_tile_count */
    void* workspace;    /* device or NULL.  With int4 weights and at least batch * n * Kp bytes here (Kp = the
                         * largest range end rounded up to 16), b is first expanded to int8 in the workspace by
                         * a small kernel and the int8 GEMM kernels run on that (same accumulators, bit for bit;
                         * worth it when m is large and the GEMM is bound by the matrix cores, not by reading b).
                         * NULL or too small: int4 weights are unpacked on their way into LDS inside the GEMM.
                         * With int8 codes on both sides, several ranges, batch == 1 and tiles * tile_rows *
                         * tile_cols * 4 bytes here (4 (m + 288) (n + 288) always suffices), the sums of finished
                         * ranges are parked in the workspace as fp32 instead of in a second register set, which
                         * keeps the largest tiles available (same result up to fp32 rounding order).
                         * Contents are undefined afterwards.  Replaces nothing in the reference, whose CUTLASS
                         * kernel converts int4 in registers (segquant/src/real_quant/real_gemm.cu:208-305). */
    int64_t workspace_bytes;
    const float* group_dequant; /* device or NULL.  Group-wise weight scales: entry [g * group_dequant_stride + n]
                         * is the de-quantisation factor 1 / scale of output column n for contraction columns
                         * [128 g, 128 g + 128).  When set, the sum of every group is multiplied by its factor
                         * before it joins the sum of its range (the range's sx and sw still divide the whole):
                         *   out[m][n] = sum_r ( sum_{g in r} f[g][n] * sum_{k in g} A_r[m][k] B[n][k] )
                         *                    / (sx_r[m] * sw_r[n]) + bias[n]
                         * Needs int8 activations, int8 weights or int4 weights with a workspace (above),
                         * a_sel 0 or 1, every range a whole number of groups, batch == 1, a float out_dtype.
                         * The reference has per-tensor and per-row weight scales only
                         * (segquant/src/real_quant/real_gemm.cu:538-638); groups exist here alone. */
    int64_t group_dequant_stride; /* floats between consecutive groups, >= n */
    const void* addend; /* device or NULL: (m, n) values of out_dtype, row stride ld_addend, batch stride
                         * batch_stride_out, added to the result before its one rounding (a residual, or the
                         * low-rank branch x L1 L2 that the reference's SVD optimiser adds to the quantised
                         * product as a separate operator, segquant/optimum/optimizer.py:731-740) */
    int64_t ld_addend;
    int64_t split_k;    /* 0: the library decides; 1: never; s > 1: the K steps of every tile are shared by s
                         * workgroups.  Splitting needs plain int8 or e4m3 codes, K ranges in multiples of 128,
                         * batch == 1 and a workspace (segq_gemm_workspace_bytes says how much: the fp32 shares,
                         * plus the parking room above per share for int8 with several ranges).  Two shares
                         * meet inside the launch: the second workgroup to arrive at a tile adds the other's
                         * share to its own, adds the bias and rounds (a + b = b + a: the same bits whoever is
                         * last).  More shares are summed in their order by a second small kernel.  For shapes
                         * whose whole tiles would leave compute units idle; no counterpart in the reference
                         * (its GemmUniversal runs one K slice per problem: mode kGemm with batch_count 1,
                         * segquant/src/real_quant/real_gemm.cu:281-285 and :424-445). */
    const void* lowrank_t;  /* device or NULL.  A low-rank branch added to the result before its one rounding:
                         *   out[m][n] += sum_{k < lowrank_rank} lowrank_t[m][k] * lowrank_l2t[n][k]
                         * computed on the matrix cores inside the epilogue (16-bit operands, fp32 sums), so the
                         * (m, n) product is never written to memory.  This is the inference-time branch of the
                         * reference's SVD optimiser, x L1 L2 with T = x L1 of shape (m, rank) and L2 of shape
                         * (rank, n), which there are two bmm launches and an addition of full-size tensors
                         * (segquant/optimum/optimizer.py:698-731).  Both matrices are in out_dtype, which must
                         * be F16 or BF16; rows 16-byte aligned.  Needs plain 8-bit codes on both sides, K ranges
                         * in multiples of 128, batch == 1; not combined with split_k.  Otherwise
                         * SEGQ_ERR_UNSUPPORTED: pass the product as addend instead. */
    int64_t ld_lowrank_t;   /* elements; multiple of 8, >= lowrank_rank */
    const void* lowrank_l2t; /* device: (n, lowrank_rank), i.e. L2 transposed, the contraction index contiguous */
    int64_t ld_lowrank_l2t;
    int32_t lowrank_rank;   /* multiple of 32, at most 512; 0 with lowrank_t == NULL */
    int32_t out_pre_op;     /* segq_pre_op applied to the result before it is encoded (out_codes only) */
    void* out_codes;        /* device or NULL.  When set, the launch writes CODES instead of floats: the (m, n)
                         * code tensor that segq_quantize would make of this GEMM's output for the linear that
                         * follows, so that neither the float output is written nor a quantise launch reads it
                         * back.  Every result is rounded to out_dtype (the dtype the output tensor would have
                         * had), out_pre_op is applied and rounded to out_dtype again, the value is multiplied by
                         * out_scale[0] and encoded as out_code_fmt: bit for bit the codes of segq_gemm followed
                         * by segq_quantize with pre_op and a static per-tensor scale.  With out_scale_neg set
                         * (DualScale) out_codes_neg is required: values >= 0 go to out_codes scaled by
                         * out_scale[0], the others to out_codes_neg scaled by out_scale_neg[0], the tensor not
                         * taken holding code(0) (segquant/src/real_quant/quantizer.cuh:178-206).  out is
                         * ignored (may be NULL).  Needs plain int8 or e4m3 codes on both sides, one range with K
                         * a multiple of 128, batch == 1, out_dtype F16 or BF16; no split_k, group factors or
                         * low-rank branch (SEGQ_ERR_UNSUPPORTED otherwise).
                         * These are the reference's chained linears, which there pass a full-size tensor
                         * through an activation kernel and a quantise kernel between the two GEMMs
                         * (backend/torch/layers/activations.py:52-57 feeding real_gemm.cu:700-705). */
    void* out_codes_neg;
    int64_t ld_out_codes;   /* bytes; >= n */
    const float* out_scale; /* device: one float */
    const float* out_scale_neg; /* device or NULL */
    int32_t out_code_fmt;   /* SEGQ_CODE_I8 | SEGQ_CODE_E4M3 */
    int32_t reserved2;
    segq_krange ranges[SEGQ_MAX_RANGES];
} segq_gemm_desc;

int segq_gemm(const segq_gemm_desc* d, segq_stream_t stream);

/* Number of tile configurations accepted in segq_gemm_desc.tile (ids 1..count). */
int segq_gemm_tile_count(void);

/* *bytes = the workspace the launch described by d would use if the caller lent as much as the
 * library can make use of (0: it has no use for one).  d is the descriptor of the launch itself;
 * its own workspace fields are ignored, nothing is enqueued.  Callers size the buffer they lend
 * with this instead of restating the library's rules.  Replaces nothing in the reference, which
 * allocates its temporaries itself (segquant/src/real_quant/real_gemm.cu:684-698, :855-865). */
int segq_gemm_workspace_bytes(const segq_gemm_desc* d, int64_t* bytes);

/* What segq_gemm(d) would launch, without launching it: the tile id the library picks (as in
 * segq_gemm_desc.tile), the number of workgroups that share the K steps of a tile (1: no split)
 * and whether finished ranges are parked in d's workspace.  Any of the three pointers may be
 * NULL.  For tools that report which kernel a measurement belongs to; no counterpart in the
 * reference. */
int segq_gemm_plan(const segq_gemm_desc* d, int32_t* tile, int32_t* splits, int32_t* parked);

/* ------------------------------------------------------------------------
 * segq_gemm for callers that cannot allocate device memory.
 *
 * No counterpart in the reference (whose operators allocate every temporary through ATen,
 * segquant/src/real_quant/real_gemm.cu:684-698).  It is for callers that cannot call hipMalloc or an
 * allocating framework routine around the launch: code under HIP graph capture, tight serving
 * loops, harnesses that forbid allocation.  Same descriptor, same kernels and same result as
 * segq_gemm called with a workspace of segq_gemm_workspace_bytes(d) bytes, but the workspace
 * (expanded int4 weights, parked sums of int8 ranges, split-K partial results) is an array of
 * SEGQ_NOALLOC_SCRATCH_BYTES that the library itself holds on every GPU it runs on, from the
 * first use on that GPU until the process ends; d->workspace is ignored.  A launch that could
 * use more than that runs with what fits, exactly as segq_gemm does when it is lent a workspace
 * of SEGQ_NOALLOC_SCRATCH_BYTES (fewer K shares; int8 ranges summed in a second register set
 * on smaller tiles instead of parked: the same result up to the order of fp32 additions); only
 * a launch that cannot run with less (an explicit split_k, group factors with int4 weights
 * beyond the array) is refused, with its status and a message, and nothing is enqueued.  The call
 * allocates nothing and frees nothing; the array's address on the current device is resolved on
 * the first call there, or ahead of time by segq_init().
 *
 * All calls on one GPU share that GPU's array and its contents are undefined between calls
 * (nothing in it needs to start at zero: every kernel writes a slot before it reads it), so two
 * such calls must not overlap on one GPU: issue them on one stream, or order the streams.
 * ---------------------------------------------------------------------- */
#define SEGQ_NOALLOC_SCRATCH_BYTES (64ll << 20)
int segq_gemm_noalloc(const segq_gemm_desc* d, segq_stream_t stream);
int64_t segq_noalloc_scratch_bytes(void); /* SEGQ_NOALLOC_SCRATCH_BYTES of the loaded library */

/* Optional set-up for the current device, outside any stream capture: reads the device's
 * properties and resolves the scratch array's address there, which the entry points otherwise do
 * on their first call on that device.  No counterpart in the reference. */
int segq_init(void);

/* Compute units and highest engine clock (kHz) of the current device, as the HIP runtime reports
 * them: what the dense 8-bit MFMA peak follows from (compute units x 4 SIMDs x 2048 operations per
 * clock x clock).  For benchmarks that state the peak they measure against; no counterpart in the
 * reference.  Either pointer may be NULL. */
int segq_device_info(int32_t* compute_units, int32_t* max_engine_clock_khz);

/* Quantise-then-multiply in one call: q writes its codes into a caller-provided
 * workspace that g reads as its a (and a_neg).  Replaces the body of
 * real_quantized_gemm_scaled / real_quantized_gemm_dual_scaled
 * (segquant/src/real_quant/real_gemm.cu:643-894) without their temporaries,
 * host synchronisation or per-call device allocation. */
int segq_linear(const segq_quant_desc* q, const segq_gemm_desc* g, segq_stream_t stream);

/* out[i] = float(e4m3(x[i])) in the dtype of x.  Replaces fake_e4m3fy
 * (segquant/src/fake_quant/quantizer_fp8.cu:34-51). */
int segq_fake_e4m3(const void* x, void* out, int32_t dtype, int64_t numel, segq_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* SEGQ_H */
