// C ABI of libsegq: argument checks, kernel selection, launches.
#include "segq_gemm_kernel.h"
#include <string.h>
#include <atomic>

namespace segq {

static thread_local char g_err[512] = "";

int fail(int status, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return status;
}

int check_launch(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(SEGQ_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return SEGQ_OK;
}

int device_cus() {
    static std::atomic<int> cus[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = cus[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cus[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

int reserve_lds(const void* kern, int bytes, unsigned long long* done) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0) dev = 0;
    const unsigned long long bit = 1ull << (dev & 63);
    if (__atomic_load_n(done, __ATOMIC_ACQUIRE) & bit) return SEGQ_OK;
    // (the call is idempotent: two threads that both find the bit clear both make it)
    if (hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess)
        return fail(SEGQ_ERR_LAUNCH, "segq_gemm: cannot reserve %d bytes of LDS", bytes);
    __atomic_fetch_or(done, bit, __ATOMIC_RELEASE);
    return SEGQ_OK;
}

int quantize_impl(const segq_quant_desc* d, hipStream_t st, const float* scale_by_value);
int quantize_many_impl(const segq_quant_desc* descs, int32_t n, hipStream_t st);
int fake_e4m3_impl(const void* x, void* out, int32_t dtype, int64_t numel, hipStream_t st);
int quantize_groups_impl(const void* w, int32_t w_dtype, int64_t n, int64_t k, void* codes, int32_t fmt, const float* scales,
                         int64_t group, hipStream_t st);
int repack_i4_impl(const void* colpacked, void* rowpacked, int64_t out, int64_t cols, hipStream_t st);

static bool is_float_dtype(int t) { return t == SEGQ_F32 || t == SEGQ_F16 || t == SEGQ_BF16; }
static bool al(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// Tile choice when the caller leaves it to the library.  The 8-wave kernels need
// K in whole 128-byte steps and 32-bit row offsets.  A launch runs in rounds of
// one tile per CU, so its time goes as rounds x tile area x a per-tile weight
// (smaller tiles move more operand bytes per MAC: measured on M = 4608, 216
// tiles of 256 x 256 beat 432 tiles of 256 x 128 by 30 %).  The 192 x 288 and
// 288 x 192 tiles exist because 4608 rows of FLUX tokens make whole rounds with
// them where 256 x 256 leaves the last round half empty.
static int choose_tile(int64_t m, int64_t n, int64_t batch, bool fold, bool wide_ok, bool plain8, int64_t k_steps = 1 << 20,
                       bool big_ok = false) {  // fold: needs a second accumulator set; big_ok: 384 x 192 serves this launch
    auto tiles = [&](int cfg) {
        const TileCfg& c = TILE_CFGS[cfg];
        return ((m + c.bm - 1) / c.bm) * ((n + c.bn - 1) / c.bn) * batch;
    };
    // (plain 8-bit operands go to the 8-wave kernels from 32 tiles of 128 x 128 up: 64 x 9216 x 3072 runs
    // 24.9 us there against 35.2 us on the general kernel)
    if (wide_ok && tiles(FIRST_WIDE_CFG + 3) >= (plain8 && !fold ? 32 : 96)) {
        // Short contractions of middling size: the plain 128 x 128 kernel needs ~100 registers, so two
        // workgroups share a CU and each one's prologue and epilogue (most of a tile's time at a dozen
        // K steps) run under the other's MFMAs.  Measured at K = 1280 .. 1536: 2048 x 10240 34.5 vs 45.5 us
        // and 4096 x 6144 44.7 vs 47-50 us for the rule below's choice; 8192 x 10240 (1280 tiles of
        // 256 x 256, five whole rounds) stays 20 % better on the big tile.
        if (plain8 && !fold && k_steps <= 12 && tiles(FIRST_WIDE_CFG) <= 512 && tiles(FIRST_WIDE_CFG + 3) >= 512) {
            // ... unless 256 x 192 tiles make whole rounds of the CUs exactly (4096 x 6144 x 1536: 512 tiles,
            // 46.4 against 50.8 us in e4m3, 48.5 against 50.8 in int8)
            const int c = FIRST_WIDE_CFG + 6;
            if (m % TILE_CFGS[c].bm == 0 && n % TILE_CFGS[c].bn == 0 && tiles(c) % device_cus() == 0) return c;
            return FIRST_WIDE_CFG + 3;
        }
        static const double weight[6] = {1.0, 1.18, 1.18, 1.45, 1.04, 1.04};
        const int64_t cus = device_cus();
        int best = -1;
        double best_cost = 0;
        for (int i = 0; i < 6; ++i) {
            if (i == 0 && fold) continue;                  // no 256 x 256 with a second accumulator set
            if (i >= 4 && (fold || !plain8)) continue;  // plain int8 or e4m3 operands, one range only
            const int cfg = FIRST_WIDE_CFG + i;
            const int64_t rounds = (tiles(cfg) + cus - 1) / cus;
            const double cost = (double)rounds * TILE_CFGS[cfg].bm * TILE_CFGS[cfg].bn * weight[i];
            if (best < 0 || cost < best_cost) {
                best = cfg;
                best_cost = cost;
            }
        }
        // 384 x 192, eight wave tiles of 96 x 96 (the fewest LDS bytes per MFMA of all tiles): taken when
        // it tiles the output exactly, in whole rounds of the CUs, and with no more rounds x area than
        // the choice above.  4608 x 12288 x 3072: three rounds instead of four of 288 x 192, e4m3 165 ->
        // 140 us; 8192^3, which it does not tile exactly, is 12 % slower on it than on 256 x 256
        const int big = FIRST_WIDE_CFG + 9;
        if (big_ok && plain8 && !fold && batch == 1 && m % TILE_CFGS[big].bm == 0 && n % TILE_CFGS[big].bn == 0 && tiles(big) % cus == 0) {
            const TileCfg& t = TILE_CFGS[best];
            const int64_t rounds = (tiles(best) + cus - 1) / cus;
            if (tiles(big) / cus * TILE_CFGS[big].bm * TILE_CFGS[big].bn <= rounds * t.bm * t.bn) return big;
        }
        return best;
    }
    return tiles(2) >= 256 ? 2 : 3;
}

// int4 weight rows (two values per byte, even k in the low nibble) -> int8 rows.
// One thread expands 16 packed bytes to 32 values.
__global__ void __launch_bounds__(256) expand_i4_kernel(const uint8_t* src, int64_t ld_src, uint8_t* dst, int64_t ld_dst,
                                                        int64_t rows, int64_t chunks_per_row) {
    const int64_t total = rows * chunks_per_row;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t row = i / chunks_per_row, c = i - row * chunks_per_row;
        const uint4 v = *reinterpret_cast<const uint4*>(src + row * ld_src + c * 16);
        const uint32_t in[4] = {v.x, v.y, v.z, v.w};
        uint32_t out[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t e = in[j] & 0x0F0F0F0Fu, o = (in[j] >> 4) & 0x0F0F0F0Fu;
            e |= (e & 0x08080808u) * 0x1Eu;  // sign-extend each nibble into its byte
            o |= (o & 0x08080808u) * 0x1Eu;
            out[2 * j] = __builtin_amdgcn_perm(o, e, 0x05010400u);      // k0 k1 k2 k3
            out[2 * j + 1] = __builtin_amdgcn_perm(o, e, 0x07030602u);  // k4 k5 k6 k7
        }
        uint4* q = reinterpret_cast<uint4*>(dst + row * ld_dst + c * 32);
        q[0] = make_uint4(out[0], out[1], out[2], out[3]);
        q[1] = make_uint4(out[4], out[5], out[6], out[7]);
    }
}

// Sum of the fp32 partial results of a split-K launch, plus bias, rounded once to the
// output type.  VEC: four columns per thread.
template <bool VEC>
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const float* part, int splits, int64_t m, int64_t n, const void* bias,
                                                            int bias_dtype, void* out, int out_dtype, int64_t ldo,
                                                            const void* addend, int64_t ldadd) {
    constexpr int W = VEC ? 4 : 1;
    const int64_t per_row = n / W;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= m * per_row) return;
    const int64_t row = i / per_row, col = (i - row * per_row) * W;
    float acc[W];
#pragma unroll
    for (int v = 0; v < W; ++v) acc[v] = 0.0f;
    for (int z = 0; z < splits; ++z) {
        const float* q = part + ((int64_t)z * m + row) * n + col;
        if constexpr (VEC) {
            const float4 t = *reinterpret_cast<const float4*>(q);
            acc[0] += t.x; acc[1] += t.y; acc[2] += t.z; acc[3] += t.w;
        } else {
            acc[0] += q[0];
        }
    }
    if (bias) {
#pragma unroll
        for (int v = 0; v < W; ++v) acc[v] += load_bias(bias, bias_dtype, col + v);
    }
    if (addend) {  // same dtype as the output
        const int64_t ea = row * ldadd + col;
#pragma unroll
        for (int v = 0; v < W; ++v) acc[v] += load_bias(addend, out_dtype, ea + v);
    }
    const int64_t e = row * ldo + col;
    if (out_dtype == SEGQ_F32) {
#pragma unroll
        for (int v = 0; v < W; ++v) static_cast<float*>(out)[e + v] = acc[v];
    } else if constexpr (VEC) {
        const bool bf = out_dtype == SEGQ_BF16;
        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(out) + e) =
            make_uint2(bf ? pack2_bf16(acc[0], acc[1]) : pack2_f16(acc[0], acc[1]), bf ? pack2_bf16(acc[2], acc[3]) : pack2_f16(acc[2], acc[3]));
    } else {
        const uint32_t two = out_dtype == SEGQ_BF16 ? pack2_bf16(acc[0], 0.0f) : pack2_f16(acc[0], 0.0f);
        static_cast<uint16_t*>(out)[e] = (uint16_t)(two & 0xffffu);
    }
}

// What a launch would do, for callers that ask before (or instead of) launching.
struct GemmPlan {
    int64_t bytes;  // workspace it would use
    int tile;       // tile id (1-based, as in segq_gemm_desc.tile)
    int splits;     // workgroups sharing the K steps of a tile (1: none)
    int parked;     // finished ranges parked in the workspace
};

// plan != nullptr: nothing is launched; *plan says what the launch would do if the caller lent
// as much workspace as the library can make use of (probe) or with d's own workspace (!probe).
static int gemm_impl(const segq_gemm_desc* d, hipStream_t st, GemmPlan* plan = nullptr, bool probe = true) {
    const bool need = plan != nullptr && probe;
    if (plan) *plan = GemmPlan{0, 0, 1, 0};
    if (!d) return fail(SEGQ_ERR_ARG, "segq_gemm: null descriptor");
    if (d->m < 0 || d->n < 0 || d->batch < 1) return fail(SEGQ_ERR_ARG, "segq_gemm: bad sizes");
    if (d->m == 0 || d->n == 0) return SEGQ_OK;
    if (d->m > 0x7fffffff / 2 || d->n > 0x7fffffff / 2) return fail(SEGQ_ERR_ARG, "segq_gemm: m or n too large");
    const bool codes_out = d->out_codes != nullptr;
    if (!d->a || !d->b || (!d->out && !codes_out)) return fail(SEGQ_ERR_ARG, "segq_gemm: null a, b or out");
    if (codes_out) {
        if ((d->out_dtype != SEGQ_BF16 && d->out_dtype != SEGQ_F16) || d->batch != 1 || !d->out_scale || d->ld_out_codes < d->n || d->split_k > 1 ||
            (d->out_code_fmt != SEGQ_CODE_I8 && d->out_code_fmt != SEGQ_CODE_E4M3) || d->out_pre_op < 0 || d->out_pre_op > SEGQ_PRE_SILU ||
            (d->out_scale_neg != nullptr) != (d->out_codes_neg != nullptr))
            return fail(SEGQ_ERR_ARG, "segq_gemm: out_codes needs out_dtype F16 or BF16, batch == 1, ld_out_codes >= n, int8 or e4m3 codes, "
                                      "out_scale, and out_scale_neg together with out_codes_neg");
    }
    if (d->n_ranges < 1 || d->n_ranges > SEGQ_MAX_RANGES) return fail(SEGQ_ERR_ARG, "segq_gemm: n_ranges %d out of range", d->n_ranges);
    const bool i8 = d->a_fmt == SEGQ_CODE_I8 && d->b_fmt == SEGQ_CODE_I8;
    const bool f8 = d->a_fmt == SEGQ_CODE_E4M3 && d->b_fmt == SEGQ_CODE_E4M3;
    const bool w4 = d->a_fmt == SEGQ_CODE_I8 && d->b_fmt == SEGQ_CODE_I4;
    if (!i8 && !f8 && !w4) return fail(SEGQ_ERR_UNSUPPORTED, "segq_gemm: no kernel for a_fmt %d with b_fmt %d", d->a_fmt, d->b_fmt);
    if (d->out_dtype != SEGQ_ACC && !is_float_dtype(d->out_dtype)) return fail(SEGQ_ERR_ARG, "segq_gemm: bad out_dtype %d", d->out_dtype);
    if (d->bias && !is_float_dtype(d->bias_dtype)) return fail(SEGQ_ERR_ARG, "segq_gemm: bad bias_dtype %d", d->bias_dtype);
    if (d->out_dtype == SEGQ_ACC && d->n_ranges != 1) return fail(SEGQ_ERR_ARG, "segq_gemm: raw accumulators need exactly one range");
    if (d->lda % 16 || d->ldb % 16 || !al(d->a, 16) || !al(d->b, 16) || (d->a_neg && !al(d->a_neg, 16)) ||
        d->batch_stride_a % 16 || d->batch_stride_b % 16)
        return fail(SEGQ_ERR_ARG, "segq_gemm: a and b need 16-byte aligned bases and row strides");
    if (!codes_out && d->ldo < d->n) return fail(SEGQ_ERR_ARG, "segq_gemm: ldo smaller than n");
    if (d->addend && (d->out_dtype == SEGQ_ACC || d->ld_addend < d->n))
        return fail(SEGQ_ERR_ARG, "segq_gemm: an addend needs a float output and ld_addend >= n");
    const bool lowrank = d->lowrank_t != nullptr || d->lowrank_rank != 0;
    if (lowrank) {
        if (!d->lowrank_t || !d->lowrank_l2t || d->lowrank_rank <= 0 || d->lowrank_rank % 32 || d->lowrank_rank > 512)
            return fail(SEGQ_ERR_ARG, "segq_gemm: the low-rank branch needs both matrices and a rank that is a multiple of 32, at most 512");
        if (d->out_dtype != SEGQ_BF16 && d->out_dtype != SEGQ_F16)
            return fail(SEGQ_ERR_UNSUPPORTED, "segq_gemm: the low-rank branch runs in the output's 16-bit dtype (out_dtype F16 or BF16)");
        if (d->ld_lowrank_t < d->lowrank_rank || d->ld_lowrank_l2t < d->lowrank_rank || d->ld_lowrank_t % 8 || d->ld_lowrank_l2t % 8 ||
            !al(d->lowrank_t, 16) || !al(d->lowrank_l2t, 16))
            return fail(SEGQ_ERR_ARG, "segq_gemm: low-rank matrices need 16-byte aligned rows of at least lowrank_rank elements");
        if (d->batch != 1 || d->split_k > 1)
            return fail(SEGQ_ERR_UNSUPPORTED, "segq_gemm: the low-rank branch needs batch == 1 and no split_k");
    }
    const bool groups = d->group_dequant != nullptr;
    if (groups) {
        if (!(i8 || w4) || d->batch != 1 || d->out_dtype == SEGQ_ACC || d->group_dequant_stride < d->n || !al(d->group_dequant, 4))
            return fail(SEGQ_ERR_UNSUPPORTED, "segq_gemm: group factors need int8 activations, one problem, a float output "
                                              "and a stride of at least n");
    }

    void* const ws = need ? reinterpret_cast<void*>(uintptr_t(256)) : d->workspace;
    const int64_t ws_bytes = need ? (int64_t)1 << 60 : d->workspace_bytes;
    GemmParams p;
    memset(&p, 0, sizeof(p));
    const int64_t kalign = w4 ? 32 : 16;
    int64_t kmax = 0, ktotal = 0;
    for (int i = 0; i < d->n_ranges; ++i) {
        const segq_krange& r = d->ranges[i];
        // the K rule of the reference's GEMM (segquant/src/real_quant/real_gemm.cu:237-247)
        if (r.k_begin < 0 || r.k_len <= 0 || r.k_begin % kalign || r.k_len % kalign)
            return fail(SEGQ_ERR_ARG, "segq_gemm: range %d: k_begin %lld and k_len %lld must be positive multiples of %lld",
                        i, (long long)r.k_begin, (long long)r.k_len, (long long)kalign);
        if (r.a_sel < 0 || r.a_sel > 3) return fail(SEGQ_ERR_ARG, "segq_gemm: range %d: bad a_sel %d", i, r.a_sel);
        if (r.a_sel == 1 && !d->a_neg) return fail(SEGQ_ERR_ARG, "segq_gemm: range %d reads a_neg, which is null", i);
        if (d->out_dtype != SEGQ_ACC && (!r.sx || !r.sw)) return fail(SEGQ_ERR_ARG, "segq_gemm: range %d has a null scale", i);
        if ((r.sx_row_stride | 1) != 1 || (r.sw_col_stride | 1) != 1) return fail(SEGQ_ERR_ARG, "segq_gemm: range %d: scale strides are 0 or 1", i);
        KRange& o = p.r[i];
        o.k0 = (int32_t)r.k_begin;
        o.k1 = (int32_t)(r.k_begin + r.k_len);
        o.a_sel = r.a_sel;
        o.sx_rs = r.sx_row_stride;
        o.sw_cs = r.sw_col_stride;
        o.sx = r.sx;
        o.sw = r.sw;
        if (r.k_begin + r.k_len > kmax) kmax = r.k_begin + r.k_len;
        ktotal += r.k_len;
    }
    if (kmax > d->lda || (w4 ? (kmax / 2 > d->ldb) : (kmax > d->ldb)))
        return fail(SEGQ_ERR_ARG, "segq_gemm: a range ends at %lld, beyond the row stride", (long long)kmax);
    // int4 weights are staged as value*16: keep |acc| below 2^31
    if (w4 && ktotal > 131071) return fail(SEGQ_ERR_UNSUPPORTED, "segq_gemm: K too large for int4 weights");
    if (kmax > 0x7fffff00) return fail(SEGQ_ERR_ARG, "segq_gemm: K too large");

    if (groups && w4) {
        const int64_t kp = (kmax + 31) & ~(int64_t)31;
        if (!ws || !al(ws, 16) || ws_bytes < d->n * kp)
            return fail(SEGQ_ERR_UNSUPPORTED, "segq_gemm: group factors with int4 weights need %lld bytes of workspace",
                        (long long)(d->n * kp));
    }
    if (w4 && ws) {
        // expand b to int8 in the caller's workspace and run the int8 kernels on it
        const int64_t kp = (kmax + 31) & ~(int64_t)31;  // whole 16-byte packed chunks
        if (al(ws, 16) && ws_bytes >= d->batch * d->n * kp && kp / 2 <= d->ldb) {
            if (plan) {  // the plan of the int8 launch on the expanded weights, plus the expansion's room
                segq_gemm_desc d8 = *d;
                d8.b_fmt = SEGQ_CODE_I8;
                d8.b = ws;
                d8.ldb = kp;
                d8.batch_stride_b = d->n * kp;
                d8.workspace = nullptr;
                d8.workspace_bytes = 0;
                const int rc = gemm_impl(&d8, st, plan, false);
                plan->bytes = d->batch * d->n * kp;
                return rc;
            }
            const int64_t chunks = kp / 32;
            for (int64_t zb = 0; zb < d->batch; ++zb) {
                const int64_t total = d->n * chunks;
                const unsigned blocks = (unsigned)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
                hipLaunchKernelGGL(expand_i4_kernel, dim3(blocks), dim3(256), 0, st,
                                   static_cast<const uint8_t*>(d->b) + zb * d->batch_stride_b, d->ldb,
                                   static_cast<uint8_t*>(d->workspace) + zb * d->n * kp, kp, d->n, chunks);
            }
            const int rc = check_launch("segq_gemm (int4 expansion)");
            if (rc != SEGQ_OK) return rc;
            segq_gemm_desc d8 = *d;
            d8.b_fmt = SEGQ_CODE_I8;
            d8.b = d->workspace;
            d8.ldb = kp;
            d8.batch_stride_b = d->n * kp;
            d8.workspace = nullptr;
            d8.workspace_bytes = 0;
            return gemm_impl(&d8, st);
        }
    }

    p.A = static_cast<const uint8_t*>(d->a);
    p.A2 = static_cast<const uint8_t*>(d->a_neg);
    p.B = static_cast<const uint8_t*>(d->b);
    p.C = d->out;
    p.bias = d->out_dtype == SEGQ_ACC ? nullptr : d->bias;
    p.M = (int32_t)d->m;
    p.N = (int32_t)d->n;
    p.lda = d->lda; p.ldb = d->ldb; p.ldc = d->ldo;
    p.bsA = d->batch_stride_a; p.bsB = d->batch_stride_b; p.bsC = d->batch_stride_out;
    p.bsSx = d->batch_stride_sx; p.bsSw = d->batch_stride_sw;
    p.out_dtype = d->out_dtype; p.bias_dtype = d->bias_dtype;
    {
        const int64_t asz = d->out_dtype == SEGQ_F32 ? 4 : 2;
        p.addend = d->addend;
        p.ldadd = d->ld_addend;
        p.vec_add = d->addend && (d->ld_addend * asz) % (4 * asz) == 0 && (d->batch_stride_out * asz) % (4 * asz) == 0 && al(d->addend, 4 * asz);
    }
    p.nr = d->n_ranges;
    const bool fold = d->n_ranges > 1;
    bool wide_ok = d->m * d->lda < (int64_t)1 << 32 && d->n * d->ldb < (int64_t)1 << 32;
    for (int i = 0; i < d->n_ranges; ++i) wide_ok = wide_ok && d->ranges[i].k_begin % 128 == 0 && d->ranges[i].k_len % 128 == 0;
    int cfg;
    bool plain8 = i8 || f8;  // both operands straight to LDS: no sign selection, no int4 unpacking
    for (int i = 0; i < d->n_ranges; ++i) plain8 = plain8 && d->ranges[i].a_sel < 2;
    // several ranges cost a second (fp32) accumulator set, and with it the biggest tiles,
    // unless the accumulators are fp32 already (plain e4m3: rescaled in place)
    const bool fold2 = fold && !(f8 && plain8);
    if (groups) {
        bool ok = wide_ok && plain8;
        for (int i = 0; i < d->n_ranges; ++i) ok = ok && d->ranges[i].a_sel < 2;
        if (!ok) return fail(SEGQ_ERR_UNSUPPORTED, "segq_gemm: group factors need ranges of whole 128-column groups and a_sel 0 or 1");
        p.grw = d->group_dequant;
        p.grw_gs = d->group_dequant_stride;
    }
    // int8 with several ranges keeps the big tiles if the caller lends a workspace to park
    // finished ranges in: one fp32 tile per workgroup
    bool park = i8 && plain8 && fold && !groups && wide_ok && d->batch == 1 && d->out_dtype != SEGQ_ACC && ws && al(ws, 16);
    auto park_fits = [&](int c) {
        if (c < FIRST_WIDE_CFG || c >= NUM_TILE_CFG) return false;
        const TileCfg& t = TILE_CFGS[c];
        const int64_t tiles = ((d->m + t.bm - 1) / t.bm) * ((d->n + t.bn - 1) / t.bn);
        return ws_bytes >= tiles * t.bm * t.bn * 4;
    };
    if (d->tile == 0) {
        if (groups) {
            // 128 x 128: at 126 registers two workgroups share a CU, and one's conversion (VALU) runs under
            // the other's MFMAs; measured 8 % (8192 x 10240 x 1280) to 25 % (8192 x 1280 x 5120) ahead
            // of 256 x 128 / 128 x 256, which are selectable by id
            cfg = FIRST_WIDE_CFG + 3;
        } else {
            cfg = park ? choose_tile(d->m, d->n, d->batch, false, wide_ok, plain8) : -1;
            park = park && park_fits(cfg);
            if (!park) cfg = choose_tile(d->m, d->n, d->batch, fold2, wide_ok, plain8, ktotal / 128, (!fold || f8) && !lowrank);
        }
    }
    else if (d->tile >= 1 && d->tile <= NUM_TILE_CFG) cfg = d->tile - 1;
    else return fail(SEGQ_ERR_ARG, "segq_gemm: tile %d is not in 0..%d", d->tile, NUM_TILE_CFG);
    // Few tokens: when the 128 x 128 tiles do not even fill the CUs once, a workgroup has its CU to
    // itself and waits on HBM latency: the int8 kernel with four LDS stages keeps three K steps in
    // flight instead of one (256 x 9216 x 1536: 14.8 -> 12.9 us, 512 x 6144 x 3072: 25.5 -> 20.4 us)
    if (d->tile == 0 && cfg == FIRST_WIDE_CFG + 3 && i8 && plain8 && !fold && !groups && !lowrank && wide_ok &&
        ((d->m + 127) / 128) * ((d->n + 127) / 128) * d->batch <= device_cus() && ktotal / 128 >= 6) {
        cfg = FIRST_WIDE_CFG + 8;
        // ... and where 128 x 96 tiles still fit the CUs once and tile the columns exactly, a third more
        // workgroups pull from memory, each with four K steps in flight (five stages)
        if (d->n % 96 == 0 && ((d->m + 127) / 128) * (d->n / 96) * d->batch <= device_cus()) cfg = FIRST_WIDE_CFG + 10;
    }
    // the 8-wave tiles that exist with the finish in output units (low-rank branch, two-way K split)
    auto tail_tile = [](int c) {
        const int w = c - FIRST_WIDE_CFG;
        return w == 0 || w == 1 || w == 3 || w == 6 || w == 7;
    };
    if (lowrank && d->tile == 0 && cfg >= FIRST_WIDE_CFG && !tail_tile(cfg)) {
        cfg = cfg == FIRST_WIDE_CFG + 2 ? FIRST_WIDE_CFG + 1 : FIRST_WIDE_CFG;
        park = park && park_fits(cfg);
    }
    // Split K: few tiles and a long contraction.  The K steps of every tile are shared by
    // `splits` workgroups (grid.y).
    //  * Two shares are finished inside the launch: each workgroup leaves its fp32 share in the
    //    workspace, and the second to arrive adds the two, adds the bias and rounds.  Workspace:
    //    two tile-sized shares per tile, one word per tile in which the first to arrive leaves the
    //    launch's stamp (a per-process counter: no clearing between launches, and a fresh workspace
    //    may hold anything) and which the second clears (so that a captured graph, which replays
    //    the launch with the stamp it was recorded with, works too).
    //  * More shares: each workgroup writes an fp32 partial result, a second kernel sums them in the
    //    order of the shares.  Workspace: the partial results.
    // Either way the parking slots of all those workgroups follow (int8 with several ranges).
    int splits = 1;
    int64_t part_bytes = 0;
    {
        const bool can = plain8 && wide_ok && d->batch == 1 && !groups && !lowrank && d->out_dtype != SEGQ_ACC && ws && al(ws, 16) &&
                         d->split_k != 1 && (d->tile == 0 || cfg >= FIRST_WIDE_CFG) && !codes_out;
        const int64_t total_steps = ktotal / 128;
        if (d->split_k > 1 && !can)
            return fail(SEGQ_ERR_UNSUPPORTED, "segq_gemm: split_k needs plain 8-bit codes, K ranges in multiples of 128, one problem, "
                                              "a float output, an 8-wave tile and a workspace");
        if (can) {
            int want = 1, scfg = cfg;
            const bool big_ok = !fold2 || park || f8;  // the 256 x 256 tile, or 256 x 128 with a second register set
            const int64_t cus = device_cus();
            auto tiles_of = [&](int c) { return ((d->m + TILE_CFGS[c].bm - 1) / TILE_CFGS[c].bm) * ((d->n + TILE_CFGS[c].bn - 1) / TILE_CFGS[c].bn); };
            if (d->split_k > 1) {
                want = (int)(d->split_k < total_steps ? d->split_k : total_steps);
                if (d->tile == 0) scfg = big_ok ? FIRST_WIDE_CFG : FIRST_WIDE_CFG + 1;
            } else if (d->tile == 0 && total_steps >= 16 && tiles_of(cfg) * 10 < cus * 9) {
                // Whole tiles would leave more than a tenth of the CUs idle: look for a big tile and a
                // number of shares that fill them.  Measured (us, random codes, 256 CUs):
                //   1024 x 3072, K 13824 twice (DualScale):  e4m3  256x192 x4 99 | 256x256 x5 130 | 128x128 176
                //                                            int8  256x192 x4 108 | 256x256 x4 125 | 128x128 184
                //   4096 x 1536, K 6144 twice:               e4m3  256x192 x2 85 | 256x256 x2 94 | 256x128 123
                // The choice minimises rounds x (K steps per share + fixed cost) x tile area / efficiency:
                // about 6 steps' worth of prologue and epilogue per workgroup, 8 more for the shares' trip
                // through memory; big tiles get more out of every byte they stream.
                auto eff = [](int c) {
                    const int area = TILE_CFGS[c].bm * TILE_CFGS[c].bn;
                    return c < FIRST_WIDE_CFG ? 0.5 : area >= 256 * 256 ? 1.0 : area >= 256 * 192 ? 0.95 : area >= 256 * 128 ? 0.85 : 0.7;
                };
                auto cost = [&](int c, int64_t s_) {
                    const int64_t wgs = tiles_of(c) * s_;
                    return (double)((wgs + cus - 1) / cus) * ((double)total_steps / s_ + 6.0 + (s_ > 1 ? 8.0 : 0.0)) *
                           TILE_CFGS[c].bm * TILE_CFGS[c].bn / eff(c);
                };
                // (the 128 x 128 tile joins for very few tokens: 64 x 9216 x 3072 in two or three shares
                // 19 us against 25 us whole)
                const int cands[4] = {FIRST_WIDE_CFG + 6, FIRST_WIDE_CFG, FIRST_WIDE_CFG + 7, FIRST_WIDE_CFG + 3};
                double best = cost(cfg, 1);
                for (int i = 0; i < (big_ok ? 4 : 1); ++i) {
                    const int c = big_ok ? cands[i] : FIRST_WIDE_CFG + 1;
                    if (c == FIRST_WIDE_CFG + 3 && (d->m > 128 || (i8 && fold))) continue;
                    int64_t s_ = cus / tiles_of(c);
                    if (s_ > total_steps / 8) s_ = total_steps / 8;
                    if (s_ > 16) s_ = 16;
                    if (s_ < 2) continue;
                    if (cost(c, s_) < best) { best = cost(c, s_); scfg = c; want = (int)s_; }
                }
            }
            const TileCfg& t = TILE_CFGS[scfg];
            const int64_t tiles = tiles_of(scfg);
            const bool need_park = i8 && fold && scfg != FIRST_WIDE_CFG + 1 && scfg != FIRST_WIDE_CFG + 2 && scfg != FIRST_WIDE_CFG + 3;
            auto shares_for = [&](int s_) {
                if (s_ == 2 && tail_tile(scfg)) return tiles * 2 * t.bm * t.bn * 4 + ((tiles * 4 + 255) & ~(int64_t)255);
                return (((int64_t)s_ * d->m * d->n * 4) + 255) & ~(int64_t)255;
            };
            auto bytes_for = [&](int s_) { return shares_for(s_) + (need_park || park ? (int64_t)s_ * tiles * t.bm * t.bn * 4 : 0); };
            while (want > 1 && bytes_for(want) > ws_bytes) --want;
            if (d->split_k > 1 && want < 2) return fail(SEGQ_ERR_ARG, "segq_gemm: workspace too small for split_k");
            if (want > 1) {
                splits = want;
                cfg = scfg;
                part_bytes = shares_for(splits);
                park = (need_park || park) && i8 && fold;
            }
        }
    }
    if (splits == 1 && d->tile != 0) park = park && park_fits(cfg);
    if (park) p.park = reinterpret_cast<float*>(static_cast<uint8_t*>(ws) + part_bytes);
    if (park) {
        // every 8-wave tile serves several ranges this way
    } else if (cfg >= FIRST_WIDE_CFG) {
        if (!wide_ok) return fail(SEGQ_ERR_UNSUPPORTED, "segq_gemm: tile %d needs K ranges in multiples of 128", cfg + 1);
        if (fold2 && cfg == FIRST_WIDE_CFG) cfg = FIRST_WIDE_CFG + 1;
        if (groups && cfg == FIRST_WIDE_CFG) cfg = FIRST_WIDE_CFG + 1;
        if (groups && cfg > FIRST_WIDE_CFG + 3)
            return fail(SEGQ_ERR_UNSUPPORTED, "segq_gemm: group factors run on tiles %d to %d", FIRST_WIDE_CFG + 2, FIRST_WIDE_CFG + 4);
    } else if (groups) {
        return fail(SEGQ_ERR_UNSUPPORTED, "segq_gemm: group factors run on tiles %d to %d", FIRST_WIDE_CFG + 2, FIRST_WIDE_CFG + 4);
    } else if (cfg >= FIRST_BIG_CFG) {
        if (!wide_ok || w4 || fold)
            return fail(SEGQ_ERR_UNSUPPORTED, "segq_gemm: tile %d needs one range, 8-bit weights and K in multiples of 128", cfg + 1);
    }
    if (lowrank) {
        // small problems, which would otherwise go to the general kernel: the smallest 8-wave tile
        if (d->tile == 0 && cfg < FIRST_WIDE_CFG && plain8 && wide_ok && splits == 1) cfg = FIRST_WIDE_CFG + 3;
        if (cfg < FIRST_WIDE_CFG || !plain8 || !wide_ok)
            return fail(SEGQ_ERR_UNSUPPORTED, "segq_gemm: the low-rank branch needs plain 8-bit codes on both sides, K ranges in multiples "
                                              "of 128 and a shape the 8-wave kernels serve; pass the product as addend instead");
        p.lr_t = static_cast<const uint16_t*>(d->lowrank_t);
        p.lr_l2 = static_cast<const uint16_t*>(d->lowrank_l2t);
        p.lr_ldt = d->ld_lowrank_t;
        p.lr_ldl = d->ld_lowrank_l2t;
        p.lr_rank = d->lowrank_rank;
    }
    if (codes_out) {
        // the epilogue that writes codes is built into two tiles of the pipelined kernels
        if (!(plain8 && wide_ok && !fold && !groups && !lowrank && splits == 1))
            return fail(SEGQ_ERR_UNSUPPORTED, "segq_gemm: out_codes needs plain int8 or e4m3 codes on both sides and one K range in "
                                              "multiples of 128; no group factors, low-rank branch or split_k");
        // 128 x 128: two workgroups share a CU, so one's epilogue (all VALU: ~40 instructions per element
        // with a GELU and two code tensors) can run under the other's MFMAs.  Measured on 4096 x 1536 ->
        // 6144 e4m3, GELU(tanh), DualScale: 66 us against 104 us on 256 x 256, one workgroup per CU
        if (d->tile == 0) cfg = FIRST_WIDE_CFG + 3;
        p.oc = d->out_codes;
        p.oc_neg = d->out_codes_neg;
        p.ldoc = d->ld_out_codes;
        p.oc_scale = d->out_scale;
        p.oc_scale_neg = d->out_scale_neg;
        p.oc_fmt = d->out_code_fmt;
        p.oc_pre = d->out_pre_op;
        p.oc_vec = d->ld_out_codes % 8 == 0 && al(d->out_codes, 8) && (!d->out_codes_neg || al(d->out_codes_neg, 8));
    }
    const TileCfg& c = TILE_CFGS[cfg];
    p.tiles_m = (int32_t)((d->m + c.bm - 1) / c.bm);
    p.tiles_n = (int32_t)((d->n + c.bn - 1) / c.bn);
    if (plan) {
        plan->bytes = part_bytes + (park ? (int64_t)splits * p.tiles_m * p.tiles_n * c.bm * c.bn * 4 : 0);
        plan->tile = cfg + 1;
        plan->splits = splits;
        plan->parked = park ? 1 : 0;
        // walk the same dispatch the launch takes, down to the kernel instance, and launch nothing:
        // the plan is refused exactly when the launch would be
        p.dry = 1;
    }
    // tiles are numbered down groups of this many tile rows, so that the 32 tiles an XCD holds at a time
    // share few operand panels; 384-row tiles reach that with half as many rows (e4m3 4608 x 12288 x 3072
    // 140.7 -> 136.2 us; other heights between 2 and 16 measured the same or worse on the 4608-token shapes)
    p.group_m = (cfg == FIRST_WIDE_CFG + 9) ? 4 : 8;
    {
        // e4m3 only (4608 x 15360 x 3072 in three ranges: 350 -> 338 us); int8, which parks its sums at the
        // boundaries, loses more to the XCDs reading different operand columns at a time than it gains
        // from spreading its stores (385 -> 397 us), and keeps the common order
        p.rot = (d->n_ranges > 1 && splits == 1 && f8) ? 1 : 0;
    }
    if ((int64_t)p.tiles_m * p.tiles_n > 0x7fffffff || d->batch > 65535) return fail(SEGQ_ERR_ARG, "segq_gemm: grid too large");
    const int64_t osz = (d->out_dtype == SEGQ_F32 || d->out_dtype == SEGQ_ACC) ? 4 : 2;
    p.vec_store = ((d->ldo * osz) % (4 * osz) == 0) && ((d->batch_stride_out * osz) % (4 * osz) == 0) && al(d->out, 4 * osz);
    p.vec_store16 = osz == 2 && d->ldo % 8 == 0 && d->batch_stride_out % 8 == 0 && al(d->out, 16);
    if (splits == 2 && tail_tile(cfg)) {
        p.splits = 2;
        p.part = static_cast<float*>(d->workspace);
        const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
        p.arrived = reinterpret_cast<unsigned int*>(static_cast<uint8_t*>(d->workspace) + tiles * 2 * c.bm * c.bn * 4);
        p.bsA = p.bsB = p.bsC = p.bsSx = p.bsSw = 0;  // blockIdx.y counts shares here, not problems
        static unsigned int g_stamp = 0x5e690000u;
        if (!p.dry) do p.stamp = __atomic_add_fetch(&g_stamp, 1u, __ATOMIC_RELAXED); while (p.stamp == 0u);  // 0 means "cleared"
        return i8 ? launch_gemm_i8(p, cfg, fold, 2, st) : launch_gemm_f8(p, cfg, fold, 2, st);
    }
    if (splits > 1) {
        p.splits = splits;
        p.C = d->workspace;
        p.ldc = d->n;
        p.bsC = d->m * d->n;
        p.bsA = p.bsB = p.bsSx = p.bsSw = 0;
        p.out_dtype = SEGQ_F32;
        p.bias = nullptr;
        p.addend = nullptr;
        p.vec_store = d->n % 4 == 0;
        p.vec_store16 = 0;
        const int rc = i8 ? launch_gemm_i8(p, cfg, fold, splits, st) : launch_gemm_f8(p, cfg, fold, splits, st);
        if (rc != SEGQ_OK || p.dry) return rc;
        const bool vec = d->n % 4 == 0 && d->ldo % 4 == 0 && al(d->out, 16);
        const int64_t items = d->m * (vec ? d->n / 4 : d->n);
        const dim3 grid((unsigned)((items + 255) / 256));
        if (vec)
            hipLaunchKernelGGL(splitk_reduce_kernel<true>, grid, dim3(256), 0, st, static_cast<const float*>(d->workspace), splits,
                               d->m, d->n, d->bias, d->bias_dtype, d->out, d->out_dtype, d->ldo, d->addend, d->ld_addend);
        else
            hipLaunchKernelGGL(splitk_reduce_kernel<false>, grid, dim3(256), 0, st, static_cast<const float*>(d->workspace), splits,
                               d->m, d->n, d->bias, d->bias_dtype, d->out, d->out_dtype, d->ldo, d->addend, d->ld_addend);
        return check_launch("segq_gemm (split-K sum)");
    }
    if (i8) return launch_gemm_i8(p, cfg, fold, d->batch, st);
    if (f8) return launch_gemm_f8(p, cfg, fold, d->batch, st);
    return launch_gemm_w4(p, cfg, fold, d->batch, st);
}

// ---- the library's own scratch memory, for segq_gemm_noalloc -------------------------------
// One array per GPU the library runs on, held until the process ends.  In host code the name
// `scratch` is only a handle for hipGetSymbolAddress: the device address it resolves to (one per
// device, each GPU holding its own copy) is what kernels, copies and fills are given.
constexpr int64_t SCRATCH_BYTES = SEGQ_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[SCRATCH_BYTES];
static void* g_scratch_ptr[64];  // resolved address per device ordinal

static int scratch_address(void** out) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
        return fail(SEGQ_ERR_LAUNCH, "segq: cannot tell the current device (or its ordinal is above 63)");
    void* ptr = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
    if (!ptr) {
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr)
            return fail(SEGQ_ERR_LAUNCH, "segq: cannot resolve the scratch array on device %d: %s", dev, hipGetErrorString(e));
        __atomic_store_n(&g_scratch_ptr[dev], ptr, __ATOMIC_RELEASE);
    }
    *out = ptr;
    return SEGQ_OK;
}

}  // namespace segq

using namespace segq;

// only the C ABI leaves the library: everything else is built with hidden visibility
#pragma GCC visibility push(default)
extern "C" {

int segq_version(void) { return 100; }

const char* segq_last_error(void) { return g_err; }

int segq_quantize(const segq_quant_desc* d, segq_stream_t stream) {
    return quantize_impl(d, static_cast<hipStream_t>(stream), nullptr);
}

int segq_quantize_many(const segq_quant_desc* descs, int32_t n, segq_stream_t stream) {
    return quantize_many_impl(descs, n, static_cast<hipStream_t>(stream));
}

static void weight_desc(segq_quant_desc* q, const void* w, int32_t w_dtype, int64_t n, int64_t k, void* codes, int32_t fmt) {
    memset(q, 0, sizeof(*q));
    q->x = w; q->x_dtype = w_dtype; q->code_fmt = fmt;
    q->rows = n; q->cols = k; q->ldx = k;
    q->codes = codes; q->ld_codes = fmt == SEGQ_CODE_I4 ? k / 2 : k;
    q->n_kseg = 1;
}

int segq_quantize_weights_scalar(const void* weights, int32_t w_dtype, int64_t n, int64_t k, void* codes,
                                 int32_t code_fmt, float scale_w, segq_stream_t stream) {
    segq_quant_desc q;
    weight_desc(&q, weights, w_dtype, n, k, codes, code_fmt);
    return quantize_impl(&q, static_cast<hipStream_t>(stream), &scale_w);
}

int segq_quantize_weights_rows(const void* weights, int32_t w_dtype, int64_t n, int64_t k, void* codes,
                               int32_t code_fmt, const float* scale_w_rows, segq_stream_t stream) {
    segq_quant_desc q;
    weight_desc(&q, weights, w_dtype, n, k, codes, code_fmt);
    q.scale = const_cast<float*>(scale_w_rows);
    q.row_stride = 1;
    return quantize_impl(&q, static_cast<hipStream_t>(stream), nullptr);
}

int segq_quantize_weights_groups(const void* weights, int32_t w_dtype, int64_t n, int64_t k, void* codes, int32_t code_fmt,
                                 const float* scales, int64_t group, segq_stream_t stream) {
    return quantize_groups_impl(weights, w_dtype, n, k, codes, code_fmt, scales, group, static_cast<hipStream_t>(stream));
}

int segq_repack_int4_cols_to_rows(const void* colpacked, void* rowpacked, int64_t out, int64_t cols, segq_stream_t stream) {
    return repack_i4_impl(colpacked, rowpacked, out, cols, static_cast<hipStream_t>(stream));
}

int segq_gemm(const segq_gemm_desc* d, segq_stream_t stream) { return gemm_impl(d, static_cast<hipStream_t>(stream)); }

int segq_gemm_tile_count(void) { return NUM_TILE_CFG; }

int segq_gemm_workspace_bytes(const segq_gemm_desc* d, int64_t* bytes) {
    if (!bytes) return fail(SEGQ_ERR_ARG, "segq_gemm_workspace_bytes: null result pointer");
    GemmPlan plan;
    const int rc = gemm_impl(d, nullptr, &plan);
    *bytes = plan.bytes;
    return rc;
}

int segq_gemm_plan(const segq_gemm_desc* d, int32_t* tile, int32_t* splits, int32_t* parked) {
    GemmPlan plan;
    const int rc = gemm_impl(d, nullptr, &plan, false);
    if (tile) *tile = plan.tile;
    if (splits) *splits = plan.splits;
    if (parked) *parked = plan.parked;
    return rc;
}

int segq_init(void) {
    void* ptr = nullptr;
    (void)device_cus();
    return scratch_address(&ptr);
}

int64_t segq_noalloc_scratch_bytes(void) { return SCRATCH_BYTES; }

int segq_device_info(int32_t* compute_units, int32_t* max_engine_clock_khz) {
    int dev = 0, cus = 0, khz = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        hipDeviceGetAttribute(&khz, hipDeviceAttributeClockRate, dev) != hipSuccess)
        return fail(SEGQ_ERR_LAUNCH, "segq_device_info: cannot read the current device's attributes");
    if (compute_units) *compute_units = cus;
    if (max_engine_clock_khz) *max_engine_clock_khz = khz;
    return SEGQ_OK;
}

int segq_gemm_noalloc(const segq_gemm_desc* d, segq_stream_t stream) {
    GemmPlan plan;
    int rc = gemm_impl(d, nullptr, &plan);
    if (rc != SEGQ_OK) return rc;
    const int64_t wish = plan.bytes;  // what the launch would use of an unlimited workspace
    segq_gemm_desc c = *d;
    c.workspace = nullptr;
    c.workspace_bytes = 0;
    if (wish > 0) {
        void* ptr = nullptr;
        rc = scratch_address(&ptr);  // resolved once per device (segq_init does it ahead of time)
        if (rc != SEGQ_OK) return rc;
        c.workspace = ptr;
        c.workspace_bytes = SCRATCH_BYTES;
    }
    // a launch that could use more than the array holds runs with what fits, as segq_gemm does with
    // a workspace of that size (fewer K shares, a second register set instead of parked sums); it
    // is refused only where it cannot run with less
    rc = gemm_impl(&c, static_cast<hipStream_t>(stream));
    if (rc != SEGQ_OK && wish > SCRATCH_BYTES) {
        char why[256];
        snprintf(why, sizeof(why), "%s", g_err);
        return fail(rc, "segq_gemm_noalloc: this launch needs more workspace than the library's scratch array holds (%lld bytes; "
                        "it could use %lld): %s; use segq_gemm with a workspace of the caller's",
                    (long long)SCRATCH_BYTES, (long long)wish, why);
    }
    return rc;
}

int segq_linear(const segq_quant_desc* q, const segq_gemm_desc* g, segq_stream_t stream) {
    if (!q || !g) return fail(SEGQ_ERR_ARG, "segq_linear: null descriptor");
    if (q->rows == 0 && g->m == 0) return SEGQ_OK;  // no token rows: nothing to quantise, nothing to multiply
    // the GEMM must consume exactly what the quantise step produces
    if (q->codes != g->a) return fail(SEGQ_ERR_ARG, "segq_linear: the GEMM must read the codes the quantise step writes");
    if (g->n_ranges < 1 || g->n_ranges > SEGQ_MAX_RANGES) return fail(SEGQ_ERR_ARG, "segq_linear: n_ranges %d out of range", g->n_ranges);
    bool reads_neg = false;
    for (int i = 0; i < g->n_ranges; ++i) reads_neg = reads_neg || g->ranges[i].a_sel == 1;
    if (reads_neg && (!q->codes_neg || q->codes_neg != g->a_neg))
        return fail(SEGQ_ERR_ARG, "segq_linear: a range reads a_neg, which is not the second code tensor the quantise step writes");
    if (q->ld_codes != g->lda || q->rows != g->m * g->batch)
        return fail(SEGQ_ERR_ARG, "segq_linear: the code tensor's rows (%lld, stride %lld) do not match the GEMM's (%lld, stride %lld)",
                    (long long)q->rows, (long long)q->ld_codes, (long long)(g->m * g->batch), (long long)g->lda);
    if (q->code_fmt != g->a_fmt) return fail(SEGQ_ERR_ARG, "segq_linear: code formats differ (%d written, %d read)", q->code_fmt, g->a_fmt);
    if (q->dynamic && g->out_dtype != SEGQ_ACC) {
        // dynamic scales are outputs of the first step: every range must divide by one of them
        const int64_t seg_rows = q->seg_rows > 0 ? q->seg_rows : q->rows;
        const int64_t extent = (seg_rows > 0 ? (q->rows - 1) / seg_rows : 0) * q->seg_stride + (seg_rows - 1) * q->row_stride +
                               (int64_t)(q->n_kseg - 1) * q->kseg_stride + 1;
        for (int i = 0; i < g->n_ranges; ++i) {
            const float* sx = g->ranges[i].sx;
            const bool in_pos = q->scale && sx >= q->scale && sx < q->scale + extent;
            const bool in_neg = q->scale_neg && sx >= q->scale_neg && sx < q->scale_neg + extent;
            if (!in_pos && !in_neg)
                return fail(SEGQ_ERR_ARG, "segq_linear: range %d divides by scales the dynamic quantise step does not write", i);
        }
    }
    const int rc = quantize_impl(q, static_cast<hipStream_t>(stream), nullptr);
    if (rc != SEGQ_OK) return rc;
    return gemm_impl(g, static_cast<hipStream_t>(stream));
}

int segq_fake_e4m3(const void* x, void* out, int32_t dtype, int64_t numel, segq_stream_t stream) {
    return fake_e4m3_impl(x, out, dtype, numel, static_cast<hipStream_t>(stream));
}

}  // extern "C"
#pragma GCC visibility pop
