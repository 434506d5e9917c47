// What the matrix cores of this device sustain with NOTHING else in the loop, against operand data:
// the ceiling a GEMM's K loop is measured against.  One workgroup of eight waves per CU (two per
// SIMD, the GEMM kernels' occupancy), every wave a 64 x 128 wave tile's worth of MFMAs per
// iteration on operands held in registers (no LDS, no memory traffic), all CUs at once.
// Prints, per operand pattern (all zero, small values, full-range random): operations per
// second and the shader clock during the launch, taken from the cycle counter (s_memtime) and the
// constant 100 MHz wall clock (s_memrealtime) read by one wave per CU at both ends.
//
// Build and run (a stand-alone program, not part of libsegq.so):
//   make -C segquant_amd/csrc mfma_ceiling && segquant_amd/mfma_ceiling
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <vector>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));

struct Clocks { unsigned long long cycles, wall; };

template <bool F8>
__global__ void __launch_bounds__(512) mfma_only(int iters, const v8i* src, int* out, Clocks* clk) {
    const int tid = threadIdx.x;
    v8i fa[4], fb[8];
    for (int i = 0; i < 4; ++i) fa[i] = src[i * 512 + tid];
    for (int i = 0; i < 8; ++i) fb[i] = src[(4 + i) * 512 + tid];
    v4i acc[8][4];
    v4f accf[8][4];
    for (int a = 0; a < 8; ++a)
        for (int b = 0; b < 4; ++b) {
            acc[a][b] = v4i{0, 0, 0, 0};
            accf[a][b] = v4f{0.f, 0.f, 0.f, 0.f};
        }
    const unsigned long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int a = 0; a < 8; ++a)
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                if constexpr (F8) {
                    accf[a][b] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[a], fa[b], accf[a][b], 0, 0, 0, 0, 0, 0);
                } else {  // a 128-byte K step of the int8 kernels: two 16 x 16 x 64 MFMAs per block
                    acc[a][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(v4i{fb[a][0], fb[a][1], fb[a][2], fb[a][3]},
                                                                     v4i{fa[b][0], fa[b][1], fa[b][2], fa[b][3]}, acc[a][b], 0, 0, 0);
                    acc[a][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(v4i{fb[a][4], fb[a][5], fb[a][6], fb[a][7]},
                                                                     v4i{fa[b][4], fa[b][5], fa[b][6], fa[b][7]}, acc[a][b], 0, 0, 0);
                }
            }
    }
    const unsigned long long c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
    int s = 0;
    for (int a = 0; a < 8; ++a)
        for (int b = 0; b < 4; ++b) s += acc[a][b][0] + acc[a][b][3] + (int)accf[a][b][1];
    out[blockIdx.x * 512 + tid] = s;
    if (tid == 0) clk[blockIdx.x] = Clocks{c1 - c0, w1 - w0};
}

int main() {
    int dev = 0, cus = 0, khz = 0;
    hipGetDevice(&dev);
    hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    hipDeviceGetAttribute(&khz, hipDeviceAttributeClockRate, dev);
    printf("device: %d CUs, highest engine clock %.2f GHz -> dense 8-bit peak %.0f TOP/s (CUs x 4 SIMDs x 2048 ops/clk x clock)\n",
           cus, khz / 1e6, cus * 4.0 * 2048 * khz * 1e3 / 1e12);
    int* out;
    v8i* src;
    Clocks* clk;
    hipMalloc(&out, cus * 512 * 4);
    hipMalloc(&src, 12 * 512 * 32);
    hipMalloc(&clk, cus * sizeof(Clocks));
    hipEvent_t e0, e1;
    hipEventCreate(&e0);
    hipEventCreate(&e1);
    std::vector<Clocks> hclk(cus);
    struct Pattern { const char* name; int range; };
    const Pattern pats[] = {{"all zero", 1}, {"values in -3..3", 7}, {"full-range random bytes", 255}};
    for (int f8 = 0; f8 < 2; ++f8)
        for (const Pattern& pt : pats) {
            std::vector<unsigned char> h(12 * 512 * 32);
            srand(12345);
            for (auto& x : h) {
                x = (unsigned char)(rand() % pt.range - pt.range / 2);
                if (f8 && (x & 0x7F) == 0x7F) x = 0x3A;  // no e4m3 NaN codes
            }
            hipMemcpy(src, h.data(), h.size(), hipMemcpyHostToDevice);
            const int iters = 4000;  // ~0.25 ms at full rate: long enough for the clock to settle under load
            auto launch = [&](int n) {
                if (f8) hipLaunchKernelGGL(mfma_only<true>, dim3(cus), dim3(512), 0, 0, n, src, out, clk);
                else hipLaunchKernelGGL(mfma_only<false>, dim3(cus), dim3(512), 0, 0, n, src, out, clk);
            };
            launch(iters);
            hipDeviceSynchronize();
            hipEventRecord(e0);
            launch(iters);
            hipEventRecord(e1);
            hipEventSynchronize(e1);
            float ms = 0;
            hipEventElapsedTime(&ms, e0, e1);
            hipMemcpy(hclk.data(), clk, cus * sizeof(Clocks), hipMemcpyDeviceToHost);
            double ghz = 0;
            for (const Clocks& c : hclk) ghz += (double)c.cycles / ((double)c.wall / 100e6) / 1e9;
            ghz /= cus;
            const double ops = 2.0 * 16 * 16 * 128 * 32 * (double)iters * 8 * cus;
            printf("%-5s %-26s %8.3f ms  %7.1f TOP/s  shader clock %.2f GHz  (%.0f %% of the pipe's cycles at that clock)\n",
                   f8 ? "e4m3" : "int8", pt.name, ms, ops / (ms * 1e-3) / 1e12, ghz,
                   100.0 * ops / (ms * 1e-3) / (cus * 4.0 * 2048 * ghz * 1e9));
            fflush(stdout);
        }
    return 0;
}
