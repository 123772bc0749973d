// Measurement aid: the MFMA rate this device sustains on its own.
//
// The published dense bf16 peak assumes the maximum clock. Under a matrix load
// the board's power limit sets the clock, and the power an MFMA draws depends
// on how many operand bits toggle: a loop of nothing but MFMAs runs measurably
// faster on constant operands than on random ones. The attention kernel's
// roofline fraction is quoted against the published peak; this probe gives the
// ceiling that is physically reachable on the data the benchmark uses
// (normally distributed bf16 operands), so the two can be read side by side.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>

#include "../../include/zdraw_hip.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kSets = 64;      // operand sets of 512 lanes x 8 bf16
constexpr int kThreads = 512;  // two waves per SIMD
constexpr int kBlocks = 256;   // one workgroup per CU

// 8 MFMAs per iteration on four independent accumulators; operands stay in registers.
// SA / SB = how many consecutive MFMAs take the same A / B operand (1 = each its own).
// RUN = how many consecutive MFMAs accumulate into the same registers (1 = the four
// accumulators in rotation).
template <int SA, int SB, int RUN = 1>
__global__ void __launch_bounds__(kThreads) mfma_probe_kernel(const bf16x8* __restrict__ data, float* out, int iters) {
    const int t = threadIdx.x;
    bf16x8 a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        a[i] = data[((blockIdx.x * 8 + i) % kSets) * kThreads + t];
        b[i] = data[((blockIdx.x * 8 + i + 3) % kSets) * kThreads + (t ^ 37)];
    }
    f32x16 o0 = {}, o1 = {}, o2 = {}, o3 = {};
    for (int it = 0; it < iters; it++) {
        if constexpr (RUN > 1) {
            // 32 MFMAs per trip of this form: every accumulator takes RUN in a row
#pragma unroll
            for (int r = 0; r < 8 / RUN; r++) {
#pragma unroll
                for (int i = 0; i < RUN; i++) o0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(RUN * r + i) & 7], b[(RUN * r + i) & 7], o0, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < RUN; i++) o1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(RUN * r + i + 1) & 7], b[(RUN * r + i + 3) & 7], o1, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < RUN; i++) o2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(RUN * r + i + 2) & 7], b[(RUN * r + i + 5) & 7], o2, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < RUN; i++) o3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(RUN * r + i + 3) & 7], b[(RUN * r + i + 7) & 7], o3, 0, 0, 0);
            }
        } else
#pragma unroll
        for (int i = 0; i < 8; i += 4) {
            o0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i / SA * SA], b[i / SB * SB], o0, 0, 0, 0);
            o1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(i + 1) / SA * SA], b[(i + 1) / SB * SB], o1, 0, 0, 0);
            o2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(i + 2) / SA * SA], b[(i + 2) / SB * SB], o2, 0, 0, 0);
            o3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(i + 3) / SA * SA], b[(i + 3) / SB * SB], o3, 0, 0, 0);
        }
        if ((it & 63) == 63) { // keep the accumulators finite
#pragma unroll
            for (int j = 0; j < 16; j++) {
                o0[j] *= 1e-3f; o1[j] *= 1e-3f; o2[j] *= 1e-3f; o3[j] *= 1e-3f;
            }
        }
    }
    float r = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) r += o0[i] + o1[i] + o2[i] + o3[i];
    out[blockIdx.x * kThreads + t] = r;
}

uint16_t to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

} // namespace

extern "C" int zdraw_hip_mfma_probe(int random_operands, int milliseconds, double* tflops) {
    if (!tflops || milliseconds <= 0) return ZDRAW_HIP_INVALID;
    *tflops = 0.0;
    const size_t n = (size_t)kSets * kThreads * 8;
    std::vector<uint16_t> host(n);
    uint64_t s = 0x9E3779B97F4A7C15ull; // xorshift + Box-Muller: N(0,1) operands
    auto uni = [&]() {
        s ^= s << 13; s ^= s >> 7; s ^= s << 17;
        return (double)((s >> 11) + 1) / 9007199254740993.0;
    };
    for (size_t i = 0; i < n; i++) {
        float v = 1.0f;
        if (random_operands) v = (float)(std::sqrt(-2.0 * std::log(uni())) * std::cos(6.283185307179586 * uni()));
        host[i] = to_bf16(v);
    }
    uint16_t* d = nullptr;
    float* out = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int rc = ZDRAW_HIP_ERR_HANDLE;
    do {
        if (hipMalloc(&d, n * 2) != hipSuccess || hipMalloc(&out, sizeof(float) * kBlocks * kThreads) != hipSuccess) break;
        if (hipMemcpy(d, host.data(), n * 2, hipMemcpyHostToDevice) != hipSuccess) break;
        if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) break;
        const int iters = 5000; // about 20 ms a launch
        const double flops = (double)kBlocks * (kThreads / 64) * iters * 8 * 32768.0;
        float total = 0.f, last = 0.f;
        bool ok = true;
        while (ok && total < (float)milliseconds) { // launches back to back; the last one is quoted
            ok = hipEventRecord(e0, nullptr) == hipSuccess;
            const bf16x8* src = reinterpret_cast<const bf16x8*>(d);
            switch (random_operands) { // 2..5: random operands, one side held over consecutive MFMAs
            case 2: mfma_probe_kernel<1, 2><<<kBlocks, kThreads>>>(src, out, iters); break;
            case 3: mfma_probe_kernel<1, 4><<<kBlocks, kThreads>>>(src, out, iters); break;
            case 4: mfma_probe_kernel<2, 1><<<kBlocks, kThreads>>>(src, out, iters); break;
            case 5: mfma_probe_kernel<1, 8><<<kBlocks, kThreads>>>(src, out, iters); break;
            case 6: mfma_probe_kernel<1, 1, 2><<<kBlocks, kThreads>>>(src, out, iters / 4); break;
            case 7: mfma_probe_kernel<1, 1, 8><<<kBlocks, kThreads>>>(src, out, iters / 4); break;
            default: mfma_probe_kernel<1, 1><<<kBlocks, kThreads>>>(src, out, iters); break;
            }
            ok = ok && hipGetLastError() == hipSuccess && hipEventRecord(e1, nullptr) == hipSuccess &&
                 hipEventSynchronize(e1) == hipSuccess && hipEventElapsedTime(&last, e0, e1) == hipSuccess;
            total += last;
        }
        if (!ok || last <= 0.f) break;
        *tflops = flops / (last * 1e-3) / 1e12;
        rc = ZDRAW_HIP_OK;
    } while (false);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (d) (void)hipFree(d);
    if (out) (void)hipFree(out);
    return rc;
}
