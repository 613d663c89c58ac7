// Probe, not part of the library: how much the FP8 matrix cores deliver at the socket power limit with each of the two
// MFMA shapes that run at 2048 FLOP per cycle and SIMD, v_mfma_f32_32x32x64_f8f6f4 and v_mfma_f32_16x16x128_f8f6f4.
// MFMAs only (operands held in registers, 256 accumulator registers per wavefront, one wavefront per SIMD, every CU),
// launched back to back for three seconds per shape; prints TFLOP/s and the socket power read from hwmon.
//   argument 0: random E4M3 operand bytes (exponent field kept small so that nothing overflows);  1: every byte 1.0
// build:  hipcc --offload-arch=gfx950 -O3 -std=c++17 -o mfma_shape_power mfma_shape_power.hip
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <chrono>
#include <thread>
#include <vector>
#include <fstream>
#include <string>
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
template <int SHAPE>
__global__ __launch_bounds__(256) void k(const int* __restrict__ src, float* out, int iters) {
    v8i a[4], b[4];
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 8; ++j) {
            a[i][j] = src[(threadIdx.x * 64 + i * 8 + j) & 16383];
            b[i][j] = src[(threadIdx.x * 64 + 32 + i * 8 + j + blockIdx.x) & 16383];
        }
    if constexpr (SHAPE == 0) {
        v16f acc[4][4];
        for (int i = 0; i < 4; ++i) for (int j = 0; j < 4; ++j) for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i], b[j], acc[i][j], 0, 0, 0, 0, 0, 0);
        }
        float s = 0; for (int i = 0; i < 4; ++i) for (int j = 0; j < 4; ++j) s += acc[i][j][0];
        out[blockIdx.x * 256 + threadIdx.x] = s;
    } else {
        v4f acc[8][8];
        v8i a2[8], b2[8];
        for (int i = 0; i < 8; ++i) for (int j = 0; j < 8; ++j) { a2[i][j] = src[(threadIdx.x * 128 + i * 8 + j + 7) & 16383]; b2[i][j] = src[(threadIdx.x * 128 + 64 + i * 8 + j + blockIdx.x * 3) & 16383]; }
        for (int i = 0; i < 8; ++i) for (int j = 0; j < 8; ++j) for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a2[i], b2[j], acc[i][j], 0, 0, 0, 0, 0, 0);
        }
        float s = 0; for (int i = 0; i < 8; ++i) for (int j = 0; j < 8; ++j) s += acc[i][j][0];
        out[blockIdx.x * 256 + threadIdx.x] = s;
    }
}
static double readf(const char* p) { std::ifstream f(p); double v = 0; f >> v; return v; }
static std::string find_hwmon() {
    for (int c = 0; c < 8; ++c) for (int h = 0; h < 10; ++h) {
        std::string p = "/sys/class/drm/card" + std::to_string(c) + "/device/hwmon/hwmon" + std::to_string(h) + "/power1_input";
        std::ifstream f(p); if (f.good()) return p;
    }
    return "";
}
int main(int argc, char** argv) {
    int* src; float* out;
    (void)hipMalloc(&src, 16384 * 4); (void)hipMalloc(&out, 256 * 256 * 4);
    std::vector<int> h(16384);
    int mode = argc > 1 ? atoi(argv[1]) : 0;   // 0 random, 1 constant
    srand(1);
    for (auto& v : h) v = mode ? 0x38383838 : ((rand() ^ (rand() << 16)) & 0xBFBFBFBF);
    (void)hipMemcpy(src, h.data(), 16384 * 4, hipMemcpyHostToDevice);
    std::string pw = find_hwmon();
    for (int shape = 0; shape < 2; ++shape) {
        const int iters = shape == 0 ? 20000 : 10000;   // per launch: 256 WGs x 4 waves x iters x 16 (or 64) MFMAs
        auto launch = [&]() { if (shape == 0) k<0><<<256, 256>>>(src, out, iters); else k<1><<<256, 256>>>(src, out, iters); };
        launch(); (void)hipDeviceSynchronize();
        auto t0 = std::chrono::steady_clock::now();
        int n = 0; double psum = 0; int pn = 0;
        while (std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() < 3.0) {
            launch(); (void)hipDeviceSynchronize(); ++n;
            if (!pw.empty() && std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() > 1.5) { psum += readf(pw.c_str()) / 1e6; ++pn; }
        }
        double dt = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
        double flop = 256.0 * 4 * iters * (shape == 0 ? 16 * 131072.0 : 64 * 65536.0) * n;
        printf("mode %d shape %s: %.0f TFLOP/s, %.0f W\n", mode, shape == 0 ? "32x32x64 " : "16x16x128", flop / dt / 1e12, pn ? psum / pn : 0.0);
        fflush(stdout);
    }
    return 0;
}
