// Probe, not part of the library: the same measurement as mfma_shape_power.hip for the bf16 shapes
// v_mfma_f32_32x32x16_bf16 and v_mfma_f32_16x16x32_bf16 (1024 FLOP per cycle and SIMD each).
// build:  hipcc --offload-arch=gfx950 -O3 -std=c++17 -o mfma_shape_power_bf16 mfma_shape_power_bf16.hip
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <chrono>
#include <vector>
#include <fstream>
#include <string>
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
template <int SHAPE>
__global__ __launch_bounds__(256) void k(const v8bf* __restrict__ src, float* out, int iters) {
    if constexpr (SHAPE == 0) {
        v8bf a[4], b[4];
        for (int i = 0; i < 4; ++i) { a[i] = src[(threadIdx.x * 8 + i) & 4095]; b[i] = src[(threadIdx.x * 8 + 4 + i + blockIdx.x) & 4095]; }
        v16f acc[4][4];
        for (int i = 0; i < 4; ++i) for (int j = 0; j < 4; ++j) for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        float s = 0; for (int i = 0; i < 4; ++i) for (int j = 0; j < 4; ++j) s += acc[i][j][0];
        out[blockIdx.x * 256 + threadIdx.x] = s;
    } else {
        v8bf a[8], b[8];
        for (int i = 0; i < 8; ++i) { a[i] = src[(threadIdx.x * 16 + i) & 4095]; b[i] = src[(threadIdx.x * 16 + 8 + i + blockIdx.x) & 4095]; }
        v4f acc[8][8];
        for (int i = 0; i < 8; ++i) for (int j = 0; j < 8; ++j) for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
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
    v8bf* src; float* out;
    (void)hipMalloc(&src, 4096 * 16); (void)hipMalloc(&out, 256 * 256 * 4);
    std::vector<unsigned short> h(4096 * 8);
    int mode = argc > 1 ? atoi(argv[1]) : 0;
    srand(1);
    for (auto& v : h) { unsigned short r = rand() & 0xffff; v = mode ? 0x3f80 : (unsigned short)((r & 0x80ff) | 0x3f00 | (r & 0x0080)); }   // random sign/mantissa, exponent near 1
    (void)hipMemcpy(src, h.data(), 4096 * 16, hipMemcpyHostToDevice);
    std::string pw = find_hwmon();
    for (int shape = 0; shape < 2; ++shape) {
        const int iters = shape == 0 ? 40000 : 20000;
        auto launch = [&]() { if (shape == 0) k<0><<<256, 256>>>(src, out, iters); else k<1><<<256, 256>>>(src, out, iters); };
        launch(); (void)hipDeviceSynchronize();
        auto t0 = std::chrono::steady_clock::now();
        int n = 0; double psum = 0; int pn = 0;
        while (std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() < 3.0) {
            launch(); (void)hipDeviceSynchronize(); ++n;
            if (!pw.empty() && std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() > 1.5) { psum += readf(pw.c_str()) / 1e6; ++pn; }
        }
        double dt = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
        double flop = 256.0 * 4 * iters * (shape == 0 ? 16 * 32768.0 : 64 * 16384.0) * n;
        printf("mode %d shape %s: %.0f TFLOP/s, %.0f W\n", mode, shape == 0 ? "32x32x16 bf16" : "16x16x32 bf16", flop / dt / 1e12, pn ? psum / pn : 0.0);
        fflush(stdout);
    }
    return 0;
}
