// A caller written against include/rocal_api_mi355x.h ALONE (compiled with -I include and nothing else of this repository),
// as a program written against rocAL's own headers would be: rocalCreate -> source -> rocalCropResizeFixed ->
// rocalColorTwistFixed -> rocalCropMirrorNormalize -> rocalVerify -> rocalRun twice, with the output tensor bound to memory
// the caller owns. Reads <dir>/meta.txt ("n H W" and one "w h" per sample) and <dir>/input.bin, writes out_b<k>.bin and
// roi_b<k>.txt per batch and prints the timers.
#include <hip/hip_runtime.h>

#include <fstream>
#include <iostream>
#include <string>
#include <vector>

#include "rocal_api_mi355x.h"

int main(int argc, char **argv) {
    if (argc < 2) return 2;
    const std::string dir = argv[1];
    unsigned n, H, W;
    std::vector<unsigned> rw, rh;
    {
        std::ifstream meta(dir + "/meta.txt");
        if (!(meta >> n >> H >> W)) return 2;
        rw.resize(n);
        rh.resize(n);
        for (unsigned i = 0; i < n; i++) meta >> rw[i] >> rh[i];
    }
    std::vector<unsigned char> host((size_t)n * H * W * 3);
    {
        std::ifstream in(dir + "/input.bin", std::ios::binary);
        in.read(reinterpret_cast<char *>(host.data()), host.size());
        if ((size_t)in.gcount() != host.size()) return 2;
    }
    rocalSetSeed(77);
    RocalContext ctx = rocalCreate(n, ROCAL_PROCESS_GPU, 0);
    if (!ctx) return 4;
    void *dev = nullptr;
    if (hipMalloc(&dev, host.size() + 64) != hipSuccess || hipMemcpy(dev, host.data(), host.size(), hipMemcpyHostToDevice) != hipSuccess) return 3;
    const int coin_v[2] = {0, 1};
    const double coin_f[2] = {0.5, 0.5};
    RocalIntParam coin = rocalCreateIntRand(coin_v, coin_f, 2);
    std::vector<float> mean{123.675f, 116.28f, 103.53f}, stdv{58.395f, 57.12f, 57.375f};
    RocalTensor src = rocalDeviceSource(ctx, W, H, false);
    RocalTensor mid = rocalCropResizeFixed(ctx, src, 64, 64, false, 0.5f, 1.2f, 0.3f, 0.7f);
    RocalTensor col = rocalColorTwistFixed(ctx, mid, 1.2f, 8.0f, 40.0f, 1.3f, false);
    RocalTensor out = rocalCropMirrorNormalize(ctx, col, 56, 56, 0.5f, 0.5f, mean, stdv, true, coin, ROCAL_NCHW, ROCAL_FP16);
    if (!src || !mid || !col || !out) {
        std::cerr << "node creation failed: " << rocalGetErrorMessage(ctx) << std::endl;
        return 6;
    }
    // the caller's own tensor (what a framework would hand over through its data pointer)
    const size_t bytes = rocalTensorDataSize(out);
    void *mine = nullptr;
    if (hipMalloc(&mine, bytes) != hipSuccess || hipMemset(mine, 0, bytes) != hipSuccess) return 3;
    if (rocalTensorSetBuffer(ctx, out, mine) != ROCAL_OK) return 9;
    if (rocalVerify(ctx) != ROCAL_OK) {
        std::cerr << "verify failed: " << rocalGetErrorMessage(ctx) << std::endl;
        return 7;
    }
    if (rocalTensorBuffer(out) != mine) return 10;
    std::cout << "intermediates_elided " << ((rocalTensorBuffer(mid) == nullptr && rocalTensorBuffer(col) == nullptr) ? 1 : 0) << std::endl;
    for (int b = 0; b < 2; b++) {
        if (rocalDeviceSourceFeed(ctx, src, dev, rw.data(), rh.data()) != ROCAL_OK || rocalRun(ctx) != ROCAL_OK) {
            std::cerr << "run failed: " << rocalGetErrorMessage(ctx) << std::endl;
            return 8;
        }
        std::vector<char> o(bytes);
        if (hipMemcpy(o.data(), mine, bytes, hipMemcpyDeviceToHost) != hipSuccess) return 3;
        std::ofstream(dir + "/out_b" + std::to_string(b) + ".bin", std::ios::binary).write(o.data(), bytes);
        const unsigned *roi = rocalTensorRoi(out);
        std::ofstream r(dir + "/roi_b" + std::to_string(b) + ".txt");
        for (unsigned i = 0; i < n; i++) r << roi[4 * i] << " " << roi[4 * i + 1] << " " << roi[4 * i + 2] << " " << roi[4 * i + 3] << "\n";
    }
    const long long unsigned upd = rocalGetParameterUpdateTime(ctx);
    const TimingInfo t = rocalGetTimingInfo(ctx);
    std::cout << "timing_us update " << upd << " process " << t.process_time << " transfer " << t.transfer_time << " load " << t.load_time << std::endl;
    const TimingInfo again = rocalGetTimingInfo(ctx);  // reading resets
    std::cout << "timing_after_reset " << again.process_time << std::endl;
    rocalRelease(ctx);
    (void)hipFree(dev);
    (void)hipFree(mine);
    std::cout << "ok" << std::endl;
    return 0;
}
