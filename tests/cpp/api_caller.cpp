// A caller written against include/rocal_api_mi355x.h ALONE (compiled with -I include and nothing else of this repository),
// as a program written against rocAL's own headers would be: rocalCreate -> source -> rocalCropResizeFixed ->
// rocalColorTwistFixed -> rocalCropMirrorNormalize -> rocalVerify -> rocalRun twice. The first batch is read as a program
// written for rocAL reads it (unit_tests.cpp:1109-1171): rocalGetOutputTensors(ctx)->at(0)->copy_data(...), dims, strides,
// copy_roi; for the second the output tensor is bound to memory the caller owns (set_mem_handle) and read from there, and
// rocalCopyToOutput must give the same bytes. Reads <dir>/meta.txt ("n H W" and one "w h" per sample) and <dir>/input.bin,
// writes out_b<k>.bin and roi_b<k>.txt per batch and prints the timers. ROCAL_BILINEAR_EDGE in the environment selects the
// edge rule of the resize.
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
    const size_t bytes = out->data_size();
    if (bytes != (size_t)n * 3 * 56 * 56 * 2 || out->data_type() != ROCAL_FP16 || out->layout() != ROCAL_NCHW || out->num_of_dims() != 4 ||
        out->batch_size() != n || out->data_type_size() != 2 || out->backend() != ROCAL_GPU)
        return 11;
    const std::vector<size_t> dims = out->dims(), strides = out->strides(), shape = out->shape();
    if (dims != std::vector<size_t>{n, 3, 56, 56} || strides != std::vector<size_t>{3 * 56 * 56 * 2, 56 * 56 * 2, 56 * 2, 2} ||
        shape != std::vector<size_t>{56, 56})
        return 12;
    if (rocalVerify(ctx) != ROCAL_OK) {
        std::cerr << "verify failed: " << rocalGetErrorMessage(ctx) << std::endl;
        return 7;
    }
    std::cout << "intermediates_elided " << ((rocalTensorBuffer(mid) == nullptr && rocalTensorBuffer(col) == nullptr) ? 1 : 0) << std::endl;
    void *mine = nullptr;  // the caller's own tensor (what a framework would hand over through its data pointer)
    if (hipMalloc(&mine, bytes) != hipSuccess || hipMemset(mine, 0, bytes) != hipSuccess) return 3;
    for (int b = 0; b < 2; b++) {
        if (b == 1) {
            out->set_mem_handle(mine);
            if (rocalTensorBuffer(out) != mine) return 10;
        }
        if (rocalDeviceSourceFeed(ctx, src, dev, rw.data(), rh.data()) != ROCAL_OK || rocalRun(ctx) != ROCAL_OK) {
            std::cerr << "run failed: " << rocalGetErrorMessage(ctx) << std::endl;
            return 8;
        }
        RocalTensorList outputs = rocalGetOutputTensors(ctx);  // waits for the batch
        if (!outputs || outputs->size() != 1 || outputs->at(0) != out) return 13;
        std::vector<char> o(bytes), o2(bytes);
        if (b == 0) {
            if (outputs->at(0)->copy_data(o.data(), ROCAL_MEMCPY_HOST) != 0) return 14;
        } else if (hipMemcpy(o.data(), mine, bytes, hipMemcpyDeviceToHost) != hipSuccess) {
            return 3;
        }
        if (rocalCopyToOutput(ctx, reinterpret_cast<unsigned char *>(o2.data()), bytes) != ROCAL_OK || o != o2) return 15;
        if (rocalCopyToOutput(ctx, reinterpret_cast<unsigned char *>(o2.data()), bytes - 1) == ROCAL_OK) return 16;  // wrong size is an error
        // a window of every sample's first plane: rows 8..15, columns 4..23
        std::vector<unsigned short> win((size_t)n * 8 * 20);
        if (outputs->at(0)->copy_data(win.data(), 4, 8, 20, 8) != 0) return 17;
        const unsigned short *full = reinterpret_cast<const unsigned short *>(o.data());
        for (unsigned i = 0; i < n; i++)
            for (unsigned y = 0; y < 8; y++)
                for (unsigned x = 0; x < 20; x++)
                    if (win[((size_t)i * 8 + y) * 20 + x] != full[(size_t)i * 3 * 56 * 56 + (y + 8) * 56 + x + 4]) return 18;
        std::ofstream(dir + "/out_b" + std::to_string(b) + ".bin", std::ios::binary).write(o.data(), bytes);
        std::vector<unsigned> roi(4 * n);
        if (outputs->at(0)->get_roi_dims_size() != 2 || outputs->at(0)->roi_type() != RocalROICordsType::ROCAL_XYWH) return 19;
        outputs->at(0)->copy_roi(roi.data());
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
