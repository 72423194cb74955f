// Test driver of the host layer, run by the test-suite as a child process.
//   host_check params <seed>            prints, as JSON, what the parameter system produces (no GPU needed)
//   host_check ring                      the shut-down protocol of the loader ring on a ring in host memory (no GPU needed)
//   host_check pipeline <scenario> <dir> builds a pipeline through the rocal* API, feeds <dir>/input.bin
//                                        twice and writes every output batch + ROI to <dir> (needs the GPU)
#include <hip/hip_runtime_api.h>

#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <sstream>
#include <string>
#include <thread>
#include <vector>

#include "rocal_host.h"
#include "nodes.h"  // internals exercised directly: ParameterFactory, ParameterVX, the parameter classes

namespace {

template <typename T>
std::string arr(const std::vector<T> &v) {
    std::ostringstream s;
    s.precision(9);
    s << "[";
    for (size_t i = 0; i < v.size(); i++) s << (i ? "," : "") << v[i];
    s << "]";
    return s.str();
}

int run_params(unsigned seed) {
    auto *pf = ParameterFactory::instance();
    pf->set_seed(seed);
    std::ostringstream js;
    js << "{";
    // 1. seed sequence: the first four values are consumed here
    std::vector<long long> seeds;
    for (int i = 0; i < 4; i++) seeds.push_back(pf->get_seed_from_seedsequence());
    js << "\"seeds\":" << arr(seeds);
    // 2. user-created uniform / custom parameters (seeds 4,5,6)
    auto *uf = static_cast<FloatParam *>(rocalCreateFloatUniformRand(0.08f, 1.0f));
    auto *ui = static_cast<IntParam *>(rocalCreateIntUniformRand(0, 1));
    const int cv[4] = {10, 20, 30, 40};
    const double cf[4] = {0.1, 0.4, 0.3, 0.2};
    auto *ci = static_cast<IntParam *>(rocalCreateIntRand(cv, cf, 4));
    std::vector<float> vf{rocalGetFloatValue(uf)};
    std::vector<int> vi{rocalGetIntValue(ui)}, vc{rocalGetIntValue(ci)};
    for (int k = 0; k < 12; k++) {
        pf->renew_parameters();
        vf.push_back(rocalGetFloatValue(uf));
        vi.push_back(rocalGetIntValue(ui));
        vc.push_back(rocalGetIntValue(ci));
    }
    js << ",\"uniform_f\":" << arr(vf) << ",\"uniform_i\":" << arr(vi) << ",\"custom_i\":" << arr(vc);
    // 3. a batch-sized mirror array on a node default (seeded with the factory seed itself)
    ParameterVX<int> mirror(0, 1);
    mirror.create_array(8);
    std::vector<int> mv;
    for (int b = 0; b < 3; b++) {
        pf->renew_parameters();
        mirror.update_array();
        mv.insert(mv.end(), mirror.values().begin(), mirror.values().end());
    }
    js << ",\"mirror_default\":" << arr(mv);
    // 4. random-resized-crop windows: user parameters first (seeds 7..10), then the crop object, whose own
    //    defaults take seeds 11..14 before being replaced
    const unsigned n = 6;
    std::vector<Roi2DCords> roi(n);
    const unsigned ws[n] = {640, 240, 333, 500, 64, 1000}, hs[n] = {480, 240, 500, 333, 48, 200};
    for (unsigned i = 0; i < n; i++) roi[i].xywh = {0, 0, ws[i], hs[i]};
    auto *area = static_cast<FloatParam *>(rocalCreateFloatUniformRand(0.08f, 1.0f));
    auto *aspect = static_cast<FloatParam *>(rocalCreateFloatUniformRand(0.75f, 1.333f));
    auto *xd = static_cast<FloatParam *>(rocalCreateFloatUniformRand(0.0f, 1.0f));
    auto *yd = static_cast<FloatParam *>(rocalCreateFloatUniformRand(0.0f, 1.0f));
    RocalRandomCropParam rrc(n);
    rrc.set_area_factor(core(area));
    rrc.set_aspect_ratio(core(aspect));
    rrc.set_x_drift_factor(core(xd));
    rrc.set_y_drift_factor(core(yd));
    rrc.create_array();
    std::vector<uint32_t> win;
    for (int b = 0; b < 3; b++) {
        pf->renew_parameters();
        rrc.set_image_dimensions(roi.data());
        rrc.update_array();
        auto w = rrc.xywh();
        win.insert(win.end(), w.begin(), w.end());
    }
    js << ",\"rrc_windows\":" << arr(win);
    // 5. factor crops (seeds 15..18 for the user parameters)
    auto *hf = static_cast<FloatParam *>(rocalCreateFloatUniformRand(0.55f, 0.95f));
    auto *wf = static_cast<FloatParam *>(rocalCreateFloatUniformRand(0.55f, 0.95f));
    auto *fx = static_cast<FloatParam *>(rocalCreateFloatUniformRand(0.01f, 0.99f));
    auto *fy = static_cast<FloatParam *>(rocalCreateFloatUniformRand(0.01f, 0.99f));
    RocalCropParam fc(n);
    fc.set_crop_height_factor(core(hf));
    fc.set_crop_width_factor(core(wf));
    fc.set_x_drift_factor(core(fx));
    fc.set_y_drift_factor(core(fy));
    fc.set_random();
    fc.create_array();
    win.clear();
    for (int b = 0; b < 2; b++) {
        pf->renew_parameters();
        fc.set_image_dimensions(roi.data());
        fc.update_array();
        auto w = fc.xywh();
        win.insert(win.end(), w.begin(), w.end());
    }
    js << ",\"factor_windows\":" << arr(win);
    // 6. anchored fixed crops and the resize size policy
    RocalCropParam fixed(n);
    fixed.crop_w = 224;
    fixed.crop_h = 200;
    fixed.set_fixed_crop(0.5f, 0.5f);
    fixed.set_image_dimensions(roi.data());
    fixed.update_array();
    js << ",\"fixed_windows\":" << arr(fixed.xywh());
    struct Probe : ResizeFamilyNode {
        using ResizeFamilyNode::adjust_out_roi_size;
    };
    std::vector<unsigned> sizes;
    const unsigned cases[][5] = {{640, 480, 256, 0, 0}, {640, 480, 0, 256, 0}, {640, 480, 300, 200, 1}, {640, 480, 256, 256, 2}, {480, 640, 256, 256, 2},
                                 {640, 480, 256, 256, 3}, {333, 500, 0, 300, 3}, {333, 500, 300, 0, 2}, {1000, 200, 256, 256, 2}};
    for (auto &c : cases)
        for (unsigned mw : {0u, 400u}) {
            unsigned w = c[2], h = c[3];
            Probe::adjust_out_roi_size(c[0], c[1], w, h, (RocalResizeScalingMode)c[4], mw, mw ? 300 : 0);
            sizes.push_back(w);
            sizes.push_back(h);
        }
    js << ",\"resize_sizes\":" << arr(sizes) << "}";
    std::cout << js.str() << std::endl;
    return 0;
}

#define HIPCHK(x)                                                            \
    if ((x) != hipSuccess) {                                                 \
        std::cerr << "HIP call failed: " #x << std::endl;                   \
        return 3;                                                            \
    }

int run_pipeline(const std::string &scenario, const std::string &dir) {
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
    HIPCHK(hipMalloc(&dev, host.size() + 64));
    HIPCHK(hipMemcpy(dev, host.data(), host.size(), hipMemcpyHostToDevice));
    RocalTensor src = rocalDeviceSource(ctx, W, H, false);
    std::vector<float> mean{123.675f, 116.28f, 103.53f}, stdv{58.395f, 57.12f, 57.375f};
    std::vector<RocalTensor> outs;
    RocalTensor mid = nullptr, mid2 = nullptr;
    // A fair coin for the mirror flags, created first so that it takes the first seed of the sequence.
    // (rocalCreateIntUniformRand(0, 1) truncates to 0 for every draw but one in 2^32, as in the reference.)
    const int coin_v[2] = {0, 1};
    const double coin_f[2] = {0.5, 0.5};
    RocalIntParam coin = rocalCreateIntRand(coin_v, coin_f, 2);
    // bounding boxes (scenarios meta_*): <dir>/boxes.txt holds, per sample, a count and then "l t r b label" lines
    const bool with_boxes = scenario.rfind("meta_", 0) == 0;
    std::vector<unsigned> box_counts(n, 0);
    std::vector<float> box_ltrb;
    std::vector<int> box_labels;
    if (with_boxes) {
        std::ifstream bf(dir + "/boxes.txt");
        for (unsigned i = 0; i < n; i++) {
            if (!(bf >> box_counts[i])) return 2;
            for (unsigned j = 0; j < box_counts[i]; j++) {
                float l, t, r, b;
                int label;
                bf >> l >> t >> r >> b >> label;
                box_ltrb.insert(box_ltrb.end(), {l, t, r, b});
                box_labels.push_back(label);
            }
        }
        if (rocalEnableBoundingBoxes(ctx) != ROCAL_OK) return 11;
    }
    if (scenario == "meta_cmn") {
        outs.push_back(rocalCropMirrorNormalize(ctx, src, 40, 48, 0.5f, 0.5f, mean, stdv, true, coin, ROCAL_NCHW, ROCAL_FP32));
    } else if (scenario == "meta_resize_flip") {
        RocalTensor a = rocalResize(ctx, src, 40, 32, false);
        outs.push_back(rocalFlipFixed(ctx, a, 1, 1, true));
    } else if (scenario == "meta_rotate") {
        outs.push_back(rocalRotateFixed(ctx, src, 30.0f, true));
    } else if (scenario == "meta_rcm") {
        outs.push_back(rocalResizeCropMirrorFixed(ctx, src, 36, 28, true, 40, 50, rocalCreateIntParameter(1)));
    } else if (scenario == "meta_crop_then_rmn") {
        RocalTensor a = rocalCropFixed(ctx, src, 30, 20, 1, false, 5, 7, 0);
        outs.push_back(rocalResizeMirrorNormalize(ctx, a, 60, 40, mean, stdv, true, ROCAL_SCALING_MODE_STRETCH, {}, 0, 0, ROCAL_LINEAR_INTERPOLATION,
                                                  rocalCreateIntParameter(1), ROCAL_NCHW, ROCAL_FP16));
    } else if (scenario == "meta_crop_resize") {
        outs.push_back(rocalCropResizeFixed(ctx, src, 64, 64, true, 0.5f, 1.2f, 0.3f, 0.7f));
    } else if (scenario == "cmn") {
        RocalIntParam mirror = coin;
        outs.push_back(rocalCropMirrorNormalize(ctx, src, 40, 48, 0.5f, 0.5f, mean, stdv, true, mirror, ROCAL_NCHW, ROCAL_FP32));
    } else if (scenario == "rrc_cmn") {
        mid = rocalCropResizeFixed(ctx, src, 64, 64, false, 0.5f, 1.2f, 0.3f, 0.7f);
        RocalIntParam mirror = coin;
        outs.push_back(rocalCropMirrorNormalize(ctx, mid, 56, 56, 0.5f, 0.5f, mean, stdv, true, mirror, ROCAL_NCHW, ROCAL_FP16));
    } else if (scenario == "rrc_twist_cmn" || scenario == "rrc_contrast_cmn" || scenario == "rrc_exposure_cmn") {
        // three nodes, two virtual tensors between them: one kernel
        mid = rocalCropResizeFixed(ctx, src, 64, 64, false, 0.5f, 1.2f, 0.3f, 0.7f);
        RocalTensor col = scenario == "rrc_twist_cmn"      ? rocalColorTwistFixed(ctx, mid, 1.2f, 8.0f, 40.0f, 1.3f, false)
                          : scenario == "rrc_contrast_cmn" ? rocalContrastFixed(ctx, mid, 1.4f, 100.0f, false)
                                                           : rocalExposureFixed(ctx, mid, 0.4f, false);
        RocalIntParam mirror = coin;
        outs.push_back(rocalCropMirrorNormalize(ctx, col, 56, 56, 0.5f, 0.5f, mean, stdv, true, mirror, ROCAL_NCHW, ROCAL_FP16));
        mid2 = col;
    } else if (scenario == "chain") {
        RocalTensor a = rocalResize(ctx, src, 40, 32, false);
        RocalTensor b = rocalColorTwistFixed(ctx, a, 1.1f, 5.0f, 30.0f, 1.2f, true);
        outs.push_back(b);
        outs.push_back(rocalFlipFixed(ctx, b, 1, 0, true));
    } else if (scenario == "rotate") {
        outs.push_back(rocalRotateFixed(ctx, src, 30.0f, true));
    } else if (scenario == "warp") {
        outs.push_back(rocalWarpAffineFixed(ctx, src, 1.05f, 0.1f, -0.08f, 0.95f, 3.0f, -2.0f, true, 48, 56));
    } else if (scenario == "rmn") {
        RocalIntParam mirror = rocalCreateIntParameter(1);
        outs.push_back(rocalResizeMirrorNormalize(ctx, src, 0, 0, mean, stdv, true, ROCAL_SCALING_MODE_STRETCH, {96, 96}, 48, 0, ROCAL_LINEAR_INTERPOLATION, mirror,
                                                  ROCAL_NCHW, ROCAL_FP16));
    } else if (scenario == "crops") {
        outs.push_back(rocalCropCenterFixed(ctx, src, 32, 24, 1, true));
        outs.push_back(rocalCropFixed(ctx, src, 30, 20, 1, true, 5, 7, 0));
        outs.push_back(rocalResizeCropMirrorFixed(ctx, src, 36, 28, true, 40, 50, rocalCreateIntParameter(1)));
        outs.push_back(rocalBrightnessFixed(ctx, src, 1.2f, 10.0f, true));
        outs.push_back(rocalContrastFixed(ctx, src, 1.3f, 70.0f, true));
    } else if (scenario == "points") {
        outs.push_back(rocalGammaFixed(ctx, src, 2.2f, true));
        outs.push_back(rocalExposureFixed(ctx, src, 0.6f, true));
        outs.push_back(rocalColorTempFixed(ctx, src, 40, true));
        RocalTensor bright = rocalBrightnessFixed(ctx, src, 0.5f, 100.0f, true);
        outs.push_back(bright);
        outs.push_back(rocalBlendFixed(ctx, src, bright, 0.3f, true));
        // a second input of another shape is refused when the graph is built, a missing one at once
        if (rocalBlendFixed(ctx, src, nullptr, 0.3f, true) != nullptr) return 14;
    } else if (scenario == "second_reader") {
        // the resized tensor feeds CropMirrorNormalize AND is the second input of a Blend node: it has two readers, so
        // resize -> CropMirrorNormalize must not be fused (the tensor has to exist for the Blend)
        mid = rocalResize(ctx, src, 40, 32, false);
        outs.push_back(rocalCropMirrorNormalize(ctx, mid, 32, 40, 0.5f, 0.5f, mean, stdv, true, rocalCreateIntParameter(0), ROCAL_NCHW, ROCAL_FP32));
        RocalTensor other = rocalResize(ctx, src, 40, 32, true, ROCAL_SCALING_MODE_STRETCH, {}, 0, 0, ROCAL_NEAREST_NEIGHBOR_INTERPOLATION);
        outs.push_back(other);
        outs.push_back(rocalBlendFixed(ctx, other, mid, 0.25f, true));
    } else if (scenario == "normalize_transpose") {
        std::vector<unsigned> hw{0, 1}, hwc{0, 1, 2};
        std::vector<float> none, m3{10.0f, 20.0f, 30.0f}, s3{2.0f, 4.0f, 8.0f};
        outs.push_back(rocalNormalize(ctx, src, hw, none, none, true));                       // per-channel statistics of every window, fp32
        outs.push_back(rocalNormalize(ctx, src, hwc, m3, s3, true, 3.0f, 1.0f, ROCAL_FP16));  // given statistics, scale and shift
        outs.push_back(rocalTranspose(ctx, src, {1, 0, 2}, true, ROCAL_NHWC));                // [N, W, H, C]
        outs.push_back(rocalTranspose(ctx, src, {2, 0, 1}, true, ROCAL_NCHW));                // [N, C, H, W]
    } else if (scenario == "ref_cases") {
        // The fixed-parameter cases of the reference's own unit tests (tests/cpp_api/unit_tests/unit_tests.cpp:605-624,730-735,
        // 745-856), all on one source, with the parameters written there.
        std::vector<float> mean128{128, 128, 128}, std12{1.2f, 1.2f, 1.2f};
        RocalIntParam m1 = rocalCreateIntParameter(1);
        outs.push_back(rocalResize(ctx, src, 400, 400, true, ROCAL_SCALING_MODE_DEFAULT, {}, 0, 0, ROCAL_LINEAR_INTERPOLATION));      // case 0
        outs.push_back(rocalResize(ctx, src, 400, 400, true, ROCAL_SCALING_MODE_DEFAULT, {}, 0, 0, ROCAL_TRIANGULAR_INTERPOLATION));  // case 0, triangular
        outs.push_back(rocalCropMirrorNormalize(ctx, src, 224, 224, 0, 0, mean128, std12, true, m1));                                 // case 25
        outs.push_back(rocalCropMirrorNormalize(ctx, src, 224, 224, 0.5f, 0.5f, mean128, std12, true, m1));                           // case 55
        outs.push_back(rocalCropResizeFixed(ctx, src, 224, 224, true, 0.25f, 1.2f, 0.6f, 0.4f));                                      // case 30
        RocalTensor rot = rocalRotateFixed(ctx, src, 45, true);                                                                       // case 31
        outs.push_back(rot);
        outs.push_back(rocalBrightnessFixed(ctx, src, 1.90f, 20, true));                                                              // case 32
        outs.push_back(rocalGammaFixed(ctx, src, 0.5f, true));                                                                        // case 33
        outs.push_back(rocalContrastFixed(ctx, src, 30, 80, true));                                                                   // case 34
        outs.push_back(rocalBlendFixed(ctx, src, rot, 0.5f, true));                                                                   // case 36
        outs.push_back(rocalWarpAffineFixed(ctx, src, 1, 1, 0.5f, 0.5f, 7, 7, true));                                                 // case 37
        outs.push_back(rocalColorTempFixed(ctx, src, 70, true));                                                                      // case 43
        outs.push_back(rocalExposureFixed(ctx, src, 1, true));                                                                        // case 46
        outs.push_back(rocalFlipFixed(ctx, src, 1, 0, true));                                                                         // case 47
        outs.push_back(rocalHueFixed(ctx, src, 150, true));                                                                           // case 48
        outs.push_back(rocalSaturationFixed(ctx, src, 0.3f, true));                                                                   // case 49
        outs.push_back(rocalColorTwistFixed(ctx, src, 0.2f, 10.0f, 100.0f, 0.25f, true));                                             // case 50
        outs.push_back(rocalCropFixed(ctx, src, 224, 224, 1, true, 0, 0, 0));                                                         // case 51
        outs.push_back(rocalCropCenterFixed(ctx, src, 224, 224, 2, true));                                                            // case 52
        outs.push_back(rocalResizeCropMirrorFixed(ctx, src, 400, 400, true, 200, 200, m1));                                           // case 53
        outs.push_back(rocalResizeMirrorNormalize(ctx, src, 400, 400, mean128, std12, true, ROCAL_SCALING_MODE_DEFAULT, {}, 0, 0,
                                                  ROCAL_LINEAR_INTERPOLATION, m1));                                                   // case 56
    } else if (scenario == "to_tensor") {
        outs.push_back(rocalResize(ctx, src, 40, 32, true));
    } else if (scenario == "errors") {
        // every line must fail the way the reference's API does: null tensor / runtime error + a message
        std::vector<float> zero_std{58.0f, 0.0f, 57.0f};
        int bad = 0;
        if (rocalCreate(n, ROCAL_PROCESS_CPU, 0) != nullptr) bad |= 1;
        if (rocalCropMirrorNormalize(ctx, src, 0, 10, 0.5f, 0.5f, mean, stdv, true) != nullptr) bad |= 2;
        if (rocalResize(ctx, src, 0, 0, true) != nullptr) bad |= 4;
        if (rocalResize(ctx, src, 10, 10, true, ROCAL_SCALING_MODE_STRETCH, {}, 5, 0) != nullptr) bad |= 8;
        if (rocalCropMirrorNormalize(ctx, nullptr, 10, 10, 0.5f, 0.5f, mean, stdv, true) != nullptr) bad |= 16;
        RocalTensor t = rocalCropMirrorNormalize(ctx, src, 10, 10, 0.5f, 0.5f, mean, zero_std, true);
        if (t == nullptr) bad |= 32;  // creation succeeds; the zero std is found in create_node()
        if (rocalVerify(ctx) != ROCAL_RUNTIME_ERROR) bad |= 64;
        if (std::string(rocalGetErrorMessage(ctx)).find("Standard deviation value cannot be 0") == std::string::npos) bad |= 128;
        if (rocalRun(nullptr) != ROCAL_CONTEXT_INVALID) bad |= 256;
        if (rocalUpdateFloatParameter(1.0f, rocalCreateFloatUniformRand(0, 1)) != ROCAL_INVALID_PARAMETER_TYPE) bad |= 512;
        std::cout << "errors_bad_mask " << bad << std::endl;
        return bad ? 5 : 0;
    } else {
        return 2;
    }
    for (auto t : outs)
        if (!t) {
            std::cerr << "node creation failed: " << rocalGetErrorMessage(ctx) << std::endl;
            return 6;
        }
    if (rocalVerify(ctx) != ROCAL_OK) {
        std::cerr << "verify failed: " << rocalGetErrorMessage(ctx) << std::endl;
        return 7;
    }
    if (mid) std::cout << "intermediate_elided " << (rocalTensorBuffer(mid) == nullptr ? 1 : 0) << std::endl;
    if (mid2) std::cout << "second_intermediate_elided " << (rocalTensorBuffer(mid2) == nullptr ? 1 : 0) << std::endl;
    for (int b = 0; b < 2; b++) {
        if (with_boxes && rocalSetBoundingBoxes(ctx, box_counts.data(), box_ltrb.data(), box_labels.data()) != ROCAL_OK) return 12;
        if (rocalDeviceSourceFeed(ctx, src, dev, rw.data(), rh.data()) != ROCAL_OK || rocalRun(ctx) != ROCAL_OK) {
            std::cerr << "run failed: " << rocalGetErrorMessage(ctx) << std::endl;
            return 8;
        }
        if (with_boxes) {
            std::vector<unsigned> counts(n);
            const unsigned total = rocalGetBoundingBoxCount(ctx, counts.data());
            std::vector<float> ltrb(4 * (size_t)total);
            std::vector<int> labels(total);
            if (rocalGetBoundingBoxCords(ctx, ltrb.data()) != ROCAL_OK || rocalGetBoundingBoxLabel(ctx, labels.data()) != ROCAL_OK) return 13;
            std::ofstream f(dir + "/boxes_b" + std::to_string(b) + ".txt");
            f.precision(9);
            size_t k = 0;
            for (unsigned i = 0; i < n; i++) {
                f << counts[i] << "\n";
                for (unsigned j = 0; j < counts[i]; j++, k++)
                    f << ltrb[4 * k] << " " << ltrb[4 * k + 1] << " " << ltrb[4 * k + 2] << " " << ltrb[4 * k + 3] << " " << labels[k] << "\n";
            }
        }
        for (size_t k = 0; k < outs.size(); k++) {
            const size_t bytes = rocalTensorDataSize(outs[k]);
            std::vector<char> out(bytes);
            HIPCHK(hipMemcpy(out.data(), rocalTensorBuffer(outs[k]), bytes, hipMemcpyDeviceToHost));
            std::ofstream f(dir + "/out" + std::to_string(k) + "_b" + std::to_string(b) + ".bin", std::ios::binary);
            f.write(out.data(), bytes);
            const unsigned *roi = rocalTensorRoi(outs[k]);
            std::ofstream r(dir + "/roi" + std::to_string(k) + "_b" + std::to_string(b) + ".txt");
            for (unsigned i = 0; i < n; i++) r << roi[4 * i] << " " << roi[4 * i + 1] << " " << roi[4 * i + 2] << " " << roi[4 * i + 3] << "\n";
        }
    }
    if (scenario == "to_tensor") {
        // the u8 output (32 rows of 40) to a planar fp16 tensor with reversed channels, then its top-left
        // 24x32 corner to an interleaved fp32 tensor; a host destination must be refused
        void *tt = nullptr;
        HIPCHK(hipMalloc(&tt, (size_t)n * 3 * 32 * 40 * 4));
        std::vector<char> out((size_t)n * 3 * 32 * 40 * 2);
        if (rocalToTensor(ctx, tt, ROCAL_NCHW, ROCAL_FP16, 1 / 58.395f, 1 / 57.12f, 1 / 57.375f, -2.0f, -1.5f, -1.0f, true, ROCAL_MEMCPY_GPU) != ROCAL_OK) return 9;
        HIPCHK(hipMemcpy(out.data(), tt, out.size(), hipMemcpyDeviceToHost));
        std::ofstream(dir + "/tt0.bin", std::ios::binary).write(out.data(), out.size());
        out.resize((size_t)n * 3 * 24 * 32 * 4);
        if (rocalToTensor(ctx, tt, ROCAL_NHWC, ROCAL_FP32, 0.5f, 0.25f, 2.0f, 1.0f, 0.0f, -3.0f, false, ROCAL_MEMCPY_GPU, 24, 32) != ROCAL_OK) return 9;
        HIPCHK(hipMemcpy(out.data(), tt, out.size(), hipMemcpyDeviceToHost));
        std::ofstream(dir + "/tt1.bin", std::ios::binary).write(out.data(), out.size());
        if (rocalToTensor(ctx, out.data(), ROCAL_NCHW, ROCAL_FP32, 1, 1, 1, 0, 0, 0, false, ROCAL_MEMCPY_HOST) != ROCAL_RUNTIME_ERROR) return 10;
        (void)hipFree(tt);
    }
    rocalRelease(ctx);
    (void)hipFree(dev);
    std::cout << "ok " << outs.size() << std::endl;
    return 0;
}

}  // namespace

// A loader thread blocked on a full ring must leave with an exception when the ring is stopped or released, never with a
// slot that is still full; release() must not free the slots before the thread has left. Prints one line per check.
int run_ring() {
    auto fill = [](PackedCircularBuffer &ring, unsigned char v) {
        for (size_t i = 0; i < 2; i++) {
            uint32_t stride = 0;
            unsigned char *p = ring.place_image(i, 5, 3, &stride);
            if (stride != 16) throw std::runtime_error("row stride");
            memset(p, v, (size_t)stride * 3);
        }
        ring.push();
    };
    bool ok = true;
    auto say = [&](const char *what, bool good) {
        std::cout << what << " " << (good ? "ok" : "FAILED") << std::endl;
        ok = ok && good;
    };
    for (int how = 0; how < 3; how++) {  // 0: stop(), 1: release(), 2: unblock_writer() while the ring stays full
        PackedCircularBuffer ring(-1, nullptr);
        ring.init(2, 4096, 3);  // depth 3: two batches fill it (the third spot is the reader's)
        fill(ring, 1);
        fill(ring, 2);
        say("level_after_two_pushes", ring.level() == 2);
        std::atomic<int> state{0};  // 1: about to block, 2: left with an exception, 3: was handed a slot
        std::string message;
        std::thread loader([&] {
            state = 1;
            try {
                uint32_t stride = 0;
                ring.place_image(0, 5, 3, &stride);
                state = 3;
            } catch (const std::exception &e) {
                message = e.what();
                state = 2;
            }
        });
        while (state.load() == 0) std::this_thread::yield();
        std::this_thread::sleep_for(std::chrono::milliseconds(50));
        say("loader_blocked_on_full_ring", state.load() == 1);
        const auto t0 = std::chrono::steady_clock::now();
        if (how == 0) ring.stop();
        else if (how == 1) ring.release();
        else ring.unblock_writer();
        loader.join();
        const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
        say(how == 0 ? "stop_wakes_loader" : how == 1 ? "release_wakes_loader" : "unblock_without_room_is_an_error", state.load() == 2 && ms < 1000.0);
        say("message", message.find(how == 2 ? "full" : "released") != std::string::npos);
        if (how == 0) {
            bool threw = false;
            try {
                ring.get_read_buffer_dev();
            } catch (const std::exception &) {
                threw = true;
            }
            say("reader_turned_away_after_stop", threw);
            ring.reset();  // a new epoch: the ring takes batches again
            fill(ring, 3);
            say("ring_usable_after_reset", ring.level() == 1 && static_cast<unsigned char *>(ring.get_read_buffer_dev())[0] == 3);
            ring.pop();
        }
        if (how == 2) {
            // the reader's side still holds both batches, oldest first
            say("oldest_batch_intact", static_cast<unsigned char *>(ring.get_read_buffer_dev())[0] == 1);
            ring.pop();
            fill(ring, 4);  // room again
            say("writer_continues_after_pop", ring.level() == 2);
        }
    }
    {
        // a consumer blocked on an empty ring is woken the same way
        PackedCircularBuffer ring(-1, nullptr);
        ring.init(2, 4096, 2);
        std::atomic<int> state{0};
        std::thread reader([&] {
            state = 1;
            try {
                ring.get_read_buffer_dev();
                state = 3;
            } catch (const std::exception &) {
                state = 2;
            }
        });
        while (state.load() == 0) std::this_thread::yield();
        std::this_thread::sleep_for(std::chrono::milliseconds(50));
        ring.release();
        reader.join();
        say("release_wakes_reader", state.load() == 2);
    }
    std::cout << (ok ? "ring ok" : "ring FAILED") << std::endl;
    return ok ? 0 : 1;
}

int main(int argc, char **argv) {
    if (argc >= 2 && !strcmp(argv[1], "ring")) return run_ring();
    if (argc >= 3 && !strcmp(argv[1], "params")) return run_params((unsigned)strtoul(argv[2], nullptr, 10));
    if (argc >= 4 && !strcmp(argv[1], "pipeline")) return run_pipeline(argv[2], argv[3]);
    std::cerr << "usage: host_check params <seed> | ring | pipeline <scenario> <dir>" << std::endl;
    return 1;
}
