// Host side of the C ABI: contexts, ops, the per-batch parameter table and kernel launches.
// One op = one node of the reference graph (create_node / update_node / process phases).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <new>
#include <string>
#include <limits>
#include <mutex>
#include <vector>

#include "rmx_common.h"
#include "rmx_launch.h"

namespace {

thread_local std::string g_err;

int fail(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_err = buf;
    return code;
}

#define HIP_TRY(expr)                                                                              \
    do {                                                                                           \
        hipError_t e_ = (expr);                                                                    \
        if (e_ != hipSuccess)                                                                      \
            return fail(RMX_ERR_HIP, "%s failed: %d (%s)", #expr, (int)e_, hipGetErrorString(e_)); \
    } while (0)

enum OpKind {
    OP_CMN = 1, OP_CROP, OP_FLIP, OP_RESIZE, OP_COLOR_TWIST, OP_BRIGHTNESS, OP_CONTRAST, OP_HUE,
    OP_SATURATION, OP_WARP_AFFINE, OP_ROTATE, OP_TO_TENSOR, OP_GAMMA, OP_EXPOSURE, OP_COLOR_TEMPERATURE, OP_BLEND, OP_NORMALIZE, OP_TRANSPOSE
};

constexpr int TABLE_RING = 4;  // updates in flight before the host has to wait on an old upload

}  // namespace

// ---- parameter table of the entry point that allocates nothing (rmx_resize_cmn_noalloc) ----
// Every GPU the library runs on holds its own copy of this array until the process ends. In host code the array's name is
// only a stand-in: its device address is asked for once per device (rmx_ctx_create) and kept in the context.
constexpr int RMX_NOALLOC_ROWS = RMX_NOALLOC_MAX_SAMPLES;
static __device__ __align__(256) unsigned char scratch[(size_t)RMX_NOALLOC_ROWS * sizeof(RmxSample)];

// The rows travel as kernel arguments (16 rows = 2 KB per launch): no staging buffer, no copy from host memory, nothing
// that a stream capture could not record.
struct RmxRowPack {
    RmxSample rows[16];
};
__global__ void __launch_bounds__(512) rmx_table_fill_kernel(RmxRowPack pack, RmxSample *table, int first, int count) {
    const uint32_t *src = reinterpret_cast<const uint32_t *>(pack.rows);
    uint32_t *dst = reinterpret_cast<uint32_t *>(table + first);
    const int words = count * (int)(sizeof(RmxSample) / 4);
    for (int i = threadIdx.x; i < words; i += blockDim.x) dst[i] = src[i];
}

// Copies a freshly packed parameter table from the pinned host ring to its device slot: 16 bytes per lane, read across
// the host link by the GPU itself. For the 4-40 KB of a table this reaches the device sooner than a copy-engine transfer
// queued on the same stream.
__global__ void __launch_bounds__(256) rmx_table_upload_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, int n16) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += gridDim.x * blockDim.x) dst[i] = src[i];
}

static std::mutex g_life_lock;  // creation and destruction of ops against the destruction of their context

struct rmx_ctx {
    int upload_kernel = 1;        // 1: tables are uploaded by rmx_table_upload_kernel, 0: by hipMemcpyAsync
    // (both under g_life_lock: a garbage collector may destroy ops and their context from different threads)
    int live_ops = 0;             // ops made on this context and not yet destroyed: they use its streams until their own end
    bool closed = false;          // rmx_ctx_destroy was called while ops were alive; the last op's end frees the context
    void *scratch_ptr = nullptr;  // device address of `scratch` on this context's device
    int device = 0;
    hipStream_t stream = nullptr;
    bool owns_stream = false;
    int num_cus = 256;
    int max_lds_per_block = 65536;
    // Launch-plan tunables (rows per wavefront strip, LDS budget of the resize fast path). Defaults are the
    // values measured best on MI355X; RMX_TUNE_* environment variables, read once when the context is
    // created and clamped to safe ranges, override them for sweeps. They change plans, never results.
    int k1_rows = 4, k1_flat_rows = 0, k3_rows = 8, k3_flat_rows = 0, tri_rows = 0, gen_rows = 8, fast_rows = 4, fast_lds = 10 * 1024, fast_wpb = 1, dma = 1, dma_lds = 10 * 1024, dma_group = 1, flat_frames = 1, deal_xcd = 1, tri_wpb = 1, tri_ring = 0, tri_tpx = 2, tri_slots = 0, tri_per_cu = 0, tri_sort = 1, warp_passes = 2, warp_wpb = 4;
};

static int tune_env(const char *name, int def, int lo, int hi) {
    const char *e = getenv(name);
    if (!e || !*e) return def;
    return std::max(lo, std::min(hi, atoi(e)));
}

struct rmx_op {
    rmx_ctx *ctx = nullptr;
    int kind = 0;
    rmx_tensor_desc src{}, dst{};
    int interp = RMX_INTERP_LINEAR;
    int roi_type = RMX_ROI_XYWH;
    uint32_t flags = 0;
    bool norm = false, quant = false;
    int n = 0;

    RmxSample *h_table[TABLE_RING] = {};  // pinned; n rows, then n source layout entries, then n side-table entries
    size_t extra_per_sample = 0;          // bytes of side table per sample (Gamma: its 256-entry table)
    std::vector<float> lut_gamma;         // Gamma: the exponent each cached table was built for (NaN = none yet)
    std::vector<uint8_t> lut_cache;       // Gamma: last table of every sample (256 powf per table are worth keeping)
    std::vector<RmxSrcLayout> layout;     // ragged source (empty: one padded tensor); copied behind the rows on every update
    std::vector<uint32_t> layout_w;       // image widths of the ragged source (a row stride may include padding)
    uint64_t ragged_bytes = 0;            // extent of the ragged source buffer
    bool slot_ragged[TABLE_RING] = {};    // what the table slot was committed with
    uint64_t slot_src_bytes[TABLE_RING] = {};
    RmxSample *d_table[TABLE_RING] = {};
    hipEvent_t uploaded[TABLE_RING] = {};
    int cur = -1;  // slot of the last update, -1 before the first
    // A launch of this op was recorded into a HIP graph: the graph's kernel node holds the address of the table slot of the
    // last update, which the ring would hand out again four updates later. Such an op keeps its parameters: updates are refused.
    bool captured = false;

    // launch plan of the last update
    rmx::KernelFn fn = nullptr;
    const char *kernel_name = "";
    rmx::KernelFn fn_fast = nullptr;  // specialisation usable when the destination base is 16-byte aligned
    const char *fast_name = "";
    int strips = 1, strip_rows = 1, tile_w = 512, lds_per_wave = 0, waves_per_block = 4;
    int aux0 = 0, aux1 = 0;
    int fast_lds = 0, fast_strips = 1, fast_rows = 8, fast_wpb = 1;  // plan of fn_fast
    int fast_aux1 = 0;                                               // aux1 of fn_fast
    // the streaming bilinear kernel in its any-width form: taken when fn_fast cannot be (a width that is not a multiple of 8,
    // a destination base off 16-byte alignment), before the general kernel
    rmx::KernelFn fn_mid = nullptr;
    const char *mid_name = "";
    int mid_lds = 0, mid_strips = 1, mid_rows = 4, mid_wpb = 1, mid_aux1 = 1;
    bool fast_needs_src16 = false;                                   // fn_fast also wants a 16-byte aligned source base
    uint64_t algo_bytes = 0;
    int tri_rows_in_flight = 0;  // streaming triangular kernel: accumulator sets (2 or 4), 0 for every other kernel
    // Point operations on whole frames (every sample's window is the whole padded image, source and destination of one
    // shape): the batch is handed to the kernel as flat_h rows of 512 pixels per sample, so that all 64 lanes work whatever the
    // image width is (224 pixels are 28 groups of 8: two rows per step keep 56 lanes busy). 0: the images' own rows.
    int flat_h = 0;
    int stats_mode = 0, stats_per_channel = 1;  // Normalize: what is computed on the device (bit 0 mean, bit 1 standard deviation)
    float stats_scale = 1.0f, stats_shift = 0.0f;
    rmx::KernelFn lds_fn[3] = {};  // kernels whose static LDS size has been asked of the runtime ([0] general, [1] fast, [2] mid)
    int lds_static[3] = {};
};

namespace {

int check_desc(const rmx_tensor_desc *d, const char *what) {
    if (!d) return fail(RMX_ERR_INVALID, "%s descriptor is NULL", what);
    if (d->n == 0 || d->h == 0 || d->w == 0) return fail(RMX_ERR_INVALID, "%s descriptor has a zero dimension", what);
    if (d->c != 3) return fail(RMX_ERR_UNSUPPORTED, "%s: only 3-channel (RGB) tensors are on the hot path (c=%u)", what, d->c);
    if (d->layout != RMX_NHWC && d->layout != RMX_NCHW) return fail(RMX_ERR_UNSUPPORTED, "%s: layout %d not supported", what, d->layout);
    if (d->dtype != RMX_FP32 && d->dtype != RMX_FP16 && d->dtype != RMX_UINT8) return fail(RMX_ERR_UNSUPPORTED, "%s: dtype %d not supported", what, d->dtype);
    return RMX_OK;
}

// Size of one table slot: n rows, n source layout entries and n side-table entries, rounded up to the 16-byte pieces in
// which the upload kernel copies it.
size_t slot_bytes(const rmx_op *op) {
    const size_t raw = (sizeof(RmxSample) + sizeof(RmxSrcLayout) + op->extra_per_sample) * (size_t)op->n;
    return (raw + 15) & ~(size_t)15;
}

int make_op(rmx_ctx *ctx, int kind, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int roi_type, rmx_op **out, size_t extra_per_sample = 0) {
    if (!ctx) return fail(RMX_ERR_INVALID, "context is NULL");
    if (!out) return fail(RMX_ERR_INVALID, "output handle pointer is NULL");
    *out = nullptr;
    int rc;
    if ((rc = check_desc(src, "source"))) return rc;
    if ((rc = check_desc(dst, "destination"))) return rc;
    if (src->dtype != RMX_UINT8 || src->layout != RMX_NHWC)
        return fail(RMX_ERR_UNSUPPORTED, "source must be uint8 NHWC (decoded RGB batch)");
    if (src->n != dst->n) return fail(RMX_ERR_INVALID, "batch size mismatch: source %u, destination %u", src->n, dst->n);
    if (roi_type != RMX_ROI_LTRB && roi_type != RMX_ROI_XYWH) return fail(RMX_ERR_INVALID, "roi_type %d invalid", roi_type);
    HIP_TRY(hipSetDevice(ctx->device));
    rmx_op *op = new (std::nothrow) rmx_op();
    if (!op) return fail(RMX_ERR_NOMEM, "out of host memory");
    op->ctx = ctx;
    {
        std::lock_guard<std::mutex> life(g_life_lock);
        ctx->live_ops++;
    }
    op->kind = kind;
    op->src = *src;
    op->dst = *dst;
    op->roi_type = roi_type;
    op->n = (int)src->n;
    op->extra_per_sample = extra_per_sample;
    // (the upload kernel moves whole 16-byte pieces: a slot is a whole number of them)
    const size_t bytes = slot_bytes(op);
    for (int i = 0; i < TABLE_RING; i++) {
        hipError_t e = hipHostMalloc((void **)&op->h_table[i], bytes, hipHostMallocDefault);
        if (e == hipSuccess) e = hipMalloc((void **)&op->d_table[i], bytes);
        if (e == hipSuccess) e = hipEventCreateWithFlags(&op->uploaded[i], hipEventDisableTiming);
        if (e != hipSuccess) {
            rmx_op_destroy(op);
            return fail(RMX_ERR_HIP, "allocating the parameter table failed: %d (%s)", (int)e, hipGetErrorString(e));
        }
        memset(op->h_table[i], 0, bytes);
    }
    *out = op;
    return RMX_OK;
}

// Next table slot; waits until the upload that last used it has completed.
int next_slot(rmx_op *op, RmxSample **row) {
    if (op->captured)
        return fail(RMX_ERR_INVALID, "a launch of this op was recorded into a HIP graph, whose replays read the parameter rows of the update before the capture: "
                                     "the op keeps those parameters (create another op for new ones, or record rmx_resize_cmn_noalloc, which carries its rows in the graph)"), -2;
    int slot = (op->cur + 1) % TABLE_RING;
    HIP_TRY(hipSetDevice(op->ctx->device));
    HIP_TRY(hipEventSynchronize(op->uploaded[slot]));
    *row = op->h_table[slot];
    return slot;
}

int commit_slot(rmx_op *op, int slot) {
    size_t bytes = sizeof(RmxSample) * (size_t)op->n;
    if (!op->layout.empty()) {
        memcpy(reinterpret_cast<char *>(op->h_table[slot]) + bytes, op->layout.data(), sizeof(RmxSrcLayout) * (size_t)op->n);
        bytes += sizeof(RmxSrcLayout) * (size_t)op->n;
    }
    if (op->extra_per_sample)  // the side table lies behind the layout entries whether or not those are in use
        bytes = (sizeof(RmxSample) + sizeof(RmxSrcLayout) + op->extra_per_sample) * (size_t)op->n;
    op->slot_ragged[slot] = !op->layout.empty();
    op->slot_src_bytes[slot] = op->ragged_bytes;
    // (Same stream as the launches. Measured against an upload stream of its own, ordered by events so that the table travels
    // under the kernels of earlier batches: the three extra event calls cost the host 18 us per update, and whole steps got
    // slower, 56.8 -> 73.0 us with a wait per batch and 38.5 -> 41.7 us without, on the RandomResizedCrop batch.)
    hipStream_t us = op->ctx->stream;
    if (op->ctx->upload_kernel) {
        const int n16 = (int)((bytes + 15) / 16);
        if ((size_t)n16 * 16 > slot_bytes(op)) return fail(RMX_ERR_INVALID, "parameter table of %zu bytes exceeds its slot of %zu", bytes, slot_bytes(op));
        hipLaunchKernelGGL(rmx_table_upload_kernel, dim3((unsigned)std::min(8, (n16 + 255) / 256)), dim3(256), 0, us,
                           reinterpret_cast<const uint4 *>(op->h_table[slot]), reinterpret_cast<uint4 *>(op->d_table[slot]), n16);
        HIP_TRY(hipGetLastError());
    } else {
        HIP_TRY(hipMemcpyAsync(op->d_table[slot], op->h_table[slot], bytes, hipMemcpyHostToDevice, us));
    }
    HIP_TRY(hipEventRecord(op->uploaded[slot], us));
    op->cur = slot;
    return RMX_OK;
}

// image size of sample i: its own when the source is ragged, the padded tensor's otherwise
inline uint32_t sample_w(const rmx_op *op, int i) { return op->layout.empty() ? op->src.w : op->layout_w[i]; }
inline uint32_t sample_h(const rmx_op *op, int i) { return op->layout.empty() ? op->src.h : op->layout[i].rows; }

// ROI in the caller's convention -> x,y,w,h clipped to the padded source tensor.
int read_roi(const rmx_op *op, const uint32_t *roi, int i, int32_t *x, int32_t *y, int32_t *w, int32_t *h) {
    const uint32_t sw = sample_w(op, i), sh = sample_h(op, i);
    if (!roi) {
        *x = 0; *y = 0; *w = (int32_t)sw; *h = (int32_t)sh;
        return RMX_OK;
    }
    uint32_t a = roi[i * 4], b = roi[i * 4 + 1], c = roi[i * 4 + 2], d = roi[i * 4 + 3];
    if (op->roi_type == RMX_ROI_LTRB) {  // l,t,r,b with r,b exclusive bounds as rocAL's width/height users read them
        if (c < a || d < b) return fail(RMX_ERR_INVALID, "sample %d: LTRB roi has r<l or b<t", i);
        c -= a;
        d -= b;
    }
    if (a >= sw || b >= sh) return fail(RMX_ERR_INVALID, "sample %d: roi origin (%u,%u) outside the %ux%u source", i, a, b, sw, sh);
    if (c > sw - a) c = sw - a;
    if (d > sh - b) d = sh - b;
    *x = (int32_t)a; *y = (int32_t)b; *w = (int32_t)c; *h = (int32_t)d;
    return RMX_OK;
}

// side table of a slot: behind the n rows and the n layout entries
inline uint8_t *slot_extra(rmx_op *op, RmxSample *rows) {
    return reinterpret_cast<uint8_t *>(rows) + (sizeof(RmxSample) + sizeof(RmxSrcLayout)) * (size_t)op->n;
}

size_t dtype_size(int dtype) { return dtype == RMX_FP32 ? 4 : dtype == RMX_FP16 ? 2 : 1; }

// Width of the x-tiles of the bilinear fast paths for a destination row of w pixels; 0 when no width fits the LDS budget.
// A lane blends 8 pixels and the lanes of a wavefront are dealt to whole rows: a tile of L = tw / 8 lanes per row runs
// floor(64 / L) rows per pass, so tiles of 128, 256 and 512 pixels keep every lane busy (1, 2 and 4 passes for 4 rows), and every
// tile is one more window to wait for. Cost of a width = passes + half the windows per strip of `rows` rows; the candidates are
// the whole row and the powers of two below it, of which those whose window fits `cap` bytes (need_of(tw)) compete. Measured on 256
// images to 299 x 299: tiles of 128 + 128 + 43 pixels 75.5 us, of 144 + 144 + 11 (the whole row halved until it fits) 86.6 us.
struct TileCost {
    int of_lanes[65];  // twice the cost of a tile of L lanes per row: a window counts half a pass
    explicit TileCost(int rows) {
        of_lanes[0] = 0;
        for (int lanes = 1; lanes <= 64; lanes++) {
            const int per_pass = 64 / lanes;
            of_lanes[lanes] = 1 + 2 * ((rows + per_pass - 1) / per_pass);
        }
    }
};
template <typename NeedOf>
int pick_tile_width(int w, const TileCost &tc, long cap, NeedOf need_of, long *need_out) {
    const int whole = std::min(std::max(w, 8), 512);
    const int cand[7] = {whole, 256, 128, 64, 32, 16, 8};
    auto tile_cost = [&tc](int t) { return tc.of_lanes[(t + 7) >> 3]; };
    int best = 0;
    long best_cost = 0;
    for (int k = 0; k < 7; k++) {
        const int tw = cand[k];
        if (k > 0 && tw >= whole) continue;
        if (best != 0 && tw < 64) break;  // (narrower tiles only where nothing wider fits)
        // whole tiles of the row (no division: cand[k] = 512 >> k for k >= 1, and the whole row is one tile unless it is cut at 512)
        const int full = (k == 0) ? (w < whole ? 0 : (whole == 512 ? w >> 9 : 1)) : (w >> (9 - k)), rest = w - full * tw;
        const long cost = (long)full * tile_cost(tw) + (rest ? tile_cost(rest) : 0);
        if (best != 0 && cost >= best_cost) continue;  // (the window's size is only asked for where it could matter)
        const long need = need_of(tw);
        if (need > cap) continue;
        best = tw;
        best_cost = cost;
        *need_out = need;
    }
    return best;
}

// Whole-frame point operations as rows of kFlatRow pixels: true (and the rows of `t` rewritten) when every sample's window
// is the whole padded source image, the destination has the source's shape, the pixels of a sample divide into whole rows
// of kFlatRow, and the source is the dense tensor. The kernel then sees flat_h rows of kFlatRow pixels per sample.
constexpr int kFlatRow = 512;  // one step of 64 lanes x 8 pixels
bool flatten_whole_frames(rmx_op *op, RmxSample *t) {
    op->flat_h = 0;
    if (!op->ctx->flat_frames || !op->layout.empty()) return false;
    if (op->src.w != op->dst.w || op->src.h != op->dst.h) return false;
    const uint64_t px = (uint64_t)op->src.w * op->src.h;
    if (px % kFlatRow != 0 || px / kFlatRow > 0x7fffff || op->src.w == (uint32_t)kFlatRow) return false;
    for (int i = 0; i < op->n; i++) {
        const RmxSample &s = t[i];
        if (s.src_x != 0 || s.src_y != 0 || s.src_w != (int32_t)op->src.w || s.src_h != (int32_t)op->src.h || s.dst_w != s.src_w || s.dst_h != s.src_h) return false;
    }
    op->flat_h = (int)(px / kFlatRow);
    for (int i = 0; i < op->n; i++) {
        t[i].src_w = t[i].dst_w = kFlatRow;
        t[i].src_h = t[i].dst_h = op->flat_h;
    }
    return true;
}

void plan_streaming(rmx_op *op, int max_rows, int rows_per_strip) {
    op->strip_rows = rows_per_strip;
    op->strips = std::max(1, (max_rows + rows_per_strip - 1) / rows_per_strip);
    op->aux0 = rows_per_strip;
    op->lds_per_wave = 0;
    op->waves_per_block = 4;
}

}  // namespace

extern "C" {

const char *rmx_last_error(void) { return g_err.c_str(); }
const char *rmx_version(void) { return "rocal-mi355x 0.1 (gfx950)"; }

int rmx_ctx_create(int device, void *stream, int own_stream, rmx_ctx **out) {
    if (!out) return fail(RMX_ERR_INVALID, "output handle pointer is NULL");
    *out = nullptr;
    int count = 0;
    HIP_TRY(hipGetDeviceCount(&count));
    if (device < 0 || device >= count) return fail(RMX_ERR_INVALID, "device %d out of range (have %d)", device, count);
    HIP_TRY(hipSetDevice(device));
    rmx_ctx *ctx = new (std::nothrow) rmx_ctx();
    if (!ctx) return fail(RMX_ERR_NOMEM, "out of host memory");
    ctx->device = device;
    if (!own_stream) {
        ctx->stream = (hipStream_t)stream;
    } else {
        hipError_t e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
        if (e != hipSuccess) {
            delete ctx;
            return fail(RMX_ERR_HIP, "hipStreamCreateWithFlags failed: %d (%s)", (int)e, hipGetErrorString(e));
        }
        ctx->owns_stream = true;
    }
    {
        // device address of the static parameter table of rmx_resize_cmn_noalloc, with this device current
        hipError_t e = hipGetSymbolAddress(&ctx->scratch_ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ctx->scratch_ptr) {
            if (ctx->owns_stream) (void)hipStreamDestroy(ctx->stream);
            delete ctx;
            return fail(RMX_ERR_HIP, "hipGetSymbolAddress(scratch) failed: %d (%s)", (int)e, hipGetErrorString(e));
        }
    }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) == hipSuccess) {
        ctx->num_cus = prop.multiProcessorCount;
        ctx->max_lds_per_block = (int)prop.sharedMemPerBlock;
        ctx->k1_rows = tune_env("RMX_TUNE_CMN_ROWS", ctx->k1_rows, 1, 64);
        ctx->k3_rows = tune_env("RMX_TUNE_COLOR_ROWS", ctx->k3_rows, 1, 64);
        ctx->k3_flat_rows = tune_env("RMX_TUNE_COLOR_FLAT_ROWS", ctx->k3_flat_rows, 0, 64);  // 0: one row for the twist, two for the linear kinds
        ctx->k1_flat_rows = tune_env("RMX_TUNE_K1_FLAT_ROWS", ctx->k1_flat_rows, 0, 16);  // rows of 512 pixels per wavefront, whole frames through the K1 kernel (0: by output type)
        ctx->tri_rows = tune_env("RMX_TUNE_TRI_ROWS", ctx->tri_rows, 0, 64);  // 0: chosen per batch
        ctx->gen_rows = tune_env("RMX_TUNE_RESIZE_ROWS", ctx->gen_rows, 1, 64);
        ctx->fast_rows = tune_env("RMX_TUNE_FAST_ROWS", ctx->fast_rows, 1, 64);
        ctx->fast_lds = tune_env("RMX_TUNE_FAST_LDS", ctx->fast_lds, 2048, 48 * 1024);
        ctx->fast_wpb = tune_env("RMX_TUNE_FAST_WPB", ctx->fast_wpb, 1, 4);
        ctx->upload_kernel = tune_env("RMX_TUNE_UPLOAD_KERNEL", ctx->upload_kernel, 0, 1);
        ctx->dma = tune_env("RMX_TUNE_DMA", ctx->dma, 0, 1);  // 0: the bilinear fast path always stages through registers
        ctx->dma_lds = tune_env("RMX_TUNE_DMA_LDS", ctx->dma_lds, 2048, 32 * 1024) & ~15;  // LDS window of a wavefront
        ctx->dma_group = tune_env("RMX_TUNE_DMA_GROUP", ctx->dma_group, 0, 16);  // windows per wavefront, 0: chosen per batch
        ctx->flat_frames = tune_env("RMX_TUNE_FLAT_FRAMES", ctx->flat_frames, 0, 1);  // 0: point operations always walk the images' own rows
        ctx->tri_wpb = tune_env("RMX_TUNE_TRI_WPB", ctx->tri_wpb, 1, 4);
        ctx->warp_passes = tune_env("RMX_TUNE_WARP_PASSES", ctx->warp_passes, 1, 8);
        ctx->warp_wpb = tune_env("RMX_TUNE_WARP_WPB", ctx->warp_wpb, 1, 4);
        ctx->tri_ring = tune_env("RMX_TUNE_TRI_RING", ctx->tri_ring, 0, 1);  // 1: always the ring kernel
        ctx->tri_tpx = tune_env("RMX_TUNE_TRI_TPX", ctx->tri_tpx, 1, 2);     // output columns per lane of the downscaling kernel
        ctx->tri_slots = tune_env("RMX_TUNE_TRI_SLOTS", ctx->tri_slots, 0, 4);  // 4: the streaming triangular kernel always keeps four rows in flight (batches that need eight go to the ring kernel)
        ctx->deal_xcd = tune_env("RMX_TUNE_DEAL_XCD", ctx->deal_xcd, 0, 1);  // samples dealt round-robin to the XCDs (0: eight runs in batch order)
        ctx->tri_sort = tune_env("RMX_TUNE_TRI_SORT", ctx->tri_sort, 0, 1);  // rows of batches of uneven cost go largest window first
        ctx->tri_per_cu = tune_env("RMX_TUNE_TRI_PER_CU", ctx->tri_per_cu, 0, 32);  // wavefronts per CU the strip planner counts on (0: by registers and LDS)
    }
    *out = ctx;
    return RMX_OK;
}

static void ctx_free(rmx_ctx *ctx) {
    (void)hipSetDevice(ctx->device);
    if (ctx->owns_stream) {
        (void)hipStreamSynchronize(ctx->stream);
        (void)hipStreamDestroy(ctx->stream);
    }
    delete ctx;
}

int rmx_ctx_destroy(rmx_ctx *ctx) {
    if (!ctx) return RMX_OK;
    {
        std::lock_guard<std::mutex> life(g_life_lock);
        if (ctx->live_ops > 0) {  // an op outlives its context (destruction order of a garbage collector): keep the streams for it
            ctx->closed = true;
            return RMX_OK;
        }
    }
    ctx_free(ctx);
    return RMX_OK;
}

int rmx_ctx_sync(rmx_ctx *ctx) {
    if (!ctx) return fail(RMX_ERR_INVALID, "context is NULL");
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    return RMX_OK;
}

void *rmx_ctx_stream(rmx_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

int rmx_op_destroy(rmx_op *op) {
    if (!op) return RMX_OK;
    (void)hipSetDevice(op->ctx->device);
    (void)hipStreamSynchronize(op->ctx->stream);
    for (int i = 0; i < TABLE_RING; i++) {
        if (op->uploaded[i]) (void)hipEventDestroy(op->uploaded[i]);
        if (op->h_table[i]) (void)hipHostFree(op->h_table[i]);
        if (op->d_table[i]) (void)hipFree(op->d_table[i]);
    }
    rmx_ctx *ctx = op->ctx;
    delete op;
    bool last;
    {
        std::lock_guard<std::mutex> life(g_life_lock);
        last = --ctx->live_ops == 0 && ctx->closed;
    }
    if (last) ctx_free(ctx);
    return RMX_OK;
}

uint64_t rmx_op_algorithmic_bytes(const rmx_op *op) { return op ? op->algo_bytes : 0; }

const char *rmx_op_plan(const rmx_op *op) {
    static thread_local char buf[256];
    if (!op) return "";
    if (op->flat_h) {  // whole frames as rows of 512 pixels
        snprintf(buf, sizeof(buf), "waves=%lld strips=%d strip_rows=%d lds_per_wave=%d waves_per_block=%d fast=%d flat_rows=%d",
                 (long long)op->n * op->strips, op->strips, op->aux0, 0, op->waves_per_block, op->fn_fast ? 1 : 0, op->flat_h);
        return buf;
    }
    if (op->fn_fast)
        snprintf(buf, sizeof(buf), "waves=%lld strips=%d strip_rows=%d lds_per_wave=%d waves_per_block=%d fast=1 group=%d",
                 (long long)op->n * op->fast_strips, op->fast_strips, op->fast_rows, op->fast_lds, op->fast_wpb, std::max(1, op->fast_aux1));
    else if (op->fn_mid)
        snprintf(buf, sizeof(buf), "waves=%lld strips=%d strip_rows=%d lds_per_wave=%d waves_per_block=%d fast=0 any_width=1 group=%d",
                 (long long)op->n * op->mid_strips, op->mid_strips, op->mid_rows, op->mid_lds, op->mid_wpb, std::max(1, op->mid_aux1));
    else {
        int len = snprintf(buf, sizeof(buf), "waves=%lld strips=%d strip_rows=%d tile_w=%d lds_per_wave=%d waves_per_block=%d fast=0",
                           (long long)op->n * op->strips, op->strips, op->strip_rows, op->tile_w, op->lds_per_wave, op->waves_per_block);
        if (op->tri_rows_in_flight && len > 0 && len < (int)sizeof(buf)) snprintf(buf + len, sizeof(buf) - len, " rows_in_flight=%d", op->tri_rows_in_flight);
    }
    return buf;
}
const char *rmx_op_kernel_name(const rmx_op *op) { return op ? (op->fn_fast ? op->fast_name : (op->fn_mid ? op->mid_name : op->kernel_name)) : ""; }

// static LDS of a kernel (bytes), asked of the runtime once per op and kernel; -1 (with the error set) when the query fails
static int static_lds_of(rmx_op *op, rmx::KernelFn fn) {
    for (int i = 0; i < 3; i++)
        if (op->lds_fn[i] == fn) return op->lds_static[i];
    hipFuncAttributes attr;
    hipError_t e = hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(fn));
    if (e != hipSuccess) {
        fail(RMX_ERR_HIP, "hipFuncGetAttributes failed: %d (%s)", (int)e, hipGetErrorString(e));
        return -1;
    }
    const int slot = (fn == op->fn_fast) ? 1 : (fn == op->fn_mid ? 2 : 0);
    op->lds_fn[slot] = fn;
    op->lds_static[slot] = (int)attr.sharedSizeBytes;
    return op->lds_static[slot];
}

// Enqueues the op's kernel with the given device table (and, for ragged sources, its layout entries).
static int launch_table(rmx_op *op, const RmxSample *table, const RmxSrcLayout *layout, const uint8_t *extra, uint64_t ragged_bytes,
                        const void *src, const void *src2, void *dst);

static int launch_impl(rmx_op *op, const void *src, const void *src2, void *dst) {
    if (op->cur < 0 || !op->fn) return fail(RMX_ERR_INVALID, "op launched before its first update");
    const bool ragged = op->slot_ragged[op->cur];
    return launch_table(op, op->d_table[op->cur], ragged ? reinterpret_cast<const RmxSrcLayout *>(op->d_table[op->cur] + op->n) : nullptr,
                        op->extra_per_sample ? slot_extra(op, op->d_table[op->cur]) : nullptr, ragged ? op->slot_src_bytes[op->cur] : 0, src, src2, dst);
}

static int launch_table(rmx_op *op, const RmxSample *table, const RmxSrcLayout *layout, const uint8_t *extra, uint64_t ragged_bytes,
                        const void *src, const void *src2, void *dst) {
    if (!src || !dst) return fail(RMX_ERR_INVALID, "source/destination buffer is NULL");
    if (!op->fn) return fail(RMX_ERR_INVALID, "op launched before its first update");
    RmxKArgs a{};
    a.src = (const uint8_t *)src;
    a.src2 = (const uint8_t *)src2;
    a.extra = extra;
    a.dst = dst;
    a.table = table;
    a.src_bytes = layout ? ragged_bytes : (uint64_t)op->src.n * op->src.h * op->src.w * op->src.c;
    a.layout = layout;
    a.n = op->n;
    a.src_h = (int)op->src.h;
    a.src_w = (int)op->src.w;
    a.dst_h = (int)op->dst.h;
    a.dst_w = (int)op->dst.w;
    if (op->flat_h) {
        a.src_h = a.dst_h = op->flat_h;
        a.src_w = a.dst_w = kFlatRow;
    }
    a.strips = op->strips;
    a.lds_bytes = op->lds_per_wave;
    a.aux0 = op->aux0;
    a.aux1 = op->aux1;
    if ((((uintptr_t)src) | ((uintptr_t)src2)) & 3u) return fail(RMX_ERR_INVALID, "the source batch must start at a 4-byte aligned address");
    if ((op->kind == OP_WARP_AFFINE || op->kind == OP_ROTATE) && (((uintptr_t)dst) & 15u)) a.aux1 &= ~1;  // packed stores need an aligned base
    // the fast specialisation wants 16-byte aligned batch bases (rows of both sides are then aligned too)
    const bool fast = op->fn_fast && (((uintptr_t)dst) & 15u) == 0 && (!op->fast_needs_src16 || (((uintptr_t)src) & 15u) == 0);
    const bool mid = !fast && op->fn_mid;
    int wpb = op->waves_per_block;
    if (fast) {
        a.strips = op->fast_strips;
        a.lds_bytes = op->fast_lds;
        a.aux0 = op->fast_rows;
        a.aux1 = op->fast_aux1;
        wpb = op->fast_wpb;
    } else if (mid) {
        a.strips = op->mid_strips;
        a.lds_bytes = op->mid_lds;
        a.aux0 = op->mid_rows;
        a.aux1 = op->mid_aux1;
        wpb = op->mid_wpb;
    }
    HIP_TRY(hipSetDevice(op->ctx->device));
    rmx::KernelFn fn = fast ? op->fn_fast : (mid ? op->fn_mid : op->fn);
    // a workgroup's LDS = the wavefronts' dynamic slices + what the kernel declares statically (coalescing slabs, colour
    // tables): fewer wavefronts per workgroup when the sum would not fit
    const int static_lds = static_lds_of(op, fn);
    if (static_lds < 0) return RMX_ERR_HIP;
    while (wpb > 1 && (size_t)a.lds_bytes * wpb + (size_t)static_lds > (size_t)op->ctx->max_lds_per_block) wpb--;
    const size_t lds = (size_t)a.lds_bytes * wpb;
    if (lds + (size_t)static_lds > (size_t)op->ctx->max_lds_per_block)
        return fail(RMX_ERR_INVALID, "plan needs %zu + %d bytes of LDS per workgroup (limit %d)", lds, static_lds, op->ctx->max_lds_per_block);
    const uint64_t waves = (uint64_t)op->n * (uint64_t)a.strips;
    const uint64_t blocks = (waves + wpb - 1) / wpb;
    if (blocks == 0 || blocks > 0x7fffffffull) return fail(RMX_ERR_INVALID, "grid of %llu workgroups is out of range", (unsigned long long)blocks);
    a.wpb = wpb;
    a.nblocks = (uint32_t)blocks;
    // reciprocals for wave_to_sample (rounded up; exact while dividend x divisor < 2^32, else the kernel divides / keeps batch order)
    auto recip = [](uint64_t d) { return (uint32_t)(((1ull << 32) + d - 1) / d); };
    a.inv_strips = (a.strips > 1 && waves * (uint64_t)a.strips < (1ull << 32)) ? recip((uint64_t)a.strips) : 0u;
    a.per_xcd = 0;
    a.inv_per_xcd = 0;
    if (op->ctx->deal_xcd && op->n >= 16 && (uint64_t)op->n * (uint64_t)(op->n / 8) < (1ull << 32)) {
        a.per_xcd = (uint32_t)(op->n / 8);
        a.inv_per_xcd = a.per_xcd > 1 ? recip(a.per_xcd) : 0u;
        if (a.per_xcd == 1) a.per_xcd = 0;  // (8..15 samples: nothing to deal)
    }
    if (op->kind == OP_NORMALIZE) {
        // moments of every sample's window (when asked for), then the FMA constants into the rows the streaming pass reads;
        // the side table of the slot holds the given statistics (6 floats per sample) and, behind them, the 64-bit counters
        const float *given = reinterpret_cast<const float *>(extra);
        unsigned long long *counters = reinterpret_cast<unsigned long long *>(const_cast<uint8_t *>(extra) + (size_t)op->n * 24);
        rmx::launch_stats(op->ctx->stream, a, counters, const_cast<RmxSample *>(table), given, op->stats_mode, op->stats_per_channel, op->stats_scale,
                          op->stats_shift, op->stats_mode != 0);
        HIP_TRY(hipGetLastError());
    }
    hipLaunchKernelGGL(fn, dim3((unsigned)blocks), dim3(wpb * RMX_WAVE), lds, op->ctx->stream, a);
    HIP_TRY(hipGetLastError());
    if (!op->captured) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(op->ctx->stream, &capturing) == hipSuccess && capturing == hipStreamCaptureStatusActive) op->captured = true;
    }
    return RMX_OK;
}

int rmx_op_launch(rmx_op *op, const void *src, void *dst) {
    if (!op) return fail(RMX_ERR_INVALID, "op is NULL");
    if (op->kind == OP_BLEND) return fail(RMX_ERR_INVALID, "a Blend node takes two sources: use rmx_op_launch2");
    return launch_impl(op, src, nullptr, dst);
}

int rmx_op_launch2(rmx_op *op, const void *src1, const void *src2, void *dst) {
    if (!op) return fail(RMX_ERR_INVALID, "op is NULL");
    if (op->kind != OP_BLEND) return fail(RMX_ERR_INVALID, "only a Blend node takes two sources");
    if (!src2) return fail(RMX_ERR_INVALID, "second source buffer is NULL");
    return launch_impl(op, src1, src2, dst);
}

/* ------------------------------------------------------------------ ragged sources */

int rmx_op_set_ragged_source(rmx_op *op, const uint64_t *offsets, const uint32_t *widths, const uint32_t *heights, uint64_t buffer_bytes) {
    return rmx_op_set_ragged_source_strided(op, offsets, widths, heights, nullptr, buffer_bytes);
}

int rmx_op_set_ragged_source_strided(rmx_op *op, const uint64_t *offsets, const uint32_t *widths, const uint32_t *heights, const uint32_t *row_strides,
                                     uint64_t buffer_bytes) {
    if (!op) return fail(RMX_ERR_INVALID, "op is NULL");
    if (op->kind == OP_BLEND) return fail(RMX_ERR_UNSUPPORTED, "a Blend node reads two padded tensors of one shape; ragged sources are not supported");
    if (!offsets && !widths && !heights) {  // back to one padded tensor
        op->layout.clear();
        op->layout_w.clear();
        op->ragged_bytes = 0;
        return RMX_OK;
    }
    if (!offsets || !widths || !heights) return fail(RMX_ERR_INVALID, "offsets, widths and heights are required together");
    std::vector<RmxSrcLayout> l((size_t)op->n);
    for (int i = 0; i < op->n; i++) {
        if (widths[i] == 0 || heights[i] == 0 || widths[i] > op->src.w || heights[i] > op->src.h)
            return fail(RMX_ERR_INVALID, "sample %d: image of %u x %u is empty or exceeds the %u x %u of the source descriptor", i, widths[i], heights[i], op->src.w, op->src.h);
        const uint32_t stride = row_strides ? row_strides[i] : widths[i] * 3u;
        if (stride < widths[i] * 3u) return fail(RMX_ERR_INVALID, "sample %d: row stride %u is shorter than a row of %u pixels", i, stride, widths[i]);
        // (the last row need not be padded)
        const uint64_t bytes = (uint64_t)stride * (heights[i] - 1) + (uint64_t)widths[i] * 3;
        if (offsets[i] > buffer_bytes || bytes > buffer_bytes - offsets[i])
            return fail(RMX_ERR_INVALID, "sample %d: %llu bytes at offset %llu do not fit the buffer of %llu bytes", i, (unsigned long long)bytes, (unsigned long long)offsets[i],
                        (unsigned long long)buffer_bytes);
        l[i].offset = offsets[i];
        l[i].row_stride = stride;
        l[i].rows = heights[i];
    }
    op->layout.swap(l);
    op->layout_w.assign(widths, widths + op->n);
    op->ragged_bytes = buffer_bytes;
    return RMX_OK;
}

/* ------------------------------------------------------------------ K1 family */

static int create_k1(rmx_ctx *ctx, int kind, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int roi_type, bool norm, rmx_op **out) {
    int rc = make_op(ctx, kind, src, dst, roi_type, out);
    if (rc) return rc;
    (*out)->norm = norm;
    (*out)->fn = rmx::select_cmn_kernel(dst->dtype, dst->layout, norm, 0, &(*out)->kernel_name);
    return RMX_OK;
}

static int update_k1(rmx_op *op, const uint32_t *roi, const float *scale, const float *bias, const uint32_t *hflip, const uint32_t *vflip,
                     bool per_sample_scale = true, bool channel_reverse = false, int *open_slot = nullptr) {
    RmxSample *t;
    int slot = next_slot(op, &t);
    if (slot < 0) return slot == -2 ? RMX_ERR_INVALID : RMX_ERR_HIP;
    uint64_t bytes = 0;
    int max_rows = 1;
    for (int i = 0; i < op->n; i++) {
        RmxSample &s = t[i];
        if (roi) {
            int rc = read_roi(op, roi, i, &s.src_x, &s.src_y, &s.src_w, &s.src_h);
            if (rc) return rc;
        } else {  // whole padded image
            s.src_x = s.src_y = 0;
            s.src_w = (int32_t)sample_w(op, i);
            s.src_h = (int32_t)sample_h(op, i);
        }
        s.dst_w = std::min<int32_t>(s.src_w, (int32_t)op->dst.w);
        s.dst_h = std::min<int32_t>(s.src_h, (int32_t)op->dst.h);
        s.src_w = s.dst_w;
        s.src_h = s.dst_h;
        s.flags = ((hflip && hflip[i]) ? RMX_S_HFLIP : 0u) | ((vflip && vflip[i]) ? RMX_S_VFLIP : 0u) | (channel_reverse ? RMX_S_CHREV : 0u);
        for (int c = 0; c < 3; c++) {
            const int k = per_sample_scale ? i * 3 + c : c;
            s.scale[c] = scale ? scale[k] : 1.0f;
            s.bias[c] = bias ? bias[k] : 0.0f;
        }
        bytes += (uint64_t)s.dst_w * s.dst_h * 3 * (1 + dtype_size(op->dst.dtype));
        max_rows = std::max(max_rows, (int)s.dst_h);
    }
    op->algo_bytes = bytes;
    int rows = op->ctx->k1_rows;
    // whole frames that are not mirrored (a mirror is a matter of rows): as rows of 512 pixels, like the colour family's
    bool flipped = false;
    for (int i = 0; i < op->n && !flipped; i++) flipped = (t[i].flags & (RMX_S_HFLIP | RMX_S_VFLIP)) != 0;
    if (!flipped && flatten_whole_frames(op, t)) {
        max_rows = op->flat_h;
        // (256 frames of 224 x 224, 1 / 2 / 4 / 8 such rows per wavefront against strips of the images' own rows: u8 -> f16 planes
        // 21.6 / 22.4 / 23.7 / 26.9 against 22.3 us, u8 -> u8 18.7 / 16.75 / 18.6 / 19.9 against 17.35 us)
        rows = op->ctx->k1_flat_rows ? op->ctx->k1_flat_rows : (op->dst.dtype == RMX_UINT8 ? 2 : 1);
    } else {
        op->flat_h = 0;
    }
    plan_streaming(op, max_rows, rows);
    // aligned specialisation: whole 8-pixel groups everywhere and 16-byte aligned destination rows
    bool aligned = op->flat_h ? true : op->dst.w % 8 == 0;
    for (int i = 0; i < op->n && aligned; i++) aligned = (t[i].dst_w % 8 == 0);
    op->fn_fast = nullptr;
    if (aligned) {
        op->fn_fast = rmx::select_cmn_kernel(op->dst.dtype, op->dst.layout, op->norm, 1, &op->fast_name);
        op->fast_strips = op->strips;
        op->fast_lds = 0;
        op->fast_rows = op->aux0;
        op->fast_wpb = op->waves_per_block;
        op->fast_needs_src16 = false;
    }
    // the same pipeline for rows of any width from 8 pixels on and a destination at any element (also what an aligned plan
    // falls back to when the destination base it is launched on is not 16-byte aligned)
    bool wide8 = true;
    for (int i = 0; i < op->n && wide8; i++) wide8 = t[i].dst_w >= 8 || t[i].dst_w <= 0 || t[i].dst_h <= 0;
    op->fn_mid = nullptr;
    if (wide8) {
        op->fn_mid = rmx::select_cmn_kernel(op->dst.dtype, op->dst.layout, op->norm, 2, &op->mid_name);
        op->mid_strips = op->strips;
        op->mid_lds = 0;
        op->mid_rows = op->aux0;
        op->mid_wpb = op->waves_per_block;
        op->mid_aux1 = op->aux1;
    }
    if (open_slot) {  // the caller fills the side table of the slot and commits it
        *open_slot = slot;
        return RMX_OK;
    }
    return commit_slot(op, slot);
}

int rmx_create_crop_mirror_normalize(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int roi_type, rmx_op **out) {
    return create_k1(ctx, OP_CMN, src, dst, roi_type, true, out);
}

int rmx_update_crop_mirror_normalize(rmx_op *op, const uint32_t *crop_roi, const float *scale, const float *bias, const uint32_t *mirror) {
    if (!op || op->kind != OP_CMN) return fail(RMX_ERR_INVALID, "op is not a CropMirrorNormalize node");
    if (!crop_roi || !scale || !bias) return fail(RMX_ERR_INVALID, "crop_roi, scale and bias arrays are required");
    return update_k1(op, crop_roi, scale, bias, mirror, nullptr);
}

int rmx_create_crop(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int roi_type, rmx_op **out) {
    return create_k1(ctx, OP_CROP, src, dst, roi_type, false, out);
}

int rmx_update_crop(rmx_op *op, const uint32_t *crop_roi) {
    if (!op || op->kind != OP_CROP) return fail(RMX_ERR_INVALID, "op is not a Crop node");
    if (!crop_roi) return fail(RMX_ERR_INVALID, "crop_roi array is required");
    return update_k1(op, crop_roi, nullptr, nullptr, nullptr, nullptr);
}

int rmx_create_flip(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int roi_type, rmx_op **out) {
    return create_k1(ctx, OP_FLIP, src, dst, roi_type, false, out);
}

int rmx_update_flip(rmx_op *op, const uint32_t *src_roi, const uint32_t *horizontal, const uint32_t *vertical) {
    if (!op || op->kind != OP_FLIP) return fail(RMX_ERR_INVALID, "op is not a Flip node");
    return update_k1(op, src_roi, nullptr, nullptr, horizontal, vertical);
}

int rmx_create_to_tensor(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, rmx_op **out) {
    return create_k1(ctx, OP_TO_TENSOR, src, dst, RMX_ROI_XYWH, true, out);
}

int rmx_update_to_tensor(rmx_op *op, const float *multiplier, const float *offset, int reverse_channels) {
    if (!op || op->kind != OP_TO_TENSOR) return fail(RMX_ERR_INVALID, "op is not a ToTensor node");
    if (!multiplier || !offset) return fail(RMX_ERR_INVALID, "multiplier and offset (3 floats each) are required");
    return update_k1(op, nullptr, multiplier, offset, nullptr, nullptr, false, reverse_channels != 0);
}

/* ------------------------------------------------------------------ Normalize */

int rmx_create_normalize(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int roi_type, rmx_op **out) {
    // side table per sample: 6 floats of given statistics + 6 counters of 8 bytes
    int rc = make_op(ctx, OP_NORMALIZE, src, dst, roi_type, out, 72);
    if (rc) return rc;
    (*out)->norm = true;
    (*out)->fn = rmx::select_cmn_kernel(dst->dtype, dst->layout, true, 0, &(*out)->kernel_name);
    return RMX_OK;
}

int rmx_update_normalize(rmx_op *op, const uint32_t *src_roi, uint32_t axis_mask, const float *mean, const float *stddev, uint32_t n_stats,
                         float scale, float shift) {
    if (!op || op->kind != OP_NORMALIZE) return fail(RMX_ERR_INVALID, "op is not a Normalize node");
    if (axis_mask != 3u && axis_mask != 7u)
        return fail(RMX_ERR_UNSUPPORTED, "axis mask %u: images are normalised over height and width (3) or height, width and channels (7)", axis_mask);
    if ((mean || stddev) && n_stats != 1 && n_stats != 3) return fail(RMX_ERR_INVALID, "given statistics hold 1 or 3 values (n_stats = %u)", n_stats);
    if (stddev)
        for (uint32_t k = 0; k < n_stats; k++)
            if (stddev[k] == 0.0f) return fail(RMX_ERR_INVALID, "standard deviation %u is 0", k);
    int slot = -1;
    int rc = update_k1(op, src_roi, nullptr, nullptr, nullptr, nullptr, true, false, &slot);
    if (rc) return rc;
    float *given = reinterpret_cast<float *>(slot_extra(op, op->h_table[slot]));
    for (int i = 0; i < op->n; i++)
        for (int c = 0; c < 3; c++) {
            given[(size_t)i * 6 + c] = mean ? mean[n_stats == 3 ? c : 0] : 0.0f;
            given[(size_t)i * 6 + 3 + c] = stddev ? stddev[n_stats == 3 ? c : 0] : 1.0f;
        }
    op->stats_mode = (mean ? 0 : 1) | (stddev ? 0 : 2);
    op->stats_per_channel = axis_mask == 3u ? 1 : 0;
    op->stats_scale = scale;
    op->stats_shift = shift;
    // the moments pass reads every source byte once more when something is computed
    if (op->stats_mode) op->algo_bytes += op->algo_bytes / (1 + dtype_size(op->dst.dtype));
    return commit_slot(op, slot);
}

/* ------------------------------------------------------------------ Transpose */

int rmx_create_transpose(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, const uint32_t *perm, int roi_type, rmx_op **out) {
    if (out) *out = nullptr;
    if (!perm) return fail(RMX_ERR_INVALID, "perm (3 axes) is required");
    const uint32_t p = perm[0] * 100 + perm[1] * 10 + perm[2];
    if (!src || !dst) return fail(RMX_ERR_INVALID, "descriptor is NULL");
    // channels stay last (NHWC-shaped output) or go to the front (NCHW-shaped output); height and width keep or swap places
    const bool swap = p == 102 || p == 210;
    if (p != 12 && p != 201 && !swap)
        return fail(RMX_ERR_UNSUPPORTED, "permutation {%u,%u,%u}: on images the channel axis goes to the front or stays at the back", perm[0], perm[1], perm[2]);
    const int want_layout = (p == 12 || p == 102) ? RMX_NHWC : RMX_NCHW;
    if (dst->layout != want_layout) return fail(RMX_ERR_INVALID, "permutation {%u,%u,%u} produces a %s tensor", perm[0], perm[1], perm[2], want_layout == RMX_NHWC ? "channels-last" : "channels-first");
    if (swap ? (dst->h < src->w || dst->w < src->h) : (dst->h < src->h || dst->w < src->w))
        return fail(RMX_ERR_INVALID, "destination of %u x %u cannot hold the permuted %u x %u source", dst->w, dst->h, src->w, src->h);
    int rc = make_op(ctx, OP_TRANSPOSE, src, dst, roi_type, out);
    if (rc) return rc;
    (*out)->aux1 = swap ? 1 : 0;
    if (swap) (*out)->fn = rmx::select_transpose_kernel(dst->dtype, dst->layout, &(*out)->kernel_name);
    else (*out)->fn = rmx::select_cmn_kernel(dst->dtype, dst->layout, false, 0, &(*out)->kernel_name);
    return RMX_OK;
}

int rmx_update_transpose(rmx_op *op, const uint32_t *src_roi) {
    if (!op || op->kind != OP_TRANSPOSE) return fail(RMX_ERR_INVALID, "op is not a Transpose node");
    if (!op->aux1) return update_k1(op, src_roi, nullptr, nullptr, nullptr, nullptr);  // a layout change of the streaming kernel
    RmxSample *t;
    int slot = next_slot(op, &t);
    if (slot < 0) return slot == -2 ? RMX_ERR_INVALID : RMX_ERR_HIP;
    uint64_t bytes = 0;
    int max_w = 1, max_h = 1;
    for (int i = 0; i < op->n; i++) {
        RmxSample &s = t[i];
        int rc = read_roi(op, src_roi, i, &s.src_x, &s.src_y, &s.src_w, &s.src_h);
        if (rc) return rc;
        s.src_w = std::min<int32_t>(s.src_w, (int32_t)op->dst.h);  // the window's width becomes the output's height
        s.src_h = std::min<int32_t>(s.src_h, (int32_t)op->dst.w);
        s.dst_w = s.src_h;
        s.dst_h = s.src_w;
        s.flags = 0;
        bytes += (uint64_t)s.src_w * s.src_h * 3 * (1 + dtype_size(op->dst.dtype));
        max_w = std::max(max_w, (int)s.src_w);
        max_h = std::max(max_h, (int)s.src_h);
    }
    op->algo_bytes = bytes;
    const int tiles_x = (max_w + 31) / 32, tiles_y = (max_h + 31) / 32;
    op->strips = tiles_x * tiles_y;
    op->aux0 = tiles_x;
    op->lds_per_wave = 0;
    op->waves_per_block = 4;
    op->fn_fast = nullptr;
    return commit_slot(op, slot);
}

/* ------------------------------------------------------------------ K2 family */

int rmx_create_resize(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int interpolation, int roi_type, uint32_t flags, rmx_op **out) {
    if (interpolation != RMX_INTERP_LINEAR && interpolation != RMX_INTERP_NEAREST && interpolation != RMX_INTERP_TRIANGULAR) {
        if (out) *out = nullptr;
        return fail(RMX_ERR_UNSUPPORTED, "interpolation %d is outside the hot path (nearest=0, linear=1, triangular=5)", interpolation);
    }
    const uint32_t chain = flags & (RMX_F_COLOR_LINEAR | RMX_F_COLOR_TWIST);
    if (chain) {
        if (out) *out = nullptr;
        if (chain == (RMX_F_COLOR_LINEAR | RMX_F_COLOR_TWIST)) return fail(RMX_ERR_INVALID, "a fused chain holds one colour node: linear or twist, not both");
        if (!(flags & RMX_F_QUANTIZE_U8)) return fail(RMX_ERR_INVALID, "a colour node in the chain reads the u8 output of the resize node: RMX_F_QUANTIZE_U8 is required");
        if (interpolation != RMX_INTERP_LINEAR) return fail(RMX_ERR_UNSUPPORTED, "the fused colour chain is built for bilinear resize only");
    }
    int rc = make_op(ctx, OP_RESIZE, src, dst, roi_type, out);
    if (rc) return rc;
    (*out)->interp = interpolation;
    (*out)->flags = flags;
    return RMX_OK;
}

// the kernels' source-coordinate law, evaluated on the host in the same fp32 operation order
static inline float src_coord_h(int u, float ratio, float off, float lo) {
    float s = (float)u * ratio;
    s = s + off;
    s = s + lo;
    return s;
}

// Upper bound of floor(c(u + d)) - floor(c(u)) for the kernels' coordinate law c(u) = u*ratio + off + lo evaluated in
// fp32: the exact coordinates lie d*ratio apart, and each computed one carries three roundings of at most half an ulp
// at a magnitude below `mag` (8 ulps of slack cover both ends). Used to size LDS windows without walking the rows.
static inline int span_bound(int d, float ratio, float mag) {
    if (d <= 0) return 1;
    return (int)std::floor((double)d * (double)ratio + 8.0 * 5.9604645e-8 * (double)mag) + 1;
}

// Static LDS the resize kernels hold besides their dynamic slices (the colour tables of a fused twist stage); the
// planners keep this much of a workgroup's LDS free.
constexpr int kStaticLdsMax = 2048;

static int plan_resize(rmx_op *op, RmxSample *t, bool norm) {
    const bool quant = (op->flags & RMX_F_QUANTIZE_U8) != 0;
    const int chain = (op->flags & RMX_F_COLOR_LINEAR) ? 1 : (op->flags & RMX_F_COLOR_TWIST) ? 2 : 0;
    // a quantised value that is not normalised is stored through an identity FMA
    const bool knorm = norm || (quant && op->dst.dtype != RMX_UINT8);
    op->norm = knorm;
    op->quant = quant && knorm;
    int max_dw = 1, max_dh = 1;
    for (int i = 0; i < op->n; i++) {
        max_dw = std::max(max_dw, (int)t[i].dst_w);
        max_dh = std::max(max_dh, (int)t[i].dst_h);
    }
    if (op->interp == RMX_INTERP_TRIANGULAR) {
        op->fn = rmx::select_resize_tri_kernel(op->dst.dtype, op->dst.layout, op->norm, op->quant, &op->kernel_name);
        if (!op->fn) return fail(RMX_ERR_UNSUPPORTED, "triangular resize kernel not available");
        // 128 output columns per wave (two per lane); ring of horizontally filtered rows per wave
        int tile_w = 128;
        float max_ry = 1.0f, max_rx = 1.0f;
        for (int i = 0; i < op->n; i++) {
            if (t[i].dst_w <= 0 || t[i].dst_h <= 0) continue;
            max_rx = std::max(max_rx, t[i].rx);
            max_ry = std::max(max_ry, t[i].ry);
        }
        const int ky = (int)std::ceil(2.0f * max_ry);
        const int kx_cap = (int)std::ceil(2.0f * max_rx);
        int ring_rows = 2;
        while (ring_rows < ky + 1) ring_rows *= 2;
        const int src_cols = std::min<int>((int)op->src.w, (int)std::ceil(tile_w * (double)max_rx) + kx_cap + 4);
        const int src_pitch = ((src_cols + 3) / 4) * 4 + 8 + 2 * ((kx_cap + 3) / 4 * 4);  // + room for the repeated border columns
        // LDS slice: coef[kx_cap][128] (only above 8 taps) | ring[ring_rows][3][128] | srcrow[3][src_pitch]
        size_t words = (size_t)(kx_cap > 8 ? kx_cap : 0) * tile_w + (size_t)ring_rows * 3 * tile_w + 3 * (size_t)src_pitch;  // 3 = rows per staging batch
        op->lds_per_wave = (int)((words * 4 + 15) / 16 * 16);
        if ((uint64_t)op->src.h * op->src.w * 3 >= (1ull << 32) || op->src.w * 3ull >= (1ull << 23) || op->src.h >= (1u << 23))
            return fail(RMX_ERR_UNSUPPORTED, "triangular resize: a source sample of %u x %u pixels is beyond the kernel's 32-bit offsets", op->src.w, op->src.h);
        if (op->lds_per_wave > op->ctx->max_lds_per_block || kx_cap > 0xffff)
            return fail(RMX_ERR_UNSUPPORTED, "triangular resize with scale %.1f x %.1f needs %d bytes of LDS per wave", max_rx, max_ry, op->lds_per_wave);
        // Downscaling variant: no ring. Usable when every sample shrinks vertically, has at most 8 horizontal
        // taps, and no source row is read by output rows more than three apart (four rows are in flight):
        // first row of r+4 strictly below the last row of r, evaluated with the kernel's own fp32 law.
        // A sample that grows vertically (two taps, several output rows per source row) needs eight rows in flight, which
        // the streaming form has for ratios from about 0.26 on: first row of r+8 strictly below the last row of r.
        bool down = kx_cap <= 8 && !op->ctx->tri_ring;
        int flight = 4;  // rows in flight the batch needs
        for (int i = 0; i < op->n && down; i++) {
            const RmxSample &s = t[i];
            if (s.dst_w <= 0 || s.dst_h <= 0) continue;
            if (!(s.ry > 0.0f)) {  // (also a NaN)
                down = false;
                break;
            }
            const int apart = s.ry >= 1.0f ? 4 : 8;
            flight = std::max(flight, apart);
            const float radius = s.ry > 1.0f ? s.ry : 1.0f;
            const float offset = (s.ry - 1) * 0.5f - radius;
            const int ksz = (int)std::ceil(radius * 2);
            const int ylo = s.src_y, yhi = s.src_y + s.src_h - 1;
            auto loc_of = [&](int r) {
                float raw = (float)(s.pc_y + r) * s.ry;
                raw = raw + offset;
                raw = raw + (float)ylo;
                return (int)std::ceil(raw);
            };
            if (s.dst_h <= apart) continue;
            // Interior rows: the first taps of rows `apart` apart lie at least floor(apart*ry - rounding slack) source rows
            // apart, which must reach past the ksz taps of the upper row. At the window's ends the clamp can fold two
            // rows onto the same source row: that happens exactly when row `apart` starts at or above the first source
            // row, or the taps of the last row but `apart` reach the last one (first taps are monotone in the row index).
            const double slack = 8.0 * 5.9604645e-8 * (double)(s.src_y + s.src_h + 2);
            if ((int)std::floor((double)apart * (double)s.ry - slack) >= ksz) {
                down = loc_of(apart) > ylo && loc_of(s.dst_h - apart - 1) + ksz - 1 < yhi;
                continue;
            }
            for (int r = 0; r + apart < s.dst_h && down; r++) {  // ratios just above 1 or just above 1/4: walk the rows
                const int last = std::max(std::min(loc_of(r) + ksz - 1, yhi), ylo);
                const int first = std::max(std::min(loc_of(r + apart), yhi), ylo);
                down = first > last;
            }
        }
        int rows = op->ctx->tri_rows > 0 ? op->ctx->tri_rows : 12;
        bool sort_rows = false;
        // Streaming form of the downscaling variant (source rows straight into LDS as raw bytes): every source row must start
        // at the same byte phase (row stride a multiple of 4), and four LDS rows of the widest tile plus the table of vertical
        // coefficients must leave room for ten wavefronts per CU at least.
        op->tri_rows_in_flight = 0;
        bool tdma = down && op->ctx->dma && op->ctx->tri_tpx == 2 && ky <= 16;
        if (flight > 4 && (!tdma || op->ctx->tri_slots == 4)) down = tdma = false;  // (only the streaming form has eight)
        if (tdma) {
            if (op->layout.empty()) tdma = (op->src.w * 3u) % 4u == 0;
            else
                for (int i = 0; i < op->n && tdma; i++) tdma = op->layout[i].row_stride % 4u == 0;
        }
        if (tdma) {
            // The widest LDS row over all tiles, by the kernel's own fp32 law for a tile's first and last tap (its byte phase
            // inside a dword is taken at its worst, 3).
            size_t pitch_max = 64;
            for (int i = 0; i < op->n && tdma; i++) {
                const RmxSample &s = t[i];
                if (s.dst_w <= 0 || s.dst_h <= 0) continue;
                const float radius = s.rx > 1.0f ? s.rx : 1.0f;
                const float offset = (s.rx - 1) * 0.5f - radius;
                const int kxi = (int)std::ceil(radius * 2);
                const int xlo = s.src_x, xhi = s.src_x + s.src_w - 1;
                auto loc_of = [&](int d) {
                    float raw = (float)d * s.rx;
                    raw = raw + offset;
                    raw = raw + (float)xlo;
                    return (int)std::ceil(raw);
                };
                for (int xt = 0; xt < (int)s.dst_w; xt += 128) {
                    const int tw = std::min(128, (int)s.dst_w - xt);
                    const int lf = loc_of(s.pc_x + xt), ll = loc_of(s.pc_x + xt + tw - 1);
                    const int cs = std::max(std::min(lf, xhi), xlo), ce = std::max(std::min(ll + kxi - 1, xhi), xlo);
                    const int nrep_l = std::max(cs - lf, 0), nrep_r = std::max(ll + kxi - 1 - ce, 0);
                    const int nd = (3 + 3 * (ce - cs + 1) + 15) >> 4;
                    const int lm = ((3 * nrep_l + 15) >> 4) << 4;
                    const int body = std::max(3 + 3 * (ll + 8 - cs) + 8, 16 * nd);
                    const int pitch = lm + (((body + 15) >> 4) << 4);
                    if (pitch > 128 * 16 || 3 * (nrep_l + nrep_r) > 64) tdma = false;
                    pitch_max = std::max(pitch_max, (size_t)pitch);
                }
            }
            // ring of four source rows (six were measured: 18 instead of 20 wavefronts per CU, a fifth slower) + vertical
            // coefficients: 64 source rows and 16 passes x 4 slots
            const size_t lds = 4 * pitch_max + (64 + 16) * (size_t)flight * 4;
            if (lds > 16 * 1024) tdma = false;
            if (tdma) {
                // Two output rows in flight instead of four when rows two apart never read the same source row. That holds
                // for a vertical ratio that is a whole or a half number: every product and sum of the kernel's coordinate
                // law is then exact in fp32 (multiples of 1/4 below 2^20), the first taps of rows two apart lie exactly
                // 2 x ratio = taps rows apart, and only the clamp at the window's ends could fold two such rows onto one
                // source row: when row 2 starts at or above the first source row, or the taps of the last row but two
                // reach the last one.
                bool two = op->ctx->tri_slots != 4 && flight == 4;
                for (int i = 0; i < op->n && two; i++) {
                    const RmxSample &s = t[i];
                    if (s.dst_w <= 0 || s.dst_h <= 2) continue;
                    const float twice = s.ry * 2.0f;
                    const int ylo = s.src_y, yhi = s.src_y + s.src_h - 1;
                    if (twice != std::floor(twice) || twice > 32.0f || (double)(s.pc_y + s.dst_h) * (double)s.ry + (double)yhi > 1048576.0) {
                        two = false;
                        break;
                    }
                    const float radius = s.ry > 1.0f ? s.ry : 1.0f;
                    const float offset = (s.ry - 1) * 0.5f - radius;
                    const int ksz = (int)std::ceil(radius * 2);
                    auto loc_of = [&](int r) {
                        float raw = (float)(s.pc_y + r) * s.ry;
                        raw = raw + offset;
                        raw = raw + (float)ylo;
                        return (int)std::ceil(raw);
                    };
                    two = loc_of(2) > ylo && loc_of((int)s.dst_h - 3) + ksz - 1 < yhi;
                }
                op->tri_rows_in_flight = two ? 2 : flight;
                op->fn = rmx::select_resize_tri_dma_kernel(op->dst.dtype, op->dst.layout, op->norm, op->quant, op->tri_rows_in_flight, &op->kernel_name);
                op->lds_per_wave = (int)lds;
            }
        }
        if (!tdma && flight > 4) down = false;  // (the kernel that stages through registers keeps four rows in flight)
        if (down && !tdma) {
            tile_w = 64 * op->ctx->tri_tpx;
            op->fn = rmx::select_resize_tri_down_kernel(op->dst.dtype, op->dst.layout, op->norm, op->quant, op->ctx->tri_tpx, &op->kernel_name);
            // LDS slice: the rows of one staging round (four 16-byte loads per lane = 4, 2 or 1 rows, by row length)
            size_t lds = 0;
            for (int i = 0; i < op->n; i++) {
                const RmxSample &s = t[i];
                if (s.dst_w <= 0 || s.dst_h <= 0) continue;
                const int kxi = (int)std::ceil(2.0f * std::max(s.rx, 1.0f));
                const int cols = std::min<int>((int)op->src.w, (int)std::ceil(tile_w * (double)std::max(s.rx, 1.0f)) + kxi + 4);
                const int pitch = ((cols + 3) / 4) * 4 + 8 + 2 * ((kxi + 3) / 4 * 4);
                // (a tile's own row can be shorter than this bound: then more rows go into a round)
                const int pads = 8 + 2 * ((kxi + 3) / 4 * 4);
                const int need = std::max(pitch, std::max(2 * std::min(pitch, 512 + pads), 4 * std::min(pitch, 256 + pads)));
                lds = std::max(lds, (size_t)need * 4);
            }
            // the staged source rows and the table of vertical coefficients (64 source rows x 4 output rows in flight)
            op->lds_per_wave = (int)((std::max<size_t>(lds, 64) + 15) / 16 * 16) + 64 * 4 * 4;
            if (op->lds_per_wave > op->ctx->max_lds_per_block)
                return fail(RMX_ERR_UNSUPPORTED, "triangular resize needs %d bytes of LDS per wave", op->lds_per_wave);
        }
        if (down) {
            // Rows per strip: a strip of R rows filters R*ratio + taps source rows, and the device runs the strips in
            // rounds of (wavefront slots) at a time; pick the R with the least rounds x rows-per-strip. Measured on
            // MI355X: a batch of equal strips that march in step runs 10-20 % slower than one whose last strip of each
            // image is a short one, so an R that leaves a remainder of at most R/2 rows is preferred.
            // A batch whose samples differ in vertical ratio (RandomResizedCrop windows: a strip of one sample filters
            // several times the source rows of a strip of another)
            float min_ry = max_ry;
            for (int i = 0; i < op->n; i++)
                if (t[i].dst_w > 0 && t[i].dst_h > 0) min_ry = std::min(min_ry, t[i].ry);
            const bool ragged_cost = max_ry > 1.5f * min_ry;
            sort_rows = ragged_cost;
            if (op->ctx->tri_rows == 0) {
                // (wavefronts per CU: 16 by the registers of the kernel that stages through registers, 20 by those of the streaming
                // one, 24 when it keeps two rows in flight)
                const int by_regs = tdma ? (op->tri_rows_in_flight == 2 ? 24 : (op->tri_rows_in_flight == 8 ? 16 : 20)) : 16;
                const int per_cu = op->ctx->tri_per_cu > 0 ? op->ctx->tri_per_cu : std::max(1, std::min(by_regs, (160 * 1024) / op->lds_per_wave));
                const long slots = (long)op->ctx->num_cus * per_cu;
                // Such a batch is only spread evenly over the device when there are several strips per wavefront slot for the
                // hardware to deal out as slots fall free. Measured on 256 such windows to 224 x 224: strips of 30 rows (one
                // per slot) 80.9 us, of 8 rows (3.5 per slot) 69.2 us.
                double best_cost = 0.0;
                for (int r = 4; r <= 64; r++) {
                    long waves = 0;
                    for (int i = 0; i < op->n; i++)
                        if (t[i].dst_w > 0 && t[i].dst_h > 0) waves += (long)((t[i].dst_w + tile_w - 1) / tile_w) * ((t[i].dst_h + r - 1) / r);
                    if (ragged_cost) {
                        // the tallest strips that still leave three per slot; two when the rows go out largest window first (below),
                        // which evens the slots out by itself (same windows, sorted: strips of 9 / 14 / 19 rows 62.8 / 57.1 / 62.8 us)
                        if (r > 4 && waves < (op->ctx->tri_sort ? 2 : 3) * slots) break;
                        rows = r;
                        continue;
                    }
                    const long rounds = std::max(1L, (waves + slots - 1) / slots);
                    const int rem = max_dh % r;
                    const double cost = (double)rounds * (r * (double)max_ry + ky) * ((rem == 0 || 2 * rem > r) ? 1.15 : 1.0);
                    if (best_cost == 0.0 || cost < best_cost) {
                        best_cost = cost;
                        rows = r;
                    }
                }
            }
        }
        op->waves_per_block = std::max(1, std::min(op->ctx->tri_wpb, op->ctx->max_lds_per_block / op->lds_per_wave));
        op->tile_w = tile_w;
        const int xtiles = (max_dw + tile_w - 1) / tile_w;
        op->aux1 = xtiles;
        op->strip_rows = rows;
        op->aux0 = op->strip_rows;
        const int ystrips = (max_dh + op->strip_rows - 1) / op->strip_rows;
        op->strips = xtiles * ystrips;
        for (int i = 0; i < op->n; i++) t[i].strip_rows = (ring_rows << 16) | kx_cap;
        // A batch whose samples differ in cost goes to the device largest window first: the hardware deals the strips out in
        // launch order as wavefront slots fall free, so the launch ends with the small windows instead of waiting for a
        // large one that started late (measured on 256 RandomResizedCrop windows: 66.4 -> 62.2 us). Only the ROWS change
        // places; each carries its sample's index (plan[2]), from which the kernels address source and destination.
        if (sort_rows && op->ctx->tri_sort) {
            std::vector<int> order(op->n);
            for (int i = 0; i < op->n; i++) order[i] = i;
            std::stable_sort(order.begin(), order.end(), [&](int x, int y) {
                return (int64_t)t[x].src_w * t[x].src_h > (int64_t)t[y].src_w * t[y].src_h;
            });
            std::vector<RmxSample> rows(t, t + op->n);
            for (int i = 0; i < op->n; i++) t[i] = rows[order[i]];
        }
        return RMX_OK;
    }
    const char *nm = nullptr;
    op->fn = (op->interp == RMX_INTERP_NEAREST)
                 ? rmx::select_resize_nearest_kernel(op->dst.dtype, op->dst.layout, op->norm, op->quant, &nm)
                 : rmx::select_resize_linear_kernel(op->dst.dtype, op->dst.layout, op->norm, op->quant, chain, &nm);
    op->kernel_name = nm;
    // Both plans below size LDS from closed-form bounds (span_bound), a handful of operations per sample: the update
    // runs once per batch on the thread that also launches, and must not cost more than the kernel it plans.
    // General kernel: x-tile of up to 64 lanes x 8 px; each wave keeps a ring of R staged source rows in LDS.
    int tile_w = std::min(((max_dw + 7) / 8) * 8, 512);
    const int budget = 16 * 1024;
    const int grows = op->ctx->gen_rows;
    int lds = 0;
    for (;;) {
        lds = 0;
        for (int i = 0; i < op->n; i++) {
            RmxSample &s = t[i];
            if (s.dst_w <= 0 || s.dst_h <= 0) {
                s.strip_rows = 1;
                continue;
            }
            // the last (narrowest) tile has the most rows per step: G = 64 / lanes per row
            const int tw_last = s.dst_w - ((s.dst_w - 1) / tile_w) * tile_w;
            const int G = 64 / ((tw_last + 7) / 8);
            const float magx = (float)(s.src_x + s.src_w + 2), magy = (float)(s.src_y + s.src_h + 2);
            const int ring = std::min<int>(s.src_h + 2, span_bound(std::min(std::min(G, grows), (int)s.dst_h) - 1, s.ry, magy) + 2);
            const int nc = std::min<int>(s.src_w, span_bound(std::min<int>(tile_w, s.dst_w) - 1, s.rx, magx) + 2);
            const int pitch = 4 + ((nc + 3) >> 2) * 4 + 4;
            s.strip_rows = ring;
            lds = std::max(lds, ring * pitch * 4);
        }
        if (lds <= budget || tile_w <= 64) break;
        tile_w = std::max(64, (tile_w / 2 + 7) / 8 * 8);
    }
    op->lds_per_wave = (lds + 15) / 16 * 16;
    if (op->lds_per_wave > op->ctx->max_lds_per_block - kStaticLdsMax)
        return fail(RMX_ERR_UNSUPPORTED, "resize plan needs %d bytes of LDS per wave", op->lds_per_wave);
    op->waves_per_block = std::max(1, std::min(4, (op->ctx->max_lds_per_block - kStaticLdsMax) / std::max(1, op->lds_per_wave)));
    op->tile_w = tile_w;
    op->aux1 = tile_w;
    // strips: short ones. A wave's steps are serialised by memory latency, so many short-lived
    // waves (several residency rounds) overlap better than one long-lived wave per slot; the
    // price is one extra window of source rows per strip. 8 rows measured best on MI355X.
    op->strip_rows = grows;
    op->aux0 = grows;
    op->strips = std::max(1, (max_dh + grows - 1) / grows);
    // fast path: every written width a multiple of 8 and aligned destination rows. Its wavefronts stage
    // the whole source window of a strip of `rows` destination rows at once; the x-tile of a sample is
    // narrowed until that window fits the LDS budget of one wavefront.
    op->fn_fast = nullptr;
    op->fn_mid = nullptr;
    if (op->interp == RMX_INTERP_LINEAR) {
        // (the kernels multiply row indices and the row stride with 24-bit multiplies)
        const bool base_ok = op->src.w * 3u < (1u << 23) && op->src.h < (1u << 23);
        bool widths8 = op->dst.w % 8 == 0;
        for (int i = 0; i < op->n && widths8; i++) widths8 = t[i].dst_w % 8 == 0;
        bool ok = base_ok && widths8;
        // 4 rows and a 10 KB slice measured best on MI355X (more, shorter-lived wavefronts per CU)
        const int rows = op->ctx->fast_rows, cap = op->ctx->fast_lds;
        const TileCost tile_cost(rows);
        int need_max = 64;
        for (int i = 0; i < op->n && ok; i++) {
            RmxSample &s = t[i];
            s.plan[0] = 8;
            if (s.dst_w % 8 != 0) {
                ok = false;
                break;
            }
            if (s.dst_w <= 0 || s.dst_h <= 0) continue;
            const float magx = (float)(s.src_x + s.src_w + 2), magy = (float)(s.src_y + s.src_h + 2);
            const int nrows = std::max(2, span_bound(std::min<int>(rows, s.dst_h) - 1, s.ry, magy) + 2);
            long need = 0;
            const int tw = pick_tile_width((int)s.dst_w, tile_cost, cap, [&](int w) {
                const int nc = std::min<int>(s.src_w, span_bound(w - 1, s.rx, magx) + 2);
                return (long)nrows * (8 + ((nc + 3) >> 2) * 4) * 4;  // bytes: one dword per pixel + replicas
            }, &need);
            if (tw == 0) {
                ok = false;  // a window this tall does not fit: the general kernel takes the batch
                break;
            }
            s.plan[0] = tw;
            need_max = std::max<int>(need_max, (int)need);
        }
        if (ok) {
            op->fn_fast = rmx::select_resize_fast_kernel(op->dst.dtype, op->dst.layout, op->norm, op->quant, chain, &op->fast_name);
            op->fast_lds = (need_max + 15) / 16 * 16;
            // interleaved fp32 output: room for the slab through which the lanes of a row exchange their runs before storing
            // (64 lanes x the 24 dwords of one lane's run; the kernel takes it from the tail of the slice)
            if (op->dst.dtype == RMX_FP32 && op->dst.layout == RMX_NHWC) op->fast_lds += 64 * 4 * 24;
            op->fast_rows = rows;
            op->fast_strips = std::max(1, (max_dh + rows - 1) / rows);
            // (default 1: a workgroup's LDS is released only when its last wavefront ends, one-wave groups keep the CU full)
            op->fast_wpb = std::max(1, std::min(op->ctx->fast_wpb, (op->ctx->max_lds_per_block - kStaticLdsMax) / std::max(1, op->fast_lds)));
            op->fast_needs_src16 = false;  // its loads only need dword alignment
            op->fast_aux1 = 0;
            if (op->fast_lds > op->ctx->max_lds_per_block - kStaticLdsMax) op->fn_fast = nullptr;
        }
        // Streaming kernel (source rows straight into LDS): needs every source row to start at the same byte phase (row stride
        // a multiple of 4). Its any-width form serves every destination; the form for whole groups and aligned rows replaces
        // the staged kernel above where that applies.
        bool dma = base_ok && op->ctx->dma;
        if (dma) {
            if (op->layout.empty()) dma = (op->src.w * 3u) % 4u == 0;
            else
                for (int i = 0; i < op->n && dma; i++) dma = op->layout[i].row_stride % 4u == 0;
        }
        if (dma) {
            // 10 KB measured best on MI355X: smaller caps cut more rows into two tiles, and the kernel's registers allow 16
            // wavefronts per CU, which 10 KB each still fit
            const int bufcap = op->ctx->dma_lds;
            int need_max = 64;
            for (int i = 0; i < op->n && dma; i++) {
                RmxSample &s = t[i];
                s.plan[1] = 8;
                if (s.dst_w <= 0 || s.dst_h <= 0) continue;
                const float magx = (float)(s.src_x + s.src_w + 2), magy = (float)(s.src_y + s.src_h + 2);
                const int nrows = std::max(2, span_bound(std::min<int>(rows, s.dst_h) - 1, s.ry, magy) + 2);
                long need = 0;
                const int tw = pick_tile_width((int)s.dst_w, tile_cost, bufcap, [&](int w) {
                    const int nc = std::min<int>(s.src_w, span_bound(w - 1, s.rx, magx) + 2);
                    return (long)nrows * (1 + ((3 + 3 * (nc + 2) + 8 + 15) >> 4)) * 16;  // margin piece + data + replicas
                }, &need);
                if (tw == 0) {
                    dma = false;
                    break;
                }
                s.plan[1] = tw;
                need_max = std::max<int>(need_max, (int)need);
            }
            if (dma && need_max <= op->ctx->max_lds_per_block - kStaticLdsMax) {
                // A wavefront works through `group` windows (of `rows` destination rows) below each other per x-tile, so that the
                // tile's x taps are computed once for all of them (1 measured best: more leave too few wavefronts to fill the chip evenly).
                const long windows = (long)op->n * ((max_dh + rows - 1) / rows);
                const int group = op->ctx->dma_group ? op->ctx->dma_group : (int)std::max<long>(1, std::min<long>(8, windows / 4096));
                const int lds = (need_max + 15) / 16 * 16;
                const int strips = std::max(1, (max_dh + rows * group - 1) / (rows * group));
                const int wpb = std::max(1, std::min(op->ctx->fast_wpb, (op->ctx->max_lds_per_block - kStaticLdsMax) / std::max(1, lds)));
                op->fn_mid = rmx::select_resize_dma_kernel(op->dst.dtype, op->dst.layout, op->norm, op->quant, chain, false, &op->mid_name);
                op->mid_lds = lds;
                op->mid_rows = rows;
                op->mid_strips = strips;
                op->mid_wpb = wpb;
                op->mid_aux1 = group;
                const char *dname = nullptr;
                rmx::KernelFn dfn = widths8 ? rmx::select_resize_dma_kernel(op->dst.dtype, op->dst.layout, op->norm, op->quant, chain, true, &dname) : nullptr;
                if (dfn) {
                    op->fn_fast = dfn;
                    op->fast_name = dname;
                    op->fast_lds = lds;
                    op->fast_rows = rows;
                    op->fast_strips = strips;
                    op->fast_wpb = wpb;
                    op->fast_aux1 = group;
                    op->fast_needs_src16 = false;
                }
            }
        }
    }
    return RMX_OK;
}

static float hue_to_sextants(float hue_deg);

// Rows and launch plan of a resize-family batch into the host table `t` (n rows); touches no device state.
static int fill_resize_rows(rmx_op *op, RmxSample *t, const uint32_t *src_roi, const uint32_t *dst_w, const uint32_t *dst_h,
                            const uint32_t *crop_roi, const float *scale, const float *bias,
                            const float *mean, const float *stddev, const uint32_t *mirror, const float *const *colour) {
    const uint32_t chain = op->flags & (RMX_F_COLOR_LINEAR | RMX_F_COLOR_TWIST);
    if (chain && !colour) return fail(RMX_ERR_INVALID, "this Resize node was created with a colour node in its chain: use rmx_update_resize_color_cmn");
    if (!chain && colour) return fail(RMX_ERR_INVALID, "this Resize node was created without a colour node in its chain");
    if (!dst_w || !dst_h) return fail(RMX_ERR_INVALID, "dst_w and dst_h arrays are required");
    if ((mean == nullptr) != (stddev == nullptr)) return fail(RMX_ERR_INVALID, "mean and stddev must be given together");
    if ((scale == nullptr) != (bias == nullptr)) return fail(RMX_ERR_INVALID, "scale and bias must be given together");
    uint64_t bytes = 0;
    const bool edge_ref = (op->flags & RMX_F_EDGE_REF) && op->interp == RMX_INTERP_LINEAR;
    for (int i = 0; i < op->n; i++) {
        RmxSample &s = t[i];
        int rc = read_roi(op, src_roi, i, &s.src_x, &s.src_y, &s.src_w, &s.src_h);
        if (rc) return rc;
        s.rs_w = (int32_t)dst_w[i];
        s.rs_h = (int32_t)dst_h[i];
        if (s.rs_w < 0 || s.rs_h < 0) return fail(RMX_ERR_INVALID, "sample %d: destination size out of range", i);
        if (crop_roi) {
            uint32_t cx = crop_roi[i * 4], cy = crop_roi[i * 4 + 1], cw = crop_roi[i * 4 + 2], chh = crop_roi[i * 4 + 3];
            if (cx > (uint32_t)s.rs_w || cy > (uint32_t)s.rs_h) return fail(RMX_ERR_INVALID, "sample %d: crop origin outside the resized image", i);
            s.pc_x = (int32_t)cx;
            s.pc_y = (int32_t)cy;
            s.dst_w = (int32_t)std::min<uint32_t>(cw, (uint32_t)s.rs_w - cx);
            s.dst_h = (int32_t)std::min<uint32_t>(chh, (uint32_t)s.rs_h - cy);
        } else {
            s.pc_x = s.pc_y = 0;
            s.dst_w = s.rs_w;
            s.dst_h = s.rs_h;
        }
        s.dst_w = std::min<int32_t>(s.dst_w, (int32_t)op->dst.w);
        s.dst_h = std::min<int32_t>(s.dst_h, (int32_t)op->dst.h);
        if (s.src_w <= 0 || s.src_h <= 0 || s.rs_w <= 0 || s.rs_h <= 0) s.dst_w = s.dst_h = 0;
        s.flags = ((mirror && mirror[i]) ? RMX_S_HFLIP : 0u) | (edge_ref ? RMX_S_EDGE_REF : 0u);
        if (s.dst_w > 0) {
            s.rx = (float)s.src_w / (float)s.rs_w;
            s.ry = (float)s.src_h / (float)s.rs_h;
            s.fsx = s.rx > 1.0f ? 1 / s.rx : 1.0f;
            s.fsy = s.ry > 1.0f ? 1 / s.ry : 1.0f;
        } else {
            s.rx = s.ry = s.fsx = s.fsy = 1.0f;
        }
        s.plan[2] = i;  // the sample this row belongs to (the triangular kernels take it from here: their rows may be reordered)
        for (int c = 0; c < 3; c++) {
            if (scale) {
                s.scale[c] = scale[i * 3 + c];
                s.bias[c] = bias[i * 3 + c];
            } else if (mean) {
                if (stddev[i * 3 + c] == 0.0f) return fail(RMX_ERR_INVALID, "sample %d: standard deviation of channel %d is 0", i, c);
                float inv = 1 / stddev[i * 3 + c];
                s.scale[c] = inv;
                s.bias[c] = -(mean[i * 3 + c] * inv);
            } else {
                s.scale[c] = 1.0f;
                s.bias[c] = 0.0f;
            }
        }
        if (chain == RMX_F_COLOR_LINEAR) {  // fma(x - c2, c0, c1)
            s.m[0] = colour[0] ? colour[0][i] : 1.0f;
            s.m[1] = colour[1] ? colour[1][i] : 0.0f;
            s.m[2] = colour[2] ? colour[2][i] : 0.0f;
            s.m[3] = 0.0f;
        } else if (chain == RMX_F_COLOR_TWIST) {  // alpha, beta, hue shift in sextants, saturation
            s.m[0] = colour[0] ? colour[0][i] : 1.0f;
            s.m[1] = colour[1] ? colour[1][i] : 0.0f;
            s.m[2] = colour[2] ? hue_to_sextants(colour[2][i]) : 0.0f;
            s.m[3] = colour[3] ? colour[3][i] : 1.0f;
        }
        // bytes of the source window actually mapped by the written window
        double fx = s.rs_w > 0 ? (double)s.dst_w / s.rs_w : 0, fy = s.rs_h > 0 ? (double)s.dst_h / s.rs_h : 0;
        bytes += (uint64_t)std::llround((double)s.src_w * s.src_h * fx * fy) * 3 +
                 (uint64_t)s.dst_w * s.dst_h * 3 * dtype_size(op->dst.dtype);
    }
    op->algo_bytes = bytes;
    return plan_resize(op, t, scale != nullptr || mean != nullptr);
}

static int update_resize_common(rmx_op *op, const uint32_t *src_roi, const uint32_t *dst_w, const uint32_t *dst_h,
                                const uint32_t *crop_roi, const float *scale, const float *bias,
                                const float *mean, const float *stddev, const uint32_t *mirror, const float *const *colour = nullptr) {
    if (!op || op->kind != OP_RESIZE) return fail(RMX_ERR_INVALID, "op is not a Resize node");
    RmxSample *t;
    int slot = next_slot(op, &t);
    if (slot < 0) return slot == -2 ? RMX_ERR_INVALID : RMX_ERR_HIP;
    int rc = fill_resize_rows(op, t, src_roi, dst_w, dst_h, crop_roi, scale, bias, mean, stddev, mirror, colour);
    if (rc) return rc;
    return commit_slot(op, slot);
}

int rmx_update_resize(rmx_op *op, const uint32_t *src_roi, const uint32_t *dst_w, const uint32_t *dst_h,
                      const uint32_t *mirror, const float *mean, const float *stddev) {
    return update_resize_common(op, src_roi, dst_w, dst_h, nullptr, nullptr, nullptr, mean, stddev, mirror);
}

int rmx_update_resize_cmn(rmx_op *op, const uint32_t *src_roi, const uint32_t *dst_w, const uint32_t *dst_h,
                          const uint32_t *crop_roi, const float *scale, const float *bias, const uint32_t *mirror) {
    if (!scale || !bias) return fail(RMX_ERR_INVALID, "scale and bias arrays are required");
    return update_resize_common(op, src_roi, dst_w, dst_h, crop_roi, scale, bias, nullptr, nullptr, mirror);
}

int rmx_update_resize_color_cmn(rmx_op *op, const uint32_t *src_roi, const uint32_t *dst_w, const uint32_t *dst_h, const uint32_t *crop_roi,
                                const float *scale, const float *bias, const uint32_t *mirror, const float *c0, const float *c1, const float *c2,
                                const float *c3) {
    if (!scale || !bias) return fail(RMX_ERR_INVALID, "scale and bias arrays are required");
    const float *colour[4] = {c0, c1, c2, c3};
    return update_resize_common(op, src_roi, dst_w, dst_h, crop_roi, scale, bias, nullptr, nullptr, mirror, colour);
}

/* ------------------------------------------------------------------ K3 family */

static int create_color(rmx_ctx *ctx, int kind, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int roi_type, rmx_op **out) {
    int rc = make_op(ctx, kind, src, dst, roi_type, out);
    if (rc) return rc;
    const bool twist = (kind == OP_COLOR_TWIST || kind == OP_HUE || kind == OP_SATURATION);
    (*out)->fn = rmx::select_color_kernel(twist ? 1 : 0, dst->dtype, dst->layout, 0, &(*out)->kernel_name);
    return RMX_OK;
}

// hue in degrees -> shift in sextants reduced to [0,6]
static float hue_to_sextants(float hue_deg) {
    float s = std::fmod(hue_deg, 360.0f);
    if (s < 0.0f) s += 360.0f;
    return s / 60.0f;
}

static int update_color(rmx_op *op, const uint32_t *roi, const float *p0, const float *p1, const float *p2, const float *p3,
                        float d0, float d1, float d2, float d3, bool hue_in_p2) {
    RmxSample *t;
    int slot = next_slot(op, &t);
    if (slot < 0) return slot == -2 ? RMX_ERR_INVALID : RMX_ERR_HIP;
    uint64_t bytes = 0;
    int max_rows = 1;
    for (int i = 0; i < op->n; i++) {
        RmxSample &s = t[i];
        int rc = read_roi(op, roi, i, &s.src_x, &s.src_y, &s.src_w, &s.src_h);
        if (rc) return rc;
        s.dst_w = std::min<int32_t>(s.src_w, (int32_t)op->dst.w);
        s.dst_h = std::min<int32_t>(s.src_h, (int32_t)op->dst.h);
        s.flags = 0;
        s.color[0] = p0 ? p0[i] : d0;
        s.color[1] = p1 ? p1[i] : d1;
        s.color[2] = p2 ? (hue_in_p2 ? hue_to_sextants(p2[i]) : p2[i]) : d2;
        s.color[3] = p3 ? p3[i] : d3;
        bytes += (uint64_t)s.dst_w * s.dst_h * 3 * (1 + dtype_size(op->dst.dtype));
        max_rows = std::max(max_rows, (int)s.dst_h);
    }
    op->algo_bytes = bytes;
    int rows = op->ctx->k3_rows;
    if (flatten_whole_frames(op, t)) {
        max_rows = op->flat_h;
        // (the twist takes one 512-pixel row per wavefront: measured on 256 frames of 224 x 224, 1 / 2 / 4 / 8 rows per
        // wavefront 20.2 / 20.3 / 20.9 / 24.4 us against 21.0 us on the images' own rows of 28 lanes)
        // (the linear kinds two: Exposure on the same frames 18.8 / 16.8 / 18.1 / 19.9 us against 17.9 us)
        const bool twist_kind = op->kind == OP_COLOR_TWIST || op->kind == OP_HUE || op->kind == OP_SATURATION;
        rows = op->ctx->k3_flat_rows ? op->ctx->k3_flat_rows : (twist_kind ? 1 : 2);
    }
    plan_streaming(op, max_rows, rows);
    // aligned specialisation: whole 8-pixel groups everywhere and 16-byte aligned destination rows
    bool aligned = op->flat_h ? true : op->dst.w % 8 == 0;
    for (int i = 0; i < op->n && aligned; i++) aligned = (t[i].dst_w % 8 == 0);
    op->fn_fast = nullptr;
    // kernel kind: 0 linear, 1 twist, 2 twist with one comparison for the hue's way back into range (no shift near one sextant)
    int kkind = 0;
    if (op->kind == OP_COLOR_TWIST || op->kind == OP_HUE || op->kind == OP_SATURATION) {
        kkind = 2;
        for (int i = 0; i < op->n && kkind == 2; i++)
            if (!(t[i].color[2] < RMX_HUE_SHIFT_LOW || t[i].color[2] >= RMX_HUE_SHIFT_HIGH)) kkind = 1;
    }
    if (aligned) {
        op->fn_fast = rmx::select_color_kernel(kkind, op->dst.dtype, op->dst.layout, 1, &op->fast_name);
        op->fast_strips = op->strips;
        op->fast_lds = 0;
        op->fast_rows = op->aux0;
        op->fast_wpb = op->waves_per_block;
        op->fast_needs_src16 = false;
    }
    // the same pipeline for rows of any width from 8 pixels on and a destination at any element
    bool wide8 = true;
    for (int i = 0; i < op->n && wide8; i++) wide8 = t[i].dst_w >= 8 || t[i].dst_w <= 0 || t[i].dst_h <= 0;
    op->fn_mid = nullptr;
    if (wide8) {
        op->fn_mid = rmx::select_color_kernel(kkind, op->dst.dtype, op->dst.layout, 2, &op->mid_name);
        op->mid_strips = op->strips;
        op->mid_lds = 0;
        op->mid_rows = op->aux0;
        op->mid_wpb = op->waves_per_block;
        op->mid_aux1 = op->aux1;
    }
    return commit_slot(op, slot);
}

int rmx_create_color_twist(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int roi_type, rmx_op **out) {
    return create_color(ctx, OP_COLOR_TWIST, src, dst, roi_type, out);
}
int rmx_update_color_twist(rmx_op *op, const uint32_t *src_roi, const float *alpha, const float *beta, const float *hue_deg, const float *sat) {
    if (!op || op->kind != OP_COLOR_TWIST) return fail(RMX_ERR_INVALID, "op is not a ColorTwist node");
    if (!alpha || !beta || !hue_deg || !sat) return fail(RMX_ERR_INVALID, "alpha, beta, hue and sat arrays are required");
    return update_color(op, src_roi, alpha, beta, hue_deg, sat, 1, 0, 0, 1, true);
}
int rmx_create_brightness(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int roi_type, rmx_op **out) {
    return create_color(ctx, OP_BRIGHTNESS, src, dst, roi_type, out);
}
int rmx_update_brightness(rmx_op *op, const uint32_t *src_roi, const float *alpha, const float *beta) {
    if (!op || op->kind != OP_BRIGHTNESS) return fail(RMX_ERR_INVALID, "op is not a Brightness node");
    if (!alpha || !beta) return fail(RMX_ERR_INVALID, "alpha and beta arrays are required");
    return update_color(op, src_roi, alpha, beta, nullptr, nullptr, 1, 0, 0, 0, false);
}
int rmx_create_contrast(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int roi_type, rmx_op **out) {
    return create_color(ctx, OP_CONTRAST, src, dst, roi_type, out);
}
int rmx_update_contrast(rmx_op *op, const uint32_t *src_roi, const float *factor, const float *center) {
    if (!op || op->kind != OP_CONTRAST) return fail(RMX_ERR_INVALID, "op is not a Contrast node");
    if (!factor || !center) return fail(RMX_ERR_INVALID, "factor and center arrays are required");
    // out = fma(x - center, factor, center)
    return update_color(op, src_roi, factor, center, center, nullptr, 1, 0, 0, 0, false);
}
int rmx_create_hue(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int roi_type, rmx_op **out) {
    return create_color(ctx, OP_HUE, src, dst, roi_type, out);
}
int rmx_update_hue(rmx_op *op, const uint32_t *src_roi, const float *hue_deg) {
    if (!op || op->kind != OP_HUE) return fail(RMX_ERR_INVALID, "op is not a Hue node");
    if (!hue_deg) return fail(RMX_ERR_INVALID, "hue array is required");
    return update_color(op, src_roi, nullptr, nullptr, hue_deg, nullptr, 1, 0, 0, 1, true);
}
int rmx_create_saturation(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int roi_type, rmx_op **out) {
    return create_color(ctx, OP_SATURATION, src, dst, roi_type, out);
}
int rmx_update_saturation(rmx_op *op, const uint32_t *src_roi, const float *sat) {
    if (!op || op->kind != OP_SATURATION) return fail(RMX_ERR_INVALID, "op is not a Saturation node");
    if (!sat) return fail(RMX_ERR_INVALID, "sat array is required");
    return update_color(op, src_roi, nullptr, nullptr, nullptr, sat, 1, 0, 0, 1, true);
}

/* ------------------------------------------------------------------ streaming neighbours of K3 / K1 */

int rmx_create_exposure(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int roi_type, rmx_op **out) {
    return create_color(ctx, OP_EXPOSURE, src, dst, roi_type, out);
}
int rmx_update_exposure(rmx_op *op, const uint32_t *src_roi, const float *factor) {
    if (!op || op->kind != OP_EXPOSURE) return fail(RMX_ERR_INVALID, "op is not an Exposure node");
    if (!factor) return fail(RMX_ERR_INVALID, "exposure factor array is required");
    // out = x * 2^factor: the multiplier is made once per sample on the host, the kernel multiplies
    std::vector<float> m((size_t)op->n);
    for (int i = 0; i < op->n; i++) m[i] = exp2f(factor[i]);
    return update_color(op, src_roi, m.data(), nullptr, nullptr, nullptr, 1, 0, 0, 0, false);
}

int rmx_create_color_temperature(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int roi_type, rmx_op **out) {
    return create_k1(ctx, OP_COLOR_TEMPERATURE, src, dst, roi_type, true, out);
}
int rmx_update_color_temperature(rmx_op *op, const uint32_t *src_roi, const int32_t *adjustment) {
    if (!op || op->kind != OP_COLOR_TEMPERATURE) return fail(RMX_ERR_INVALID, "op is not a ColorTemperature node");
    if (!adjustment) return fail(RMX_ERR_INVALID, "adjustment array is required");
    // red + adj, green, blue - adj: a per-channel offset with unit scale, which is what the K1 kernel computes
    std::vector<float> bias((size_t)op->n * 3);
    for (int i = 0; i < op->n; i++) {
        bias[(size_t)i * 3 + 0] = (float)adjustment[i];
        bias[(size_t)i * 3 + 1] = 0.0f;
        bias[(size_t)i * 3 + 2] = -(float)adjustment[i];
    }
    return update_k1(op, src_roi, nullptr, bias.data(), nullptr, nullptr);
}

static int create_point(rmx_ctx *ctx, int kind, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int roi_type, rmx_op **out) {
    int rc = make_op(ctx, kind, src, dst, roi_type, out, kind == OP_GAMMA ? 256 : 0);
    if (rc) return rc;
    (*out)->fn = rmx::select_point_kernel(kind == OP_BLEND ? 1 : 0, dst->dtype, dst->layout, 0, &(*out)->kernel_name);
    if (kind == OP_GAMMA) {
        (*out)->lut_gamma.assign((size_t)(*out)->n, std::numeric_limits<float>::quiet_NaN());
        (*out)->lut_cache.assign((size_t)(*out)->n * 256, 0);
    }
    return RMX_OK;
}

// rows and launch plan of a one-pass op that writes the source window to the destination's origin
static int update_point(rmx_op *op, const uint32_t *roi, const float *p0, const float *gamma) {
    RmxSample *t;
    int slot = next_slot(op, &t);
    if (slot < 0) return slot == -2 ? RMX_ERR_INVALID : RMX_ERR_HIP;
    uint64_t bytes = 0;
    int max_rows = 1;
    const int sources = op->kind == OP_BLEND ? 2 : 1;
    uint8_t *lut = slot_extra(op, t);
    for (int i = 0; i < op->n; i++) {
        RmxSample &s = t[i];
        int rc = read_roi(op, roi, i, &s.src_x, &s.src_y, &s.src_w, &s.src_h);
        if (rc) return rc;
        s.dst_w = std::min<int32_t>(s.src_w, (int32_t)op->dst.w);
        s.dst_h = std::min<int32_t>(s.src_h, (int32_t)op->dst.h);
        s.flags = 0;
        s.color[0] = p0 ? p0[i] : 0.0f;
        s.color[1] = s.color[2] = s.color[3] = 0.0f;
        if (gamma) {
            // lut[v] = u8 store (round to nearest even, saturate) of powf(v/255, gamma)*255; rebuilt only when the sample's
            // exponent changed since the last update (a fixed gamma costs 256 powf per sample once, not per batch)
            uint8_t *mine = op->lut_cache.data() + (size_t)i * 256;
            if (!(op->lut_gamma[i] == gamma[i])) {
                for (int v = 0; v < 256; v++) {
                    float r = rintf(powf((float)v / 255.0f, gamma[i]) * 255.0f);
                    r = !(r > 0.0f) ? 0.0f : (r > 255.0f ? 255.0f : r);  // a NaN becomes 0
                    mine[v] = (uint8_t)r;
                }
                op->lut_gamma[i] = gamma[i];
            }
            memcpy(lut + (size_t)i * 256, mine, 256);
        }
        bytes += (uint64_t)s.dst_w * s.dst_h * 3 * (sources + dtype_size(op->dst.dtype));
        max_rows = std::max(max_rows, (int)s.dst_h);
    }
    op->algo_bytes = bytes;
    int rows = op->ctx->k3_rows;
    if (flatten_whole_frames(op, t)) {  // whole frames as rows of 512 pixels, as the colour family takes them
        max_rows = op->flat_h;
        // (256 frames of 224 x 224, 1 / 2 / 4 / 8 such rows per wavefront against the images' own rows: Gamma 16.9 / 17.2 / 18.7 /
        // 20.6 against 18.1 us, Blend 24.4 / 22.8 / 25.0 / 27.1 against 23.9 us)
        rows = op->ctx->k3_flat_rows ? op->ctx->k3_flat_rows : (op->kind == OP_GAMMA ? 1 : 2);
    }
    plan_streaming(op, max_rows, rows);
    bool aligned = op->flat_h ? true : op->dst.w % 8 == 0;
    for (int i = 0; i < op->n && aligned; i++) aligned = (t[i].dst_w % 8 == 0);
    op->fn_fast = nullptr;
    if (aligned) {
        op->fn_fast = rmx::select_point_kernel(op->kind == OP_BLEND ? 1 : 0, op->dst.dtype, op->dst.layout, 1, &op->fast_name);
        op->fast_strips = op->strips;
        op->fast_lds = 0;
        op->fast_rows = op->aux0;
        op->fast_wpb = op->waves_per_block;
        op->fast_needs_src16 = false;
    }
    // the same pipeline for rows of any width from 8 pixels on and a destination at any element
    bool wide8 = true;
    for (int i = 0; i < op->n && wide8; i++) wide8 = t[i].dst_w >= 8 || t[i].dst_w <= 0 || t[i].dst_h <= 0;
    op->fn_mid = nullptr;
    if (wide8) {
        op->fn_mid = rmx::select_point_kernel(op->kind == OP_BLEND ? 1 : 0, op->dst.dtype, op->dst.layout, 2, &op->mid_name);
        op->mid_strips = op->strips;
        op->mid_lds = 0;
        op->mid_rows = op->aux0;
        op->mid_wpb = op->waves_per_block;
        op->mid_aux1 = op->aux1;
    }
    return commit_slot(op, slot);
}

int rmx_create_gamma(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int roi_type, rmx_op **out) {
    return create_point(ctx, OP_GAMMA, src, dst, roi_type, out);
}
int rmx_update_gamma(rmx_op *op, const uint32_t *src_roi, const float *gamma) {
    if (!op || op->kind != OP_GAMMA) return fail(RMX_ERR_INVALID, "op is not a Gamma node");
    if (!gamma) return fail(RMX_ERR_INVALID, "gamma array is required");
    return update_point(op, src_roi, nullptr, gamma);
}

int rmx_create_blend(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int roi_type, rmx_op **out) {
    return create_point(ctx, OP_BLEND, src, dst, roi_type, out);
}
int rmx_update_blend(rmx_op *op, const uint32_t *src_roi, const float *ratio) {
    if (!op || op->kind != OP_BLEND) return fail(RMX_ERR_INVALID, "op is not a Blend node");
    if (!ratio) return fail(RMX_ERR_INVALID, "ratio array is required");
    return update_point(op, src_roi, ratio, nullptr);
}

/* ------------------------------------------------------------------ K4 family */

static int create_warp(rmx_ctx *ctx, int kind, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int interpolation, int roi_type, rmx_op **out) {
    if (interpolation != RMX_INTERP_LINEAR && interpolation != RMX_INTERP_NEAREST) {
        if (out) *out = nullptr;
        return fail(RMX_ERR_UNSUPPORTED, "warp interpolation %d is outside the hot path (nearest=0, linear=1)", interpolation);
    }
    int rc = make_op(ctx, kind, src, dst, roi_type, out);
    if (rc) return rc;
    (*out)->interp = interpolation;
    (*out)->fn = rmx::select_warp_kernel(interpolation, dst->dtype, dst->layout, false, &(*out)->kernel_name);
    return RMX_OK;
}

static int update_warp(rmx_op *op, const uint32_t *roi, const float *affine, const float *angle, const uint32_t *dst_w, const uint32_t *dst_h) {
    RmxSample *t;
    int slot = next_slot(op, &t);
    if (slot < 0) return slot == -2 ? RMX_ERR_INVALID : RMX_ERR_HIP;
    uint64_t bytes = 0;
    int max_dw = 1, max_dh = 1;
    double worst_box = 0;
    // The form that loads the source box straight into LDS as packed bytes needs every source row to start at the same byte
    // phase (row stride a multiple of 4).
    bool raw = op->ctx->dma != 0;
    if (raw) {
        if (op->layout.empty()) raw = (op->src.w * 3u) % 4u == 0;
        else
            for (int i = 0; i < op->n && raw; i++) raw = op->layout[i].row_stride % 4u == 0;
    }
    op->fn = rmx::select_warp_kernel(op->interp, op->dst.dtype, op->dst.layout, raw, &op->kernel_name);
    for (int i = 0; i < op->n; i++) {
        RmxSample &s = t[i];
        int rc = read_roi(op, roi, i, &s.src_x, &s.src_y, &s.src_w, &s.src_h);
        if (rc) return rc;
        s.dst_w = std::min<int32_t>(dst_w ? (int32_t)dst_w[i] : s.src_w, (int32_t)op->dst.w);
        s.dst_h = std::min<int32_t>(dst_h ? (int32_t)dst_h[i] : s.src_h, (int32_t)op->dst.h);
        if (s.src_w <= 0 || s.src_h <= 0) s.dst_w = s.dst_h = 0;
        s.flags = 0;
        if (affine) {
            // rocAL's fill order x0,y0,x1,y1,o0,o1 -> M = [[x0,x1,o0],[y0,y1,o1]]
            const float *a = affine + i * 6;
            s.m[0] = a[0]; s.m[1] = a[2]; s.m[2] = a[4];
            s.m[3] = a[1]; s.m[4] = a[3]; s.m[5] = a[5];
        } else {
            float rad = angle[i] * 0.017453292519943295f;
            float c = std::cos(rad), sn = std::sin(rad);
            s.m[0] = c;  s.m[1] = -sn; s.m[2] = 0.0f;
            s.m[3] = sn; s.m[4] = c;   s.m[5] = 0.0f;
        }
        bytes += (uint64_t)s.src_w * s.src_h * 3 + (uint64_t)s.dst_w * s.dst_h * 3 * dtype_size(op->dst.dtype);
        max_dw = std::max(max_dw, (int)s.dst_w);
        max_dh = std::max(max_dh, (int)s.dst_h);
        // LDS need of a destination tile (32 x 16*passes): bounding box of its image under M, margins, and the
        // repeated column and row
        const double th = 16.0 * op->ctx->warp_passes;
        double bw = 32.0 * std::fabs(s.m[0]) + th * std::fabs(s.m[1]) + 6.0;
        double bh = 32.0 * std::fabs(s.m[3]) + th * std::fabs(s.m[4]) + 6.0;
        if (std::isfinite(bw) && std::isfinite(bh)) {
            bw = std::min(bw, (double)s.src_w + 1);
            bh = std::min(bh, (double)s.src_h + 1);
            if (raw) {
                // (packed bytes: rows of whole 16-byte pieces from the dword that holds the box's first pixel; boxes of up to
                // kWarpRawPieces pieces per row are staged at that pitch; in dwords, like the other form)
                const double pieces = std::ceil((3.0 + 3.0 * (bw + 1.0)) / 16.0);
                worst_box = std::max(worst_box, (pieces <= rmx::kWarpRawPieces ? (double)rmx::kWarpRawPieces : pieces) * 4.0 * bh);
            } else {
                // (boxes of up to 60 dwords per row are staged at a pitch of 60, see the kernel)
                const double pitch = std::ceil(bw / 4) * 4 + 4;
                worst_box = std::max(worst_box, (pitch <= 60.0 ? 60.0 : pitch) * bh);
            }
        }
    }
    op->algo_bytes = bytes;
    const int cap = 16 * 1024;  // per wave (16 loads per lane); bigger boxes fall back to global gathers inside the kernel
    int need = (int)std::min<double>(worst_box * 4 + (raw ? 16 : 0), (double)cap);
    op->lds_per_wave = std::max(256, (need + 15) / 16 * 16);
    op->waves_per_block = std::max(1, std::min(op->ctx->warp_wpb, op->ctx->max_lds_per_block / op->lds_per_wave));
    const int passes = op->ctx->warp_passes;
    const int tiles_x = (max_dw + 31) / 32, tiles_y = (max_dh + 16 * passes - 1) / (16 * passes);
    op->strips = tiles_x * tiles_y;
    op->aux0 = tiles_x;
    // aux1 bit 0: the shapes allow packed 16-byte stores (whole 8-pixel groups, rows a multiple of 8 pixels wide);
    // bits 8..: passes of 16 rows per tile
    bool aligned = op->dst.w % 8 == 0;
    for (int i = 0; i < op->n && aligned; i++) aligned = (t[i].dst_w % 8 == 0);
    op->aux1 = (aligned ? 1 : 0) | (passes << 8);
    return commit_slot(op, slot);
}

int rmx_create_warp_affine(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int interpolation, int roi_type, rmx_op **out) {
    return create_warp(ctx, OP_WARP_AFFINE, src, dst, interpolation, roi_type, out);
}
int rmx_update_warp_affine(rmx_op *op, const uint32_t *src_roi, const float *affine, const uint32_t *dst_w, const uint32_t *dst_h) {
    if (!op || op->kind != OP_WARP_AFFINE) return fail(RMX_ERR_INVALID, "op is not a WarpAffine node");
    if (!affine) return fail(RMX_ERR_INVALID, "affine array is required");
    return update_warp(op, src_roi, affine, nullptr, dst_w, dst_h);
}
int rmx_create_rotate(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int interpolation, int roi_type, rmx_op **out) {
    return create_warp(ctx, OP_ROTATE, src, dst, interpolation, roi_type, out);
}
int rmx_update_rotate(rmx_op *op, const uint32_t *src_roi, const float *angle_deg, const uint32_t *dst_w, const uint32_t *dst_h) {
    if (!op || op->kind != OP_ROTATE) return fail(RMX_ERR_INVALID, "op is not a Rotate node");
    if (!angle_deg) return fail(RMX_ERR_INVALID, "angle array is required");
    return update_warp(op, src_roi, nullptr, angle_deg, dst_w, dst_h);
}

/* ------------------------------------------------------------------ one entry point that allocates nothing */

int rmx_resize_cmn_noalloc(rmx_ctx *ctx, const rmx_tensor_desc *src_desc, const rmx_tensor_desc *dst_desc, int interpolation, int roi_type,
                           uint32_t flags, const void *src, void *dst, const uint32_t *src_roi, const uint32_t *dst_w, const uint32_t *dst_h,
                           const uint32_t *crop_roi, const float *scale, const float *bias, const uint32_t *mirror) {
    if (!ctx) return fail(RMX_ERR_INVALID, "context is NULL");
    int rc;
    if ((rc = check_desc(src_desc, "source"))) return rc;
    if ((rc = check_desc(dst_desc, "destination"))) return rc;
    if (src_desc->dtype != RMX_UINT8 || src_desc->layout != RMX_NHWC) return fail(RMX_ERR_UNSUPPORTED, "source must be uint8 NHWC (decoded RGB batch)");
    if (src_desc->n != dst_desc->n) return fail(RMX_ERR_INVALID, "batch size mismatch: source %u, destination %u", src_desc->n, dst_desc->n);
    if (src_desc->n > (uint32_t)RMX_NOALLOC_ROWS)
        return fail(RMX_ERR_INVALID, "batch of %u samples exceeds the %d rows of the static parameter table (RMX_NOALLOC_MAX_SAMPLES)", src_desc->n, RMX_NOALLOC_ROWS);
    if (roi_type != RMX_ROI_LTRB && roi_type != RMX_ROI_XYWH) return fail(RMX_ERR_INVALID, "roi_type %d invalid", roi_type);
    if (interpolation != RMX_INTERP_LINEAR && interpolation != RMX_INTERP_NEAREST && interpolation != RMX_INTERP_TRIANGULAR)
        return fail(RMX_ERR_UNSUPPORTED, "interpolation %d is outside the hot path (nearest=0, linear=1, triangular=5)", interpolation);
    if (flags & ~(uint32_t)(RMX_F_QUANTIZE_U8 | RMX_F_EDGE_REF)) return fail(RMX_ERR_UNSUPPORTED, "only RMX_F_QUANTIZE_U8 and RMX_F_EDGE_REF are supported here");
    if (!scale || !bias) return fail(RMX_ERR_INVALID, "scale and bias arrays are required");
    if (!ctx->scratch_ptr) return fail(RMX_ERR_INVALID, "the context holds no address of the static parameter table");
    HIP_TRY(hipSetDevice(ctx->device));
    // an op that lives on this call's stack: same packing, same planner, same kernels as rmx_create_resize + rmx_update_resize_cmn
    rmx_op op;
    op.ctx = ctx;
    op.kind = OP_RESIZE;
    op.src = *src_desc;
    op.dst = *dst_desc;
    op.roi_type = roi_type;
    op.n = (int)src_desc->n;
    op.interp = interpolation;
    op.flags = flags;
    RmxSample rows[RMX_NOALLOC_ROWS];  // host side of the table, on this call's stack (64 KiB)
    memset(rows, 0, sizeof(RmxSample) * (size_t)op.n);
    rc = fill_resize_rows(&op, rows, src_roi, dst_w, dst_h, crop_roi, scale, bias, nullptr, nullptr, mirror, nullptr);
    if (rc) return rc;
    RmxSample *table = static_cast<RmxSample *>(ctx->scratch_ptr);  // the address asked of the runtime, never the array's name
    for (int first = 0; first < op.n; first += 16) {
        RmxRowPack pack;
        const int count = std::min(16, op.n - first);
        memcpy(pack.rows, rows + first, sizeof(RmxSample) * (size_t)count);
        hipLaunchKernelGGL(rmx_table_fill_kernel, dim3(1), dim3(512), 0, ctx->stream, pack, table, first, count);
        HIP_TRY(hipGetLastError());
    }
    return launch_table(&op, table, nullptr, nullptr, 0, src, nullptr, dst);
}

/* ------------------------------------------------------------------ measurement helper */

int rmx_copy_bytes(rmx_ctx *ctx, const void *src, void *dst, size_t nbytes) {
    if (!ctx || !src || !dst) return fail(RMX_ERR_INVALID, "context/source/destination is NULL");
    if (nbytes % 16 != 0) return fail(RMX_ERR_INVALID, "nbytes must be a multiple of 16");
    if ((((uintptr_t)src) | ((uintptr_t)dst)) & 15u) return fail(RMX_ERR_INVALID, "buffers must be 16-byte aligned");
    HIP_TRY(hipSetDevice(ctx->device));
    rmx::launch_copy(ctx->stream, src, dst, nbytes, ctx->num_cus);
    HIP_TRY(hipGetLastError());
    return RMX_OK;
}

int rmx_stream_probe(rmx_ctx *ctx, int mode, const void *src, void *dst, size_t nbytes, int groups_per_cu) {
    if (!ctx || !src || !dst) return fail(RMX_ERR_INVALID, "context/source/destination is NULL");
    if (mode < 0 || mode > 2) return fail(RMX_ERR_INVALID, "mode must be 0 (copy), 1 (read only) or 2 (write only)");
    if (groups_per_cu < 0 || groups_per_cu > 64) return fail(RMX_ERR_INVALID, "groups_per_cu out of range (0..64)");
    if (nbytes % 16 != 0) return fail(RMX_ERR_INVALID, "nbytes must be a multiple of 16");
    if ((((uintptr_t)src) | ((uintptr_t)dst)) & 15u) return fail(RMX_ERR_INVALID, "buffers must be 16-byte aligned");
    HIP_TRY(hipSetDevice(ctx->device));
    rmx::launch_stream(ctx->stream, mode, src, dst, nbytes, ctx->num_cus, groups_per_cu);
    HIP_TRY(hipGetLastError());
    return RMX_OK;
}

}  // extern "C"
