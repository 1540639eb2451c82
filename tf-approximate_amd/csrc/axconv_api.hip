// C-ABI entry points of libaxconv_hip.so: validation, geometry, planning, workspace carving, launches.
#include "axconv_internal.h"

#include <math.h>
#include <stdlib.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <map>
#include <mutex>
#include <string>
#include <tuple>
#include <vector>

using namespace axc;

struct axc_table {
    uint16_t *dev_tableT; // [257 filter code][256 input code]; row 256 is zero
    int device;
};

// Workspace of axc_conv2d_minmax_static: a fixed array in the library's device image, one copy per GPU, held until
// the process ends.  In host code this name is only a handle for hipGetSymbolAddress; the address each device
// reports is what kernels and copies get.
constexpr size_t kStaticScratchBytes = (size_t)32 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace axc {
int device_cus()
{
    static std::atomic<int> cached[64];   // per device; 0 = not asked yet
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess)
        return 256;
    const int slot = dev & 63;
    cus = cached[slot].load(std::memory_order_relaxed);
    if (cus > 0)
        return cus;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
        return 256;
    cached[slot].store(cus, std::memory_order_relaxed);
    return cus;
}

// LDS a workgroup may take and the shader clock of the current device, as the runtime reports them (cached); the
// gfx950 figures where it reports nothing.
static int device_attribute_cached(std::atomic<int> (&cached)[64], hipDeviceAttribute_t attr, int fallback)
{
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess)
        return fallback;
    const int slot = dev & 63;
    v = cached[slot].load(std::memory_order_relaxed);
    if (v > 0)
        return v;
    if (hipDeviceGetAttribute(&v, attr, dev) != hipSuccess || v <= 0)
        return fallback;
    cached[slot].store(v, std::memory_order_relaxed);
    return v;
}
int device_lds_bytes()
{
    static std::atomic<int> cached[64];
    return device_attribute_cached(cached, hipDeviceAttributeMaxSharedMemoryPerBlock, 160 * 1024);
}
double device_clock_hz()
{
    static std::atomic<int> cached[64];
    return 1e3 * (double)device_attribute_cached(cached, hipDeviceAttributeClockRate, 2400000);
}
} // namespace axc

namespace {

thread_local std::string g_last_error;

int fail(int status, const char *msg)
{
    g_last_error = msg;
    return status;
}

int fail_hip(hipError_t e, const char *what)
{
    g_last_error = std::string(what) + ": " + hipGetErrorString(e);
    return AXC_RUNTIME_ERROR;
}

#define AXC_HIP(call)                                \
    do {                                             \
        hipError_t e_ = (call);                      \
        if (e_ != hipSuccess)                        \
            return fail_hip(e_, #call);              \
    } while (0)

// Device address of `scratch` on the current device, looked up once per device with that device current.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};

int static_scratch(void **ptr)
{
    int dev = 0;
    AXC_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices)
        return fail(AXC_RUNTIME_ERROR, "device index out of range for the static workspace");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        AXC_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p)
            return fail(AXC_RUNTIME_ERROR, "hipGetSymbolAddress returned no address for the static workspace");
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return AXC_OK;
}

// ---- the word through which a LUT-GEMM launch reports a wait between its wavefronts that ran out ----
// Host memory the device can write, one word per GPU, allocated when the first table is created on that GPU (a launch
// call allocates nothing).  A launch call that finds the word set reports the failure - of an EARLIER launch on that
// GPU, whose output is incomplete - clears it and does nothing else.
std::mutex g_wait_mutex;
uint32_t *g_wait_host[kMaxDevices] = {};
uint32_t *g_wait_dev[kMaxDevices] = {};
std::atomic<uint32_t> g_wait_limit{1u << 20};   // polls per wait, ~150 cycles each: far beyond any fill or epilogue

int wait_error_alloc()
{
    int dev = 0;
    AXC_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices)
        return AXC_OK;   // launches on such a device run without the report
    std::lock_guard<std::mutex> lock(g_wait_mutex);
    if (g_wait_host[dev])
        return AXC_OK;
    void *host = nullptr, *devp = nullptr;
    AXC_HIP(hipHostMalloc(&host, 64, hipHostMallocMapped));
    memset(host, 0, 64);
    const hipError_t e = hipHostGetDevicePointer(&devp, host, 0);
    if (e != hipSuccess) {
        (void)hipHostFree(host);
        return fail_hip(e, "hipHostGetDevicePointer");
    }
    g_wait_host[dev] = static_cast<uint32_t *>(host);
    g_wait_dev[dev] = static_cast<uint32_t *>(devp);
    return AXC_OK;
}

// The device's view of the word (null if there is none), after reporting what an earlier launch left in it.
int wait_error_check(uint32_t **dev_word)
{
    *dev_word = nullptr;
    int dev = 0;
    AXC_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices)
        return AXC_OK;
    uint32_t *host = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_wait_mutex);
        host = g_wait_host[dev];
        *dev_word = g_wait_dev[dev];
    }
    if (!host)
        return AXC_OK;
    const uint32_t code = __atomic_exchange_n(host, 0u, __ATOMIC_RELAXED);
    if (code != 0u) {
        char msg[200];
        snprintf(msg, sizeof(msg), "an earlier LUT-GEMM launch on this device gave up a wait between its wavefronts "
                 "(code %u): its output is incomplete", code);
        return fail(AXC_RUNTIME_ERROR, msg);
    }
    return AXC_OK;
}

// ---- profiling: events around each kernel, on the launch stream ----
struct ProfEntry {
    std::vector<std::pair<hipEvent_t, hipEvent_t>> pending;
    double total_ms = 0.0;
    int64_t launches = 0;
};
std::mutex g_prof_mutex;
std::atomic<bool> g_prof_enabled{false};
std::map<std::string, ProfEntry> g_prof;

struct ProfScope {
    const char *name;
    hipStream_t stream;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    bool on;
    ProfScope(const char *n, hipStream_t s) : name(n), stream(s), on(g_prof_enabled.load())
    {
        if (!on)
            return;
        if (hipEventCreate(&e0) != hipSuccess) {
            on = false;
        } else if (hipEventCreate(&e1) != hipSuccess) {
            (void)hipEventDestroy(e0);
            on = false;
        } else {
            (void)hipEventRecord(e0, stream);
        }
    }
    ~ProfScope()
    {
        if (!on)
            return;
        (void)hipEventRecord(e1, stream);
        std::lock_guard<std::mutex> lock(g_prof_mutex);
        g_prof[name].pending.emplace_back(e0, e1);
    }
};

void prof_drain_locked(ProfEntry &pe)
{
    for (auto &ev : pe.pending) {
        float ms = 0.0f;
        if (hipEventSynchronize(ev.second) == hipSuccess && hipEventElapsedTime(&ms, ev.first, ev.second) == hipSuccess) {
            pe.total_ms += ms;
            pe.launches += 1;
        }
        (void)hipEventDestroy(ev.first);
        (void)hipEventDestroy(ev.second);
    }
    pe.pending.clear();
}

// A table lives in the memory of the device that was current when it was created.
int check_table_device(const axc_table *table)
{
    int dev = 0;
    AXC_HIP(hipGetDevice(&dev));
    if (dev != table->device)
        return fail(AXC_INVALID_ARGUMENT, "the truth table was created on another device than the current one");
    return AXC_OK;
}

// ---- quantization parameters (approx_ops_types.h:29-49,135-197) ----
// Every float operation rounds on its own (volatile), as in the reference build.
void nudge(float min, float max, float *nudged_min, float *nudged_max, float *scale, int *zero_point)
{
    const float qmin = 0.0f, qmax = 255.0f;
    volatile float range = max - min;
    volatile float sc = range / (qmax - qmin);
    volatile float ratio = min / sc;
    volatile float zp_from_min = qmin - ratio;
    int zp;
    if (zp_from_min < qmin)
        zp = 0;
    else if (zp_from_min > qmax)
        zp = 255;
    else
        zp = (int)(uint16_t)roundf(zp_from_min);
    volatile float lo = (qmin - (float)zp) * sc;
    volatile float hi = (qmax - (float)zp) * sc;
    *nudged_min = lo;
    *nudged_max = hi;
    *scale = sc;
    *zero_point = zp;
}

void var_quant_props(float min, float max, float *scale, float *inv_scale, float *offset)
{
    float s = 0.0f, inv = 0.0f, nmin = 0.0f, nmax = 0.0f;
    int zp = 0;
    if (min != 0.0f || max != 0.0f) {
        nudge(min, max, &nmin, &nmax, &s, &zp);
        volatile float i = 1.0f / s;
        inv = i;
    }
    *scale = s;
    *inv_scale = inv;
    *offset = nmin;
}

int host_quantize(float v, float offset, float inv_scale)
{
    volatile float d = v - offset;
    volatile float pr = d * inv_scale;
    volatile float t = pr + 0.5f;
    float tt = t;
    if (!(tt > 0.0f))
        return 0;
    if (tt >= 255.0f)
        return 255;
    return (int)tt;
}

// ---- geometry (approx_nn_conv_ops.cpp:254-404) ----
int windowed_output_size(int64_t in, int64_t filter, int64_t dilation, int64_t stride, int padding,
                         int64_t *out, int64_t *before, int64_t *after)
{
    const int64_t eff = (filter - 1) * dilation + 1;
    if (padding == AXC_PAD_VALID) {
        *out = (in - eff + stride) / stride;
        *before = *after = 0;
    } else if (padding == AXC_PAD_SAME) {
        *out = (in + stride - 1) / stride;
        int64_t needed = (*out - 1) * stride + eff - in;
        if (needed < 0)
            needed = 0;
        *before = needed / 2;
        *after = needed - *before;
    } else {
        *out = (in + *before + *after - eff + stride) / stride;
    }
    if (*out < 0)
        return fail(AXC_INVALID_ARGUMENT, "Computed output size would be negative");
    return AXC_OK;
}

int geometry(const axc_conv2d_desc *d, axc_conv2d_dims *o)
{
    if (!d || !o)
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    if (d->data_format != AXC_FORMAT_NHWC && d->data_format != AXC_FORMAT_NCHW)
        return fail(AXC_INVALID_ARGUMENT, "Invalid data format");
    const bool nhwc = d->data_format == AXC_FORMAT_NHWC;
    const int iN = 0, iC = nhwc ? 3 : 1, iH = nhwc ? 1 : 2, iW = nhwc ? 2 : 3;
    if (d->strides[iN] != 1 || d->strides[iC] != 1)
        return fail(AXC_INVALID_ARGUMENT,
                    "Current implementation does not yet support strides in the batch and depth dimensions.");
    if (d->strides[iH] <= 0 || d->strides[iW] <= 0)
        return fail(AXC_INVALID_ARGUMENT, "Row and column strides should be larger than 0.");
    if (d->dilations[iN] != 1 || d->dilations[iC] != 1)
        return fail(AXC_INVALID_ARGUMENT,
                    "Current implementation does not yet support dilations in the batch and depth dimensions.");
    if (d->dilations[iH] <= 0 || d->dilations[iW] <= 0)
        return fail(AXC_INVALID_ARGUMENT, "Dilated rates should be larger than 0.");
    if (d->padding != AXC_PAD_VALID && d->padding != AXC_PAD_SAME && d->padding != AXC_PAD_EXPLICIT)
        return fail(AXC_INVALID_ARGUMENT, "Invalid padding");
    for (int i = 0; i < 4; ++i) {
        if (d->input_shape[i] < 0 || d->input_shape[i] > INT32_MAX)
            return fail(AXC_INVALID_ARGUMENT, "input is too large");
        if (d->filter_shape[i] < 0 || d->filter_shape[i] > INT32_MAX)
            return fail(AXC_INVALID_ARGUMENT, "filter is too large");
    }
    const int64_t in_depth = d->input_shape[iC], patch_depth = d->filter_shape[2];
    if (patch_depth <= 0 || in_depth % patch_depth != 0)
        return fail(AXC_INVALID_ARGUMENT, "input depth must be evenly divisible by filter depth");

    o->batch = (int32_t)d->input_shape[iN];
    o->input_rows = (int32_t)d->input_shape[iH];
    o->input_cols = (int32_t)d->input_shape[iW];
    o->in_depth = (int32_t)in_depth;
    o->filter_rows = (int32_t)d->filter_shape[0];
    o->filter_cols = (int32_t)d->filter_shape[1];
    o->patch_depth = (int32_t)patch_depth;
    o->out_depth = (int32_t)d->filter_shape[3];
    o->stride_rows = d->strides[iH];
    o->stride_cols = d->strides[iW];
    o->dilation_rows = d->dilations[iH];
    o->dilation_cols = d->dilations[iW];
    o->pad_rows_before = o->pad_rows_after = o->pad_cols_before = o->pad_cols_after = 0;
    if (d->padding == AXC_PAD_EXPLICIT) {
        o->pad_rows_before = d->explicit_paddings[2 * iH];
        o->pad_rows_after = d->explicit_paddings[2 * iH + 1];
        o->pad_cols_before = d->explicit_paddings[2 * iW];
        o->pad_cols_after = d->explicit_paddings[2 * iW + 1];
    }
    int rc = windowed_output_size(o->input_rows, o->filter_rows, o->dilation_rows, o->stride_rows, d->padding,
                                  &o->out_rows, &o->pad_rows_before, &o->pad_rows_after);
    if (rc != AXC_OK)
        return rc;
    return windowed_output_size(o->input_cols, o->filter_cols, o->dilation_cols, o->stride_cols, d->padding,
                                &o->out_cols, &o->pad_cols_before, &o->pad_cols_after);
}

// Checks shared by every launch entry point; the reference's messages where it has them.
int validate_for_launch(const axc_conv2d_desc *d, const axc_conv2d_dims &dm, bool depthwise)
{
    if (d->num_bits != 8)
        return fail(AXC_INVALID_ARGUMENT, "only num_bits = 8 is supported");
    if (d->data_format != AXC_FORMAT_NHWC)
        return fail(AXC_UNIMPLEMENTED, "Generic conv implementation only supports NHWC tensor format for now.");
    if (depthwise) {
        if (d->filter_shape[3] != 1 || dm.patch_depth != dm.in_depth)
            return fail(AXC_INVALID_ARGUMENT, "depthwise filter must be [rows, cols, in_depth, 1]");
    } else if (dm.in_depth != dm.patch_depth) {
        return fail(AXC_UNIMPLEMENTED, "Generic conv implementation does not support grouped convolutions for now.");
    }
    if (d->padding == AXC_PAD_EXPLICIT)
        return fail(AXC_UNIMPLEMENTED, "Explicit padding is not implemented.");
    const int64_t patch_len = (int64_t)dm.filter_rows * dm.filter_cols * dm.patch_depth;
    if (patch_len > (int64_t)(16 * 1024 * 1024) / (int64_t)sizeof(float))
        return fail(AXC_INVALID_ARGUMENT, "ApproxConv2DOp: Patch too large for buffer");
    if (patch_len >= 32768) // 32768 * 65535 would overflow the int32 accumulator
        return fail(AXC_INVALID_ARGUMENT, "patch length must be below 32768 for int32 accumulation");
    if (dm.input_rows >= 32768 || dm.input_cols >= 32768 || dm.pad_rows_before >= 16384 ||
        dm.pad_cols_before >= 16384)
        return fail(AXC_INVALID_ARGUMENT, "image dimensions must be below 32768");
    const int64_t out_elems = (int64_t)dm.batch * dm.out_rows * dm.out_cols * (depthwise ? dm.in_depth : dm.out_depth);
    const int64_t in_elems = (int64_t)dm.batch * dm.input_rows * dm.input_cols * dm.in_depth;
    if (out_elems >= ((int64_t)1 << 40) || in_elems >= ((int64_t)1 << 40))
        return fail(AXC_INVALID_ARGUMENT, "tensor too large");
    // the dense kernel addresses the quantized input with 32-bit byte offsets
    const int64_t xq_bytes = ((int64_t)dm.batch * dm.input_rows + 1) * dm.input_cols * ((dm.in_depth + 3) / 4) * 4;
    if (!depthwise && xq_bytes >= ((int64_t)1 << 31))
        return fail(AXC_INVALID_ARGUMENT, "input too large: more than 2^31 quantized activations");
    return AXC_OK;
}

ConvGeom make_geom(const axc_conv2d_dims &dm)
{
    ConvGeom g;
    g.N = dm.batch; g.H = dm.input_rows; g.W = dm.input_cols; g.C = dm.in_depth;
    g.KH = dm.filter_rows; g.KW = dm.filter_cols; g.Co = dm.out_depth;
    g.OH = (int)dm.out_rows; g.OW = (int)dm.out_cols;
    g.sh = dm.stride_rows; g.sw = dm.stride_cols; g.dh = dm.dilation_rows; g.dw = dm.dilation_cols;
    g.ph = (int)dm.pad_rows_before; g.pw = (int)dm.pad_cols_before;
    g.C4 = (g.C + 3) / 4;
    g.M = (int64_t)g.N * g.OH * g.OW;
    g.K = g.KH * g.KW * g.C;
    return g;
}


// Forced tile width (0 = the planner chooses): set by axc_set_tile_columns; the environment variable
// AXC_TILE_COLUMNS gives its initial value, read once when the library is loaded.
std::atomic<int> g_forced_nt{[] {
    const char *env = std::getenv("AXC_TILE_COLUMNS");
    const int v = env ? std::atoi(env) : 0;
    return (v == 16 || v == 32 || v == 64) ? v : 0;
}()};

// Pre-expanded rows (lutgemm_px_kernel.hip): 0 = the planner decides, 1 = every layer that can run that way does,
// -1 = never.  Set by axc_set_preexpand; AXC_PREEXPAND gives the initial value, read once when the library is loaded.
std::atomic<int> g_px_mode{[] {
    const char *env = std::getenv("AXC_PREEXPAND");
    const int v = env ? std::atoi(env) : 0;
    return (v == 1 || v == -1) ? v : 0;
}()};
constexpr size_t kPxMaxBytes = (size_t)2 << 30;     // most memory a layer's pre-expanded rows may take
// Rows up to this size stay in the memory-side cache between the launch that writes them and the one that reads
// them; larger sets are read from memory, and the cost model is less sure of them: they must promise a gain.
constexpr size_t kPxCachedBytes = (size_t)192 << 20;

// Tile plan: columns per tile (16/32/64) and rows per tile, by a cost model in LDS/VALU cycles.
// Derive cost per fill is constant; lookup cost per fill grows with the wavefront-rows a SIMD carries.
DensePlan compute_plan(const ConvGeom &g, int cus, int forced_nt, int px_mode, double clock_hz)
{
    DensePlan best{};
    double best_cost = 1e300;
    const int taps = g.KH * g.KW;
    const bool px_possible = (g.C4 & 1) == 0 &&
                             (size_t)((g.Co + 15) / 16) * (size_t)(taps * g.C4 / 2) * 65536 <= kPxMaxBytes;
    const bool want_px = px_mode > 0 && px_possible && (forced_nt == 0 || forced_nt == 16);
    for (int nt : {16, 32, 64}) {
        if (forced_nt == 16 || forced_nt == 32 || forced_nt == 64) {
            if (nt != forced_nt)
                continue;
        } else if (nt > 16 && nt / 2 >= g.Co) {
            continue; // half the columns of a wider tile would be padding
        }
        const int R = 2 * (64 / nt), ks = 64 / nt, subs = 4 / ks;
        const int n_col = (g.Co + nt - 1) / nt;
        const int fills = taps * g.C4 * subs;
        const int64_t cap_wrows = (int64_t)kDenseWaves * R; // wavefront-rows (64 pixels each) per tile
        const int64_t total_wrows = (g.M + 63) / 64;
        const int64_t min_tiles = (total_wrows + cap_wrows - 1) / cap_wrows;
        // candidate row-tile counts: the minimum, and counts that fill whole rounds of CUs, alone or together with
        // a split of K
        std::vector<int64_t> cands{min_tiles};
        for (int64_t rounds = 1; rounds <= 48; ++rounds) {
            for (int split : {1, 2, 3, 4, 6, 8, 12, 16}) {
                if (split > 1 && rounds > 2)
                    break;
                const int64_t n_row = (rounds * cus) / ((int64_t)n_col * split);
                if (n_row > min_tiles && n_row <= total_wrows)
                    cands.push_back(n_row);
                if (split == 1 && n_row + 1 > min_tiles && n_row + 1 <= total_wrows)
                    cands.push_back(n_row + 1);
            }
        }
        if (total_wrows > min_tiles)
            cands.push_back(total_wrows);
        for (int64_t n_row : cands) {
            const int64_t wrows = (total_wrows + n_row - 1) / n_row;  // per tile
            const double per_simd = (double)((wrows + 3) / 4);          // wavefront-rows on the busiest SIMD
            // Cycles, fitted to the LUT-GEMM launch times of ~85 layer shapes run both ways (mean error 3.5 %).
            // Per fill: barrier + expanding + staging, then the lookups; per tile: geometry, the first fills, the
            // turn and store of the outputs, which grow with the tile's rows.  (What a launch costs whatever its
            // plan, ~25 000 cycles, is left out.)
            const double per_fill = 1658.0 + per_simd * 247.0;
            // Splitting K over tiles keeps the tiles tall (many lookups per expanded fill) when M alone does not
            // give every CU a tile; the int32 partial sums then cost one more pass over (k_splits + 1) outputs.
            for (int ks : {1, 2, 3, 4, 6, 8, 12, 16}) {
                if (want_px && nt != 16)
                    break;  // pre-expanded rows are asked for wherever they are possible: 16 columns
                int fps = (fills + ks - 1) / ks;
                if (want_px && ks > 1)
                    fps += fps & 1;   // a K split covers whole pre-expanded fills: pairs of fills
                if (ks > 1 && (fps < 8 || (int64_t)(ks - 1) * fps >= fills))
                    continue;
                const int64_t tiles = n_row * n_col * ks;
                const int64_t rounds = (tiles + cus - 1) / cus;
                double cost = (double)rounds * ((double)fps * per_fill + 2200.0 + per_simd * 1876.0);
                // the extra pass of a K split (fitted: 13 900 cycles + 6.8 TB/s), and a margin: split only for a gain
                const double split_cost = ks > 1 ? 17000.0 + (double)(ks + 1) * (double)g.M * g.Co * 4.0 * 3.5e-4 : 0.0;
                cost += split_cost;
                // The same tiles out of pre-expanded rows (16 columns, whole K, channel quads in pairs): a phase
                // covers two fills and neither expands nor stages (8 200 cycles at 13 wavefront-rows per SIMD,
                // 2 800 at 2).  The rows cost 512 bytes of memory per filter element, written once per call: by
                // workgroups that ride in the patch-sum launch (measured: +1.5 us, then 7 TB/s), beyond ~400 MB
                // more slowly or by a launch of their own (6.5 us, 4.5 TB/s); and every row comes out of memory at
                // least once, at 3 TB/s where no two tiles share rows.  Sets too large to stay in the memory-side
                // cache between the two launches must promise 2 %.
                int px = 0;
                if (px_possible && px_mode >= 0 && nt == 16 && (ks == 1 || (fps & 1) == 0)) {
                    const double px_bytes = (double)n_col * (double)(fills / 2) * 65536.0;
                    double px_cost = (double)rounds * ((double)(fps / 2) * (1790.0 + per_simd * 493.0) + per_simd * 1980.0);
                    const double stream = px_bytes / 3.0e12 * clock_hz;
                    px_cost = (px_cost > stream ? px_cost : stream) + split_cost;
                    const double margin = px_bytes > (double)kPxCachedBytes ? 0.98 : 1.0;
                    px_cost += (px_bytes <= 400e6 ? 1.5e-6 + px_bytes / 7e12 : 6.5e-6 + px_bytes / 4.5e12) * clock_hz;
                    if (px_mode > 0 || px_cost < cost * margin) {
                        cost = px_cost;
                        px = 1;
                    }
                }
                if (cost < best_cost) {
                    best_cost = cost;
                    best.cost = (float)cost;
                    best.px = px;
                    best.nt = nt;
                    best.rows_per_tile = (int)(wrows * 64);
                    best.n_row_tiles = (int)((total_wrows + wrows - 1) / wrows);
                    best.n_col_tiles = n_col;
                    best.fills = fills;
                    best.k_splits = ks;
                    best.fills_per_split = fps;
                    const int64_t all = (int64_t)best.n_row_tiles * n_col * ks;
                    best.grid = (int)(all < cus ? all : cus);
                }
            }
        }
    }
    return best;
}

// The plan depends on (taps, channel quads, columns, pixels, CUs, forced width) only: looked up instead of
// recomputed on every workspace query and launch.
constexpr int kPxModeGlobal = 99;   // "whatever axc_set_preexpand says"
DensePlan make_plan(const ConvGeom &g, int cus, int px_mode = kPxModeGlobal)
{
    struct Key {
        int taps, c4, co, cus, forced, px_mode;
        int64_t m;
        bool operator<(const Key &o) const
        {
            return std::tie(taps, c4, co, cus, forced, px_mode, m) <
                   std::tie(o.taps, o.c4, o.co, o.cus, o.forced, o.px_mode, o.m);
        }
    };
    static std::mutex mu;
    static std::map<Key, DensePlan> cache;
    const Key key{g.KH * g.KW, g.C4, g.Co, cus, g_forced_nt.load(std::memory_order_relaxed),
                  px_mode == kPxModeGlobal ? g_px_mode.load(std::memory_order_relaxed) : px_mode, g.M};
    {
        std::lock_guard<std::mutex> lock(mu);
        auto it = cache.find(key);
        if (it != cache.end())
            return it->second;
    }
    const DensePlan plan = compute_plan(g, cus, key.forced, key.px_mode, device_clock_hz());
    std::lock_guard<std::mutex> lock(mu);
    if (cache.size() >= 4096)
        cache.clear();
    cache[key] = plan;
    return plan;
}

inline size_t align_up(size_t v) { return (v + 255) & ~(size_t)255; }

struct DenseWorkspace {
    size_t sub_off, xq_off, psum_off, wq_off, fsum_off, layer_off, part_off, px_off, px_bytes;
    size_t total;        // everything, the pre-expanded rows (last) included
    size_t total_no_px;  // what a launch needs that does without them
};

// sub_bytes: room for the pixels a strided 1x1 filter reads, gathered into a dense tensor (see prepare_dense)
DenseWorkspace dense_workspace(const ConvGeom &g, const DensePlan &plan, size_t sub_bytes, int flat_row_bytes)
{
    DenseWorkspace w;
    size_t off = 0;
    w.sub_off = off; off += align_up(sub_bytes);
    w.xq_off = off;   // + the zero-point row; the flat layout's last quad may reach a few bytes past its row
    off += align_up(flat_row_bytes ? ((size_t)g.N * g.H + 1) * flat_row_bytes + 16
                                   : ((size_t)g.N * g.H + 1) * g.C4 * g.W * 4);
    w.psum_off = off; off += align_up((size_t)g.M * 4); // patch sums: one float per output pixel
    w.wq_off = off; off += align_up((size_t)plan.n_col_tiles * plan.fills * 64 * 2);
    w.fsum_off = off; off += align_up((size_t)g.Co * 4);
    w.layer_off = off;  // layer entry point: partial (min, max) pairs of both tensors, then the LayerQuant
    off += align_up((size_t)4 * kMinMaxBlocks * sizeof(float)) + align_up(sizeof(LayerQuant));
    w.part_off = off;   // int32 partial sums of the K splits
    if (plan.k_splits > 1)
        off += align_up((size_t)plan.k_splits * (size_t)g.M * g.Co * 4);
    w.total_no_px = off;
    w.px_off = off;
    w.px_bytes = plan.px ? (size_t)plan.n_col_tiles * (size_t)(plan.fills / 2) * 65536 : 0;
    off += align_up(w.px_bytes);
    w.total = off;
    return w;
}

struct PreparedDense {
    axc_conv2d_dims dims;
    ConvGeom g;          // what the pre-pass kernels see
    ConvGeom g_full;     // the layer as given (differs from g when the input is subsampled first)
    ConvGeom gk;         // what the planner and the LUT-GEMM kernels see (differs from g in the flat layout)
    int flat_row_bytes;  // > 0: xq in the flat layout, rows of this many bytes
    bool subsample;
    DensePlan plan;
    DenseWorkspace ws;
    bool empty;
};

// A 1x1 filter with a stride only ever reads every stride-th pixel, and never needs padding: the op equals the 1x1
// stride-1 op on the subsampled input.  Those pixels are gathered into the workspace first (element_bytes each:
// floats, or bytes for the codes entry point), and every kernel then sees a dense, unpadded stride-1 layer with a
// quarter (stride 2) of the pixels to quantize and sum.  allow_subsample = false keeps the layer as given (callers
// with their own padding origin).
int prepare_dense(const axc_conv2d_desc *desc, PreparedDense *pd, bool allow_subsample = true, int element_bytes = 4,
                  int px_mode = kPxModeGlobal)
{
    const bool allow_flat = allow_subsample;   // both are for callers that leave the padding origin to the library
    int rc = geometry(desc, &pd->dims);
    if (rc != AXC_OK)
        return rc;
    rc = validate_for_launch(desc, pd->dims, false);
    if (rc != AXC_OK)
        return rc;
    pd->g = pd->g_full = make_geom(pd->dims);
    pd->subsample = false;
    pd->empty = pd->g.M * pd->g.Co == 0; // approx_nn_conv_ops.cpp:449
    if (pd->empty || pd->g.K == 0) {
        pd->plan = DensePlan{};
        pd->ws = DenseWorkspace{};
        return AXC_OK;
    }
    size_t sub_bytes = 0;
    if (allow_subsample && pd->g.KH == 1 && pd->g.KW == 1 && (pd->g.sh > 1 || pd->g.sw > 1) && pd->g.ph == 0 &&
        pd->g.pw == 0) {
        pd->subsample = true;
        pd->g.H = pd->g.OH;
        pd->g.W = pd->g.OW;
        pd->g.sh = pd->g.sw = 1;
        sub_bytes = (size_t)pd->g.M * pd->g.C * element_bytes;
    }
    // Channel counts that are no multiple of four (3-channel stems) would pad every pixel to whole quads: a quarter
    // of a 3-channel layer's lookups would hit the null weight.  With a filter dilation of 1 along the row, the KW * C
    // codes under one filter row are contiguous in a pixel-major byte layout instead, and are cut into quads as one
    // run: 21 -> 24 slots per row of a 7x7x3 filter where quads per pixel give 28.  The kernels then see a filter of
    // KH taps over ceil(KW * C / 4) quads and read their activation dwords at byte granularity.  Not with a
    // caller-defined padding origin (it may be negative).
    pd->gk = pd->g;
    pd->flat_row_bytes = 0;
    {
        const ConvGeom &g = pd->g;
        const int run = g.KW * g.C, quads = (run + 3) / 4;
        const int64_t row_bytes = std::max<int64_t>((int64_t)(g.pw + g.W) * g.C, (int64_t)(g.OW - 1) * g.sw * g.C + 4 * quads);
        const int64_t rb4 = (row_bytes + 3) & ~(int64_t)3;
        const bool flat_ok = allow_flat && !pd->subsample && (g.C & 3) != 0 && g.dw == 1 && g.pw >= 0;
        if (flat_ok && quads < g.KW * g.C4 && ((int64_t)g.N * g.H + 2) * rb4 < ((int64_t)1 << 31)) {
            pd->flat_row_bytes = (int)rb4;
            pd->gk.KW = 1;
            pd->gk.C = run;       // the filter as [KH][KW * C][Co]
            pd->gk.C4 = quads;
        }
        // Pre-expanded rows want the quads in pairs.  An odd count (3x3x3: 9 codes, 3 quads, no fewer than the three
        // one-channel quads of the other layout) may take one more quad, all null weights (its channels lie beyond
        // KW * C), where the planner then picks those rows and expects the layer to be faster for it.
        const int64_t row_bytes_p = std::max<int64_t>((int64_t)(g.pw + g.W) * g.C, (int64_t)(g.OW - 1) * g.sw * g.C + 4 * (quads + 1));
        const int64_t rb4_p = (row_bytes_p + 3) & ~(int64_t)3;
        if (flat_ok && (quads & 1) && quads >= 3 && ((int64_t)g.N * g.H + 2) * rb4_p < ((int64_t)1 << 31)) {
            ConvGeom gp = pd->g;
            gp.KW = 1;
            gp.C = run;
            gp.C4 = quads + 1;
            const DensePlan padded = make_plan(gp, device_cus(), px_mode), plain = make_plan(pd->gk, device_cus(), px_mode);
            if (padded.px && padded.cost < plain.cost) {
                pd->gk = gp;
                pd->flat_row_bytes = (int)rb4_p;
            }
        }
    }
    pd->plan = make_plan(pd->gk, device_cus(), px_mode);
    pd->ws = dense_workspace(pd->g, pd->plan, sub_bytes, pd->flat_row_bytes);
    return AXC_OK;
}

enum class DenseOut { Float, AccI32 };

int run_dense(const axc_table *table, const axc_conv2d_desc *desc, const float *input, const float *filter,
              const uint8_t *input_codes, const uint8_t *filter_codes, int input_zero_code,
              float in_min, float in_max, float f_min, float f_max, float *out_f, int32_t *out_i,
              void *workspace, size_t workspace_bytes, void *stream_v, bool layer_mode = false,
              const float *bias = nullptr, int activation = AXC_ACT_NONE, const int *pad_before_override = nullptr)
{
    if (!table || !desc)
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    if (int rc_dev = check_table_device(table))
        return rc_dev;
    if (activation != AXC_ACT_NONE && activation != AXC_ACT_RELU)
        return fail(AXC_INVALID_ARGUMENT, "unknown activation");
    const bool codes_mode = input_codes != nullptr;
    uint32_t *wait_word = nullptr;
    if (int rc_wait = wait_error_check(&wait_word))
        return rc_wait;
    PreparedDense pd;
    int rc = prepare_dense(desc, &pd, pad_before_override == nullptr, codes_mode ? 1 : 4);
    if (rc != AXC_OK)
        return rc;
    if (pd.empty)
        return AXC_OK;
    if (pd.plan.px && workspace_bytes < pd.ws.total) {
        // No room for the pre-expanded rows: the layer runs the kernel that expands inside its tiles, with the tile
        // shape and K split the planner prices for THAT kernel, if the workspace holds what that plan needs (its K
        // split may ask for partial sums the other plan has none of); otherwise with the plan at hand.
        PreparedDense alt;
        rc = prepare_dense(desc, &alt, pad_before_override == nullptr, codes_mode ? 1 : 4, -1);
        if (rc == AXC_OK && workspace_bytes >= alt.ws.total)
            pd = alt;
    }
    if (pad_before_override) { // a caller with its own padding rule (tf1 AxConv2D); the plan does not depend on it
        pd.g.ph = pad_before_override[0];
        pd.g.pw = pad_before_override[1];
    }
    if ((!codes_mode && (!input || !filter)) || (codes_mode && !filter_codes) || (!out_f && !out_i))
        return fail(AXC_INVALID_ARGUMENT, "null tensor pointer");
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    const ConvGeom &g = pd.g;

    axc_quant_props qp;
    memset(&qp, 0, sizeof(qp));
    if (!codes_mode) {
        axc_quant_props_compute(in_min, in_max, f_min, f_max, &qp);
    } else {
        if (input_zero_code < 0 || input_zero_code > 255)
            return fail(AXC_INVALID_ARGUMENT, "input_zero_code must be in [0, 255]");
        qp.input_zero_code = input_zero_code;
    }

    if (g.K == 0) { // no taps: every sum is empty
        const int64_t n = g.M * g.Co;
        // a fill kernel rather than hipMemsetAsync: callers may capture the stream into a graph
        AXC_HIP(launch_fill_u32(out_i ? reinterpret_cast<uint32_t *>(out_i) : reinterpret_cast<uint32_t *>(out_f), n, 0u,
                                stream));
        return AXC_OK;
    }
    // a workspace without room for the pre-expanded rows still serves: the layer then runs without them
    const bool use_px = pd.plan.px && workspace_bytes >= pd.ws.total;
    if (workspace_bytes < pd.ws.total_no_px || (!workspace && pd.ws.total_no_px))
        return fail(AXC_INVALID_ARGUMENT, "workspace too small (see axc_conv2d_workspace_bytes)");
    if (((uintptr_t)workspace & 255) != 0)
        return fail(AXC_INVALID_ARGUMENT, "workspace must be 256-byte aligned");

    char *ws = static_cast<char *>(workspace);
    uint32_t *xq = reinterpret_cast<uint32_t *>(ws + pd.ws.xq_off);
    float *psum = reinterpret_cast<float *>(ws + pd.ws.psum_off);
    uint16_t *wq = reinterpret_cast<uint16_t *>(ws + pd.ws.wq_off);
    float *fsum = reinterpret_cast<float *>(ws + pd.ws.fsum_off);

    const uint32_t zp4 = phys_row((uint32_t)qp.input_zero_code) * 0x01010101u;
    // by-value quantization of the two tensors (op entry points); the layer entry point computes its own on the device
    TensorQuant tq_in = {qp.input_offset, qp.input_inv_scale, qp.input_scale, 0.0f, 0u, zp4};
    TensorQuant tq_f = {qp.filter_offset, qp.filter_inv_scale, qp.filter_scale, 0.0f, 0u, 0u};
    LayerQuant *lq_dev = nullptr;
    if (layer_mode) { // min / max of the whole input tensor, as the layer computes them, whatever the filter reads
        ProfScope ps("layer_quant", stream);
        float *partials = reinterpret_cast<float *>(ws + pd.ws.layer_off);
        lq_dev = reinterpret_cast<LayerQuant *>(ws + pd.ws.layer_off + align_up((size_t)4 * kMinMaxBlocks * sizeof(float)));
        const ConvGeom &gf = pd.g_full;
        AXC_HIP(launch_layer_quant(input, (int64_t)gf.N * gf.H * gf.W * gf.C, filter, (int64_t)g.K * g.Co, g.K, partials,
                                   lq_dev, stream));
    }
    if (pd.subsample) {
        ProfScope ps("subsample", stream);
        const ConvGeom &gf = pd.g_full;
        void *sub = ws + pd.ws.sub_off;
        AXC_HIP(launch_subsample(codes_mode ? static_cast<const void *>(input_codes) : static_cast<const void *>(input),
                                 codes_mode ? 1 : 4, gf.N, gf.H, gf.W, gf.C, gf.sh, gf.sw, g.H, g.W, sub, stream));
        if (codes_mode)
            input_codes = static_cast<const uint8_t *>(sub);
        else
            input = static_cast<const float *>(sub);
    }
    const bool flat = pd.flat_row_bytes > 0;
    const ConvGeom &gk = pd.gk;   // the layer as the LUT-GEMM kernels and the filter packing see it
    bool quantized_by_patch_sums = false, filter_done = false, px_done = false;
    uint16_t *const px_rows = use_px ? reinterpret_cast<uint16_t *>(ws + pd.ws.px_off) : nullptr;
    if (out_f && !codes_mode) {
        // carries the filter pre-pass, and with it the pre-expanded rows, along when it can
        ProfScope ps(flat ? "patch_sums_flat" : "patch_sums", stream);
        const FilterJob job = {filter, filter_codes, &pd.plan, tq_f, wq, fsum, table->dev_tableT, px_rows};
        if (flat)   // the patch sums write the flat layout where they hold the rows anyway, else the pass below does
            AXC_HIP(launch_patch_sums(input, g, tq_in, lq_dev, psum, stream, xq, &quantized_by_patch_sums, nullptr,
                                      nullptr, pd.flat_row_bytes));
        else
            AXC_HIP(launch_patch_sums(input, g, tq_in, lq_dev, psum, stream, xq, &quantized_by_patch_sums, &job,
                                      &filter_done, 0, &px_done));
    }
    if (flat && !quantized_by_patch_sums) {
        ProfScope ps("quantize_flat_rows", stream);
        AXC_HIP(launch_quantize_flat_rows(input, codes_mode ? input_codes : nullptr, g, g.pw, pd.flat_row_bytes, tq_in,
                                          lq_dev, reinterpret_cast<uint8_t *>(xq), stream));
    } else if (flat) {
        // written by the patch-sum launch
    } else if (codes_mode) {
        ProfScope ps("codes_relayout", stream);
        AXC_HIP(launch_codes_relayout(input_codes, g, zp4, xq, stream));
    } else if (!quantized_by_patch_sums) {
        ProfScope ps("quantize_relayout", stream);
        AXC_HIP(launch_quantize_relayout(input, g, tq_in, lq_dev, xq, nullptr, stream));
    }
    if (!filter_done) {
        ProfScope ps("filter_pack", stream);
        AXC_HIP(launch_filter_pack(codes_mode ? nullptr : filter, filter_codes, gk, pd.plan, tq_f, lq_dev, wq,
                                   (out_f && !codes_mode) ? fsum : nullptr, stream, table->dev_tableT, px_rows, &px_done));
    }

    DenseParams p;
    p.g = gk;
    p.g.ph = g.ph;   // a caller's own padding origin (never with the flat layout)
    p.g.pw = g.pw;
    p.plan = pd.plan;
    p.xq = xq;
    p.psum = psum;
    p.wq = wq;
    p.fsum = fsum;
    p.tableT = table->dev_tableT;
    p.out_f = out_f;
    p.out_i = out_i;
    p.s1xs2 = qp.s1xs2;
    p.m1 = qp.m1;
    p.m2 = qp.m2;
    {
        volatile float km = (float)g.K * qp.m1xm2;
        p.k_m1xm2 = km;
    }
    p.zp4 = zp4;
    p.lq_dev = lq_dev;
    p.bias = bias;
    p.relu = activation == AXC_ACT_RELU ? 1 : 0;
    {
        const int64_t step = 64 * (kDenseWaves / 2), ohow = (int64_t)g.OH * g.OW;
        p.step_n = (int)(step / ohow);
        p.step_oh = (int)((step % ohow) / g.OW);
        p.step_ow = (int)(step % g.OW);
    }
    p.px_rows = nullptr;
    p.px_bytes = 0;
    p.spin_limit = g_wait_limit.load(std::memory_order_relaxed);
    p.wait_error = wait_word;
    if (use_px) {
        if (!px_done) {
            ProfScope ps("px_expand_rows", stream);
            AXC_HIP(launch_px_expand_rows(wq, table->dev_tableT, pd.plan, px_rows, stream));
        }
        p.px_rows = px_rows;
        p.px_bytes = (uint32_t)pd.ws.px_bytes;
    }
    if (flat) {
        p.xq_bytes = (uint32_t)((size_t)g.N * g.H * pd.flat_row_bytes);
        p.row_step = pd.flat_row_bytes;
        p.addr_unit = 1;
        p.quad_bytes = 4;
        p.zp_tail_bytes = (uint32_t)pd.flat_row_bytes + 16;
        p.flat_col_bytes = g.sw * g.C;
    } else {
        p.xq_bytes = (uint32_t)((size_t)g.N * g.H * g.C4 * g.W * 4);
        p.row_step = g.C4 * g.W;
        p.addr_unit = 4;
        p.quad_bytes = (uint32_t)g.W * 4u;
        p.zp_tail_bytes = (uint32_t)g.C4 * (uint32_t)g.W * 4u;
        p.flat_col_bytes = 0;
    }
    p.wq_bytes = (uint32_t)((size_t)pd.plan.n_col_tiles * pd.plan.fills * 128);
    {
        // Short-K layers with many tiles per workgroup (1x1 with few channels on large images) spend a quarter of
        // every tile draining their output stores, and workgroups that run in lockstep do so all at once, above
        // what memory takes.  Starting every second group of workgroups a third of a tile late keeps the two halves
        // out of step for the whole launch: the stores of one overlap the lookups of the other (measured -8.5 % per
        // tile at K = 32, of which the late start gives back a third of a tile once).  Not worth it with fewer
        // tiles per workgroup or longer K.
        const DensePlan &pl = pd.plan;
        const int64_t tiles = (int64_t)pl.n_row_tiles * pl.n_col_tiles * pl.k_splits;
        p.stagger_sleeps = 0;
        p.stagger_groups = 2;
        if (use_px && pl.k_splits == 1 && tiles >= (int64_t)2 * pl.grid) {
            // Out of pre-expanded rows, with any K and from two tiles per workgroup on: four groups, each one sleep
            // period (~8 000 cycles, about what a tile's output stores take) behind the one before it (measured:
            // 1x1 64->256 @56x56 -8 %, 128->512 @28x28 -3 %, the other multi-tile layers -0.5 to -2 %).
            p.stagger_sleeps = 1;
            p.stagger_groups = 4;
        } else if (pl.k_splits == 1 && pl.fills <= 16 && tiles >= (int64_t)8 * pl.grid) {
            const double per_simd = (double)((pl.rows_per_tile / 64 + 3) / 4);
            const double tile_cycles = (double)pl.fills * (1700.0 + per_simd * 290.0) + 6000.0; // the planner's model
            const int sleeps = (int)(0.45 * tile_cycles / 8128.0 + 0.5);
            p.stagger_sleeps = sleeps < 1 ? 1 : (sleeps > 8 ? 8 : sleeps);
        }
    }
    if (pd.plan.k_splits > 1) {
        int32_t *part = reinterpret_cast<int32_t *>(ws + pd.ws.part_off);
        p.out_f = nullptr;
        p.out_i = part;
        if (use_px) {
            ProfScope ps("lutgemm_px", stream);
            AXC_HIP(launch_dense_px(p, true, stream));
        } else {
            ProfScope ps("lutgemm_expand", stream);
            AXC_HIP(launch_dense(p, true, stream));
        }
        ProfScope ps("splitk_epilogue", stream);
        AXC_HIP(launch_splitk_epilogue(p, part, out_f, out_i, stream));
        return AXC_OK;
    }
    if (use_px) {
        ProfScope ps("lutgemm_px", stream);
        AXC_HIP(launch_dense_px(p, out_i != nullptr, stream));
        return AXC_OK;
    }
    {
        ProfScope ps("lutgemm_expand", stream);
        AXC_HIP(launch_dense(p, out_i != nullptr, stream));
    }
    return AXC_OK;
}

struct DepthwiseWorkspace {
    size_t wcodes_off, fsum_off, layer_off, total;
};

DepthwiseWorkspace depthwise_workspace(int taps, int C)
{
    DepthwiseWorkspace w;
    size_t off = 0;
    w.wcodes_off = off; off += align_up((size_t)taps * C);
    w.fsum_off = off; off += align_up((size_t)C * 4);
    w.layer_off = off;  // layer entry point: partial (min, max) pairs of both tensors, then the LayerQuant
    off += align_up((size_t)4 * kMinMaxBlocks * sizeof(float)) + align_up(sizeof(LayerQuant));
    w.total = off;
    return w;
}

int run_depthwise(const axc_table *table, const axc_conv2d_desc *desc, const float *input, const float *filter,
                  float in_min, float in_max, float f_min, float f_max, float *out_f, int32_t *out_i,
                  void *workspace, size_t workspace_bytes, void *stream_v, bool layer_mode = false,
                  const float *bias = nullptr, int activation = AXC_ACT_NONE)
{
    if (!table || !desc)
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    if (int rc_dev = check_table_device(table))
        return rc_dev;
    if (activation != AXC_ACT_NONE && activation != AXC_ACT_RELU)
        return fail(AXC_INVALID_ARGUMENT, "unknown activation");
    axc_conv2d_dims dm;
    int rc = geometry(desc, &dm);
    if (rc != AXC_OK)
        return rc;
    rc = validate_for_launch(desc, dm, true);
    if (rc != AXC_OK)
        return rc;
    const int C = dm.in_depth, taps = dm.filter_rows * dm.filter_cols;
    const int64_t M = (int64_t)dm.batch * dm.out_rows * dm.out_cols;
    if (M * C == 0)
        return AXC_OK;
    if (!input || !filter || (!out_f && !out_i))
        return fail(AXC_INVALID_ARGUMENT, "null tensor pointer");
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    if (taps == 0) {
        // a fill kernel rather than hipMemsetAsync: callers may capture the stream into a graph
        AXC_HIP(launch_fill_u32(out_f ? reinterpret_cast<uint32_t *>(out_f) : reinterpret_cast<uint32_t *>(out_i), M * C, 0u,
                                stream));
        return AXC_OK;
    }
    const DepthwiseWorkspace dws = depthwise_workspace(taps, C);
    if (workspace_bytes < dws.total || !workspace)
        return fail(AXC_INVALID_ARGUMENT, "workspace too small (see axc_depthwise_conv2d_workspace_bytes)");
    if (((uintptr_t)workspace & 255) != 0)
        return fail(AXC_INVALID_ARGUMENT, "workspace must be 256-byte aligned");
    axc_quant_props qp;
    axc_quant_props_compute(in_min, in_max, f_min, f_max, &qp);
    char *ws = static_cast<char *>(workspace);
    uint8_t *wcodes = reinterpret_cast<uint8_t *>(ws + dws.wcodes_off);
    float *fsum = reinterpret_cast<float *>(ws + dws.fsum_off);
    const TensorQuant tq_in = {qp.input_offset, qp.input_inv_scale, qp.input_scale, 0.0f, 0u, 0u};
    const TensorQuant tq_f = {qp.filter_offset, qp.filter_inv_scale, qp.filter_scale, 0.0f, 0u, 0u};
    LayerQuant *lq_dev = nullptr;
    if (layer_mode) {
        ProfScope ps("layer_quant", stream);
        float *partials = reinterpret_cast<float *>(ws + dws.layer_off);
        lq_dev = reinterpret_cast<LayerQuant *>(ws + dws.layer_off + align_up((size_t)4 * kMinMaxBlocks * sizeof(float)));
        AXC_HIP(launch_layer_quant(input, (int64_t)dm.batch * dm.input_rows * dm.input_cols * C, filter,
                                   (int64_t)taps * C, taps, partials, lq_dev, stream));
    }
    {
        ProfScope ps("depthwise_filter", stream);
        AXC_HIP(launch_depthwise_filter(filter, taps, C, tq_f, lq_dev, wcodes, fsum, stream));
    }
    DepthwiseParams p;
    p.N = dm.batch; p.H = dm.input_rows; p.W = dm.input_cols; p.C = C;
    p.KH = dm.filter_rows; p.KW = dm.filter_cols; p.OH = (int)dm.out_rows; p.OW = (int)dm.out_cols;
    p.sh = dm.stride_rows; p.sw = dm.stride_cols; p.dh = dm.dilation_rows; p.dw = dm.dilation_cols;
    p.ph = (int)dm.pad_rows_before; p.pw = (int)dm.pad_cols_before;
    p.M = M;
    p.x = input; p.wcodes = wcodes; p.fsum = fsum; p.tableT = table->dev_tableT;
    p.out_f = out_f; p.out_i = out_i;
    p.in_q = tq_in;
    p.s1xs2 = qp.s1xs2; p.m1 = qp.m1; p.m2 = qp.m2;
    {
        volatile float km = (float)taps * qp.m1xm2;
        p.k_m1xm2 = km;
    }
    p.lq_dev = lq_dev;
    p.bias = bias;
    p.relu = activation == AXC_ACT_RELU ? 1 : 0;
    const int cus = device_cus();
    const int64_t blocks_needed = (M * C + kBlockThreads - 1) / kBlockThreads;
    const int grid = (int)(blocks_needed < cus ? blocks_needed : cus);
    {
        ProfScope ps("depthwise_lut", stream);
        AXC_HIP(launch_depthwise(p, out_i != nullptr, grid, stream));
    }
    return AXC_OK;
}

} // namespace

// ---------------------------------------------------------------------------------------------

extern "C" {

const char *axc_status_string(int status)
{
    switch (status) {
    case AXC_OK: return "OK";
    case AXC_INVALID_ARGUMENT: return "INVALID_ARGUMENT";
    case AXC_UNIMPLEMENTED: return "UNIMPLEMENTED";
    case AXC_RUNTIME_ERROR: return "RUNTIME_ERROR";
    default: return "UNKNOWN";
    }
}

const char *axc_last_error(void) { return g_last_error.c_str(); }

int axc_table_create(const uint16_t *host_table, axc_table **out)
{
    if (!host_table || !out)
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    // transpose to weight-code major: tableT[b][a] = T[(a << 8) | b]
    std::vector<uint16_t> t((size_t)kTableRows * 256, 0); // row 256 stays zero: the null weight's row
    for (int a = 0; a < 256; ++a)
        for (int b = 0; b < 256; ++b)
            t[(size_t)b * 256 + a] = host_table[(size_t)a * 256 + b];
    axc_table *tab = new axc_table;
    tab->dev_tableT = nullptr;
    hipError_t e = hipGetDevice(&tab->device);
    if (e == hipSuccess)
        e = hipMalloc(reinterpret_cast<void **>(&tab->dev_tableT), kTableAllocBytes);
    if (e == hipSuccess)
        e = hipMemcpy(tab->dev_tableT, t.data(), kTableAllocBytes, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        if (tab->dev_tableT)
            (void)hipFree(tab->dev_tableT);
        delete tab;
        return fail_hip(e, "table upload");
    }
    // set-up time is where the static workspace's address on this device is looked up (the lookup may load the
    // device image); a failure here is reported by axc_conv2d_minmax_static, which looks again
    void *unused = nullptr;
    (void)static_scratch(&unused);
    (void)wait_error_alloc();   // without the word, launches run with no report of a wait that ran out
    *out = tab;
    return AXC_OK;
}

int axc_table_create_from_file(const char *filename, int num_bits, axc_table **out)
{
    if (!out)
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    if (num_bits != 8)
        return fail(AXC_INVALID_ARGUMENT, "only num_bits = 8 is supported");
    std::vector<uint16_t> t(65536, 0);
    if (!filename || !filename[0]) {
        for (uint32_t i = 0; i < 65536u; ++i)
            t[i] = (uint16_t)((i >> 8) * (i & 0xFFu));
    } else {
        FILE *f = fopen(filename, "rb");
        if (!f)
            return fail(AXC_INVALID_ARGUMENT, "ApproxTF: Couldn't read the lookup table!");
        std::vector<unsigned char> raw(kTableBytes);
        const size_t got = fread(raw.data(), 1, kTableBytes, f);
        fclose(f);
        if (got != (size_t)kTableBytes)
            return fail(AXC_INVALID_ARGUMENT, "ApproxTF: Couldn't read the lookup table!");
        for (int i = 0; i < 65536; ++i)
            t[i] = (uint16_t)(raw[2 * i] | (raw[2 * i + 1] << 8));
    }
    return axc_table_create(t.data(), out);
}

int axc_table_destroy(axc_table *table)
{
    if (!table)
        return AXC_OK;
    hipError_t e = hipFree(table->dev_tableT);
    delete table;
    if (e != hipSuccess)
        return fail_hip(e, "hipFree");
    return AXC_OK;
}

int axc_quant_props_compute(float input_min, float input_max, float filter_min, float filter_max,
                            axc_quant_props *out)
{
    if (!out)
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    var_quant_props(input_min, input_max, &out->input_scale, &out->input_inv_scale, &out->input_offset);
    var_quant_props(filter_min, filter_max, &out->filter_scale, &out->filter_inv_scale, &out->filter_offset);
    volatile float s = out->input_scale * out->filter_scale;
    out->s1xs2 = s;
    out->m1 = out->input_offset;
    out->m2 = out->filter_offset;
    volatile float mm = out->m1 * out->m2;
    out->m1xm2 = mm;
    out->input_zero_code = host_quantize(0.0f, out->input_offset, out->input_inv_scale);
    return AXC_OK;
}

int axc_conv2d_geometry(const axc_conv2d_desc *desc, axc_conv2d_dims *dims) { return geometry(desc, dims); }

int axc_conv2d_workspace_bytes(const axc_conv2d_desc *desc, size_t *bytes)
{
    if (!bytes)
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    // enough for every entry point that takes this workspace: with and without the subsampled copy a strided 1x1
    // filter gets, floats or codes
    PreparedDense pd, pd_plain;
    int rc = prepare_dense(desc, &pd);
    if (rc != AXC_OK)
        return rc;
    rc = prepare_dense(desc, &pd_plain, false);
    if (rc != AXC_OK)
        return rc;
    *bytes = pd.ws.total > pd_plain.ws.total ? pd.ws.total : pd_plain.ws.total;
    return AXC_OK;
}

int axc_fake_approx_conv2d(const axc_table *table, const axc_conv2d_desc *desc, const float *input,
                           const float *filter, const float *bias, int activation, float *output, void *workspace,
                           size_t workspace_bytes, void *stream)
{
    if (!output)
        return fail(AXC_INVALID_ARGUMENT, "null tensor pointer");
    return run_dense(table, desc, input, filter, nullptr, nullptr, 0, 0.0f, 0.0f, 0.0f, 0.0f, output, nullptr, workspace,
                     workspace_bytes, stream, true, bias, activation);
}

int axc_fake_approx_depthwise_conv2d(const axc_table *table, const axc_conv2d_desc *desc, const float *input,
                                     const float *filter, const float *bias, int activation, float *output,
                                     void *workspace, size_t workspace_bytes, void *stream)
{
    if (!output)
        return fail(AXC_INVALID_ARGUMENT, "null tensor pointer");
    return run_depthwise(table, desc, input, filter, 0.0f, 0.0f, 0.0f, 0.0f, output, nullptr, workspace,
                         workspace_bytes, stream, true, bias, activation);
}

// tf1 AxConv2D: filter origin offsets of ReferenceAxConvFunctor (tf1/axqconv/axqconv.cc:153-163), C integer division
static void axconv_tf1_pads(const ConvGeom &g, int padding, int pads[2])
{
    const int extra = padding == AXC_PAD_VALID ? 1 : 0;
    pads[0] = ((g.OH - 1) * g.sh + g.KH - g.H + extra) / 2;
    pads[1] = ((g.OW - 1) * g.sw + g.KW - g.W + extra) / 2;
}

int axc_axconv2d_quint8(const axc_table *table, const axc_conv2d_desc *desc, const uint8_t *input,
                        const uint8_t *filter, int32_t offset_input, int32_t offset_filter, int32_t *output,
                        void *workspace, size_t workspace_bytes, void *stream)
{
    if (!desc)
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    // AxQuantizedConv2DOp's attribute checks (tf1/axqconv/axqconv.cc:297-325)
    if (desc->strides[1] != desc->strides[2])
        return fail(AXC_INVALID_ARGUMENT, "Current implementation only supports equal length strides in the row and "
                                          "column dimensions.");
    if (desc->dilations[1] != 1 || desc->dilations[2] != 1)
        return fail(AXC_INVALID_ARGUMENT, "Current implementation only supports dilated rate as 1 in the row and "
                                          "column dimensions.");
    if (desc->padding != AXC_PAD_SAME && desc->padding != AXC_PAD_VALID)
        return fail(AXC_INVALID_ARGUMENT, "padding must be SAME or VALID");
    if (offset_input < 0 || offset_input > 255) // the reference stores it in a quint8 for taps outside the image (:215)
        return fail(AXC_INVALID_ARGUMENT, "offset_input must be in [0, 255]");
    PreparedDense pd;
    int rc = prepare_dense(desc, &pd, false);
    if (rc != AXC_OK)
        return rc;
    if (pd.empty)
        return AXC_OK;
    if (!input || !filter || !output)
        return fail(AXC_INVALID_ARGUMENT, "null tensor pointer");
    int pads[2];
    axconv_tf1_pads(pd.g, desc->padding, pads);
    rc = run_dense(table, desc, nullptr, nullptr, input, filter, offset_input, 0.0f, 0.0f, 0.0f, 0.0f, nullptr, output,
                   workspace, workspace_bytes, stream, false, nullptr, AXC_ACT_NONE, pads);
    if (rc != AXC_OK || pd.g.K == 0)
        return rc;
    pd.g.ph = pads[0];
    pd.g.pw = pads[1];
    char *ws = static_cast<char *>(workspace);
    ProfScope ps("axconv_correction", static_cast<hipStream_t>(stream));
    AXC_HIP(launch_axconv_correction(input, filter, pd.g, offset_input, offset_filter,
                                     reinterpret_cast<int32_t *>(ws + pd.ws.psum_off),
                                     reinterpret_cast<int32_t *>(ws + pd.ws.fsum_off), output,
                                     static_cast<hipStream_t>(stream)));
    return AXC_OK;
}

// AxTune of ApproximateSelector::init (tf1/axqconv/approximate_selector.h:52-85): weight column w is replaced by
// the column whose products are closest to exact multiplication by w (sum of absolute errors over all inputs); on a
// tie the weight's own column wins, otherwise the lowest column index.
// Here as a 256 x 256 error matrix built column by column, then one arg-min per row.
int axc_table_tune_weights(const uint16_t *table, uint16_t *tuned)
{
    if (!table || !tuned)
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    // columns of the source table, contiguous: col[c][i] = table[i][c] (table and tuned may be the same buffer)
    std::vector<int32_t> col((size_t)256 * 256);
    for (int i = 0; i < 256; ++i)
        for (int c = 0; c < 256; ++c)
            col[(size_t)c * 256 + i] = table[(size_t)i * 256 + c];
    // err[w][c] = sum_i |i * w - col[c][i]|   (at most 256 * 65535, fits int32)
    std::vector<int32_t> err((size_t)256 * 256);
    for (int c = 0; c < 256; ++c) {
        const int32_t *cc = &col[(size_t)c * 256];
        for (int w = 0; w < 256; ++w) {
            int32_t e = 0, exact = 0;
            for (int i = 0; i < 256; ++i, exact += w) {
                const int32_t d = exact - cc[i];
                e += d < 0 ? -d : d;
            }
            err[(size_t)w * 256 + c] = e;
        }
    }
    for (int w = 0; w < 256; ++w) {
        const int32_t *ew = &err[(size_t)w * 256];
        int best = (int)(std::min_element(ew, ew + 256) - ew);   // the first of the smallest
        if (ew[w] == ew[best])
            best = w;                                            // the weight's own column wins a tie
        const int32_t *cb = &col[(size_t)best * 256];
        for (int i = 0; i < 256; ++i)
            tuned[(size_t)i * 256 + w] = (uint16_t)cb[i];
    }
    return AXC_OK;
}

// FloatToQuantizedUnclamped<quint8>(0.0f, range_min, range_max) (tf1/axqconv/quantization_utils.h:49-64): the range
// is widened by 256/255 in double, and the code of 0.0f is minus the rounded (half away from zero) code of range_min.
int axc_quint8_zero_point(float range_min, float range_max, int32_t *zero_point)
{
    if (!zero_point)
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    if (range_min == range_max) {
        *zero_point = 0;
        return AXC_OK;
    }
    const double steps = 256.0;
    const float width = range_max - range_min;                   // float, as in the reference
    const double range = (double)width * (steps / (steps - 1.0));
    const double range_scale = steps / range;
    *zero_point = (int32_t)(int64_t)(round(0.0 * range_scale) - round((double)range_min * range_scale));
    return AXC_OK;
}

// QuantizationRangeForMultiplication<quint8, quint8, qint32> (tf1/axqconv/quantization_utils.h:114-140): one level of
// the product is one level of a times one level of b, all in float.
int axc_qint32_range_for_multiplication(float min_a, float max_a, float min_b, float max_b, float *min_c,
                                        float *max_c)
{
    if (!min_c || !max_c)
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    volatile float a_level = (max_a - min_a) / (float)(int64_t)255;
    volatile float b_level = (max_b - min_b) / (float)(int64_t)255;
    volatile float c_level = a_level * b_level;
    volatile float lo = c_level * (float)(int64_t)INT32_MIN;
    volatile float hi = c_level * (float)(int64_t)INT32_MAX;
    *min_c = lo;
    *max_c = hi;
    return AXC_OK;
}

int axc_conv2d_tile_plan(const axc_conv2d_desc *desc, int32_t plan[8])
{
    if (!plan)
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    PreparedDense pd;
    int rc = prepare_dense(desc, &pd);
    if (rc != AXC_OK)
        return rc;
    plan[0] = pd.plan.nt;
    plan[1] = pd.plan.rows_per_tile;
    plan[2] = pd.plan.n_row_tiles;
    plan[3] = pd.plan.n_col_tiles;
    plan[4] = pd.plan.k_splits;
    plan[5] = pd.plan.grid;
    plan[6] = pd.plan.k_splits > 1 ? pd.plan.fills_per_split : pd.plan.fills;
    plan[7] = pd.plan.px ? (px_free_running(pd.plan, pd.gk.KH * pd.gk.KW) ? 2 : 1) : 0;
    return AXC_OK;
}

int axc_set_wait_limit(uint32_t polls)
{
    g_wait_limit.store(polls, std::memory_order_relaxed);
    return AXC_OK;
}

int axc_set_tile_columns(int columns)
{
    if (columns != 0 && columns != 16 && columns != 32 && columns != 64)
        return fail(AXC_INVALID_ARGUMENT, "tile columns must be 0 (planner's choice), 16, 32 or 64");
    g_forced_nt.store(columns, std::memory_order_relaxed);
    return AXC_OK;
}

int axc_set_preexpand(int mode)
{
    if (mode < -1 || mode > 1)
        return fail(AXC_INVALID_ARGUMENT, "preexpand mode must be 0 (planner's choice), 1 (whenever possible) or -1 (never)");
    g_px_mode.store(mode, std::memory_order_relaxed);
    return AXC_OK;
}

int axc_depthwise_conv2d_workspace_bytes(const axc_conv2d_desc *desc, size_t *bytes)
{
    if (!bytes)
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    axc_conv2d_dims dm;
    int rc = geometry(desc, &dm);
    if (rc != AXC_OK)
        return rc;
    rc = validate_for_launch(desc, dm, true);
    if (rc != AXC_OK)
        return rc;
    *bytes = depthwise_workspace(dm.filter_rows * dm.filter_cols, dm.in_depth).total;
    return AXC_OK;
}

int axc_conv2d_minmax(const axc_table *table, const axc_conv2d_desc *desc, const float *input,
                      const float *filter, float input_min, float input_max, float filter_min, float filter_max,
                      float *output, void *workspace, size_t workspace_bytes, void *stream)
{
    return run_dense(table, desc, input, filter, nullptr, nullptr, 0, input_min, input_max, filter_min,
                     filter_max, output, nullptr, workspace, workspace_bytes, stream);
}

int axc_conv2d_minmax_bias_act(const axc_table *table, const axc_conv2d_desc *desc, const float *input,
                               const float *filter, float input_min, float input_max, float filter_min,
                               float filter_max, const float *bias, int activation, float *output, void *workspace,
                               size_t workspace_bytes, void *stream)
{
    if (!output)
        return fail(AXC_INVALID_ARGUMENT, "null tensor pointer");
    return run_dense(table, desc, input, filter, nullptr, nullptr, 0, input_min, input_max, filter_min,
                     filter_max, output, nullptr, workspace, workspace_bytes, stream, false, bias, activation);
}

int axc_depthwise_conv2d_minmax_bias_act(const axc_table *table, const axc_conv2d_desc *desc, const float *input,
                                         const float *filter, float input_min, float input_max, float filter_min,
                                         float filter_max, const float *bias, int activation, float *output,
                                         void *workspace, size_t workspace_bytes, void *stream)
{
    if (!output)
        return fail(AXC_INVALID_ARGUMENT, "null tensor pointer");
    return run_depthwise(table, desc, input, filter, input_min, input_max, filter_min, filter_max, output,
                         nullptr, workspace, workspace_bytes, stream, false, bias, activation);
}

int axc_conv2d_static_workspace_limit(size_t *bytes)
{
    if (!bytes)
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    *bytes = kStaticScratchBytes;
    return AXC_OK;
}

int axc_conv2d_minmax_static(const axc_table *table, const axc_conv2d_desc *desc, const float *input,
                             const float *filter, float input_min, float input_max, float filter_min,
                             float filter_max, float *output, void *stream)
{
    if (!table || !desc)
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    PreparedDense pd;
    int rc = prepare_dense(desc, &pd);
    if (rc != AXC_OK)
        return rc;
    size_t needed = pd.plan.px ? pd.ws.total : pd.ws.total_no_px;
    if (pd.plan.px && needed > kStaticScratchBytes) {
        // without room for pre-expanded rows the layer runs as run_dense re-plans it, or as planned minus the rows
        PreparedDense alt;
        rc = prepare_dense(desc, &alt, true, 4, -1);
        if (rc != AXC_OK)
            return rc;
        needed = std::min(alt.ws.total, pd.ws.total_no_px);
    }
    if (needed > kStaticScratchBytes) {
        char msg[200];
        snprintf(msg, sizeof(msg), "layer needs %zu bytes of workspace, the static workspace holds %zu: use "
                 "axc_conv2d_minmax with a caller-owned workspace", needed, kStaticScratchBytes);
        return fail(AXC_INVALID_ARGUMENT, msg);
    }
    void *ws = nullptr;
    rc = static_scratch(&ws);
    if (rc != AXC_OK)
        return rc;
    // Every byte of the workspace a launch reads is written by that launch first (codes, sums, packed filter,
    // partial sums), so what the previous call left in the array needs no clearing.
    return run_dense(table, desc, input, filter, nullptr, nullptr, 0, input_min, input_max, filter_min, filter_max,
                     output, nullptr, ws, kStaticScratchBytes, stream);
}

int axc_conv2d_minmax_acc_i32(const axc_table *table, const axc_conv2d_desc *desc, const float *input,
                              const float *filter, float input_min, float input_max, float filter_min,
                              float filter_max, int32_t *acc, void *workspace, size_t workspace_bytes,
                              void *stream)
{
    return run_dense(table, desc, input, filter, nullptr, nullptr, 0, input_min, input_max, filter_min,
                     filter_max, nullptr, acc, workspace, workspace_bytes, stream);
}

int axc_conv2d_codes_acc_i32(const axc_table *table, const axc_conv2d_desc *desc, const uint8_t *input_codes,
                             const uint8_t *filter_codes, int input_zero_code, int32_t *acc, void *workspace,
                             size_t workspace_bytes, void *stream)
{
    if (!input_codes || !filter_codes) {
        // distinguish "empty output" from a null pointer only after geometry
        PreparedDense pd;
        int rc = prepare_dense(desc, &pd);
        if (rc != AXC_OK)
            return rc;
        if (pd.empty)
            return AXC_OK;
        return fail(AXC_INVALID_ARGUMENT, "null tensor pointer");
    }
    return run_dense(table, desc, nullptr, nullptr, input_codes, filter_codes, input_zero_code, 0, 0, 0, 0,
                     nullptr, acc, workspace, workspace_bytes, stream);
}

int axc_depthwise_conv2d_minmax(const axc_table *table, const axc_conv2d_desc *desc, const float *input,
                                const float *filter, float input_min, float input_max, float filter_min,
                                float filter_max, float *output, void *workspace, size_t workspace_bytes,
                                void *stream)
{
    return run_depthwise(table, desc, input, filter, input_min, input_max, filter_min, filter_max, output,
                         nullptr, workspace, workspace_bytes, stream);
}

int axc_depthwise_conv2d_minmax_acc_i32(const axc_table *table, const axc_conv2d_desc *desc,
                                        const float *input, const float *filter, float input_min,
                                        float input_max, float filter_min, float filter_max, int32_t *acc,
                                        void *workspace, size_t workspace_bytes, void *stream)
{
    return run_depthwise(table, desc, input, filter, input_min, input_max, filter_min, filter_max, nullptr, acc,
                         workspace, workspace_bytes, stream);
}

int axc_quantize(const float *values, int64_t n, float min, float max, uint8_t *codes, void *stream)
{
    if (n < 0 || (n > 0 && (!values || !codes)))
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    float scale, inv, offset;
    var_quant_props(min, max, &scale, &inv, &offset);
    AXC_HIP(launch_quantize_flat(values, n, offset, inv, codes, static_cast<hipStream_t>(stream)));
    return AXC_OK;
}

int axc_profile_enable(int enable)
{
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    g_prof_enabled = enable != 0;
    return AXC_OK;
}

int axc_profile_reset(void)
{
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    for (auto &kv : g_prof)
        prof_drain_locked(kv.second);
    g_prof.clear();
    return AXC_OK;
}

int axc_profile_read(int index, char *name, size_t name_bytes, double *total_ms, int64_t *launches)
{
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    if (index < 0 || (size_t)index >= g_prof.size())
        return AXC_INVALID_ARGUMENT; // end of list; not an error worth a message
    auto it = g_prof.begin();
    std::advance(it, index);
    prof_drain_locked(it->second);
    if (name && name_bytes) {
        strncpy(name, it->first.c_str(), name_bytes - 1);
        name[name_bytes - 1] = 0;
    }
    if (total_ms)
        *total_ms = it->second.total_ms;
    if (launches)
        *launches = it->second.launches;
    return AXC_OK;
}

int axc_lds_gather_peak(double *lookups_per_second, void *stream)
{
    if (!lookups_per_second)
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    *lookups_per_second = 0.0;
    AXC_HIP(run_lds_gather_peak(lookups_per_second, static_cast<hipStream_t>(stream), false));
    return AXC_OK;
}

int axc_lds_read_peak(double *bytes_per_second, void *stream)
{
    if (!bytes_per_second)
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    *bytes_per_second = 0.0;
    AXC_HIP(run_lds_gather_peak(bytes_per_second, static_cast<hipStream_t>(stream), true));
    return AXC_OK;
}

int axc_valu_issue_peak(double *lane_ops_per_second, void *stream)
{
    if (!lane_ops_per_second)
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    *lane_ops_per_second = 0.0;
    AXC_HIP(run_valu_issue_peak(lane_ops_per_second, kDenseAccumulateMix, static_cast<hipStream_t>(stream)));
    return AXC_OK;
}

int axc_lookup_mix_peak(double *lookups_per_second, void *stream)
{
    if (!lookups_per_second)
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    *lookups_per_second = 0.0;
    AXC_HIP(run_lookup_mix_peak(lookups_per_second, static_cast<hipStream_t>(stream)));
    return AXC_OK;
}

int axc_dense_accumulate_ops_per_lookup(double *ops)
{
    if (!ops)
        return fail(AXC_INVALID_ARGUMENT, "null argument");
    *ops = kDenseAccumulateMix == 0 ? 1.0 : 0.75;
    return AXC_OK;
}

int axc_device_info(int *compute_units, int *lds_bytes_per_workgroup, int *clock_khz)
{
    int dev = 0;
    AXC_HIP(hipGetDevice(&dev));
    int v = 0;
    if (compute_units) {
        AXC_HIP(hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev));
        *compute_units = v;
    }
    if (lds_bytes_per_workgroup) {
        AXC_HIP(hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev));
        *lds_bytes_per_workgroup = v;
    }
    if (clock_khz) {
        AXC_HIP(hipDeviceGetAttribute(&v, hipDeviceAttributeClockRate, dev));
        *clock_khz = v;
    }
    return AXC_OK;
}

} // extern "C"
