// Standalone harness: drives axconv::ApproxConv2DOp (the TensorFlow-free op shell) on seeded synthetic layers.
//
//   axconv_harness [--layer config1|northstar|dw] [--table FILE] [--seed S] [--reps R]
//
// It follows the recipe of the reference's only test (tf2/test/test_table_approx_conv_2d.py:39-62): draw
// random tensors, fake-quantize them with their min/max, run the op with the exact table t[a][b] = a*b and
// compare with an ordinary convolution of the fake-quantized tensors; the expected max-normalized L-infinity
// error is ~1e-6 (tf2/README.md:31).  The ordinary convolution is a plain fp64 loop on the host, so the check
// is only run for layers small enough for it.  Larger layers are timed: HIP events around R launches.
// Exit status 0 = check passed (or timing only), 1 = check failed, 2 = setup error.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "approx_conv2d_op.h"

namespace {

#define HIP_OK(expr)                                                                                  \
    do {                                                                                              \
        hipError_t e_ = (expr);                                                                       \
        if (e_ != hipSuccess) {                                                                       \
            std::fprintf(stderr, "%s failed: %s\n", #expr, hipGetErrorString(e_));                    \
            std::exit(2);                                                                             \
        }                                                                                             \
    } while (0)

// Nudged quantization range as the op computes it (tf2/src/approx_ops_types.h:29-49).
struct Nudged {
    float min, max, scale;
};
Nudged nudge(float mn, float mx)
{
    const float qmin = 0.0f, qmax = 255.0f;
    Nudged r;
    r.scale = (mx - mn) / (qmax - qmin);
    const float zp_real = qmin - mn / r.scale;
    float zp;
    if (zp_real < qmin)
        zp = qmin;
    else if (zp_real > qmax)
        zp = qmax;
    else
        zp = std::round(zp_real);
    r.min = (qmin - zp) * r.scale;
    r.max = (qmax - zp) * r.scale;
    return r;
}

// Clamp to the nudged range and snap to its grid: what the op's callers feed it.
void fake_quantize(std::vector<float> &v, float mn, float mx)
{
    const Nudged n = nudge(mn, mx);
    for (float &x : v) {
        const float c = std::min(std::max(x, n.min), n.max);
        x = std::floor((c - n.min) / n.scale + 0.5f) * n.scale + n.min;
    }
}

class HarnessContext : public axconv::OpContext {
public:
    explicit HarnessContext(hipStream_t s) : m_stream(s) {}
    ~HarnessContext() override { release(); }
    float *allocate_output(const std::vector<int64_t> &shape) override
    {
        size_t n = 1;
        for (int64_t d : shape)
            n *= (size_t)d;
        return static_cast<float *>(allocate_temp(n * sizeof(float)));
    }
    void *allocate_temp(size_t bytes) override
    {
        void *p = nullptr;
        if (hipMalloc(&p, bytes ? bytes : 1) != hipSuccess)
            return nullptr;
        m_blocks.push_back(p);
        return p;
    }
    void *stream() override { return m_stream; }
    void release()
    {
        for (void *p : m_blocks)
            (void)hipFree(p);
        m_blocks.clear();
    }

private:
    hipStream_t m_stream;
    std::vector<void *> m_blocks;
};

struct Layer {
    const char *name;
    int n, h, w, c, kh, kw, co, stride;
    float in_lo, in_hi, f_sigma, f_range;
    bool depthwise;
    bool check; // small enough for the fp64 host convolution
};

const Layer kLayers[] = {
    {"config1", 1, 32, 32, 16, 3, 3, 32, 1, -1.0f, 1.0f, 0.1f, 0.3f, false, true},
    {"northstar", 64, 56, 56, 64, 3, 3, 64, 1, -1.0f, 1.0f, 0.1f, 0.3f, false, false},
    {"dw", 2, 28, 28, 32, 3, 3, 1, 1, -1.0f, 1.0f, 0.1f, 0.3f, true, true},
};

// Attribute validation of the shell (no GPU needed): every rejected attribute set must come back with the
// reference's message (tf2/src/approx_nn_conv_ops.cpp:266-303).
int selftest()
{
    struct Case {
        const char *what;
        axconv::ApproxConv2DAttrs attrs;
        const char *expect; // nullptr = must be accepted
    };
    auto base = []() {
        axconv::ApproxConv2DAttrs a;
        a.strides = {1, 1, 1, 1};
        a.padding = "SAME";
        return a;
    };
    std::vector<Case> cases;
    cases.push_back({"defaults", base(), nullptr});
    { auto a = base(); a.strides = {1, 1, 1}; cases.push_back({"3 strides", a, "Sliding window strides must specify 4 dimensions"}); }
    { auto a = base(); a.dilations = {1, 1}; cases.push_back({"2 dilations", a, "Sliding window dilations field must specify 4 dimensions"}); }
    { auto a = base(); a.strides = {2, 1, 1, 1}; cases.push_back({"batch stride", a, "Current implementation does not yet support strides in the batch and depth dimensions."}); }
    { auto a = base(); a.strides = {1, 0, 1, 1}; cases.push_back({"zero stride", a, "Row and column strides should be larger than 0."}); }
    { auto a = base(); a.dilations = {1, 1, 1, 2}; cases.push_back({"depth dilation", a, "Current implementation does not yet support dilations in the batch and depth dimensions."}); }
    { auto a = base(); a.dilations = {1, 0, 1, 1}; cases.push_back({"zero dilation", a, "Dilated rates should be larger than 0."}); }
    { auto a = base(); a.data_format = "NHCW"; cases.push_back({"data format", a, "Invalid data format"}); }
    { auto a = base(); a.explicit_paddings = {0, 0, 1, 1, 1, 1, 0, 0}; cases.push_back({"stray explicit paddings", a, "explicit_paddings attribute must be empty if the padding attribute is not EXPLICIT"}); }
    int failed = 0;
    for (const Case &c : cases) {
        axconv::ApproxConv2DParameters params;
        const axconv::Status st = axconv::InitApproxConv2DParameters(c.attrs, &params);
        const bool ok = c.expect ? (!st.ok() && st.code == AXC_INVALID_ARGUMENT && st.message == c.expect) : st.ok();
        std::printf("%-26s %s\n", c.what, ok ? "ok" : "MISMATCH");
        if (!ok) {
            std::printf("    got: [%d] %s\n", st.code, st.message.c_str());
            ++failed;
        }
    }
    std::printf(failed ? "FAILED\n" : "OK\n");
    return failed ? 1 : 0;
}

void usage()
{
    std::printf("usage: axconv_harness [--layer config1|northstar|dw] [--table FILE] [--seed S] [--reps R]\n"
                "  --layer   seeded synthetic layer (default config1: 1x32x32x16 -> 32, 3x3, stride 1, SAME)\n"
                "  --table   256x256 little-endian uint16 truth table file; default: the exact table a*b,\n"
                "            for which the result is checked against an fp64 convolution on the host\n"
                "  --reps    timed launches (default 20)\n"
                "  --selftest  check the shell's attribute validation against the reference's messages (no GPU)\n");
}

} // namespace

int main(int argc, char **argv)
{
    std::string layer_name = "config1", table_file;
    uint64_t seed = 1;
    int reps = 20;
    for (int i = 1; i < argc; ++i) {
        const std::string a = argv[i];
        if (a == "--help" || a == "-h") {
            usage();
            return 0;
        } else if (a == "--selftest") {
            return selftest();
        } else if (a == "--layer" && i + 1 < argc) {
            layer_name = argv[++i];
        } else if (a == "--table" && i + 1 < argc) {
            table_file = argv[++i];
        } else if (a == "--seed" && i + 1 < argc) {
            seed = std::strtoull(argv[++i], nullptr, 10);
        } else if (a == "--reps" && i + 1 < argc) {
            reps = std::atoi(argv[++i]);
        } else {
            usage();
            return 2;
        }
    }
    const Layer *L = nullptr;
    for (const Layer &l : kLayers)
        if (layer_name == l.name)
            L = &l;
    if (!L) {
        usage();
        return 2;
    }

    // ---- seeded tensors, fake-quantized as the op's callers do ----
    std::mt19937_64 rng(seed);
    std::uniform_real_distribution<float> uni(L->in_lo, L->in_hi);
    std::normal_distribution<float> nor(0.0f, L->f_sigma);
    std::vector<float> x((size_t)L->n * L->h * L->w * L->c), f((size_t)L->kh * L->kw * L->c * L->co);
    for (float &v : x)
        v = uni(rng);
    for (float &v : f)
        v = nor(rng);
    const float in_min = L->in_lo, in_max = L->in_hi, f_min = -L->f_range, f_max = L->f_range;
    fake_quantize(x, in_min, in_max);
    fake_quantize(f, f_min, f_max);

    // ---- the op ----
    axconv::ApproxConv2DAttrs attrs;
    attrs.strides = {1, L->stride, L->stride, 1};
    attrs.padding = "SAME";
    attrs.mul_map_file = table_file;
    attrs.depthwise = L->depthwise;
    std::vector<uint16_t> exact;
    const bool exact_table = table_file.empty();
    if (exact_table) {
        exact.resize(65536);
        for (int a = 0; a < 256; ++a)
            for (int b = 0; b < 256; ++b)
                exact[(size_t)a * 256 + b] = (uint16_t)(a * b);
    }
    axconv::ApproxConv2DOp op = exact_table ? axconv::ApproxConv2DOp(attrs, exact.data()) : axconv::ApproxConv2DOp(attrs);
    if (!op.status().ok()) {
        std::fprintf(stderr, "op construction failed: %s\n", op.status().message.c_str());
        return 2;
    }

    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    axconv::DeviceTensor dx, df, dy;
    dx.shape = {L->n, L->h, L->w, L->c};
    df.shape = {L->kh, L->kw, L->c, L->co};
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&dx.data), x.size() * sizeof(float)));
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&df.data), f.size() * sizeof(float)));
    HIP_OK(hipMemcpy(dx.data, x.data(), x.size() * sizeof(float), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(df.data, f.data(), f.size() * sizeof(float), hipMemcpyHostToDevice));

    HarnessContext ctx(stream);
    axconv::Status st = op.Compute(&ctx, dx, df, in_min, in_max, f_min, f_max, &dy);
    if (!st.ok()) {
        std::fprintf(stderr, "Compute failed: %s\n", st.message.c_str());
        return 2;
    }
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<float> y((size_t)dy.num_elements());
    HIP_OK(hipMemcpy(y.data(), dy.data, y.size() * sizeof(float), hipMemcpyDeviceToHost));
    const int oh = (int)dy.shape[1], ow = (int)dy.shape[2], oc = (int)dy.shape[3];
    std::printf("layer %s: input %dx%dx%dx%d, filter %dx%dx%dx%d%s -> output %dx%dx%dx%d\n", L->name, L->n, L->h,
                L->w, L->c, L->kh, L->kw, L->c, L->co, L->depthwise ? " (depthwise)" : "", L->n, oh, ow, oc);

    int status = 0;
    if (exact_table && L->check) {
        // ordinary convolution of the fake-quantized tensors, fp64, SAME padding
        const int ph = std::max(0, ((oh - 1) * L->stride + L->kh - L->h)) / 2;
        const int pw = std::max(0, ((ow - 1) * L->stride + L->kw - L->w)) / 2;
        double max_err = 0.0, max_ref = 0.0;
        for (int n = 0; n < L->n; ++n)
            for (int r = 0; r < oh; ++r)
                for (int c = 0; c < ow; ++c)
                    for (int o = 0; o < oc; ++o) {
                        double acc = 0.0;
                        for (int kh = 0; kh < L->kh; ++kh)
                            for (int kw = 0; kw < L->kw; ++kw) {
                                const int ih = r * L->stride - ph + kh, iw = c * L->stride - pw + kw;
                                if (ih < 0 || ih >= L->h || iw < 0 || iw >= L->w)
                                    continue;
                                const float *px = &x[(((size_t)n * L->h + ih) * L->w + iw) * L->c];
                                if (L->depthwise) {
                                    acc += (double)px[o] * f[((size_t)kh * L->kw + kw) * L->c + o];
                                } else {
                                    const float *pf = &f[(((size_t)kh * L->kw + kw) * L->c) * L->co + o];
                                    for (int ci = 0; ci < L->c; ++ci)
                                        acc += (double)px[ci] * pf[(size_t)ci * L->co];
                                }
                            }
                        const double got = y[(((size_t)n * oh + r) * ow + c) * oc + o];
                        max_err = std::max(max_err, std::fabs(got - acc));
                        max_ref = std::max(max_ref, std::fabs(acc));
                    }
        const double linf = max_err / std::max(max_ref, 1e-30);
        std::printf("exact table vs fp64 convolution: max-normalized Linf = %.3g (bound 1e-5)\n", linf);
        if (!(linf <= 1e-5))
            status = 1;
    }

    // ---- timing ----
    if (reps > 0) {
        hipEvent_t e0, e1;
        HIP_OK(hipEventCreate(&e0));
        HIP_OK(hipEventCreate(&e1));
        for (int i = 0; i < 3; ++i) {
            ctx.release();
            st = op.Compute(&ctx, dx, df, in_min, in_max, f_min, f_max, &dy);
        }
        HIP_OK(hipStreamSynchronize(stream));
        // allocate once outside the timed region: the op itself never allocates
        ctx.release();
        std::vector<HarnessContext *> ctxs;
        for (int i = 0; i < reps; ++i)
            ctxs.push_back(new HarnessContext(stream));
        HIP_OK(hipEventRecord(e0, stream));
        for (int i = 0; i < reps && st.ok(); ++i)
            st = op.Compute(ctxs[i], dx, df, in_min, in_max, f_min, f_max, &dy);
        HIP_OK(hipEventRecord(e1, stream));
        HIP_OK(hipEventSynchronize(e1));
        float ms = 0.0f;
        HIP_OK(hipEventElapsedTime(&ms, e0, e1));
        for (HarnessContext *c : ctxs)
            delete c;
        if (!st.ok()) {
            std::fprintf(stderr, "Compute failed: %s\n", st.message.c_str());
            return 2;
        }
        const double macs = (double)L->n * oh * ow * oc * L->kh * L->kw * (L->depthwise ? 1 : L->c);
        std::printf("%d launches (hipMalloc of output and workspace inside the timed region): %.4f ms each, %.1f approximate GMAC/s\n",
                    reps, ms / reps, macs / (ms / reps * 1e-3) / 1e9);
    }
    (void)hipFree(dx.data);
    (void)hipFree(df.data);
    std::printf(status == 0 ? "OK\n" : "FAILED\n");
    return status;
}
