// C ABI of the FFT-convolution library: argument checking, FFT-size planning,
// frequency-buffer ownership and the stage schedule of the three passes.
// Everything the reference spreads over fbcunn/SpatialConvolutionFFT.lua
// (planning, buffers), fbcunn/SpatialConvolutionFBFFT.lua (the three passes) and
// the FFI/luaT bindings (src/fft/FFTWrapperLua.cpp, src/MM.cu,
// src/ConvolutionBias.cu) sits behind these entry points.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>
#include <new>
#include <string>

#include "../../include/fbfftconv.h"
#include "kernels.h"

namespace fbfc {

static thread_local std::string g_kernel_log;
void kernel_log_clear() { g_kernel_log.clear(); }
void kernel_log_add(const char *name, long grid_items)
{
    char buf[128];
    std::snprintf(buf, sizeof buf, "%s%s grid=%ld", g_kernel_log.empty() ? "" : "; ", name, grid_items);
    g_kernel_log += buf;
}
const char *kernel_log_get() { return g_kernel_log.c_str(); }

// Per-launch timing (kernels.h): the list of event pairs the launches of this thread draw from while a
// pass with per-launch timing runs.
struct LaunchEvents {
    hipEvent_t *ev;
    int n, used;
};
static thread_local LaunchEvents g_launch_events = {nullptr, 0, 0};
bool launch_events_next(hipEvent_t *start, hipEvent_t *stop)
{
    LaunchEvents &l = g_launch_events;
    if (l.ev == nullptr || l.used + 2 > l.n) return false;
    *start = l.ev[l.used];
    *stop = l.ev[l.used + 1];
    l.used += 2;
    return true;
}

}  // namespace fbfc

namespace {

thread_local std::string g_last_error;

int fail(int code, const std::string &msg)
{
    g_last_error = msg;
    return code;
}

int fail_hip(hipError_t e, const char *what)
{
    return fail(FBFC_ERR_HIP, std::string(what) + ": " + hipGetErrorString(e));
}

constexpr int kMinFft = 8;
constexpr int kMaxFft = 128;
constexpr int kMaxTileFft = 32;

// fbcunn/SpatialConvolutionFFT.lua:875-882 (2^i, i = 1..10)
int next_power_of_2(int v)
{
    for (int i = 1; i <= 10; ++i)
        if ((1 << i) >= v) return 1 << i;
    return -1;
}

int imax(int a, int b) { return a > b ? a : b; }

// One launch transforms all planes of a tensor and addresses a frequency row of its spectrum with
// 32-bit byte offsets: batch * tiles * planes (and out_planes * in_planes) must stay below
// fft_max_planes(n).  Checked when the plan is made, so that an oversized layer is refused with the
// numbers in the message instead of failing at its first pass.
// complex buffers are read and written as 8-byte (re, im) pairs
bool complex_aligned(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 7) == 0; }

int planes_limit(int n, long batch, long tiles, long in_planes, long out_planes)
{
    const long lim = fbfc::fft_max_planes(n);
    const long vb = batch * tiles;  // at most 2^31 * 2^31: no overflow in long
    const long cand[3] = {vb * in_planes, vb * out_planes, out_planes * in_planes};
    const char *what[3] = {"batch x tiles x input planes", "batch x tiles x output planes",
                           "output planes x input planes"};
    for (int i = 0; i < 3; ++i) {
        if (vb > lim || cand[i] > lim) {
            char buf[200];
            std::snprintf(buf, sizeof buf,
                          "%s = %ld planes exceed the %ld one FFT of size %d can take in a launch "
                          "(split the batch)", what[i], cand[i], lim, n);
            return fail(FBFC_ERR_UNSUPPORTED_SIZE, buf);
        }
    }
    return FBFC_OK;
}

int plan_query(const fbfc_conv_desc *d, fbfc_plan_info *info)
{
    if (d == nullptr || info == nullptr) return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    if (d->batch < 1 || d->in_planes < 1 || d->out_planes < 1 || d->in_h < 1 || d->in_w < 1 ||
        d->k_h < 1 || d->k_w < 1)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "sizes must be positive");
    if (d->stride_h != 1 || d->stride_w != 1)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "fft only supports stride-1 convolutions atm");
    if (d->pad_h < 0 || d->pad_w < 0)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "padding must be non-negative");
    if (d->pad_h >= d->k_h || d->pad_w >= d->k_w)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "Padding must be smaller than kernel");
    const int out_h = d->in_h + 2 * d->pad_h - d->k_h + 1;
    const int out_w = d->in_w + 2 * d->pad_w - d->k_w + 1;
    if (out_h < 1 || out_w < 1)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "kernel larger than padded input");
    // prepareFBFFTSizeAndBuffers: square, power of two, covers every operand
    int need = imax(imax(d->in_h + 2 * d->pad_h, d->in_w + 2 * d->pad_w), imax(d->k_h, d->k_w));
    need = imax(need, imax(out_h, out_w));
    int n = next_power_of_2(need);
    if (n < 0) return fail(FBFC_ERR_UNSUPPORTED_SIZE, "Too large a convolution dimensions");
    if (n < kMinFft) n = kMinFft;  // a larger canvas gives the same convolution
    if (n > kMaxFft) {
        char buf[96];
        std::snprintf(buf, sizeof buf, "FFT size %d not supported (8..%d)", n, kMaxFft);
        return fail(FBFC_ERR_UNSUPPORTED_SIZE, buf);
    }
    const int lim = planes_limit(n, d->batch, 1, d->in_planes, d->out_planes);
    if (lim != FBFC_OK) return lim;
    const size_t q = (size_t)n * (n / 2 + 1);
    info->fft_size = n;
    info->n_freq = (int)q;
    info->out_h = out_h;
    info->out_w = out_w;
    info->input_freq_bytes = q * d->batch * d->in_planes * 8;
    info->weight_freq_bytes = q * d->out_planes * d->in_planes * 8;
    info->output_freq_bytes = q * d->batch * d->out_planes * 8;
    info->scratch_bytes = fbfc::bias_grad_scratch_bytes(d->batch, d->out_planes);
    info->tiles_h = 1;
    info->tiles_w = 1;
    info->backward_freq_bytes = info->input_freq_bytes + info->weight_freq_bytes;
    return FBFC_OK;
}

void set_geometry(fbfc_plan *p, int tile_h, int tile_w);

bool fft_size_ok(int n) { return n == 8 || n == 16 || n == 32 || n == 64 || n == 128; }
bool fft_size_tiny(int n) { return n == 2 || n == 4; }

int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Tiled plans (fbcunn/SpatialConvolutionFFTTiled.lua:445-560, 618-672, 745-777): the tile is the
// window that is transformed; consecutive windows are tile - kernel + 1 apart (overlap-save), so a
// window yields that many finished rows / columns of the result.
int plan_query_tiled(const fbfc_conv_desc *d, int tile_h, int tile_w, fbfc_plan_info *info)
{
    const int rc = plan_query(d, info);
    // an image too large for one FFT is exactly what tiling is for
    if (rc != FBFC_OK && rc != FBFC_ERR_UNSUPPORTED_SIZE) return rc;
    const int out_h = d->in_h + 2 * d->pad_h - d->k_h + 1;
    const int out_w = d->in_w + 2 * d->pad_w - d->k_w + 1;
    char buf[160];
    if (tile_h < 1 || tile_w < 1) return fail(FBFC_ERR_INVALID_ARGUMENT, "both tile sizes must be specified");
    if (tile_h < d->k_h || tile_w < d->k_w)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "Tiling cannot be smaller than kernel !");
    if (tile_h > out_h || tile_w > out_w) {
        std::snprintf(buf, sizeof buf, "Tile size too large (%dx%d) for output (%dx%d)", tile_h, tile_w, out_h,
                      out_w);
        return fail(FBFC_ERR_INVALID_ARGUMENT, buf);
    }
    int n = next_power_of_2(imax(tile_h, tile_w));
    if (n < 0 || n > kMaxTileFft) {
        std::snprintf(buf, sizeof buf, "tile FFT size not supported (tiles up to %d)", kMaxTileFft);
        return fail(FBFC_ERR_UNSUPPORTED_SIZE, buf);
    }
    if (n < kMinFft) n = kMinFft;
    const int step_h = tile_h - d->k_h + 1, step_w = tile_w - d->k_w + 1;
    const size_t q = (size_t)n * (n / 2 + 1);
    // output tiles (updateOutput, accGradParameters) and gradInput tiles (updateGradInput)
    const size_t nt_out = (size_t)ceil_div(out_h, step_h) * ceil_div(out_w, step_w);
    const size_t nt_in = (size_t)ceil_div(d->in_h, step_h) * ceil_div(d->in_w, step_w);
    const size_t nt = nt_out > nt_in ? nt_out : nt_in;
    const int lim = planes_limit(n, d->batch, (long)nt, d->in_planes, d->out_planes);
    if (lim != FBFC_OK) return lim;
    info->fft_size = n;
    info->n_freq = (int)q;
    info->out_h = out_h;
    info->out_w = out_w;
    info->input_freq_bytes = q * d->batch * nt * d->in_planes * 8;
    info->weight_freq_bytes = q * d->out_planes * d->in_planes * 8;
    info->output_freq_bytes = q * d->batch * nt * d->out_planes * 8;
    info->scratch_bytes = fbfc::bias_grad_scratch_bytes(d->batch, d->out_planes);
    info->tiles_h = ceil_div(out_h, step_h);
    info->tiles_w = ceil_div(out_w, step_w);
    info->backward_freq_bytes = 0;  // a tiled backward() runs as its two passes
    return FBFC_OK;
}

}  // namespace

// What one pass transforms and contracts.  For an untiled plan the operands are whole planes and
// vbatch is the batch; for a tiled plan they are windows and vbatch = batch * tiles.
struct pass_geom {
    int vbatch;
    // forward-FFT operands that depend on tiling (the weight operand never does)
    int a_h, a_w, a_pad_u, a_pad_l;   // input (fprop, accGrad) resp. gradOutput (bprop)
    fbfc::Window a_win;
    int g_h, g_w;                     // accGrad only: gradOutput
    fbfc::Window g_win;
    // inverse FFT
    int r_h, r_w, r_pad_u, r_pad_l;
    fbfc::Window r_win;
};

struct fbfc_plan {
    fbfc_conv_desc d;
    fbfc_plan_info info;
    bool tiled;
    bool iterated;   // tiled, passes run as fused kernels: no feature-map spectra, only w_freq, part and scratch
    float *part;     // iterated: partial gradWeight results, acc_ranges x F x P x kh x kw floats
    int acc_ranges;
    pass_geom fprop, bprop, accgrad;
    int device;
    float *in_freq, *w_freq, *out_freq, *res_freq, *scratch;
    float *bw_gi, *bw_gw;  // result spectra of fbfc_backward's single-grid stages (fbfc_plan_prepare_backward)
    unsigned reuse;
    bool have_in, have_w, have_out;  // which forward spectra are valid in their buffer
    int timed;  // > 0: repetitions per stage between two events; < 0: every launch timed by its own dispatch
    hipEvent_t ev[FBFC_NUM_STAGES + 1];
    hipEvent_t kev[2 * 16];  // per-launch timing: a (start, stop) pair for each of up to 16 launches of a pass
    bool ev_made;
    float stage_ms[FBFC_NUM_STAGES];
    char stage_kernel[FBFC_NUM_STAGES][160];  // what each stage of the last pass launched
};

namespace {

// Records stage boundaries when the plan is timed.
struct StageTimer {
    fbfc_plan *p;
    hipStream_t s;
    int n;
    int slot[FBFC_NUM_STAGES];
    int first_ev[FBFC_NUM_STAGES + 1];  // per-launch timing: events used before each recorded stage
    StageTimer(fbfc_plan *plan, hipStream_t stream) : p(plan), s(stream), n(0)
    {
        for (auto &name : p->stage_kernel) name[0] = 0;
        fbfc::kernel_log_clear();
        if (p->timed) {
            for (float &m : p->stage_ms) m = 0.0f;
            if (p->timed > 0) {
                (void)hipEventRecord(p->ev[0], s);
            } else {
                fbfc::g_launch_events = {p->kev, (int)(sizeof p->kev / sizeof p->kev[0]), 0};
                first_ev[0] = 0;
            }
        }
    }
    ~StageTimer() { fbfc::g_launch_events = {nullptr, 0, 0}; }
    // number of back-to-back launches of each stage (1 unless the plan is timed)
    int reps() const { return p->timed > 0 ? p->timed : 1; }
    // after the first of several repetitions: what it logged is the stage's launch list
    std::string first_log;
    void keep_log() { first_log = fbfc::kernel_log_get(); }
    void done(int stage)
    {
        // what the stage launched (once, whatever the number of timed repetitions: the first entries)
        std::snprintf(p->stage_kernel[stage], sizeof p->stage_kernel[stage], "%s",
                      first_log.empty() ? fbfc::kernel_log_get() : first_log.c_str());
        first_log.clear();
        fbfc::kernel_log_clear();
        if (!p->timed) return;
        slot[n] = stage;
        ++n;
        if (p->timed > 0) (void)hipEventRecord(p->ev[n], s);
        else first_ev[n] = fbfc::g_launch_events.used;
    }
    int finish()
    {
        if (!p->timed) return FBFC_OK;
        if (p->timed < 0) {
            // every launch carried its own (start, stop) pair: a stage is the sum of its launches
            fbfc::g_launch_events = {nullptr, 0, 0};
            hipError_t e = hipStreamSynchronize(s);
            if (e != hipSuccess) return fail_hip(e, "hipStreamSynchronize");
            for (int i = 0; i < n; ++i) {
                float sum = 0.0f;
                for (int k = first_ev[i]; k < first_ev[i + 1]; k += 2) {
                    float ms = 0.0f;
                    e = hipEventElapsedTime(&ms, p->kev[k], p->kev[k + 1]);
                    if (e != hipSuccess) return fail_hip(e, "hipEventElapsedTime");
                    sum += ms;
                }
                p->stage_ms[slot[i]] = sum;
            }
            return FBFC_OK;
        }
        hipError_t e = hipEventSynchronize(p->ev[n]);
        if (e != hipSuccess) return fail_hip(e, "hipEventSynchronize");
        for (int i = 0; i < n; ++i) {
            float ms = 0.0f;
            e = hipEventElapsedTime(&ms, p->ev[i], p->ev[i + 1]);
            if (e != hipSuccess) return fail_hip(e, "hipEventElapsedTime");
            p->stage_ms[slot[i]] = ms / (float)reps();
        }
        return FBFC_OK;
    }
};

#define FBFC_TRY(expr, what)                                   \
    do {                                                       \
        hipError_t e_ = (expr);                                \
        if (e_ != hipSuccess) return fail_hip(e_, what);       \
    } while (0)

// A stage of a pass: launched once, or tm.reps() times back to back when the plan is timed
// (every stage is a pure function of its inputs, so repeating it changes no result).
#define FBFC_STAGE(tm, expr, what)                             \
    do {                                                       \
        for (int r_ = 0; r_ < (tm).reps(); ++r_) {             \
            if (r_ == 1) (tm).keep_log();                      \
            hipError_t e_ = (expr);                            \
            if (e_ != hipSuccess) return fail_hip(e_, what);   \
        }                                                      \
    } while (0)

fbfc::Window make_window(int d1, int nty, int ntx, int step_y, int step_x, int off_y, int off_x, int img_h,
                         int img_w)
{
    fbfc::Window w;
    w.on = 1;
    w.d1 = d1;
    w.nt = nty * ntx;
    w.ntx = ntx;
    w.step_y = step_y;
    w.step_x = step_x;
    w.off_y = off_y;
    w.off_x = off_x;
    w.img_h = img_h;
    w.img_w = img_w;
    w.remap = 0;  // decided per launch
    return w;
}

void set_geometry(fbfc_plan *p, int tile_h, int tile_w)
{
    const fbfc_conv_desc &d = p->d;
    const int oh = p->info.out_h, ow = p->info.out_w;
    pass_geom &f = p->fprop, &b = p->bprop, &a = p->accgrad;
    if (!p->tiled) {
        f.vbatch = b.vbatch = a.vbatch = d.batch;
        f.a_h = d.in_h; f.a_w = d.in_w; f.a_pad_u = d.pad_h; f.a_pad_l = d.pad_w;
        f.r_h = oh; f.r_w = ow;
        b.a_h = oh; b.a_w = ow;
        b.r_h = d.in_h; b.r_w = d.in_w; b.r_pad_u = d.pad_h; b.r_pad_l = d.pad_w;
        a.a_h = d.in_h; a.a_w = d.in_w; a.a_pad_u = d.pad_h; a.a_pad_l = d.pad_w;
        a.g_h = oh; a.g_w = ow;
        a.r_h = d.k_h; a.r_w = d.k_w;
        return;
    }
    const int sh = tile_h - d.k_h + 1, sw = tile_w - d.k_w + 1;
    // updateOutput: output tiles sh x sw; input windows tile_h x tile_w whose corner is the tile's
    // corner moved up-left by the padding (SpatialConvolutionFFTTiled.lua:521-537)
    const int nty = ceil_div(oh, sh), ntx = ceil_div(ow, sw);
    f.vbatch = d.batch * nty * ntx;
    f.a_h = tile_h; f.a_w = tile_w;
    f.a_win = make_window(d.in_planes, nty, ntx, sh, sw, -d.pad_h, -d.pad_w, d.in_h, d.in_w);
    f.r_h = sh; f.r_w = sw;
    f.r_win = make_window(d.out_planes, nty, ntx, sh, sw, 0, 0, oh, ow);
    // updateGradInput: gradInput tiles sh x sw; gradOutput windows reach kernel - 1 further up-left,
    // and the tile is read kernel - 1 rows / columns into the circular result (:638-658, :420-431)
    const int mty = ceil_div(d.in_h, sh), mtx = ceil_div(d.in_w, sw);
    b.vbatch = d.batch * mty * mtx;
    b.a_h = tile_h; b.a_w = tile_w;
    b.a_win = make_window(d.out_planes, mty, mtx, sh, sw, d.pad_h - (d.k_h - 1), d.pad_w - (d.k_w - 1), oh, ow);
    b.r_h = sh; b.r_w = sw; b.r_pad_u = d.k_h - 1; b.r_pad_l = d.k_w - 1;
    b.r_win = make_window(d.in_planes, mty, mtx, sh, sw, 0, 0, d.in_h, d.in_w);
    // accGradParameters: gradOutput tiles sh x sw against the input windows of updateOutput; the sum
    // over tiles joins the sum over the batch in the contraction (:758-777)
    a.vbatch = f.vbatch;
    a.a_h = tile_h; a.a_w = tile_w;
    a.a_win = f.a_win;
    a.g_h = sh; a.g_w = sw;
    a.g_win = make_window(d.out_planes, nty, ntx, sh, sw, 0, 0, oh, ow);
    a.r_h = d.k_h; a.r_w = d.k_w;
}

}  // namespace

extern "C" {

const char *fbfc_version(void) { return "fbfftconv 0.1 (gfx950)"; }

const char *fbfc_last_error(void) { return g_last_error.c_str(); }

const char *fbfc_last_launch(void) { return fbfc::kernel_log_get(); }

int fbfc_plan_query(const fbfc_conv_desc *desc, fbfc_plan_info *info)
{
    return plan_query(desc, info);
}

int fbfc_plan_query_tiled(const fbfc_conv_desc *desc, int tile_h, int tile_w, fbfc_plan_info *info)
{
    if (desc == nullptr || info == nullptr) return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    return plan_query_tiled(desc, tile_h, tile_w, info);
}

static int plan_create(const fbfc_conv_desc *desc, int tile_h, int tile_w, fbfc_plan **out, bool iterated = false)
{
    if (out == nullptr) return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    *out = nullptr;
    fbfc_plan_info info;
    const bool tiled = tile_h > 0 || tile_w > 0;
    const int rc = tiled ? fbfc_plan_query_tiled(desc, tile_h, tile_w, &info) : plan_query(desc, &info);
    if (rc != FBFC_OK) return rc;
    size_t part_bytes = 0;
    int acc_ranges = 0;
    if (iterated) {
        // the fused passes keep the spectra of the feature maps on chip: the plan owns the weight spectrum,
        // the partial gradWeight results of accGradParameters and the bias gradient's workspace
        const int nt_out = info.tiles_h * info.tiles_w;
        acc_ranges = fbfc::fused_accgrad_ranges(info.fft_size, desc->batch * nt_out, desc->out_planes, desc->in_planes);
        part_bytes = (size_t)acc_ranges * desc->out_planes * desc->in_planes * desc->k_h * desc->k_w * sizeof(float);
        info.input_freq_bytes = 0;
        info.output_freq_bytes = 0;
        info.scratch_bytes += part_bytes;
    }
    fbfc_plan *p = new (std::nothrow) fbfc_plan();
    if (p == nullptr) return fail(FBFC_ERR_OUT_OF_MEMORY, "host allocation failed");
    std::memset(p, 0, sizeof *p);
    p->d = *desc;
    p->info = info;
    p->tiled = tiled;
    p->iterated = iterated;
    p->acc_ranges = acc_ranges;
    set_geometry(p, tile_h, tile_w);
    hipError_t e = hipGetDevice(&p->device);
    if (e == hipSuccess) e = fbfc::fft_prepare_device();
    if (e == hipSuccess) e = fbfc::bias_grad_noalloc_prepare();
    if (e == hipSuccess && iterated) e = fbfc::fused_prepare_device();
    if (e == hipSuccess && !iterated) e = hipMalloc(reinterpret_cast<void **>(&p->in_freq), info.input_freq_bytes);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&p->w_freq), info.weight_freq_bytes);
    if (e == hipSuccess && !iterated) e = hipMalloc(reinterpret_cast<void **>(&p->out_freq), info.output_freq_bytes);
    if (e == hipSuccess && iterated) e = hipMalloc(reinterpret_cast<void **>(&p->part), part_bytes);
    if (e == hipSuccess && iterated)
        e = hipMalloc(reinterpret_cast<void **>(&p->scratch), fbfc::bias_grad_scratch_bytes(desc->batch, desc->out_planes));
    if (e != hipSuccess) {
        const bool oom = (e == hipErrorOutOfMemory);
        (void)hipGetLastError();
        fbfc_plan_destroy(p);
        // the reference reports "Not enough memory for FFT buffers" (SpatialConvolutionFFT.lua:687)
        if (oom) return fail(FBFC_ERR_OUT_OF_MEMORY, "Not enough memory for FFT buffers");
        return fail_hip(e, "plan allocation");
    }
    *out = p;
    return FBFC_OK;
}

int fbfc_plan_create(const fbfc_conv_desc *desc, fbfc_plan **out) { return plan_create(desc, 0, 0, out); }

int fbfc_plan_create_tiled(const fbfc_conv_desc *desc, int tile_h, int tile_w, fbfc_plan **out)
{
    if (tile_h < 1 || tile_w < 1) return fail(FBFC_ERR_INVALID_ARGUMENT, "both tile sizes must be specified");
    return plan_create(desc, tile_h, tile_w, out);
}

int fbfc_plan_create_tiled_iterated(const fbfc_conv_desc *desc, int tile_h, int tile_w, fbfc_plan **out)
{
    if (tile_h < 1 || tile_w < 1) return fail(FBFC_ERR_INVALID_ARGUMENT, "both tile sizes must be specified");
    return plan_create(desc, tile_h, tile_w, out, true);
}

int fbfc_plan_destroy(fbfc_plan *p)
{
    if (p == nullptr) return FBFC_OK;
    if (p->part) (void)hipFree(p->part);
    if (p->in_freq) (void)hipFree(p->in_freq);
    if (p->w_freq) (void)hipFree(p->w_freq);
    if (p->out_freq) (void)hipFree(p->out_freq);
    if (p->res_freq) (void)hipFree(p->res_freq);
    if (p->scratch) (void)hipFree(p->scratch);
    if (p->bw_gi) (void)hipFree(p->bw_gi);
    if (p->bw_gw) (void)hipFree(p->bw_gw);
    if (p->ev_made) {
        for (hipEvent_t &ev : p->ev) (void)hipEventDestroy(ev);
        for (hipEvent_t &ev : p->kev) (void)hipEventDestroy(ev);
    }
    delete p;
    return FBFC_OK;
}

int fbfc_plan_get_info(const fbfc_plan *p, fbfc_plan_info *info)
{
    if (p == nullptr || info == nullptr) return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    *info = p->info;
    return FBFC_OK;
}

int fbfc_plan_set_reuse(fbfc_plan *p, unsigned flags)
{
    if (p == nullptr) return fail(FBFC_ERR_INVALID_ARGUMENT, "null plan");
    if (flags & ~(unsigned)FBFC_REUSE_ALL) return fail(FBFC_ERR_INVALID_ARGUMENT, "unknown memory reuse policy");
    // the fused passes keep no spectrum that could be reused: like the reference's module
    // (SpatialConvolutionFFTTiledIterated.lua:47-48) they override any policy with "none"
    if (p->iterated) return FBFC_OK;
    if (flags != 0 && p->res_freq == nullptr) {
        // With reuse, a pass must not overwrite a spectrum a later pass wants: its
        // result goes to a buffer of its own (the reference keys such buffers by
        // "isOutputOfAlgorithm", SpatialConvolutionFBFFT.lua:382-399).
        size_t bytes = p->info.input_freq_bytes;
        if (p->info.weight_freq_bytes > bytes) bytes = p->info.weight_freq_bytes;
        if (p->info.output_freq_bytes > bytes) bytes = p->info.output_freq_bytes;
        hipError_t e = hipMalloc(reinterpret_cast<void **>(&p->res_freq), bytes);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return fail(FBFC_ERR_OUT_OF_MEMORY, "Not enough memory for FFT buffers");
        }
    }
    p->reuse = flags;
    p->have_in = p->have_w = p->have_out = false;
    return FBFC_OK;
}

int fbfc_plan_set_timed(fbfc_plan *p, int on)
{
    if (p == nullptr) return fail(FBFC_ERR_INVALID_ARGUMENT, "null plan");
    if (on && !p->ev_made) {
        for (hipEvent_t &ev : p->ev) FBFC_TRY(hipEventCreate(&ev), "hipEventCreate");
        for (hipEvent_t &ev : p->kev) FBFC_TRY(hipEventCreate(&ev), "hipEventCreate");
        p->ev_made = true;
    }
    p->timed = on;
    return FBFC_OK;
}

int fbfc_plan_stage_kernel(const fbfc_plan *p, int stage, char *name, size_t n)
{
    if (p == nullptr || name == nullptr || n == 0) return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    if (stage < 0 || stage >= FBFC_NUM_STAGES) return fail(FBFC_ERR_INVALID_ARGUMENT, "no such stage");
    std::snprintf(name, n, "%s", p->stage_kernel[stage]);
    return FBFC_OK;
}

int fbfc_debug_force_contraction_kernel(int variant)
{
    if (variant != -1 && variant != 0 && variant != 1 && variant != 2 && variant != 4 && variant != 8 && variant != 9)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "contraction kernel variant must be -1, 0, 1, 2, 4, 8 or 9");
    fbfc::cgemm_force_variant(variant);
    return FBFC_OK;
}

int fbfc_debug_force_spectrum_streaming(int mode)
{
    if (mode != -1 && mode != 1) return fail(FBFC_ERR_INVALID_ARGUMENT, "spectrum streaming mode must be -1 or 1");
    fbfc::spectrum_stream_force(mode);
    return FBFC_OK;
}

int fbfc_plan_stage_ms(const fbfc_plan *p, float *ms, int n)
{
    if (p == nullptr || ms == nullptr || n < 0) return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    for (int i = 0; i < n; ++i) ms[i] = (i < FBFC_NUM_STAGES) ? p->stage_ms[i] : 0.0f;
    return FBFC_OK;
}

// the weight operand of updateOutput / updateGradInput: never windowed
static fbfc::FwdArgs weight_args(const fbfc_plan *p, const float *weight)
{
    const fbfc_conv_desc &d = p->d;
    return fbfc::FwdArgs{weight, p->w_freq, (long)d.out_planes * d.in_planes, d.k_h, d.k_w, 0, 0, {}, 1};
}

int fbfc_update_output(fbfc_plan *p, const float *input, const float *weight, const float *bias,
                       float *output, void *stream)
{
    if (p == nullptr || input == nullptr || weight == nullptr || output == nullptr)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const fbfc_conv_desc &d = p->d;
    const pass_geom &g = p->fprop;
    const int N = p->info.fft_size;
    // the contraction leaves out the frequencies that are conjugates of others (Hermitian symmetry
    // along ky in the columns kx = 0 and N/2); the inverse transform does not read them
    const int QH = fbfc::hermitian_count(N);
    const fbfc::FreqMap fm = fbfc::hermitian_map(N);
    StageTimer tm(p, s);
    if (p->iterated) {
        // weight spectrum, then one kernel: windows of the input -> spectra -> sum over input planes of
        // I conj(W) -> inverse transform, bias, output tiles
        FBFC_STAGE(tm, fbfc::launch_rfft2d_one(N, weight_args(p, weight), s), "rfft2d(weight)");
        tm.done(FBFC_STAGE_FFT_A);
        fbfc::FusedConvArgs fa = {};
        fa.small = input; fa.big = output; fa.w_freq = p->w_freq; fa.bias = bias;
        fa.small_win = g.a_win; fa.big_win = g.r_win;
        fa.small_h = g.a_h; fa.small_w = g.a_w;
        fa.big_h = g.r_h; fa.big_w = g.r_w; fa.big_pad_u = g.r_pad_u; fa.big_pad_l = g.r_pad_l;
        fa.n_small = d.in_planes; fa.n_big = d.out_planes; fa.w_stride_small = 1; fa.w_stride_big = d.in_planes;
        fa.out_planes = d.out_planes; fa.in_planes = d.in_planes;
        fa.vbatch = g.vbatch; fa.conj_w = 1; fa.alpha = 1.0f / ((float)N * (float)N);
        FBFC_STAGE(tm, fbfc::launch_fused_conv(N, fa, s), "fused updateOutput");
        tm.done(FBFC_STAGE_MM);
        return tm.finish();
    }
    const fbfc::FwdArgs fin = {input, p->in_freq, (long)g.vbatch * d.in_planes, g.a_h, g.a_w, g.a_pad_u,
                               g.a_pad_l, g.a_win, 1};
    const fbfc::FwdArgs fw = weight_args(p, weight);
    // both forward FFTs in one launch
    FBFC_STAGE(tm, fbfc::launch_rfft2d_pair(N, fin, fw, s), "rfft2d(input, weight)");
    tm.done(FBFC_STAGE_FFT_A);
    p->have_in = true;
    p->have_w = true;
    float *res = p->reuse ? p->res_freq : p->out_freq;
    // a new forward pass starts a new step: a spectrum of gradOutput left in the plan belongs to
    // the previous one, whatever the reuse policy
    p->have_out = false;
    // O[b][f] = 1/N^2 sum_p I[b][p] conj(W[f][p])   (SpatialConvolutionFBFFT.lua:157-164)
    FBFC_STAGE(tm, fbfc::launch_cgemm_freq_map(0, p->in_freq, p->w_freq, res, QH, fm, g.vbatch, d.out_planes,
                                     d.in_planes, 1.0f / ((float)N * (float)N), 0, s), "cgemm(fprop)");
    tm.done(FBFC_STAGE_MM);
    const fbfc::InvArgs inv = {res, output, (long)g.vbatch * d.out_planes, g.r_h, g.r_w, g.r_pad_u, g.r_pad_l,
                               bias, d.out_planes, g.r_win, nullptr, nullptr, 0.0f, 0, 0};
    FBFC_STAGE(tm, fbfc::launch_irfft2d_args(N, inv, s), "irfft2d(output)");
    tm.done(FBFC_STAGE_IFFT);
    return tm.finish();
}

int fbfc_update_grad_input(fbfc_plan *p, const float *grad_output, const float *weight,
                           float *grad_input, void *stream)
{
    if (p == nullptr || grad_output == nullptr || weight == nullptr || grad_input == nullptr)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const fbfc_conv_desc &d = p->d;
    const pass_geom &g = p->bprop;
    const int N = p->info.fft_size;
    // the contraction leaves out the frequencies that are conjugates of others (Hermitian symmetry
    // along ky in the columns kx = 0 and N/2); the inverse transform does not read them
    const int QH = fbfc::hermitian_count(N);
    const fbfc::FreqMap fm = fbfc::hermitian_map(N);
    StageTimer tm(p, s);
    if (p->iterated) {
        FBFC_STAGE(tm, fbfc::launch_rfft2d_one(N, weight_args(p, weight), s), "rfft2d(weight)");
        tm.done(FBFC_STAGE_FFT_A);
        fbfc::FusedConvArgs fa = {};
        fa.small = grad_output; fa.big = grad_input; fa.w_freq = p->w_freq; fa.bias = nullptr;
        fa.small_win = g.a_win; fa.big_win = g.r_win;
        fa.small_h = g.a_h; fa.small_w = g.a_w;
        fa.big_h = g.r_h; fa.big_w = g.r_w; fa.big_pad_u = g.r_pad_u; fa.big_pad_l = g.r_pad_l;
        fa.n_small = d.out_planes; fa.n_big = d.in_planes; fa.w_stride_small = d.in_planes; fa.w_stride_big = 1;
        fa.out_planes = d.out_planes; fa.in_planes = d.in_planes;
        fa.vbatch = g.vbatch; fa.conj_w = 0; fa.alpha = 1.0f / ((float)N * (float)N);
        FBFC_STAGE(tm, fbfc::launch_fused_conv(N, fa, s), "fused updateGradInput");
        tm.done(FBFC_STAGE_MM);
        return tm.finish();
    }
    const fbfc::FwdArgs fgo = {grad_output, p->out_freq, (long)g.vbatch * d.out_planes, g.a_h, g.a_w,
                               g.a_pad_u, g.a_pad_l, g.a_win, 1};
    const fbfc::FwdArgs fw = weight_args(p, weight);
    const bool need_w = !((p->reuse & FBFC_REUSE_WEIGHT) && p->have_w);
    if (need_w) {
        FBFC_STAGE(tm, fbfc::launch_rfft2d_pair(N, fgo, fw, s), "rfft2d(gradOutput, weight)");
    } else {
        FBFC_STAGE(tm, fbfc::launch_rfft2d_one(N, fgo, s), "rfft2d(gradOutput)");
    }
    tm.done(FBFC_STAGE_FFT_A);
    // a tiled updateGradInput transforms other windows of gradOutput than accGradParameters does
    p->have_out = !p->tiled;
    p->have_w = true;
    float *res = p->reuse ? p->res_freq : p->in_freq;
    if (!p->reuse) p->have_in = false;
    // GI[b][p] = 1/N^2 sum_f GO[b][f] W[f][p]   (SpatialConvolutionFBFFT.lua:244-251)
    FBFC_STAGE(tm, fbfc::launch_cgemm_freq_map(1, p->out_freq, p->w_freq, res, QH, fm, g.vbatch, d.in_planes,
                                     d.out_planes, 1.0f / ((float)N * (float)N), 0, s), "cgemm(bprop)");
    tm.done(FBFC_STAGE_MM);
    const fbfc::InvArgs inv = {res, grad_input, (long)g.vbatch * d.in_planes, g.r_h, g.r_w, g.r_pad_u,
                               g.r_pad_l, nullptr, 1, g.r_win, nullptr, nullptr, 0.0f, 0, 0};
    FBFC_STAGE(tm, fbfc::launch_irfft2d_args(N, inv, s), "irfft2d(gradInput)");
    tm.done(FBFC_STAGE_IFFT);
    return tm.finish();
}

// reuse_go: the spectrum of gradOutput that updateGradInput just left in the plan is taken as is
static int acc_grad_parameters(fbfc_plan *p, const float *input, const float *grad_output,
                               float *grad_weight, float *grad_bias, float scale, bool reuse_go,
                               void *stream)
{
    if (p == nullptr || input == nullptr || grad_output == nullptr || grad_weight == nullptr)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const fbfc_conv_desc &d = p->d;
    const pass_geom &g = p->accgrad;
    const int N = p->info.fft_size;
    // the contraction leaves out the frequencies that are conjugates of others (Hermitian symmetry
    // along ky in the columns kx = 0 and N/2); the inverse transform does not read them
    const int QH = fbfc::hermitian_count(N);
    const fbfc::FreqMap fm = fbfc::hermitian_map(N);
    StageTimer tm(p, s);
    if (p->iterated) {
        fbfc::FusedAccArgs fa = {};
        fa.input = input; fa.grad_output = grad_output; fa.grad_weight = grad_weight; fa.part = p->part;
        fa.in_win = g.a_win; fa.go_win = g.g_win;
        fa.in_h = g.a_h; fa.in_w = g.a_w; fa.go_h = g.g_h; fa.go_w = g.g_w; fa.kh = d.k_h; fa.kw = d.k_w;
        fa.out_planes = d.out_planes; fa.in_planes = d.in_planes; fa.vbatch = g.vbatch; fa.nranges = p->acc_ranges;
        fa.alpha = scale / ((float)N * (float)N);
        FBFC_STAGE(tm, fbfc::launch_fused_accgrad(N, fa, s), "fused accGradParameters");
        tm.done(FBFC_STAGE_MM);
        if (grad_bias != nullptr) {
            // no spectrum of gradOutput exists to read the plane sums from: the stand-alone reduction
            FBFC_STAGE(tm, fbfc::launch_bias_grad(grad_output, grad_bias, scale, d.batch, d.out_planes,
                                                  p->info.out_h * p->info.out_w, p->scratch, s), "bias grad");
            tm.done(FBFC_STAGE_BIAS_GRAD);
        }
        return tm.finish();
    }
    const fbfc::FwdArgs fgo = {grad_output, p->out_freq, (long)g.vbatch * d.out_planes, g.g_h, g.g_w, 0, 0,
                               g.g_win, 1};
    const fbfc::FwdArgs fin = {input, p->in_freq, (long)g.vbatch * d.in_planes, g.a_h, g.a_w, g.a_pad_u,
                               g.a_pad_l, g.a_win, 1};
    const bool need_go = !(((p->reuse & FBFC_REUSE_OUTPUT) || reuse_go) && p->have_out);
    const bool need_in = !((p->reuse & FBFC_REUSE_INPUT) && p->have_in);
    if (need_go && need_in) {
        FBFC_STAGE(tm, fbfc::launch_rfft2d_pair(N, fgo, fin, s), "rfft2d(gradOutput, input)");
        tm.done(FBFC_STAGE_FFT_A);
    } else if (need_go) {
        FBFC_STAGE(tm, fbfc::launch_rfft2d_one(N, fgo, s), "rfft2d(gradOutput)");
        tm.done(FBFC_STAGE_FFT_A);
    } else if (need_in) {
        FBFC_STAGE(tm, fbfc::launch_rfft2d_one(N, fin, s), "rfft2d(input)");
        tm.done(FBFC_STAGE_FFT_B);
    }
    p->have_in = true;
    float *res = p->reuse ? p->res_freq : p->w_freq;
    if (!p->reuse) p->have_w = false;
    // GW[f][p] = scale/N^2 sum_b conj(GO[b][f]) I[b][p]   (SpatialConvolutionFBFFT.lua:337-344)
    FBFC_STAGE(tm, fbfc::launch_cgemm_freq_map(2, p->out_freq, p->in_freq, res, QH, fm, d.out_planes, d.in_planes,
                                     g.vbatch, scale / ((float)N * (float)N), 0, s), "cgemm(accGrad)");
    tm.done(FBFC_STAGE_MM);
    fbfc::InvArgs inv = {res, grad_weight, (long)d.out_planes * d.in_planes, g.r_h, g.r_w, 0, 0, nullptr, 1, {},
                         nullptr, nullptr, 0.0f, 0, 0};
    if (grad_bias != nullptr) {
        // gradBias[f] = scale * sum_b DC(gradOutput[b][f]) is read off the spectrum of gradOutput by a
        // few extra workgroups of the inverse-FFT launch
        inv.go_freq = p->out_freq;
        inv.grad_bias = grad_bias;
        inv.scale = scale;
        inv.batch = g.vbatch;
        inv.out_planes = d.out_planes;
    }
    FBFC_STAGE(tm, fbfc::launch_irfft2d_args(N, inv, s), "irfft2d(gradWeight) + bias grad");
    tm.done(FBFC_STAGE_IFFT);
    // the spectrum of gradOutput is good for the accGradParameters that follows the updateGradInput
    // of the same gradOutput, once: a second accGradParameters transforms its own
    p->have_out = false;
    return tm.finish();
}

int fbfc_acc_grad_parameters(fbfc_plan *p, const float *input, const float *grad_output,
                             float *grad_weight, float *grad_bias, float scale, void *stream)
{
    return acc_grad_parameters(p, input, grad_output, grad_weight, grad_bias, scale, false, stream);
}

// The buffers the one-grid-per-stage backward pass writes its two product spectra to (it reads all
// three operand spectra in one launch, so neither result may overwrite one of them).  Made here, on the
// plan's device, never inside a pass.
int fbfc_plan_prepare_backward(fbfc_plan *p)
{
    if (p == nullptr) return fail(FBFC_ERR_INVALID_ARGUMENT, "null plan");
    if (p->tiled || (p->bw_gi != nullptr && p->bw_gw != nullptr)) return FBFC_OK;
    int current = 0;
    FBFC_TRY(hipGetDevice(&current), "hipGetDevice");
    if (current != p->device) FBFC_TRY(hipSetDevice(p->device), "hipSetDevice");
    hipError_t e = hipSuccess;
    if (p->bw_gi == nullptr) e = hipMalloc(reinterpret_cast<void **>(&p->bw_gi), p->info.input_freq_bytes);
    if (e == hipSuccess && p->bw_gw == nullptr)
        e = hipMalloc(reinterpret_cast<void **>(&p->bw_gw), p->info.weight_freq_bytes);
    if (e != hipSuccess) (void)hipGetLastError();
    if (current != p->device) (void)hipSetDevice(current);
    if (e == hipErrorOutOfMemory) return fail(FBFC_ERR_OUT_OF_MEMORY, "Not enough memory for FFT buffers");
    if (e != hipSuccess) return fail_hip(e, "backward buffers");
    return FBFC_OK;
}

int fbfc_backward(fbfc_plan *p, const float *input, const float *grad_output, const float *weight,
                  float *grad_input, float *grad_weight, float *grad_bias, float scale, void *stream)
{
    if (p == nullptr || input == nullptr || grad_output == nullptr || weight == nullptr ||
        grad_input == nullptr || grad_weight == nullptr)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    if (p->tiled || p->bw_gi == nullptr || p->bw_gw == nullptr) {
        const int rc = fbfc_update_grad_input(p, grad_output, weight, grad_input, stream);
        if (rc != FBFC_OK) return rc;
        // updateGradInput leaves FFT(gradOutput) in the plan (have_out; not for tiled plans, whose two
        // passes window gradOutput differently)
        return acc_grad_parameters(p, input, grad_output, grad_weight, grad_bias, scale, true, stream);
    }
    // Untiled: both passes share FFT(gradOutput) and have the same FFT size, so each stage is one grid:
    // the (up to) three forward transforms, the two contractions, the two inverse transforms.  Every
    // plane and every frequency goes through the code its own pass would run.
    hipStream_t s = static_cast<hipStream_t>(stream);
    const fbfc_conv_desc &d = p->d;
    const pass_geom &gb = p->bprop, &ga = p->accgrad;
    const int N = p->info.fft_size;
    const int QH = fbfc::hermitian_count(N);
    const fbfc::FreqMap fm = fbfc::hermitian_map(N);
    StageTimer tm(p, s);
    const fbfc::FwdArgs fgo = {grad_output, p->out_freq, (long)gb.vbatch * d.out_planes, gb.a_h, gb.a_w,
                               gb.a_pad_u, gb.a_pad_l, gb.a_win, 1};
    const fbfc::FwdArgs fw = weight_args(p, weight);
    const fbfc::FwdArgs fin = {input, p->in_freq, (long)ga.vbatch * d.in_planes, ga.a_h, ga.a_w, ga.a_pad_u,
                               ga.a_pad_l, ga.a_win, 1};
    const bool need_w = !((p->reuse & FBFC_REUSE_WEIGHT) && p->have_w);
    const bool need_in = !((p->reuse & FBFC_REUSE_INPUT) && p->have_in);
    if (need_w && need_in) {
        FBFC_STAGE(tm, fbfc::launch_rfft2d_triple(N, fgo, fw, fin, s), "rfft2d(gradOutput, weight, input)");
    } else if (need_w) {
        FBFC_STAGE(tm, fbfc::launch_rfft2d_pair(N, fgo, fw, s), "rfft2d(gradOutput, weight)");
    } else if (need_in) {
        // the two passes would transform these in two launches of their own
        FBFC_STAGE(tm, fbfc::launch_rfft2d_each(N, fgo, fin, s), "rfft2d(gradOutput, input)");
    } else {
        FBFC_STAGE(tm, fbfc::launch_rfft2d_one(N, fgo, s), "rfft2d(gradOutput)");
    }
    tm.done(FBFC_STAGE_FFT_A);
    p->have_in = p->have_w = true;
    const float norm = 1.0f / ((float)N * (float)N);
    // GI[b][p] = 1/N^2 sum_f GO[b][f] W[f][p];  GW[f][p] = scale/N^2 sum_b conj(GO[b][f]) I[b][p]
    // (SpatialConvolutionFBFFT.lua:244-251, 337-344)
    const fbfc::MmArgs mgi = {p->out_freq, p->w_freq, p->bw_gi, gb.vbatch, d.in_planes, d.out_planes, norm, 0};
    const fbfc::MmArgs mgw = {p->out_freq, p->in_freq, p->bw_gw, d.out_planes, d.in_planes, ga.vbatch,
                              scale * norm, 0};
    FBFC_STAGE(tm, fbfc::launch_cgemm_backward(mgi, mgw, QH, fm, s), "cgemm(bprop, accGrad)");
    tm.done(FBFC_STAGE_MM);
    const fbfc::InvArgs igi = {p->bw_gi, grad_input, (long)gb.vbatch * d.in_planes, gb.r_h, gb.r_w, gb.r_pad_u,
                               gb.r_pad_l, nullptr, 1, gb.r_win, nullptr, nullptr, 0.0f, 0, 0};
    fbfc::InvArgs igw = {p->bw_gw, grad_weight, (long)d.out_planes * d.in_planes, ga.r_h, ga.r_w, 0, 0, nullptr, 1,
                         {}, nullptr, nullptr, 0.0f, 0, 0};
    if (grad_bias != nullptr) {
        igw.go_freq = p->out_freq;
        igw.grad_bias = grad_bias;
        igw.scale = scale;
        igw.batch = ga.vbatch;
        igw.out_planes = d.out_planes;
    }
    FBFC_STAGE(tm, fbfc::launch_irfft2d_two(N, igi, igw, s), "irfft2d(gradInput, gradWeight) + bias grad");
    tm.done(FBFC_STAGE_IFFT);
    p->have_out = false;
    return tm.finish();
}

static int fft2d_impl(const float *real, long planes, int h, int w, int pad_u, int pad_l, int fft_size,
                      float *freq, void *stream)
{
    if (real == nullptr || freq == nullptr) return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    if (!complex_aligned(freq)) return fail(FBFC_ERR_INVALID_ARGUMENT, "the complex buffer must be 8-byte aligned");
    if (!fft_size_ok(fft_size) && !fft_size_tiny(fft_size))
        return fail(FBFC_ERR_UNSUPPORTED_SIZE, "FBFFT error: unsupported size");
    if (planes < 1 || h < 1 || w < 1 || pad_u < 0 || pad_l < 0 || h + pad_u > fft_size ||
        w + pad_l > fft_size)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "plane plus padding must fit the FFT size");
    FBFC_TRY(fbfc::fft_prepare_device(), "device set-up");
    if (fft_size_tiny(fft_size)) {
        FBFC_TRY(fbfc::launch_rfft2d_tiny(fft_size, real, freq, planes, h, w, pad_u, pad_l,
                                          static_cast<hipStream_t>(stream)), "rfft2d");
        return FBFC_OK;
    }
    FBFC_TRY(fbfc::launch_rfft2d(fft_size, real, freq, planes, h, w, pad_u, pad_l,
                                 static_cast<hipStream_t>(stream)), "rfft2d");
    return FBFC_OK;
}

int fbfc_fft2d(const float *real, long planes, int h, int w, int pad_u, int pad_l, int fft_size,
               float *freq, void *stream)
{
    fbfc::kernel_log_clear();
    return fft2d_impl(real, planes, h, w, pad_u, pad_l, fft_size, freq, stream);
}

static int ifft2d_impl(const float *freq, long planes, int h, int w, int pad_u, int pad_l, int fft_size,
                       float *real, const float *bias, int bias_period, void *stream)
{
    if (real == nullptr || freq == nullptr) return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    if (!complex_aligned(freq)) return fail(FBFC_ERR_INVALID_ARGUMENT, "the complex buffer must be 8-byte aligned");
    if (!fft_size_ok(fft_size) && !fft_size_tiny(fft_size))
        return fail(FBFC_ERR_UNSUPPORTED_SIZE, "FBFFT error: unsupported size");
    if (planes < 1 || h < 1 || w < 1 || pad_u < 0 || pad_l < 0 || h + pad_u > fft_size ||
        w + pad_l > fft_size)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "plane plus padding must fit the FFT size");
    if (bias != nullptr && bias_period < 1) return fail(FBFC_ERR_INVALID_ARGUMENT, "bias_period must be positive");
    FBFC_TRY(fbfc::fft_prepare_device(), "device set-up");
    if (fft_size_tiny(fft_size)) {
        FBFC_TRY(fbfc::launch_irfft2d_tiny(fft_size, freq, real, planes, h, w, pad_u, pad_l, bias, bias_period,
                                           static_cast<hipStream_t>(stream)), "irfft2d");
        return FBFC_OK;
    }
    FBFC_TRY(fbfc::launch_irfft2d(fft_size, freq, real, planes, h, w, pad_u, pad_l, bias, bias_period,
                                  static_cast<hipStream_t>(stream)), "irfft2d");
    return FBFC_OK;
}

int fbfc_ifft2d(const float *freq, long planes, int h, int w, int pad_u, int pad_l, int fft_size,
                float *real, const float *bias, int bias_period, void *stream)
{
    fbfc::kernel_log_clear();
    return ifft2d_impl(freq, planes, h, w, pad_u, pad_l, fft_size, real, bias, bias_period, stream);
}

// fbfft leaves a 2-D spectrum as (planes, N/2+1, N): rows = the halved axis.  Which axis that is
// depends on the size (test/test_FFTModule.lua:238-241): see layout_kernels.hip.
static int planes_layout_mode(int n) { return (n < 8 || n > 32) ? 1 : 2; }

size_t fbfc_planes_layout_workspace_bytes(long planes, int fft_size)
{
    if (planes < 1 || (!fft_size_ok(fft_size) && !fft_size_tiny(fft_size))) return 0;
    return (size_t)planes * fft_size * (fft_size / 2 + 1) * 8;
}

int fbfc_fft2d_planes(const float *real, long planes, int h, int w, int pad_u, int pad_l, int fft_size,
                      float *freq_planes, float *workspace, void *stream)
{
    if (freq_planes == nullptr || workspace == nullptr) return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    if (!complex_aligned(freq_planes))
        return fail(FBFC_ERR_INVALID_ARGUMENT, "the complex buffer must be 8-byte aligned");
    fbfc::kernel_log_clear();
    const int rc = fft2d_impl(real, planes, h, w, pad_u, pad_l, fft_size, workspace, stream);
    if (rc != FBFC_OK) return rc;
    FBFC_TRY(fbfc::launch_freq_to_planes(workspace, freq_planes, planes, fft_size * (fft_size / 2 + 1), fft_size,
                                         planes_layout_mode(fft_size), static_cast<hipStream_t>(stream)),
             "layout conversion");
    return FBFC_OK;
}

int fbfc_ifft2d_planes(const float *freq_planes, long planes, int h, int w, int pad_u, int pad_l, int fft_size,
                       float *real, float *workspace, void *stream)
{
    if (freq_planes == nullptr || workspace == nullptr || real == nullptr)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    if (!complex_aligned(freq_planes) || !complex_aligned(workspace))
        return fail(FBFC_ERR_INVALID_ARGUMENT, "the complex buffer must be 8-byte aligned");
    if (!fft_size_ok(fft_size) && !fft_size_tiny(fft_size))
        return fail(FBFC_ERR_UNSUPPORTED_SIZE, "FBFFT error: unsupported size");
    // everything the inverse transform would refuse is refused before the conversion is launched
    if (planes < 1 || h < 1 || w < 1 || pad_u < 0 || pad_l < 0 || h + pad_u > fft_size || w + pad_l > fft_size)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "plane plus padding must fit the FFT size");
    fbfc::kernel_log_clear();
    FBFC_TRY(fbfc::launch_planes_to_freq(freq_planes, workspace, planes, fft_size * (fft_size / 2 + 1), fft_size,
                                         planes_layout_mode(fft_size), static_cast<hipStream_t>(stream)),
             "layout conversion");
    return ifft2d_impl(workspace, planes, h, w, pad_u, pad_l, fft_size, real, nullptr, 1, stream);
}

static int transpose_mm_impl(const float *A, const float *B, float *C, int n_freq, int m, int n, int k,
                             float inv_norm, int conj_trans_a, int conj_trans_b, int accumulate, void *stream);

size_t fbfc_transpose_mm_planes_workspace_bytes(int n_freq, int m, int n, int k)
{
    if (n_freq < 1 || m < 1 || n < 1 || k < 1) return 0;
    return (size_t)n_freq * 8 * ((size_t)m * k + (size_t)k * n + (size_t)m * n);
}

int fbfc_transpose_mm_planes(const float *A, const float *B, float *C, int n_freq, int m, int n, int k,
                             float inv_norm, int conj_trans_a, int conj_trans_b, int accumulate,
                             float *workspace, void *stream)
{
    if (A == nullptr || B == nullptr || C == nullptr || workspace == nullptr)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    if (n_freq < 1 || m < 1 || n < 1 || k < 1) return fail(FBFC_ERR_INVALID_ARGUMENT, "sizes must be positive");
    if (!complex_aligned(A) || !complex_aligned(B) || !complex_aligned(C) || !complex_aligned(workspace))
        return fail(FBFC_ERR_INVALID_ARGUMENT, "complex operands must be 8-byte aligned");
    if (conj_trans_a && conj_trans_b)
        return fail(FBFC_ERR_UNSUPPORTED_DIMENSION, "conjugate-transposing both operands is not supported");
    hipStream_t s = static_cast<hipStream_t>(stream);
    float *wa = workspace;
    float *wb = wa + (size_t)n_freq * m * k * 2;
    float *wc = wb + (size_t)n_freq * k * n * 2;
    fbfc::kernel_log_clear();
    FBFC_TRY(fbfc::launch_planes_to_freq(A, wa, (long)m * k, n_freq, 0, 0, s), "layout conversion (A)");
    FBFC_TRY(fbfc::launch_planes_to_freq(B, wb, (long)k * n, n_freq, 0, 0, s), "layout conversion (B)");
    if (accumulate) FBFC_TRY(fbfc::launch_planes_to_freq(C, wc, (long)m * n, n_freq, 0, 0, s), "layout conversion (C)");
    const int rc = transpose_mm_impl(wa, wb, wc, n_freq, m, n, k, inv_norm, conj_trans_a, conj_trans_b, accumulate,
                                     stream);
    if (rc != FBFC_OK) return rc;
    FBFC_TRY(fbfc::launch_freq_to_planes(wc, C, (long)m * n, n_freq, 0, 0, s), "layout conversion (C)");
    return FBFC_OK;
}

static bool fft1d_size_ok(int n) { return n >= 2 && n <= 128 && (n & (n - 1)) == 0; }

int fbfc_fft1d(const float *real, long rows, int n, int pad_l, int fft_size, float *freq, void *stream)
{
    fbfc::kernel_log_clear();
    if (real == nullptr || freq == nullptr) return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    if (!fft1d_size_ok(fft_size)) return fail(FBFC_ERR_UNSUPPORTED_SIZE, "FBFFT error: unsupported size");
    if (rows < 1 || n < 1 || pad_l < 0 || n + pad_l > fft_size)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "row plus padding must fit the FFT size");
    FBFC_TRY(fbfc::launch_rfft1d(fft_size, real, freq, rows, n, pad_l, static_cast<hipStream_t>(stream)),
             "rfft1d");
    return FBFC_OK;
}

int fbfc_ifft1d(const float *freq, long rows, int n, int pad_l, int fft_size, float *real, void *stream)
{
    fbfc::kernel_log_clear();
    if (real == nullptr || freq == nullptr) return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    if (!fft1d_size_ok(fft_size)) return fail(FBFC_ERR_UNSUPPORTED_SIZE, "FBFFT error: unsupported size");
    if (rows < 1 || n < 1 || pad_l < 0 || n + pad_l > fft_size)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "row plus padding must fit the FFT size");
    FBFC_TRY(fbfc::launch_irfft1d(fft_size, freq, real, rows, n, pad_l, static_cast<hipStream_t>(stream)),
             "irfft1d");
    return FBFC_OK;
}

static int transpose_mm_impl(const float *A, const float *B, float *C, int n_freq, int m, int n, int k,
                             float inv_norm, int conj_trans_a, int conj_trans_b, int accumulate, void *stream)
{
    if (A == nullptr || B == nullptr || C == nullptr) return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    if (!complex_aligned(A) || !complex_aligned(B) || !complex_aligned(C))
        return fail(FBFC_ERR_INVALID_ARGUMENT, "complex operands must be 8-byte aligned");
    if (n_freq < 1 || m < 1 || n < 1 || k < 1) return fail(FBFC_ERR_INVALID_ARGUMENT, "sizes must be positive");
    if (conj_trans_a && conj_trans_b)
        return fail(FBFC_ERR_UNSUPPORTED_DIMENSION, "conjugate-transposing both operands is not supported");
    const int mode = conj_trans_b ? 0 : (conj_trans_a ? 2 : 1);
    FBFC_TRY(fbfc::launch_cgemm_freq(mode, A, B, C, n_freq, m, n, k, inv_norm, accumulate ? 1 : 0,
                                     static_cast<hipStream_t>(stream)), "cgemm");
    return FBFC_OK;
}

int fbfc_transpose_mm(const float *A, const float *B, float *C, int n_freq, int m, int n, int k,
                      float inv_norm, int conj_trans_a, int conj_trans_b, int accumulate, void *stream)
{
    fbfc::kernel_log_clear();
    return transpose_mm_impl(A, B, C, n_freq, m, n, k, inv_norm, conj_trans_a, conj_trans_b, accumulate, stream);
}

// ---- direct convolution -------------------------------------------------------------------------
static int direct_check(const fbfc_conv_desc *d)
{
    if (d == nullptr) return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    if (d->batch < 1 || d->in_planes < 1 || d->out_planes < 1 || d->in_h < 1 || d->in_w < 1 || d->k_h < 1 ||
        d->k_w < 1 || d->stride_h < 1 || d->stride_w < 1)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "sizes must be positive");
    if (d->pad_h < 0 || d->pad_w < 0) return fail(FBFC_ERR_INVALID_ARGUMENT, "padding must be non-negative");
    if (d->in_h + 2 * d->pad_h < d->k_h || d->in_w + 2 * d->pad_w < d->k_w)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "kernel larger than padded input");
    return FBFC_OK;
}

static_assert(sizeof(fbfc_conv_desc) == 11 * sizeof(int), "the direct kernels read the descriptor as 11 ints");

int fbfc_direct_update_output(const fbfc_conv_desc *desc, const float *input, const float *weight,
                              const float *bias, float *output, void *stream)
{
    const int rc = direct_check(desc);
    if (rc != FBFC_OK) return rc;
    if (input == nullptr || weight == nullptr || output == nullptr) return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    fbfc::kernel_log_clear();
    FBFC_TRY(fbfc::launch_direct_fprop(reinterpret_cast<const int *>(desc), input, weight, bias, output,
                                       static_cast<hipStream_t>(stream)), "direct updateOutput");
    return FBFC_OK;
}

int fbfc_direct_update_grad_input(const fbfc_conv_desc *desc, const float *grad_output, const float *weight,
                                  float *grad_input, void *stream)
{
    const int rc = direct_check(desc);
    if (rc != FBFC_OK) return rc;
    if (grad_output == nullptr || weight == nullptr || grad_input == nullptr)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    fbfc::kernel_log_clear();
    FBFC_TRY(fbfc::launch_direct_bprop(reinterpret_cast<const int *>(desc), grad_output, weight, grad_input,
                                       static_cast<hipStream_t>(stream)), "direct updateGradInput");
    return FBFC_OK;
}

int fbfc_direct_acc_grad_parameters(const fbfc_conv_desc *desc, const float *input, const float *grad_output,
                                    float *grad_weight, float *grad_bias, float scale, float *scratch,
                                    void *stream)
{
    const int rc = direct_check(desc);
    if (rc != FBFC_OK) return rc;
    if (input == nullptr || grad_output == nullptr || grad_weight == nullptr)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    if (grad_bias != nullptr && scratch == nullptr)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "the bias gradient needs its workspace");
    fbfc::kernel_log_clear();
    hipStream_t s = static_cast<hipStream_t>(stream);
    FBFC_TRY(fbfc::launch_direct_accgrad(reinterpret_cast<const int *>(desc), input, grad_output, grad_weight, scale,
                                         s), "direct accGradParameters");
    if (grad_bias != nullptr) {
        const int o_h = (desc->in_h + 2 * desc->pad_h - desc->k_h) / desc->stride_h + 1;
        const int o_w = (desc->in_w + 2 * desc->pad_w - desc->k_w) / desc->stride_w + 1;
        FBFC_TRY(fbfc::launch_bias_grad(grad_output, grad_bias, scale, desc->batch, desc->out_planes, o_h * o_w,
                                        scratch, s), "bias grad");
    }
    return FBFC_OK;
}

int fbfc_update_output_bias(float *output, const float *bias, int batch, int planes, int h, int w,
                            void *stream)
{
    if (output == nullptr || bias == nullptr) return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    if (batch < 1 || planes < 1 || h < 1 || w < 1) return fail(FBFC_ERR_INVALID_ARGUMENT, "sizes must be positive");
    FBFC_TRY(fbfc::launch_bias_add(output, bias, batch, planes, h * w, static_cast<hipStream_t>(stream)),
             "bias add");
    return FBFC_OK;
}

int fbfc_update_output_bias_strided(float *output, const float *bias, int batch, int planes, int h, int w,
                                    long stride_b, long stride_f, long stride_h, long stride_w,
                                    long bias_stride, void *stream)
{
    if (output == nullptr || bias == nullptr) return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    if (batch < 1 || planes < 1 || h < 1 || w < 1) return fail(FBFC_ERR_INVALID_ARGUMENT, "sizes must be positive");
    FBFC_TRY(fbfc::launch_bias_add_strided(output, bias, batch, planes, h, w, stride_b, stride_f, stride_h,
                                           stride_w, bias_stride, static_cast<hipStream_t>(stream)),
             "bias add");
    return FBFC_OK;
}

int fbfc_acc_grad_parameters_bias_strided(const float *grad_output, float *grad_bias, float scale, int batch,
                                          int planes, int h, int w, long stride_b, long stride_f,
                                          long stride_h, long stride_w, long bias_stride, float *scratch,
                                          void *stream)
{
    if (grad_output == nullptr || grad_bias == nullptr || scratch == nullptr)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    if (batch < 1 || planes < 1 || h < 1 || w < 1) return fail(FBFC_ERR_INVALID_ARGUMENT, "sizes must be positive");
    FBFC_TRY(fbfc::launch_bias_grad_strided(grad_output, grad_bias, scale, batch, planes, h, w, stride_b,
                                            stride_f, stride_h, stride_w, bias_stride, scratch,
                                            static_cast<hipStream_t>(stream)), "bias grad");
    return FBFC_OK;
}

size_t fbfc_bias_grad_scratch_bytes(int batch, int planes)
{
    if (batch < 1 || planes < 1) return 0;
    return fbfc::bias_grad_scratch_bytes(batch, planes);
}

int fbfc_acc_grad_parameters_bias(const float *grad_output, float *grad_bias, float scale, int batch,
                                  int planes, int h, int w, float *scratch, void *stream)
{
    if (grad_output == nullptr || grad_bias == nullptr || scratch == nullptr)
        return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    if (batch < 1 || planes < 1 || h < 1 || w < 1) return fail(FBFC_ERR_INVALID_ARGUMENT, "sizes must be positive");
    FBFC_TRY(fbfc::launch_bias_grad(grad_output, grad_bias, scale, batch, planes, h * w, scratch,
                                    static_cast<hipStream_t>(stream)), "bias grad");
    return FBFC_OK;
}

int fbfc_acc_grad_parameters_bias_noalloc(const float *grad_output, float *grad_bias, float scale,
                                          int batch, int planes, int h, int w, void *stream)
{
    if (grad_output == nullptr || grad_bias == nullptr) return fail(FBFC_ERR_INVALID_ARGUMENT, "null argument");
    if (batch < 1 || planes < 1 || h < 1 || w < 1) return fail(FBFC_ERR_INVALID_ARGUMENT, "sizes must be positive");
    if (planes > fbfc::bias_grad_noalloc_max_planes()) {
        char buf[160];
        std::snprintf(buf, sizeof buf,
                      "%d planes exceed the %d the fixed workspace holds; use fbfc_acc_grad_parameters_bias "
                      "with a workspace of your own", planes, fbfc::bias_grad_noalloc_max_planes());
        return fail(FBFC_ERR_UNSUPPORTED_SIZE, buf);
    }
    FBFC_TRY(fbfc::launch_bias_grad_noalloc(grad_output, grad_bias, scale, batch, planes, h * w,
                                            static_cast<hipStream_t>(stream)), "bias grad (fixed workspace)");
    return FBFC_OK;
}

}  // extern "C"
