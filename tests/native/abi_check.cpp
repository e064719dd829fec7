// C ABI check without Python or torch: a plain HIP host program that links
// libascan.so through include/ascan.h, drives every compute entry point with buffers
// from hipMalloc on a stream of its own, and compares the results with the
// sequential fp64 loops of the test oracle (oracle/seqscan.c).  Also checks the
// status codes of invalid calls.  Exit status 0 and a final "ok" line on success.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "ascan.h"

extern "C" {
void seq_forward_from_f32(const float* g, const float* x, const float* init, double* out, int64_t rows, int64_t T,
                          int reverse);
void seq_backward_from_f32(const float* g, const float* state, const float* init, const float* dout, double* dg,
                           double* dx, double* dinit, int64_t rows, int64_t T);
void seq_forward_sigmoid_f32(const float* z, const float* x, const float* init, double* out, int64_t rows, int64_t T);
void seq_backward_sigmoid_f32(const float* z, const float* state, const float* init, const float* dout, double* dz,
                              double* dx, double* dinit, int64_t rows, int64_t T);
void seq_forward_exp_f32(const float* z, const float* x, const float* init, double* out, int64_t rows, int64_t T);
void seq_backward_exp_f32(const float* z, const float* state, const float* init, const float* dout, double* dz,
                          double* dx, double* dinit, int64_t rows, int64_t T);
void seq_forward_lerp_f32(const float* z, const float* v, const float* init, double* out, int64_t rows, int64_t T);
void seq_backward_lerp_f32(const float* z, const float* v, const float* state, const float* init, const float* dout,
                           double* dz, double* dv, double* dinit, int64_t rows, int64_t T);
void seq_forward_expnorm_f32(const float* z, const float* v, const float* init, double* out, int64_t rows, int64_t T);
void seq_backward_expnorm_f32(const float* z, const float* v, const float* state, const float* init, const float* dout,
                           double* dz, double* dv, double* dinit, int64_t rows, int64_t T);
}

#define HIP_OK(call)                                                                          \
    do {                                                                                      \
        hipError_t e_ = (call);                                                               \
        if (e_ != hipSuccess) {                                                               \
            std::fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_)); \
            std::exit(2);                                                                     \
        }                                                                                     \
    } while (0)

#define EXPECT(cond)                                                           \
    do {                                                                       \
        if (!(cond)) {                                                         \
            std::fprintf(stderr, "%s:%d check failed: %s\n", __FILE__, __LINE__, #cond); \
            std::exit(1);                                                      \
        }                                                                      \
    } while (0)

namespace {

struct Lcg {
    uint64_t s;
    float uniform() {  // [0, 1)
        s = s * 6364136223846793005ull + 1442695040888963407ull;
        return (float)((s >> 40) & 0xFFFFFF) / 16777216.0f;
    }
};

struct DeviceBuffer {
    void* p = nullptr;
    size_t bytes = 0;
    explicit DeviceBuffer(size_t n) : bytes(n) { HIP_OK(hipMalloc(&p, n ? n : 1)); }
    ~DeviceBuffer() { (void)hipFree(p); }
    DeviceBuffer(const DeviceBuffer&) = delete;
    DeviceBuffer& operator=(const DeviceBuffer&) = delete;
};

void upload(DeviceBuffer& d, const std::vector<float>& h, hipStream_t s) {
    HIP_OK(hipMemcpyAsync(d.p, h.data(), h.size() * sizeof(float), hipMemcpyHostToDevice, s));
}
std::vector<float> download(const DeviceBuffer& d, size_t n, hipStream_t s) {
    std::vector<float> h(n);
    HIP_OK(hipMemcpyAsync(h.data(), d.p, n * sizeof(float), hipMemcpyDeviceToHost, s));
    HIP_OK(hipStreamSynchronize(s));
    return h;
}

double worst(const std::vector<float>& got, const std::vector<double>& want) {
    double scale = 1.0, err = 0.0;
    for (double w : want) scale = std::fmax(scale, std::fabs(w));
    for (size_t i = 0; i < want.size(); ++i) err = std::fmax(err, std::fabs((double)got[i] - want[i]));
    return err / scale;
}

// One problem through forward, reverse and backward, with and without an
// initial state, with and without the workspace; every result against the loops.
void check_problem(int64_t rows, int64_t T, bool with_initial, hipStream_t stream) {
    std::printf("rows=%lld T=%lld initial=%d\n", (long long)rows, (long long)T, (int)with_initial);
    std::fflush(stdout);
    const size_t n = (size_t)rows * (size_t)T;
    Lcg rng{(uint64_t)(rows * 1000003 + T)};
    std::vector<float> g(n), x(n), d(n), init(rows);
    for (size_t i = 0; i < n; ++i) {
        g[i] = rng.uniform();
        x[i] = 2.0f * rng.uniform() - 1.0f;
        d[i] = 2.0f * rng.uniform() - 1.0f;
    }
    for (auto& v : init) v = 4.0f * rng.uniform() - 2.0f;
    const float* init_host = with_initial ? init.data() : nullptr;

    DeviceBuffer dg_in(n * 4), dx_in(n * 4), dd_in(n * 4), dinit_in(rows * 4);
    DeviceBuffer out(n * 4), rev(n * 4), d_gates(n * 4), d_tokens(n * 4), d_init(rows * 4);
    upload(dg_in, g, stream);
    upload(dx_in, x, stream);
    upload(dd_in, d, stream);
    upload(dinit_in, init, stream);
    const void* init_dev = with_initial ? dinit_in.p : nullptr;

    const size_t ws_bytes = ascan_workspace_bytes(rows, T, ASCAN_F32);
    DeviceBuffer ws(ws_bytes);
    void* ws_ptr = ws_bytes ? ws.p : nullptr;

    if (with_initial) {
        EXPECT(ascan_forward_from(dg_in.p, dx_in.p, init_dev, out.p, rows, T, ASCAN_F32, 0, ws_ptr, ws_bytes, stream) == ASCAN_OK);
        EXPECT(ascan_forward_from(dg_in.p, dx_in.p, init_dev, rev.p, rows, T, ASCAN_F32, 1, ws_ptr, ws_bytes, stream) == ASCAN_OK);
        EXPECT(ascan_backward_from(dg_in.p, out.p, init_dev, dd_in.p, d_gates.p, d_tokens.p, d_init.p, rows, T, ASCAN_F32,
                                   ws_ptr, ws_bytes, stream) == ASCAN_OK);
    } else if (ws_bytes) {
        EXPECT(ascan_forward_split(dg_in.p, dx_in.p, out.p, rows, T, ASCAN_F32, 0, ws_ptr, ws_bytes, stream) == ASCAN_OK);
        EXPECT(ascan_forward_split(dg_in.p, dx_in.p, rev.p, rows, T, ASCAN_F32, 1, ws_ptr, ws_bytes, stream) == ASCAN_OK);
        EXPECT(ascan_backward_split(dg_in.p, out.p, dd_in.p, d_gates.p, d_tokens.p, rows, T, ASCAN_F32, ws_ptr, ws_bytes,
                                    stream) == ASCAN_OK);
    } else {
        EXPECT(ascan_forward(dg_in.p, dx_in.p, out.p, rows, T, ASCAN_F32, 0, stream) == ASCAN_OK);
        EXPECT(ascan_forward(dg_in.p, dx_in.p, rev.p, rows, T, ASCAN_F32, 1, stream) == ASCAN_OK);
        EXPECT(ascan_backward(dg_in.p, out.p, dd_in.p, d_gates.p, d_tokens.p, rows, T, ASCAN_F32, stream) == ASCAN_OK);
    }
    const std::vector<float> h_out = download(out, n, stream), h_rev = download(rev, n, stream);
    const std::vector<float> h_dg = download(d_gates, n, stream), h_dx = download(d_tokens, n, stream);

    std::vector<double> t_out(n), t_rev(n), t_dg(n), t_dx(n), t_di(rows);
    seq_forward_from_f32(g.data(), x.data(), init_host, t_out.data(), rows, T, 0);
    seq_forward_from_f32(g.data(), x.data(), init_host, t_rev.data(), rows, T, 1);
    // the backward pass consumes the states the GPU produced
    seq_backward_from_f32(g.data(), h_out.data(), init_host, d.data(), t_dg.data(), t_dx.data(), t_di.data(), rows, T);
    const double tol = 2e-5;
    EXPECT(worst(h_out, t_out) <= tol);
    EXPECT(worst(h_rev, t_rev) <= tol);
    EXPECT(worst(h_dx, t_dx) <= tol);
    EXPECT(worst(h_dg, t_dg) <= tol);
    if (with_initial) EXPECT(worst(download(d_init, rows, stream), t_di) <= tol);

    // Backward pass of the reverse scan: the loops run on the sequences flipped in time.
    {
        EXPECT(ascan_backward_reverse(dg_in.p, rev.p, init_dev, dd_in.p, d_gates.p, d_tokens.p, with_initial ? d_init.p : nullptr,
                                      rows, T, ASCAN_F32, ws_ptr, ws_bytes, stream) == ASCAN_OK);
        auto flipped = [&](const std::vector<float>& v) {
            std::vector<float> f(v.size());
            for (int64_t r = 0; r < rows; ++r)
                for (int64_t t = 0; t < T; ++t) f[r * T + t] = v[r * T + (T - 1 - t)];
            return f;
        };
        const std::vector<float> fg = flipped(g), fs = flipped(h_rev), fd = flipped(d);
        std::vector<double> f_dg(n), f_dx(n);
        seq_backward_from_f32(fg.data(), fs.data(), init_host, fd.data(), f_dg.data(), f_dx.data(), t_di.data(), rows, T);
        for (int64_t r = 0; r < rows; ++r)
            for (int64_t t = 0; t < T; ++t) {
                t_dg[r * T + t] = f_dg[r * T + (T - 1 - t)];
                t_dx[r * T + t] = f_dx[r * T + (T - 1 - t)];
            }
        EXPECT(worst(download(d_tokens, n, stream), t_dx) <= tol);
        EXPECT(worst(download(d_gates, n, stream), t_dg) <= tol);
        if (with_initial) EXPECT(worst(download(d_init, rows, stream), t_di) <= tol);
    }
    if (ws_bytes) {
        unsigned char header[64];
        HIP_OK(hipMemcpy(header, ws.p, sizeof(header), hipMemcpyDeviceToHost));
        EXPECT(ascan_workspace_timeouts(header) == 0u);
    }
}

// The gated entry points (sigmoid gate; sigmoid gate with interpolated values; exponential gates) and the
// split-row forward scan whose table is the library's static array.
void check_gated_and_static(int64_t rows, int64_t T, hipStream_t stream) {
    std::printf("gated rows=%lld T=%lld\n", (long long)rows, (long long)T);
    std::fflush(stdout);
    const size_t n = (size_t)rows * (size_t)T;
    Lcg rng{(uint64_t)(rows * 7919 + T)};
    std::vector<float> z(n), x(n), d(n), init(rows);
    for (size_t i = 0; i < n; ++i) {
        z[i] = 8.0f * rng.uniform() - 3.0f;
        x[i] = 2.0f * rng.uniform() - 1.0f;
        d[i] = 2.0f * rng.uniform() - 1.0f;
    }
    for (auto& v : init) v = 4.0f * rng.uniform() - 2.0f;
    DeviceBuffer dz_in(n * 4), dx_in(n * 4), dd_in(n * 4), dinit_in(rows * 4);
    DeviceBuffer out(n * 4), d_z(n * 4), d_x(n * 4), d_init(rows * 4);
    upload(dz_in, z, stream);
    upload(dx_in, x, stream);
    upload(dd_in, d, stream);
    upload(dinit_in, init, stream);
    const size_t ws_bytes = ascan_workspace_bytes(rows, T, ASCAN_F32);
    DeviceBuffer ws(ws_bytes);
    void* ws_ptr = ws_bytes ? ws.p : nullptr;
    std::vector<double> t_out(n), t_dz(n), t_dx(n), t_di(rows);
    const double tol = 4e-5;  // the in-kernel sigmoid (about 2 ulp) enters every gate

    EXPECT(ascan_forward_gated(dz_in.p, dx_in.p, dinit_in.p, out.p, rows, T, ASCAN_F32, ASCAN_GATE_SIGMOID, ws_ptr,
                               ws_bytes, stream) == ASCAN_OK);
    EXPECT(ascan_backward_gated(dz_in.p, out.p, dinit_in.p, dd_in.p, d_z.p, d_x.p, d_init.p, rows, T, ASCAN_F32,
                                ASCAN_GATE_SIGMOID, ws_ptr, ws_bytes, stream) == ASCAN_OK);
    std::vector<float> h_out = download(out, n, stream);
    seq_forward_sigmoid_f32(z.data(), x.data(), init.data(), t_out.data(), rows, T);
    seq_backward_sigmoid_f32(z.data(), h_out.data(), init.data(), d.data(), t_dz.data(), t_dx.data(), t_di.data(), rows, T);
    EXPECT(worst(h_out, t_out) <= tol);
    EXPECT(worst(download(d_z, n, stream), t_dz) <= tol);
    EXPECT(worst(download(d_x, n, stream), t_dx) <= tol);
    EXPECT(worst(download(d_init, rows, stream), t_di) <= tol);

    EXPECT(ascan_forward_gated(dz_in.p, dx_in.p, dinit_in.p, out.p, rows, T, ASCAN_F32, ASCAN_GATE_SIGMOID_LERP, ws_ptr,
                               ws_bytes, stream) == ASCAN_OK);
    EXPECT(ascan_backward_lerp(dz_in.p, dx_in.p, out.p, dinit_in.p, dd_in.p, d_z.p, d_x.p, d_init.p, rows, T, ASCAN_F32,
                               ws_ptr, ws_bytes, stream) == ASCAN_OK);
    h_out = download(out, n, stream);
    seq_forward_lerp_f32(z.data(), x.data(), init.data(), t_out.data(), rows, T);
    seq_backward_lerp_f32(z.data(), x.data(), h_out.data(), init.data(), d.data(), t_dz.data(), t_dx.data(), t_di.data(),
                          rows, T);
    EXPECT(worst(h_out, t_out) <= tol);
    EXPECT(worst(download(d_z, n, stream), t_dz) <= tol);
    EXPECT(worst(download(d_x, n, stream), t_dx) <= tol);
    EXPECT(worst(download(d_init, rows, stream), t_di) <= tol);

    // exponential gate: the stored values are logarithms of gates in (0, 1]
    {
        std::vector<float> logs(n);
        for (size_t i = 0; i < n; ++i) logs[i] = -0.25f * std::fabs(z[i]);
        upload(dz_in, logs, stream);
        EXPECT(ascan_forward_gated(dz_in.p, dx_in.p, dinit_in.p, out.p, rows, T, ASCAN_F32, ASCAN_GATE_EXP, ws_ptr,
                                   ws_bytes, stream) == ASCAN_OK);
        EXPECT(ascan_backward_gated(dz_in.p, out.p, dinit_in.p, dd_in.p, d_z.p, d_x.p, d_init.p, rows, T, ASCAN_F32,
                                    ASCAN_GATE_EXP, ws_ptr, ws_bytes, stream) == ASCAN_OK);
        h_out = download(out, n, stream);
        seq_forward_exp_f32(logs.data(), x.data(), init.data(), t_out.data(), rows, T);
        seq_backward_exp_f32(logs.data(), h_out.data(), init.data(), d.data(), t_dz.data(), t_dx.data(), t_di.data(), rows,
                             T);
        EXPECT(worst(h_out, t_out) <= tol);
        EXPECT(worst(download(d_z, n, stream), t_dz) <= tol);
        EXPECT(worst(download(d_x, n, stream), t_dx) <= tol);
        EXPECT(worst(download(d_init, rows, stream), t_di) <= tol);
    }

    // exponential gate with the input scale sqrt(1 - gate^2): logarithms strictly below zero
    {
        std::vector<float> logs(n);
        for (size_t i = 0; i < n; ++i) logs[i] = -0.25f * std::fabs(z[i]) - 1e-3f;
        upload(dz_in, logs, stream);
        EXPECT(ascan_forward_gated(dz_in.p, dx_in.p, dinit_in.p, out.p, rows, T, ASCAN_F32, ASCAN_GATE_EXP_NORM, ws_ptr,
                                   ws_bytes, stream) == ASCAN_OK);
        EXPECT(ascan_backward_gated_values(dz_in.p, dx_in.p, out.p, dinit_in.p, dd_in.p, d_z.p, d_x.p, d_init.p, rows, T,
                                           ASCAN_F32, ASCAN_GATE_EXP_NORM, ws_ptr, ws_bytes, stream) == ASCAN_OK);
        h_out = download(out, n, stream);
        seq_forward_expnorm_f32(logs.data(), x.data(), init.data(), t_out.data(), rows, T);
        seq_backward_expnorm_f32(logs.data(), x.data(), h_out.data(), init.data(), d.data(), t_dz.data(), t_dx.data(),
                                 t_di.data(), rows, T);
        EXPECT(worst(h_out, t_out) <= tol);
        EXPECT(worst(download(d_z, n, stream), t_dz) <= tol);
        EXPECT(worst(download(d_x, n, stream), t_dx) <= tol);
        EXPECT(worst(download(d_init, rows, stream), t_di) <= tol);
    }

    // static-table forward scan: stored values in [0, 1) as gates (x from a zero state)
    std::vector<float> g(n);
    for (size_t i = 0; i < n; ++i) g[i] = rng.uniform();
    upload(dz_in, g, stream);
    EXPECT(ascan_forward_split_static(dz_in.p, dx_in.p, out.p, rows, T, ASCAN_F32, 0, stream) == ASCAN_OK);
    seq_forward_from_f32(g.data(), x.data(), nullptr, t_out.data(), rows, T, 0);
    EXPECT(worst(download(out, n, stream), t_out) <= 2e-5);
}

void check_status_codes(hipStream_t stream) {
    DeviceBuffer a(4096), b(4096), c(4096);
    EXPECT(ascan_abi_version() == ASCAN_ABI_VERSION);
    EXPECT(ascan_forward(nullptr, b.p, c.p, 1, 16, ASCAN_F32, 0, stream) == ASCAN_ERR_NULL_POINTER);
    EXPECT(ascan_forward(a.p, b.p, c.p, 1, 16, 99, 0, stream) == ASCAN_ERR_BAD_DTYPE);
    EXPECT(ascan_forward(a.p, b.p, c.p, -1, 16, ASCAN_F32, 0, stream) == ASCAN_ERR_BAD_SHAPE);
    EXPECT(ascan_forward((char*)a.p + 2, b.p, c.p, 1, 16, ASCAN_F32, 0, stream) == ASCAN_ERR_MISALIGNED);
    EXPECT(ascan_backward(a.p, b.p, c.p, nullptr, a.p, 1, 16, ASCAN_F32, stream) == ASCAN_ERR_NULL_POINTER);
    // outputs may not overlap inputs or each other; buffers that merely touch are fine
    EXPECT(ascan_forward(a.p, b.p, a.p, 1, 16, ASCAN_F32, 0, stream) == ASCAN_ERR_OVERLAP);
    EXPECT(ascan_forward(a.p, b.p, (char*)b.p + 32, 1, 16, ASCAN_F32, 0, stream) == ASCAN_ERR_OVERLAP);
    EXPECT(ascan_backward(a.p, b.p, c.p, (char*)a.p + 1024, (char*)a.p + 1024 + 60, 1, 16, ASCAN_F32, stream) ==
           ASCAN_ERR_OVERLAP);
    EXPECT(ascan_backward(a.p, b.p, c.p, (char*)c.p + 60, (char*)a.p + 1024, 1, 16, ASCAN_F32, stream) ==
           ASCAN_ERR_OVERLAP);
    EXPECT(ascan_forward(a.p, (char*)a.p + 64, (char*)a.p + 128, 1, 16, ASCAN_F32, 0, stream) == ASCAN_OK);
    EXPECT(ascan_backward(a.p, (char*)a.p + 64, (char*)a.p + 128, (char*)a.p + 192, (char*)a.p + 256, 1, 16, ASCAN_F32,
                          stream) == ASCAN_OK);
    // empty problems are accepted without touching any pointer
    EXPECT(ascan_forward(nullptr, nullptr, nullptr, 0, 16, ASCAN_F32, 0, stream) == ASCAN_OK);
    EXPECT(ascan_backward(nullptr, nullptr, nullptr, nullptr, nullptr, 4, 0, ASCAN_F32, stream) == ASCAN_OK);
    EXPECT(ascan_workspace_bytes(100000, 4096, ASCAN_F32) == 0);
    EXPECT(ascan_workspace_bytes(100000, 65536, ASCAN_F32) > 0);
    EXPECT(ascan_workspace_bytes(2, 1 << 20, ASCAN_F32) > 0);
    EXPECT(ascan_status_string(ASCAN_ERR_MISALIGNED) != nullptr);
    // gates: unknown code; a sigmoid gate with a complex dtype; the interpolating gate without its values
    EXPECT(ascan_forward_gated(a.p, b.p, nullptr, c.p, 1, 16, ASCAN_F32, 9, nullptr, 0, stream) == ASCAN_ERR_BAD_ACTIVATION);
    EXPECT(ascan_forward_gated(a.p, b.p, nullptr, c.p, 1, 16, ASCAN_C64, ASCAN_GATE_SIGMOID_LERP, nullptr, 0, stream) ==
           ASCAN_ERR_BAD_ACTIVATION);
    EXPECT(ascan_backward_gated(a.p, b.p, nullptr, c.p, (char*)a.p + 1024, (char*)a.p + 2048, nullptr, 1, 16, ASCAN_F32,
                                ASCAN_GATE_SIGMOID_LERP, nullptr, 0, stream) == ASCAN_ERR_BAD_ACTIVATION);
    EXPECT(ascan_backward_lerp(a.p, nullptr, b.p, nullptr, c.p, (char*)a.p + 1024, (char*)a.p + 2048, nullptr, 1, 16,
                               ASCAN_F32, nullptr, 0, stream) == ASCAN_ERR_NULL_POINTER);
    EXPECT(ascan_backward_gated(a.p, b.p, nullptr, c.p, (char*)a.p + 1024, (char*)a.p + 2048, nullptr, 1, 16, ASCAN_F32,
                                ASCAN_GATE_EXP_NORM, nullptr, 0, stream) == ASCAN_ERR_BAD_ACTIVATION);
    EXPECT(ascan_backward_gated_values(a.p, (char*)a.p + 3072, b.p, nullptr, c.p, (char*)a.p + 1024, (char*)a.p + 2048,
                                       nullptr, 1, 16, ASCAN_F32, ASCAN_GATE_EXP, nullptr, 0, stream) ==
           ASCAN_ERR_BAD_ACTIVATION);
    EXPECT(ascan_backward_gated_values(a.p, nullptr, b.p, nullptr, c.p, (char*)a.p + 1024, (char*)a.p + 2048, nullptr, 1,
                                       16, ASCAN_F32, ASCAN_GATE_EXP_NORM, nullptr, 0, stream) == ASCAN_ERR_NULL_POINTER);
    // the static-table entry point refuses what does not fit its array
    EXPECT(ascan_forward_split_static(a.p, b.p, c.p, 128, 1 << 24, ASCAN_F32, 0, stream) == ASCAN_ERR_TOO_LARGE);
}

}  // namespace

int main() {
    int count = 0;
    HIP_OK(hipGetDeviceCount(&count));
    EXPECT(count > 0);
    HIP_OK(hipSetDevice(0));
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));  // default priority
    check_status_codes(stream);
    const int64_t problems[][2] = {{7, 1}, {5, 37}, {300, 1024}, {64, 4099}, {33, 65536}, {3, 300000}, {1, 1 << 20}};
    for (const auto& p : problems) {
        check_problem(p[0], p[1], false, stream);
        check_problem(p[0], p[1], true, stream);
    }
    const int64_t gated[][2] = {{9, 40}, {300, 1024}, {64, 4099}, {12, 65536}, {3, 300000}};
    for (const auto& p : gated) check_gated_and_static(p[0], p[1], stream);
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipStreamDestroy(stream));
    std::printf("ok\n");
    return 0;
}
