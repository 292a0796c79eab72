// Stand-alone consumer of the C ABI (include/oeq_amd.h): no Python and no torch at run time.
//
// Reads a kernel bundle written by tests/test_cabi_standalone_gpu.py
//   <dir>/kernels.hip   generated HIP source
//   <dir>/bundle.txt    problem dims, kernel descriptors, batch size
//   <dir>/{x,y,w,g}.bin inputs, <dir>/{z,dx,dy,dw}.bin expected results (raw little-endian floats)
// compiles the source with oeq_jit_compile, runs oeq_tp_forward / oeq_tp_backward on plain
// hipMalloc'ed buffers and compares with the expected values (max normalised error); when the set has
// second-order kernels, oeq_tp_double_backward is checked against sums of first-order calls.
//
// Build: hipcc -O2 -std=c++17 -Iinclude tests/cabi/cabi_roundtrip.cpp -o tests/cabi/cabi_roundtrip \
//        -Lopenequivariance_amd -loeq_amd -Wl,-rpath,'$ORIGIN/../../openequivariance_amd'
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <sstream>
#include <string>
#include <vector>

#include "oeq_amd.h"

#define CHECK_HIP(x)                                                                   \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));               \
            return 2;                                                                  \
        }                                                                              \
    } while (0)
#define CHECK_OEQ(x)                                                                   \
    do {                                                                               \
        if ((x) != 0) {                                                                \
            std::fprintf(stderr, "%s: %s\n", #x, oeq_last_error());                    \
            return 3;                                                                  \
        }                                                                              \
    } while (0)

static std::vector<float> read_floats(const std::string& path) {
    std::ifstream f(path, std::ios::binary | std::ios::ate);
    if (!f) { std::fprintf(stderr, "cannot open %s\n", path.c_str()); std::exit(4); }
    size_t bytes = (size_t)f.tellg();
    std::vector<float> v(bytes / sizeof(float));
    f.seekg(0);
    f.read((char*)v.data(), (std::streamsize)bytes);
    return v;
}

static double normalized_error(const std::vector<float>& got, const std::vector<float>& want) {
    double num = 0.0, den = 0.0;
    for (size_t i = 0; i < want.size(); ++i) {
        num = std::fmax(num, std::fabs((double)got[i] - (double)want[i]));
        den = std::fmax(den, std::fabs((double)want[i]));
    }
    return den > 0.0 ? num / den : num;
}

int main(int argc, char** argv) {
    if (argc < 2) { std::fprintf(stderr, "usage: %s <bundle dir>\n", argv[0]); return 1; }
    const std::string dir = argv[1];

    std::ifstream src_file(dir + "/kernels.hip");
    std::stringstream src;
    src << src_file.rdbuf();

    std::ifstream b(dir + "/bundle.txt");
    oeq_problem_dims dims{};
    long long batch = 0;
    int n_descs = 0;
    b >> dims.L1_dim >> dims.L2_dim >> dims.L3_dim >> dims.weight_numel >> dims.elem_size >> dims.shared_weights >>
        dims.deterministic >> dims.wpartial_per_block >> batch >> n_descs;
    std::vector<std::string> names(n_descs);
    std::vector<oeq_kernel_desc> descs(n_descs);
    for (int i = 0; i < n_descs; ++i) {
        b >> descs[i].role >> names[i] >> descs[i].block_threads >> descs[i].units_per_block >> descs[i].max_blocks >>
            descs[i].grid_multiple;
    }
    for (int i = 0; i < n_descs; ++i) descs[i].kernel_name = names[i].c_str();
    if (!b || dims.elem_size != 4) { std::fprintf(stderr, "bad bundle\n"); return 1; }

    const char* opts[] = {"-O3", "--std=c++17", "-ffp-contract=fast", "-Xclang", "-target-feature", "-Xclang",
                          "-packed-fp32-ops"};
    void* code = nullptr;
    size_t code_size = 0;
    CHECK_OEQ(oeq_jit_compile(src.str().c_str(), "gfx950", opts, 7, &code, &code_size));
    oeq_kernels* k = nullptr;
    CHECK_OEQ(oeq_kernels_create(code, code_size, &dims, descs.data(), n_descs, &k));
    oeq_free(code);

    const auto x = read_floats(dir + "/x.bin"), y = read_floats(dir + "/y.bin"), w = read_floats(dir + "/w.bin"),
               g = read_floats(dir + "/g.bin");
    const auto z_ref = read_floats(dir + "/z.bin"), dx_ref = read_floats(dir + "/dx.bin"),
               dy_ref = read_floats(dir + "/dy.bin"), dw_ref = read_floats(dir + "/dw.bin");
    float *dX, *dY, *dW, *dG, *dZ, *gX, *gY, *gW;
    void* ws = nullptr;
    auto bytes = [](const std::vector<float>& v) { return v.size() * sizeof(float); };
    CHECK_HIP(hipMalloc(&dX, bytes(x)));
    CHECK_HIP(hipMalloc(&dY, bytes(y)));
    CHECK_HIP(hipMalloc(&dW, bytes(w)));
    CHECK_HIP(hipMalloc(&dG, bytes(g)));
    CHECK_HIP(hipMalloc(&dZ, bytes(z_ref)));
    CHECK_HIP(hipMalloc(&gX, bytes(x)));
    CHECK_HIP(hipMalloc(&gY, bytes(y)));
    CHECK_HIP(hipMalloc(&gW, bytes(w)));
    CHECK_HIP(hipMemcpy(dX, x.data(), bytes(x), hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(dY, y.data(), bytes(y), hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(dW, w.data(), bytes(w), hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(dG, g.data(), bytes(g), hipMemcpyHostToDevice));
    size_t ws_bytes = oeq_tp_backward_workspace_bytes(k, batch);
    if (ws_bytes) CHECK_HIP(hipMalloc(&ws, ws_bytes));

    hipStream_t stream;
    CHECK_HIP(hipStreamCreate(&stream));
    CHECK_OEQ(oeq_tp_forward(k, batch, dX, dY, dW, dZ, stream));
    CHECK_OEQ(oeq_tp_backward(k, batch, dX, gX, dY, gY, dW, gW, dG, ws, ws_bytes, stream));
    CHECK_HIP(hipStreamSynchronize(stream));

    std::vector<float> z(z_ref.size()), dx(x.size()), dy(y.size()), dw(w.size());
    CHECK_HIP(hipMemcpy(z.data(), dZ, bytes(z), hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(dx.data(), gX, bytes(dx), hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(dy.data(), gY, bytes(dy), hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(dw.data(), gW, bytes(dw), hipMemcpyDeviceToHost));
    const double e[4] = {normalized_error(z, z_ref), normalized_error(dx, dx_ref), normalized_error(dy, dy_ref),
                         normalized_error(dw, dw_ref)};
    std::printf("errors z=%.3g dx=%.3g dy=%.3g dw=%.3g\n", e[0], e[1], e[2], e[3]);
    double e2[2] = {0, 0};
    if (oeq_has_double_backward(k)) {
        // Second-order kernels against the first-order entry points, with the first-order gradients as
        // cotangents (A, B, C) = (dX, dY, dW): d/d(dZ) = F(A,Y,W) + F(X,B,W) + F(X,Y,C) and
        // d/dX = dX-part of backward(X,B,W;dZ) + dX-part of backward(X,Y,C;dZ).
        float *hX, *hY, *hW, *hG, *tZ, *tX, *tY, *tW;
        CHECK_HIP(hipMalloc(&hX, bytes(x)));
        CHECK_HIP(hipMalloc(&hY, bytes(y)));
        CHECK_HIP(hipMalloc(&hW, bytes(w)));
        CHECK_HIP(hipMalloc(&hG, bytes(g)));
        CHECK_HIP(hipMalloc(&tZ, bytes(g)));
        CHECK_HIP(hipMalloc(&tX, bytes(x)));
        CHECK_HIP(hipMalloc(&tY, bytes(y)));
        CHECK_HIP(hipMalloc(&tW, bytes(w)));
        // shared weights: kernel B leaves partial weight gradients in a workspace for the ordered reduction
        const size_t dd_bytes = oeq_tp_double_backward_workspace_bytes(k, batch);
        void* dd_ws = nullptr;
        if (dd_bytes) CHECK_HIP(hipMalloc(&dd_ws, dd_bytes));
        CHECK_OEQ(oeq_tp_double_backward(k, batch, dX, dY, dW, dG, gX, gY, gW, hX, hY, hW, hG, dd_ws, dd_bytes, stream));
        CHECK_HIP(hipStreamSynchronize(stream));
        std::vector<float> gg(g.size()), ddx(x.size()), gg_ref(g.size(), 0.f), ddx_ref(x.size(), 0.f), t(g.size()),
            tx(x.size());
        CHECK_HIP(hipMemcpy(gg.data(), hG, bytes(gg), hipMemcpyDeviceToHost));
        CHECK_HIP(hipMemcpy(ddx.data(), hX, bytes(ddx), hipMemcpyDeviceToHost));
        const float* fw[3][3] = {{gX, dY, dW}, {dX, gY, dW}, {dX, dY, gW}};
        for (auto& o : fw) {
            CHECK_OEQ(oeq_tp_forward(k, batch, o[0], o[1], o[2], tZ, stream));
            CHECK_HIP(hipStreamSynchronize(stream));
            CHECK_HIP(hipMemcpy(t.data(), tZ, bytes(t), hipMemcpyDeviceToHost));
            for (size_t i = 0; i < t.size(); ++i) gg_ref[i] += t[i];
        }
        const float* bw[2][2] = {{gY, dW}, {dY, gW}};
        for (auto& o : bw) {
            CHECK_OEQ(oeq_tp_backward(k, batch, dX, tX, o[0], tY, o[1], tW, dG, ws, ws_bytes, stream));
            CHECK_HIP(hipStreamSynchronize(stream));
            CHECK_HIP(hipMemcpy(tx.data(), tX, bytes(tx), hipMemcpyDeviceToHost));
            for (size_t i = 0; i < tx.size(); ++i) ddx_ref[i] += tx[i];
        }
        e2[0] = normalized_error(gg, gg_ref);
        e2[1] = normalized_error(ddx, ddx_ref);
        std::printf("second order: d/d(dZ)=%.3g d/dX=%.3g\n", e2[0], e2[1]);
    } else {
        std::printf("second order: no fused kernels in this set\n");
    }
    oeq_kernels_destroy(k);
    for (double v : e2)
        if (!(v <= 1e-5)) { std::printf("FAILED\n"); return 6; }
    for (double v : e)
        if (!(v <= 1e-5)) { std::printf("FAILED\n"); return 5; }
    std::printf("OK\n");
    return 0;
}
