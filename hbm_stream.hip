// Stream ceilings of the GPU's memory system, measured with plain kernels: what a read-only, a write-only
// and a copy kernel reach, as sequential sweeps and as one 384 KB chunk per block (the shape of the
// convolution's per-node edge data). bench.py runs this program (built by __graft_entry__.build()) and
// puts its JSON line into the bench record; profiles/hbm_ceiling.md summarises it.
//
// The same program also reports `read_with_writes_*`: the chunk read again while the blocks write an eighth, half or all
// of what they read (the convolution forward writes 12 % of its traffic, its backward 57 %): on this part any
// share of writes brings a read stream down to about the copy rate, so a kernel's mix of reads and writes,
// not only its byte count, decides which ceiling applies. And `valu_fixed_work_ms`: a fixed amount of
// independent fp32 multiply-adds (plain v_fma_f32, two waves per SIMD) on every SIMD: the rate at which the vector
// units issue them under sustained load, which also tells boxes with different sustained clocks apart.
//
// `./hbm_stream accumulate` instead runs three kernels that add 8.6 GB worth of values into a buffer small
// enough to stay in the L2 caches: float atomics from all blocks on one 512 KB buffer, float atomics with each
// XCD's blocks on their own 512 KB slice, and plain read-modify-write of 1024 private 16 KB slices. Under
// rocprofv3 --pmc WRITE_SIZE / FETCH_SIZE they show where such updates are carried out: in the L2 (traffic =
// the buffer, once) or on the memory side (traffic = every update).
//
// `./hbm_stream pipes` asks whether FP32 matrix instructions (v_mfma_f32_16x16x4_f32) and FP32 vector instructions
// overlap on a SIMD: the same counts of each alone, interleaved one to eight inside a wave, and in phases of 64 and
// 512, with one and with two waves per SIMD on every SIMD. (They do not on MI355X: every arrangement takes the sum.)
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <numeric>
#include <random>
#include <string>
#include <vector>

typedef float __attribute__((ext_vector_type(4))) f4;

#define CHECK(x)                                                                        \
    do {                                                                                \
        hipError_t e_ = (x);                                                            \
        if (e_ != hipSuccess) {                                                         \
            std::fprintf(stderr, "%s failed: %s\n", #x, hipGetErrorString(e_));         \
            return 1;                                                                   \
        }                                                                               \
    } while (0)

__global__ __launch_bounds__(256) void read_sweep(const f4* __restrict__ p, size_t n, float* out) {
    f4 acc = {0, 0, 0, 0};
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) acc += __builtin_nontemporal_load(p + i);
    if (acc.x + acc.y + acc.z + acc.w == 123.456f) *out = 1.f;
}

__global__ __launch_bounds__(256) void write_sweep(f4* __restrict__ p, size_t n) {
    const f4 v = {1, 2, 3, 4};
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) __builtin_nontemporal_store(v, p + i);
}

__global__ __launch_bounds__(256) void copy_sweep(const f4* __restrict__ a, f4* __restrict__ b, size_t n) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
        __builtin_nontemporal_store(__builtin_nontemporal_load(a + i), b + i);
}

// one chunk per block, chunks taken in the order `perm` gives
template <int WRITE>
__global__ __launch_bounds__(128) void chunks(const f4* __restrict__ a, f4* __restrict__ b, const int* __restrict__ perm,
                                              int chunk_f4, float* out) {
    const long c = perm[blockIdx.x];
    const f4* src = a + c * chunk_f4;
    f4* dst = b + c * chunk_f4;
    f4 acc = {0, 0, 0, 0};
    for (int i = threadIdx.x; i < chunk_f4; i += 128) {
        const f4 v = __builtin_nontemporal_load(src + i);
        if (WRITE) __builtin_nontemporal_store(v, dst + i);
        else acc += v;
    }
    if (!WRITE && acc.x + acc.y + acc.z + acc.w == 123.456f) *out = 1.f;
}

// one chunk per block, read; of every WRITE_EVERY 16-byte pieces read, one is written (0: none)
template <int WRITE_EVERY>
__global__ __launch_bounds__(128) void chunks_mixed(const f4* __restrict__ a, f4* __restrict__ b, const int* __restrict__ perm,
                                                    int chunk_f4, float* out) {
    const long c = perm[blockIdx.x];
    const f4* src = a + c * chunk_f4;
    f4* dst = b + c * chunk_f4;
    f4 acc = {0, 0, 0, 0};
    for (int i = threadIdx.x; i < chunk_f4; i += 128) {
        const f4 v = __builtin_nontemporal_load(src + i);
        acc += v;
        // whole 2 KB rows of the block are written or skipped, so that written lines are written in full
        if (WRITE_EVERY && (i / 128) % WRITE_EVERY == 0) __builtin_nontemporal_store(v, dst + i);
    }
    if (acc.x + acc.y + acc.z + acc.w == 123.456f) *out = 1.f;
}

// 8 independent chains of 65 536 multiply-adds per lane: 524 288 wave instructions per wave
__global__ __launch_bounds__(256) void valu_fixed_work(float* out, float seed) {
    float x[8];
    for (int q = 0; q < 8; ++q) x[q] = seed + threadIdx.x * 1e-3f + q;
    for (int it = 0; it < 65536; ++it) {
        #pragma unroll
        for (int q = 0; q < 8; ++q) x[q] = __builtin_fmaf(x[q], 0.999f, 0.001f);
    }
    float t = 0.f;
    for (int q = 0; q < 8; ++q) t += x[q];
    if (t == 123.456f) *out = t;
}

__global__ __launch_bounds__(256) void atomics_shared(float* p, int n_floats, int rounds) {
    for (int r = 0; r < rounds; ++r)
        for (int i = threadIdx.x; i < n_floats; i += 256) unsafeAtomicAdd(p + i, 1.0f);
}

__global__ __launch_bounds__(256) void atomics_per_xcd(float* p, int n_floats, int rounds) {
    float* q = p + (size_t)(blockIdx.x % 8) * n_floats;  // workgroups go to the XCDs round-robin
    for (int r = 0; r < rounds; ++r)
        for (int i = threadIdx.x; i < n_floats; i += 256) unsafeAtomicAdd(q + i, 1.0f);
}

__global__ __launch_bounds__(256) void rmw_private(float* p, int n_floats, int rounds) {
    float* q = p + (size_t)blockIdx.x * n_floats;
    for (int r = 0; r < rounds; ++r)
        for (int i = threadIdx.x; i < n_floats; i += 256) q[i] += 1.0f;
}

static int accumulate_modes() {
    const int n = 128 * 1024;         // 512 KB of floats: the shared buffer, and each of the 8 per-XCD slices
    const int n_private = 4096;       // 16 KB of floats per block in the third kernel
    const int blocks = 1024;
    // the largest footprint of the three kernels: 8 slices of n floats, or one private slice per block
    const size_t bytes = sizeof(float) * std::max((size_t)8 * n, (size_t)blocks * n_private);
    float* p = nullptr;
    CHECK(hipMalloc(&p, bytes));
    CHECK(hipMemset(p, 0, bytes));
    hipEvent_t a, b;
    (void)hipEventCreate(&a);
    (void)hipEventCreate(&b);
    const char* names[3] = {"atomics_shared", "atomics_per_xcd", "rmw_private"};
    for (int mode = 0; mode < 3; ++mode) {
        (void)hipEventRecord(a);
        if (mode == 0) atomics_shared<<<blocks, 256>>>(p, n, 16);
        if (mode == 1) atomics_per_xcd<<<blocks, 256>>>(p, n, 16);
        if (mode == 2) rmw_private<<<blocks, 256>>>(p, n_private, 512);
        (void)hipEventRecord(b);
        (void)hipEventSynchronize(b);
        float ms = 0.f;
        (void)hipEventElapsedTime(&ms, a, b);
        std::printf("%s: %.3f ms for 8.59 GB of updates (%.0f GB/s)\n", names[mode], ms, 8589.9 / ms);
    }
    return 0;
}

typedef float v4f __attribute__((ext_vector_type(4)));
// MODE 0: matrix instructions only; 1: vector only; 2: one matrix instruction then eight vector ones, repeated;
// 3: 64 matrix instructions, then 512 vector ones. Per iteration every mode that has them issues 64 and 512.
template <int MODE>
__global__ __launch_bounds__(256) void pipes_kernel(float* out, float seed, int iters) {
    v4f g[4];
    for (int i = 0; i < 4; ++i) g[i] = v4f{0, 0, 0, 0};
    float x[8];
    for (int q = 0; q < 8; ++q) x[q] = seed + threadIdx.x * 1e-3f + q;
    const float a = seed, b = seed * 0.5f;
    for (int it = 0; it < iters; ++it) {
        if (MODE == 0 || MODE == 3) {
#pragma unroll
            for (int m = 0; m < 64; ++m) g[m & 3] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, g[m & 3], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (MODE == 1 || MODE == 3) {
#pragma unroll
            for (int v = 0; v < 64; ++v)
#pragma unroll
                for (int q = 0; q < 8; ++q) x[q] = __builtin_fmaf(x[q], 0.999f, 0.001f);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (MODE == 2) {
#pragma unroll
            for (int m = 0; m < 64; ++m) {
                g[m & 3] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, g[m & 3], 0, 0, 0);
#pragma unroll
                for (int q = 0; q < 8; ++q) x[q] = __builtin_fmaf(x[q], 0.999f, 0.001f);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    float t = 0;
    for (int q = 0; q < 8; ++q) t += x[q];
    for (int i = 0; i < 4; ++i) t += g[i][0] + g[i][1] + g[i][2] + g[i][3];
    if (t == 123.456f) out[0] = t;
}

template <int MODE>
static float pipes_ms(int blocks, float* d) {
    hipEvent_t a, b;
    (void)hipEventCreate(&a);
    (void)hipEventCreate(&b);
    pipes_kernel<MODE><<<blocks, 256>>>(d, 1.0f, 16);
    (void)hipDeviceSynchronize();
    (void)hipEventRecord(a);
    pipes_kernel<MODE><<<blocks, 256>>>(d, 1.0f, 2000);
    (void)hipEventRecord(b);
    (void)hipEventSynchronize(b);
    float ms = 0.f;
    (void)hipEventElapsedTime(&ms, a, b);
    return ms;
}

static int pipes_modes() {
    float* d = nullptr;
    CHECK(hipMalloc(&d, 1024));
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    for (int waves = 1; waves <= 2; ++waves) {
        const int blocks = prop.multiProcessorCount * waves;  // 4 waves per block: one per SIMD
        std::printf("waves per SIMD %d, 128 000 matrix and 1 024 000 vector instructions per wave: matrix only %.3f ms, "
                    "vector only %.3f ms, interleaved in one wave %.3f ms, in phases %.3f ms\n",
                    waves, pipes_ms<0>(blocks, d), pipes_ms<1>(blocks, d), pipes_ms<2>(blocks, d), pipes_ms<3>(blocks, d));
    }
    return 0;
}

template <typename F>
static float median_ms(F launch, int iters = 7) {
    hipEvent_t a, b;
    (void)hipEventCreate(&a);
    (void)hipEventCreate(&b);
    launch();
    launch();
    (void)hipDeviceSynchronize();
    std::vector<float> ts;
    for (int i = 0; i < iters; ++i) {
        (void)hipEventRecord(a);
        launch();
        (void)hipEventRecord(b);
        (void)hipEventSynchronize(b);
        float ms = 0.f;
        (void)hipEventElapsedTime(&ms, a, b);
        ts.push_back(ms);
    }
    std::sort(ts.begin(), ts.end());
    return ts[ts.size() / 2];
}

int main(int argc, char** argv) {
    if (argc > 1 && std::string(argv[1]) == "accumulate") return accumulate_modes();
    if (argc > 1 && std::string(argv[1]) == "pipes") return pipes_modes();
    const int n_chunks = 21000, chunk_bytes = 384 * 1024;  // 8.26 GB per buffer
    const int chunk_f4 = chunk_bytes / 16;
    const size_t bytes = (size_t)n_chunks * chunk_bytes, n = bytes / 16;
    f4 *a = nullptr, *b = nullptr;
    float* out = nullptr;
    int* dperm = nullptr;
    CHECK(hipMalloc(&a, bytes));
    CHECK(hipMalloc(&b, bytes));
    CHECK(hipMalloc(&out, 4));
    CHECK(hipMalloc(&dperm, n_chunks * sizeof(int)));
    CHECK(hipMemset(a, 1, bytes));
    CHECK(hipMemset(b, 0, bytes));
    const double gb = bytes / 1e9;
    double best_r = 0, best_w = 0, best_c = 0;
    for (int grid : {1024, 2048, 4096, 8192, 32768}) {
        best_r = std::max(best_r, gb / median_ms([&] { read_sweep<<<grid, 256>>>(a, n, out); }) * 1e3);
        best_w = std::max(best_w, gb / median_ms([&] { write_sweep<<<grid, 256>>>(b, n); }) * 1e3);
        best_c = std::max(best_c, 2 * gb / median_ms([&] { copy_sweep<<<grid, 256>>>(a, b, n); }) * 1e3);
    }
    std::vector<int> perm(n_chunks);
    std::iota(perm.begin(), perm.end(), 0);
    CHECK(hipMemcpy(dperm, perm.data(), n_chunks * sizeof(int), hipMemcpyHostToDevice));
    const double seq_r = gb / median_ms([&] { chunks<0><<<n_chunks, 128>>>(a, b, dperm, chunk_f4, out); }) * 1e3;
    const double seq_c = 2 * gb / median_ms([&] { chunks<1><<<n_chunks, 128>>>(a, b, dperm, chunk_f4, out); }) * 1e3;
    std::mt19937 gen(1);
    std::shuffle(perm.begin(), perm.end(), gen);
    CHECK(hipMemcpy(dperm, perm.data(), n_chunks * sizeof(int), hipMemcpyHostToDevice));
    const double sc_r = gb / median_ms([&] { chunks<0><<<n_chunks, 128>>>(a, b, dperm, chunk_f4, out); }) * 1e3;
    const double sc_c = 2 * gb / median_ms([&] { chunks<1><<<n_chunks, 128>>>(a, b, dperm, chunk_f4, out); }) * 1e3;
    const double memcpy_c = 2 * gb / median_ms([&] { (void)hipMemcpyAsync(b, a, bytes, hipMemcpyDeviceToDevice, 0); }) * 1e3;
    // bytes read plus bytes written, per second, with writes for 1/8, 1/2 and all of the data read
    const double mix8 = (1 + 1.0 / 8) * gb / median_ms([&] { chunks_mixed<8><<<n_chunks, 128>>>(a, b, dperm, chunk_f4, out); }) * 1e3;
    const double mix2 = (1 + 1.0 / 2) * gb / median_ms([&] { chunks_mixed<2><<<n_chunks, 128>>>(a, b, dperm, chunk_f4, out); }) * 1e3;
    const double mix1 = 2 * gb / median_ms([&] { chunks_mixed<1><<<n_chunks, 128>>>(a, b, dperm, chunk_f4, out); }) * 1e3;
    const double mix0 = gb / median_ms([&] { chunks_mixed<0><<<n_chunks, 128>>>(a, b, dperm, chunk_f4, out); }) * 1e3;
    // two waves on every SIMD: 2 x 524 288 instructions of 4 issue cycles each per SIMD
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;
    const float valu_ms = median_ms([&] { valu_fixed_work<<<cus * 2, 256>>>(out, 1.0f); });
    // wave64 multiply-adds that one SIMD issues per microsecond, and the same as a chip-wide fp32 rate
    const double valu_per_simd_us = 2.0 * 524288.0 / (valu_ms * 1e3);
    const double valu_tflops = (double)cus * 8 * 524288.0 * 64 * 2 / (valu_ms * 1e-3) / 1e12;
    std::printf("{\"unit\": \"GB/s\", \"buffer_gb\": %.2f, \"read_sweep\": %.0f, \"write_sweep\": %.0f, \"copy_sweep\": %.0f, "
                "\"read_chunks_sequential\": %.0f, \"copy_chunks_sequential\": %.0f, \"read_chunks_scattered\": %.0f, "
                "\"copy_chunks_scattered\": %.0f, \"hipMemcpy_d2d\": %.0f, \"read_with_writes_0\": %.0f, "
                "\"read_with_writes_1_8\": %.0f, \"read_with_writes_1_2\": %.0f, \"read_with_writes_1_1\": %.0f, "
                "\"valu_fixed_work_ms\": %.4f, \"valu_wave64_fma_per_simd_per_us\": %.1f, \"valu_fp32_tflops_unpacked\": %.1f, "
                "\"compute_units\": %d, \"clock_khz_nominal\": %d}\n",
                gb, best_r, best_w, best_c, seq_r, seq_c, sc_r, sc_c, memcpy_c, mix0, mix8, mix2, mix1, valu_ms, valu_per_simd_us, valu_tflops, cus,
                prop.clockRate);
    return 0;
}
