// A host program that uses libkiln_marlin_gemm through include/kiln_w4a16.h and the HIP runtime
// alone: the counterpart of the reference's own harness, which links its static library and
// compares the kernel with a baseline (crates/kiln-marlin-gemm/tests/parity.rs:54-158).
//
//   c_abi_harness gemm    DIR M K N G      one call, result against DIR/y_f32.bin
//   c_abi_harness threads DIR M K N G T    T host threads (own stream, workspace and output each)
//                                          enter the library at the same moment, first on a plan
//                                          cache that has never seen the shape; every result must
//                                          equal a serial call bit for bit
// DIR holds a_bf16.bin [M,K], b_packed.bin [K*N/8 int32], s_tiled.bin [(K/G)*N f16], y_f32.bin [M,N]
// (the CPU oracle's f32 result).  Bound, as everywhere: per row max|y - bf16(y_ref)| <= 1e-2 max|y_ref|.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include "kiln_w4a16.h"

#define CHECK_HIP(call)                                                                          \
    do {                                                                                         \
        hipError_t e_ = (call);                                                                  \
        if (e_ != hipSuccess) {                                                                  \
            std::fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_)); \
            std::exit(2);                                                                        \
        }                                                                                        \
    } while (0)

static std::vector<unsigned char> read_file(const std::string &path, size_t want) {
    std::FILE *f = std::fopen(path.c_str(), "rb");
    if (!f) {
        std::fprintf(stderr, "cannot open %s\n", path.c_str());
        std::exit(2);
    }
    std::vector<unsigned char> buf(want);
    const size_t got = std::fread(buf.data(), 1, want, f);
    const bool more = std::fgetc(f) != EOF;
    std::fclose(f);
    if (got != want || more) {
        std::fprintf(stderr, "%s: expected exactly %zu bytes\n", path.c_str(), want);
        std::exit(2);
    }
    return buf;
}

static float bf16_to_f32(uint16_t b) {
    const uint32_t u = (uint32_t)b << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}
static uint16_t f32_to_bf16(float f) {  // round to nearest even, as crates/kiln-model/src/quantized.rs:260-265
    uint32_t u;
    std::memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

struct Problem {
    int m, k, n, g;
    void *a, *b, *s;  // device
};

struct Call {
    hipStream_t stream = nullptr;
    void *ws = nullptr, *c = nullptr;
    std::vector<uint16_t> out;
};

static void make_call(const Problem &p, Call *c) {
    CHECK_HIP(hipStreamCreate(&c->stream));
    const size_t ws_bytes = kiln_w4a16_workspace_bytes(p.m, p.n, p.k), zeroed = kiln_w4a16_workspace_zeroed_bytes();
    CHECK_HIP(hipMalloc(&c->ws, ws_bytes));
    CHECK_HIP(hipMemset(c->ws, 0, zeroed));  // once; every call leaves the prefix zero again
    if (ws_bytes > zeroed) CHECK_HIP(hipMemset((char *)c->ws + zeroed, 0xA5, ws_bytes - zeroed));  // the rest may hold anything
    CHECK_HIP(hipMalloc(&c->c, (size_t)p.m * p.n * 2));
    CHECK_HIP(hipMemset(c->c, 0xFF, (size_t)p.m * p.n * 2));
    c->out.resize((size_t)p.m * p.n);
}

static int run_gemm(const Problem &p, Call *c) {
    return kiln_marlin_w4a16_gemm(p.a, p.b, c->c, p.s, p.m, p.n, p.k, c->ws, p.g, 0, c->stream, -1, -1, -1, 16);
}

static void fetch(const Problem &p, Call *c) {
    CHECK_HIP(hipStreamSynchronize(c->stream));
    CHECK_HIP(hipMemcpy(c->out.data(), c->c, c->out.size() * 2, hipMemcpyDeviceToHost));
}

static double worst_row_error(const Problem &p, const std::vector<uint16_t> &y, const float *y_ref) {
    double worst = 0.0;
    for (int r = 0; r < p.m; ++r) {
        double row_max = 0.0, diff = 0.0;
        for (int j = 0; j < p.n; ++j) {
            const double want = bf16_to_f32(f32_to_bf16(y_ref[(size_t)r * p.n + j]));
            const double got = bf16_to_f32(y[(size_t)r * p.n + j]);
            if (!std::isfinite(got)) return INFINITY;
            row_max = std::fmax(row_max, std::fabs(want));
            diff = std::fmax(diff, std::fabs(got - want));
        }
        worst = std::fmax(worst, diff / std::fmax(row_max, 1e-30));
    }
    return worst;
}

int main(int argc, char **argv) {
    if (argc < 7) {
        std::fprintf(stderr, "usage: %s gemm|threads DIR M K N G [T]\n", argv[0]);
        return 2;
    }
    const std::string mode = argv[1], dir = argv[2];
    Problem p{std::atoi(argv[3]), std::atoi(argv[4]), std::atoi(argv[5]), std::atoi(argv[6]), nullptr, nullptr, nullptr};
    const int threads = argc > 7 ? std::atoi(argv[7]) : 4;
    const size_t groups = p.g == -1 ? 1 : (size_t)p.k / p.g;
    const size_t a_bytes = (size_t)p.m * p.k * 2, b_bytes = (size_t)p.k * p.n / 2, s_bytes = groups * p.n * 2;
    const auto a = read_file(dir + "/a_bf16.bin", a_bytes);
    const auto b = read_file(dir + "/b_packed.bin", b_bytes);
    const auto s = read_file(dir + "/s_tiled.bin", s_bytes);
    const auto y_ref = read_file(dir + "/y_f32.bin", (size_t)p.m * p.n * 4);
    CHECK_HIP(hipSetDevice(0));
    CHECK_HIP(hipMalloc(&p.a, a_bytes));
    CHECK_HIP(hipMalloc(&p.b, b_bytes));
    CHECK_HIP(hipMalloc(&p.s, s_bytes));
    CHECK_HIP(hipMemcpy(p.a, a.data(), a_bytes, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(p.b, b.data(), b_bytes, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(p.s, s.data(), s_bytes, hipMemcpyHostToDevice));
    std::printf("%s m=%d k=%d n=%d g=%d\n", mode.c_str(), p.m, p.k, p.n, p.g);
    std::fflush(stdout);

    std::vector<Call> calls(mode == "threads" ? threads : 0);
    if (mode == "threads") {
        for (Call &c : calls) make_call(p, &c);
        std::atomic<int> ready{0}, failed{0};
        std::vector<std::thread> pool;
        for (int t = 0; t < threads; ++t)
            pool.emplace_back([&, t] {
                CHECK_HIP(hipSetDevice(0));
                ready.fetch_add(1);
                while (ready.load() < threads) {}  // all enter the library together, on a cold plan cache
                for (int i = 0; i < 64; ++i)
                    if (run_gemm(p, &calls[t]) != KILN_W4A16_OK) failed.fetch_add(1);
            });
        for (std::thread &t : pool) t.join();
        for (Call &c : calls) fetch(p, &c);
        if (failed.load()) {
            std::printf("FAIL: %d calls returned an error\n", failed.load());
            return 1;
        }
    }

    Call serial;
    make_call(p, &serial);
    const int status = run_gemm(p, &serial);
    if (status != KILN_W4A16_OK) {
        std::printf("FAIL: status %d (%s)\n", status, kiln_w4a16_status_string(status));
        return 1;
    }
    fetch(p, &serial);
    const double err = worst_row_error(p, serial.out, reinterpret_cast<const float *>(y_ref.data()));
    std::printf("worst row error %.3e\n", err);
    if (!(err <= 1e-2)) {
        std::printf("FAIL: above 1e-2\n");
        return 1;
    }
    for (size_t t = 0; t < calls.size(); ++t)
        if (std::memcmp(calls[t].out.data(), serial.out.data(), serial.out.size() * 2) != 0) {
            std::printf("FAIL: thread %zu's result differs from the serial call\n", t);
            return 1;
        }
    std::printf("OK\n");
    return 0;
}
