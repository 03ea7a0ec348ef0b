// Stand-alone driver of the layer for profilers: no Python, no PyTorch, only the host mirror's C API and the HIP runtime.
//
//   tf_layer_probe <libtitanic_moe_hip.so> [rows=4] [passes=64] [batches=16] [copies=4] [skew=0] [request=1]
//
// Builds the benchmark geometry (H 4096, E 256, top-6, I 2048, one shared expert) with pseudo-random operands (valid FP4 /
// FP8 / UE8M0 codes: the values do not matter to a profiler, the routing is as spread as with real weights; skew > 0 adds the
// selection bias -skew * ln(1 + expert), which concentrates the routes on the first experts; request > 1: every `request`
// consecutive rows are one request's draft tokens, a shared base row plus noise of 0.3 times its spread, so that their routes
// overlap as the speculative-verify workload's do), runs `passes`
// eager passes of the layer's own schedule cycling through `batches` input batches, prints the mean durations the library's
// marks give, and finally launches `copies` plain copies of 256 MiB (tf_probe_copy) so that a hardware-counter run holds a
// kernel whose traffic is known: 268,435,456 bytes fetched and as many written per launch.
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cmath>
#include <cstring>
#include <vector>
#include "../../../include/titanic_moe.h"

extern "C" {
void* tfh_layer_create(const char*, const ca_geometry*, int, const void* const*, int, int, int, int, int, int, int, char*, size_t);
void tfh_layer_destroy(void*);
int tfh_layer_set_tokens(void*, const int64_t*, int, const int32_t*, char*, size_t);
int tfh_layer_run(void*, uint64_t, char*, size_t);
int tfh_layer_profile_marks(void*, const uint64_t*, int, int, int, float*, char*, size_t);
long long tfh_layer_tap(void*, const char*, void*, size_t, char*, size_t);
void tfh_layer_keep_intermediate(void*, int);
}

typedef uint32_t u4v __attribute__((ext_vector_type(4)));
__global__ void __launch_bounds__(256) tf_probe_copy(const u4v* __restrict__ src, u4v* __restrict__ dst, size_t vectors) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < vectors; i += (size_t)gridDim.x * blockDim.x) dst[i] = src[i];
}

namespace {
struct Rng {
    uint64_t s;
    uint64_t next() { uint64_t z = (s += 0x9E3779B97F4A7C15ull); z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull; z = (z ^ (z >> 27)) * 0x94D049BB133111EBull; return z ^ (z >> 31); }
};
std::vector<uint8_t> random_bytes(size_t n, Rng& r, uint8_t and_mask, uint8_t base, uint8_t range) {
    std::vector<uint8_t> v(n);
    size_t i = 0;
    for (; i + 8 <= n; i += 8) {
        uint64_t w = r.next();
        for (int j = 0; j < 8; ++j, w >>= 8) v[i + j] = range ? (uint8_t)(base + (w & 0xff) % range) : (uint8_t)(w & and_mask);
    }
    for (uint64_t w = r.next(); i < n; ++i, w >>= 8) v[i] = range ? (uint8_t)(base + (w & 0xff) % range) : (uint8_t)(w & and_mask);
    return v;
}
uint16_t to_bf16(float f) { uint32_t b; std::memcpy(&b, &f, 4); return (uint16_t)((b + 0x7fffu + ((b >> 16) & 1u)) >> 16); }
std::vector<uint16_t> random_bf16(size_t n, Rng& r, float amplitude) {
    std::vector<uint16_t> v(n);
    for (size_t i = 0; i < n; ++i) v[i] = to_bf16(((float)(r.next() >> 40) / (float)(1 << 24) * 2.f - 1.f) * amplitude);
    return v;
}
#define HIP_OK(call) do { hipError_t e_ = (call); if (e_ != hipSuccess) { std::fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(e_)); return 1; } } while (0)
}  // namespace

int main(int argc, char** argv) {
    if (argc < 2) { std::fprintf(stderr, "usage: %s <libtitanic_moe_hip.so> [rows] [passes] [batches] [copies] [skew] [request]\n", argv[0]); return 2; }
    const int rows = argc > 2 ? std::atoi(argv[2]) : 4, passes = argc > 3 ? std::atoi(argv[3]) : 64;
    const int batches = argc > 4 ? std::atoi(argv[4]) : 16, copies = argc > 5 ? std::atoi(argv[5]) : 4;
    const float skew = argc > 6 ? (float)std::atof(argv[6]) : 0.f;
    const int request = argc > 7 ? std::atoi(argv[7]) : 1;
    if (rows < 1 || rows > 16384 || passes < 1 || batches < 1 || batches > 64 || copies < 0 || request < 1 || rows % request) { std::fprintf(stderr, "arguments out of range\n"); return 2; }
    const ca_geometry g = {4096, 256, 6, 2048, 2048, 0, 1.0f, 128, 128, 128, -1, 10.f};
    const size_t H = g.hidden, E = g.experts, I = g.intermediate, S = g.shared_intermediate;
    Rng rng{0x7469746eull};
    std::fprintf(stderr, "operands...\n");
    const std::vector<uint16_t> gate_w = random_bf16(E * H, rng, 0.05f);
    std::vector<float> bias(E, 0.f);
    for (size_t e = 0; e < E; ++e) bias[e] = -skew * std::log(1.f + (float)e);
    const std::vector<uint8_t> w13 = random_bytes(E * 2 * I * H / 2, rng, 0xff, 0, 0), s13 = random_bytes(E * 2 * I * H / 32, rng, 0, 117, 4);
    const std::vector<uint8_t> w2 = random_bytes(E * H * I / 2, rng, 0xff, 0, 0), s2 = random_bytes(E * H * I / 32, rng, 0, 117, 4);
    // E4M3 codes with the top exponent bit clear: finite, magnitude below 2
    const std::vector<uint8_t> sh_w13 = random_bytes(2 * S * H, rng, 0xbf, 0, 0), sh_s13 = random_bytes((2 * S / g.shared_bn) * (H / g.shared_bk), rng, 0, 118, 3);
    const std::vector<uint8_t> sh_w2 = random_bytes(H * S, rng, 0xbf, 0, 0), sh_s2 = random_bytes((H / g.shared_bn) * (S / g.shared_bk), rng, 0, 118, 3);
    const void* operands[11] = {gate_w.data(), bias.data(), bias.data(), w13.data(), s13.data(), w2.data(), s2.data(),
                                sh_w13.data(), sh_s13.data(), sh_w2.data(), sh_s2.data()};
    char error[512] = "";
    std::fprintf(stderr, "layer...\n");
    void* layer = tfh_layer_create(argv[1], &g, rows, operands, 0, 1, 1, 1, 0, 1, 1, error, sizeof error);
    if (!layer) { std::fprintf(stderr, "layer: %s\n", error); return 1; }
    tfh_layer_keep_intermediate(layer, 0);      // many rows: no BF16 copy of the routed intermediate (a tap of the tests), as in the benchmark
    std::vector<int64_t> tokens((size_t)rows);
    for (int i = 0; i < rows; ++i) tokens[i] = i;
    if (tfh_layer_set_tokens(layer, tokens.data(), rows, nullptr, error, sizeof error)) { std::fprintf(stderr, "tokens: %s\n", error); return 1; }
    std::vector<uint64_t> inputs;
    for (int b = 0; b < batches; ++b) {
        std::vector<uint16_t> x = random_bf16((size_t)rows * H, rng, 2.f);
        if (request > 1) {
            auto value = [](uint16_t v) { const uint32_t b = (uint32_t)v << 16; float f; std::memcpy(&f, &b, 4); return f; };
            for (int r = 0; r < rows; ++r) {
                if (r % request == 0) continue;                          // a request's first row is its base
                const uint16_t* base = &x[(size_t)(r - r % request) * H];
                for (size_t c = 0; c < H; ++c) x[(size_t)r * H + c] = to_bf16(value(base[c]) + 0.3f * value(x[(size_t)r * H + c]));
            }
        }
        void* d = nullptr;
        HIP_OK(hipMalloc(&d, x.size() * 2));
        HIP_OK(hipMemcpy(d, x.data(), x.size() * 2, hipMemcpyHostToDevice));
        inputs.push_back((uint64_t)d);
    }
    double tiles = 0, active = 0, routes = 0;        // tiles, experts with rows and live routes a pass, averaged over the batches
    std::vector<int32_t> tile_base(E + 1), ids((size_t)rows * g.topk);
    for (int b = 0; b < batches; ++b) {
        if (tfh_layer_run(layer, inputs[b], error, sizeof error)) { std::fprintf(stderr, "run: %s\n", error); return 1; }
        if (tfh_layer_tap(layer, "tile_base", tile_base.data(), tile_base.size() * 4, error, sizeof error) < 0) { std::fprintf(stderr, "tap: %s\n", error); return 1; }
        if (tfh_layer_tap(layer, "ids", ids.data(), ids.size() * 4, error, sizeof error) < 0) { std::fprintf(stderr, "tap: %s\n", error); return 1; }
        tiles += tile_base[E];
        std::vector<char> seen(E, 0);
        for (int32_t e : ids) if (e >= 0 && e < (int32_t)E) { routes += 1; if (!seen[e]) { seen[e] = 1; active += 1; } }
    }
    tiles /= batches; active /= batches; routes /= batches;
    // algorithmic bytes of the two launches of the routed experts.  Few rows (streaming launches; the shared expert streams in
    // them): every 16-row tile's expert weights and scales once, the shared expert's once, the rows' codes, intermediates and
    // outputs.  Many rows (grouped GEMM; the shared expert runs in kernels of its own): every expert with rows streams its
    // weights and scales once, the token codes are read once a route, the intermediate is FP8 codes and block scales.
    const double K = g.topk;
    // owners of at most eight rows: the shared expert's up / gate weights stream in the front-end launch, not in the FC1 launch
    const bool early_shared = rows <= 64 && H <= 5120;
    double fc1_bytes, fc2_bytes;
    if (rows <= 64) {
        fc1_bytes = tiles * (2.0 * I * H / 2 + 2.0 * I * H / 32) + (early_shared ? 0.0 : 2.0 * S * H) + rows * (2.0 * H + K * I * 2 + 2.0 * S);
        fc2_bytes = tiles * (1.0 * H * I / 2 + 1.0 * H * I / 32) + 1.0 * H * S + rows * (K * I * 2 + K * H * 2 + 2.0 * S + 2.0 * H);
    } else {
        fc1_bytes = active * (2.0 * I * H / 2 + 2.0 * I * H / 32) + routes * (H + H / 128.0) + routes * (I + I / 128.0);
        fc2_bytes = active * (1.0 * H * I / 2 + 1.0 * H * I / 32) + routes * (I + I / 128.0) + routes * H * 2.0;
    }
    std::printf("{\"tiles\": %.3f, \"active_experts\": %.3f, \"routes\": %.1f, \"fc1_algorithmic_bytes\": %.0f, \"fc2_algorithmic_bytes\": %.0f}\n",
                tiles, active, routes, fc1_bytes, fc2_bytes);
    float ms[6] = {0, 0, 0, 0, 0, 0};
    if (rows <= 64) {
        if (tfh_layer_profile_marks(layer, inputs.data(), batches, passes, 0, ms, error, sizeof error)) { std::fprintf(stderr, "profile: %s\n", error); return 1; }
    } else {       // many rows: another schedule (no marks); the passes are there for the profiler
        for (int i = 0; i < passes; ++i)
            if (tfh_layer_run(layer, inputs[i % batches], error, sizeof error)) { std::fprintf(stderr, "run: %s\n", error); return 1; }
    }
    std::printf("{\"rows\": %d, \"passes\": %d, \"front_end_ms\": %.6f, \"fc1_ms\": %.6f, \"fc2_ms\": %.6f, \"sum_ms\": %.6f, \"pass_ms\": %.6f}\n",
                rows, passes, ms[0], ms[1], ms[2], ms[3], ms[4]);
    if (copies > 0) {
        const size_t bytes = (size_t)256 << 20;
        void *src = nullptr, *dst = nullptr;
        HIP_OK(hipMalloc(&src, bytes));
        HIP_OK(hipMalloc(&dst, bytes));
        HIP_OK(hipMemset(src, 0x5a, bytes));
        for (int i = 0; i < copies; ++i) tf_probe_copy<<<4096, 256>>>((const u4v*)src, (u4v*)dst, bytes / 16);
        HIP_OK(hipDeviceSynchronize());
        HIP_OK(hipFree(src));
        HIP_OK(hipFree(dst));
    }
    for (uint64_t d : inputs) HIP_OK(hipFree((void*)d));
    tfh_layer_destroy(layer);
    return 0;
}
