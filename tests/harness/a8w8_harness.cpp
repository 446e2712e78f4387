// Host harness for libmi355a8w8, in the shape of the reference's demo executables:
// same flags, same launch / validation / benchmark printouts
// (opus_gemm/block_scale_gemm/gemm_a8w8_blockscale_host.cc:128-294), so that a user of
//   gemm_a8w8_blockscale.exe -b 1 -m 4096 -n 4096 -k 4096 -v 1
// finds the same command line and the same lines of output.  One source builds three programs:
//   gemm_a8w8_blockscale.exe   1x128 / 128x128 block scales, fp32 C (the reference program)
//   gemm_a8w8_8wave.exe        dense GEMM, --scale-mode tensor|rowcol|mx|mxt, bf16 C
//                              (mxt: the row-major MX scales are re-ordered into the tiled layout
//                              inside the timed loop, then the GEMM runs on the tiled scales)
//   flatmm_a8w8.exe            skinny-M GEMM over pre-shuffled weights, bf16 C
// This is test infrastructure: validation (-v 1) calls the CPU oracle, exactly as the
// reference program calls its own gemm_ref (host.cc:260-281).
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

#include "../../include/mi355_a8w8.h"

// CPU oracle (oracle/a8w8_oracle.c)
extern "C" {
void orc_encode_vec(const float*, uint8_t*, size_t, int, int);
void orc_gemm_ref(const uint8_t*, const uint8_t*, const float*, const float*, float*, int, int, int, int, int, int, int,
                  int, int, int, int, int, int, int);
void orc_gemm_ref_mx(const uint8_t*, const uint8_t*, const uint8_t*, const uint8_t*, float*, int, int, int, int, int,
                     int, int, int, int, int, int);
float orc_bf16_to_f32(uint16_t);
int orc_num_threads(void);
}

#ifndef HARNESS_KIND
#define HARNESS_KIND 0   // 0 block scale, 1 dense 8-wave, 2 flatmm
#endif

// Every runtime and library call is checked; a failure names the call site and ends the program with status 1,
// which is what the reference program does on a HIP error (host.cc:17-26).
static void require_hip(hipError_t err, const char* what, int line)
{
    if (err == hipSuccess) return;
    fprintf(stderr, "%s failed at line %d: %s\n", what, line, hipGetErrorString(err));
    exit(1);
}
static void require_a8w8(int status, const char* what, int line)
{
    if (status == A8W8_OK) return;
    fprintf(stderr, "%s failed at line %d: %s\n", what, line, a8w8_status_string(status));
    exit(1);
}
#define CHECK_HIP(call) require_hip((call), #call, __LINE__)
#define CHECK_A8W8(call) require_a8w8((call), #call, __LINE__)

// Seeded replacement for the reference's rand_vector (host.cc:32-44, unseeded there): splitmix64
// stream -> uniform [lo, hi); Box-Muller for normals.
struct Rng {
    uint64_t s;
    explicit Rng(uint64_t seed) : s(seed) {}
    uint64_t next()
    {
        uint64_t z = (s += 0x9E3779B97F4A7C15ull);
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    float uniform(float lo, float hi) { return lo + (hi - lo) * (float)((next() >> 40) * (1.0 / 16777216.0)); }
    float normal()
    {
        float u1 = uniform(1e-7f, 1.0f), u2 = uniform(0.f, 1.f);
        return sqrtf(-2.0f * logf(u1)) * cosf(6.28318530718f * u2);
    }
};

static void fill_uniform_fp8(std::vector<uint8_t>& q, Rng& r, float lo, float hi)
{
    std::vector<float> x(q.size());
    for (auto& v : x) v = r.uniform(lo, hi);
    orc_encode_vec(x.data(), q.data(), x.size(), 0, 0);
}

// per-row amax/448 quantisation of N(0,1) values (configs 2 and 5)
static void quant_rows(std::vector<uint8_t>& q, std::vector<float>& scale, int rows, int k, Rng& r)
{
    std::vector<float> x((size_t)rows * k);
    for (auto& v : x) v = r.normal();
    for (int i = 0; i < rows; ++i) {
        float amax = 0.f;
        for (int p = 0; p < k; ++p) amax = fmaxf(amax, fabsf(x[(size_t)i * k + p]));
        scale[i] = amax / 448.0f;
        for (int p = 0; p < k; ++p) x[(size_t)i * k + p] /= scale[i];
    }
    orc_encode_vec(x.data(), q.data(), x.size(), 0, 0);
}

// MX: values N(0,1) * 2^U(-4,4) per 32-block, exponent e = ceil(log2(amax/448)) (config 4)
static void quant_mx(std::vector<uint8_t>& q, std::vector<uint8_t>& e8, int rows, int k, Rng& r)
{
    std::vector<float> x((size_t)rows * k);
    for (int i = 0; i < rows; ++i)
        for (int g = 0; g < k / 32; ++g) {
            const float s = exp2f(r.uniform(-4.f, 4.f));
            float amax = 0.f;
            float* blk = &x[(size_t)i * k + g * 32];
            for (int p = 0; p < 32; ++p) { blk[p] = r.normal() * s; amax = fmaxf(amax, fabsf(blk[p])); }
            int e = -127;
            if (amax > 0.f) {
                int ex; const float f = frexpf(amax / 448.0f, &ex);
                e = f == 0.5f ? ex - 1 : ex;
                e = e < -127 ? -127 : (e > 127 ? 127 : e);
            }
            e8[(size_t)i * (k / 32) + g] = (uint8_t)(e + 127);
            for (int p = 0; p < 32; ++p) blk[p] = ldexpf(blk[p], -e);
        }
    orc_encode_vec(x.data(), q.data(), x.size(), 0, 0);
}

// valid_vector (host.cc:46-63) with the tolerance as a parameter pair: |ref - out| <= rel*|ref| + abs.
// `allowed` is the number of elements that may miss it: 0 everywhere except for MX inputs, where
// the matrix cores' own accumulation error (about 5e-5 of sum|a||b|s) pushes a few outputs that
// cancel to almost zero past the absolute term; those may be at most 0.1% of the tile.
static bool valid_vector(const float* ref, const float* out, size_t n, float rel, float abs_, size_t allowed = 0)
{
    size_t errors = 0;
    for (size_t i = 0; i < n; ++i) {
        const float diff = fabsf(ref[i] - out[i]);
        if (!(diff <= rel * fabsf(ref[i]) + abs_)) {
            if (errors < 10 && allowed == 0)
                printf("Error at %zu: ref=%.6f, result=%.6f, diff=%.6f\n", i, ref[i], out[i], diff);
            ++errors;
            if (allowed == 0 && errors >= 10) break;
        }
    }
    if (allowed && errors) printf("%zu of %zu elements beyond tolerance (allowed %zu)\n", errors, n, allowed);
    return errors <= allowed;
}

// A pair of HIP events on the default stream (the stream every launch of this program uses).
struct StreamTimer {
    hipEvent_t first{}, last{};
    StreamTimer()
    {
        CHECK_HIP(hipEventCreate(&first));
        CHECK_HIP(hipEventCreate(&last));
    }
    ~StreamTimer()
    {
        (void)hipEventDestroy(first);
        (void)hipEventDestroy(last);
    }
    void begin() { CHECK_HIP(hipEventRecord(first)); }
    float end_ms()
    {
        float ms = 0.f;
        CHECK_HIP(hipEventRecord(last));
        CHECK_HIP(hipEventSynchronize(last));
        CHECK_HIP(hipEventElapsedTime(&ms, first, last));
        return ms;
    }
};

// The reference's timing protocol (benchmark_kernel, host.cc:92-126): untimed warm-up launches (200 there), then
// `iterations` launches (100 there) between two events; returns the mean time of one launch in ms.
template <class F>
static float benchmark(F launch, int warmup, int iterations)
{
    for (int i = 0; i < warmup; ++i) launch(i);
    CHECK_HIP(hipDeviceSynchronize());
    StreamTimer timer;
    timer.begin();
    for (int i = 0; i < iterations; ++i) launch(i);
    return timer.end_ms() / (float)iterations;
}

template <class T>
static T* to_device(const std::vector<T>& h)
{
    T* d = nullptr;
    CHECK_HIP(hipMalloc(&d, h.size() * sizeof(T) + 16));
    CHECK_HIP(hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice));
    return d;
}

int main(int argc, char** argv)
{
    // defaults of the reference program (host.cc:134-138) for the block-scale build
    int M = HARNESS_KIND == 2 ? 16 : 256, N = HARNESS_KIND == 2 ? 16384 : 512, K = HARNESS_KIND == 2 ? 7168 : 256;
    int batch = HARNESS_KIND == 0 ? 8 : 1, verify = 0, seed = 0xA8A8, rotate = 4;
    int iters = 100, warmup = 200;      // the reference's protocol (host.cc:92-94); --iters / --warmup change it
    std::string scale_mode = HARNESS_KIND == 0 ? "block" : "rowcol";

    // Flags take their value as the next argument ("-m 4096") or after an equals sign ("-m=4096"), as in the
    // reference program (host.cc:140-173); unknown arguments are ignored there and here.
    struct Option {
        const char* short_name;
        const char* long_name;
        int* number;
        std::string* text;
    };
    const Option options[] = {
        {"-m", "--m", &M, nullptr},          {"-n", "--n", &N, nullptr},
        {"-k", "--k", &K, nullptr},          {"-b", "--b", &batch, nullptr},
        {"-v", "--verify", &verify, nullptr}, {nullptr, "--scale-mode", nullptr, &scale_mode},
        {nullptr, "--seed", &seed, nullptr}, {nullptr, "--rotate-buffers", &rotate, nullptr},
        {nullptr, "--iters", &iters, nullptr}, {nullptr, "--warmup", &warmup, nullptr},
    };
    for (int i = 1; i < argc; ++i) {
        const std::string arg = argv[i];
        const size_t eq = arg.find('=');
        const std::string name = arg.substr(0, eq);
        for (const Option& o : options) {
            if (!((o.short_name && name == o.short_name) || (o.long_name && name == o.long_name))) continue;
            std::string value;
            if (eq != std::string::npos) value = arg.substr(eq + 1);
            else if (i + 1 < argc) value = argv[++i];
            if (o.number) *o.number = atoi(value.c_str());
            else *o.text = value;
            break;
        }
    }
    if (M <= 0 || N <= 0 || K <= 0 || batch <= 0) {
        fprintf(stderr, "Invalid problem size: M, N, K and batch must be positive.\n");
        return 1;
    }
    if (iters <= 0 || warmup < 0) {
        fprintf(stderr, "--iters must be positive and --warmup non-negative.\n");
        return 1;
    }
    int mode = A8W8_SCALE_ROWCOL;
    if (HARNESS_KIND == 0 || scale_mode == "block") mode = A8W8_SCALE_BLOCK_1x128_128x128;
    else if (scale_mode == "tensor") mode = A8W8_SCALE_TENSOR;
    else if (scale_mode == "mx" || scale_mode == "mxt") mode = A8W8_SCALE_MX_E8M0_1x32;
    else if (scale_mode != "rowcol") { fprintf(stderr, "unknown --scale-mode %s\n", scale_mode.c_str()); return 1; }
    if (mode == A8W8_SCALE_BLOCK_1x128_128x128 && (N % 128 != 0 || K % 128 != 0)) {
        fprintf(stderr, "M/N/K must be multiples of GROUP_M/GROUP_N/GROUP_K (1,128,128) for scale factors.\n");
        return 1;
    }
    if (HARNESS_KIND == 2 && batch != 1) { fprintf(stderr, "flatmm harness runs batch 1\n"); return 1; }

    CHECK_A8W8(a8w8_init(-1));      // device set-up outside the timed loop
    Rng rng((uint64_t)seed);
    const size_t a_elems = (size_t)batch * M * K, b_elems = (size_t)batch * N * K, c_elems = (size_t)batch * M * N;
    std::vector<uint8_t> host_a(a_elems), host_b(b_elems);
    std::vector<float> sfa_f, sfb_f;
    std::vector<uint8_t> sfa_e, sfb_e;
    a8w8_gemm_args args{};
    args.m = M; args.n = N; args.k = K; args.batch = batch;
    args.stride_a = K; args.stride_b = K; args.stride_c = N;
    args.stride_a_batch = M * K; args.stride_b_batch = N * K; args.stride_c_batch = M * N;
    args.scale_mode = mode;
    args.c_dtype = HARNESS_KIND == 0 ? A8W8_C_FP32 : A8W8_C_BF16;

    if (mode == A8W8_SCALE_BLOCK_1x128_128x128) {
        // the reference's inputs: A~U[0,1), B~U[-.5,.5), scales~U[.8,1.2) (host.cc:207-210)
        fill_uniform_fp8(host_a, rng, 0.f, 1.f);
        fill_uniform_fp8(host_b, rng, -0.5f, 0.5f);
        sfa_f.resize((size_t)batch * (K / 128) * M);
        sfb_f.resize((size_t)batch * (N / 128) * (K / 128));
        for (auto& v : sfa_f) v = rng.uniform(0.8f, 1.2f);
        for (auto& v : sfb_f) v = rng.uniform(0.8f, 1.2f);
        args.stride_sfa = M; args.stride_sfb = K / 128;
        args.stride_sfa_batch = M * (K / 128); args.stride_sfb_batch = (N / 128) * (K / 128);
    } else if (mode == A8W8_SCALE_MX_E8M0_1x32) {
        if (K % 32 != 0) { fprintf(stderr, "K must be a multiple of 32 for MX scales.\n"); return 1; }
        sfa_e.resize((size_t)batch * M * (K / 32));
        sfb_e.resize((size_t)batch * N * (K / 32));
        quant_mx(host_a, sfa_e, batch * M, K, rng);
        quant_mx(host_b, sfb_e, batch * N, K, rng);
        args.stride_sfa = K / 32; args.stride_sfb = K / 32;
        args.stride_sfa_batch = M * (K / 32); args.stride_sfb_batch = N * (K / 32);
    } else {
        sfa_f.resize((size_t)batch * M);
        sfb_f.resize((size_t)batch * N);
        quant_rows(host_a, sfa_f, batch * M, K, rng);
        quant_rows(host_b, sfb_f, batch * N, K, rng);
        args.stride_sfa = 0; args.stride_sfb = 1;
        args.stride_sfa_batch = M; args.stride_sfb_batch = N;
        if (mode == A8W8_SCALE_TENSOR) {   // one scale per tensor: keep the bytes, use the first row's scale
            sfa_f.assign((size_t)batch, sfa_f[0]);
            sfb_f.assign((size_t)batch, sfb_f[0]);
            args.stride_sfb = 0; args.stride_sfa_batch = 1; args.stride_sfb_batch = 1;
        }
    }

    uint8_t* dev_a = to_device(host_a);
    std::vector<uint8_t*> dev_b_copies;
    if (HARNESS_KIND == 2) {
        std::vector<uint8_t> shuf(host_b.size());
        CHECK_A8W8(a8w8_preshuffle_b(host_b.data(), shuf.data(), N, K));
        for (int r = 0; r < (rotate < 1 ? 1 : rotate); ++r) dev_b_copies.push_back(to_device(shuf));
        args.b_preshuffled = 1;
    } else {
        dev_b_copies.push_back(to_device(host_b));
    }
    void* dev_sfa = mode == A8W8_SCALE_MX_E8M0_1x32 ? (void*)to_device(sfa_e) : (void*)to_device(sfa_f);
    void* dev_sfb = mode == A8W8_SCALE_MX_E8M0_1x32 ? (void*)to_device(sfb_e) : (void*)to_device(sfb_f);
    const size_t c_bytes = c_elems * (args.c_dtype == A8W8_C_FP32 ? 4 : 2);
    void* dev_c = nullptr;
    CHECK_HIP(hipMalloc(&dev_c, c_bytes));
    args.a = dev_a; args.b = dev_b_copies[0]; args.c = dev_c; args.sfa = dev_sfa; args.sfb = dev_sfb;

    // mxt: tiled copies of the scales, rebuilt from the row-major arrays by every launch
    const bool tiled = scale_mode == "mxt";
    uint8_t *dev_ta = nullptr, *dev_tb = nullptr;
    const size_t ta_bytes = tiled ? a8w8_mx_tiled_bytes(M, K) : 0, tb_bytes = tiled ? a8w8_mx_tiled_bytes(N, K) : 0;
    if (tiled) {
        CHECK_HIP(hipMalloc(&dev_ta, ta_bytes * batch));
        CHECK_HIP(hipMalloc(&dev_tb, tb_bytes * batch));
    }
    auto launch = [&](int i) {
        a8w8_gemm_args local = args;
        local.b = dev_b_copies[(size_t)i % dev_b_copies.size()];
        if (tiled) {
            for (int b = 0; b < batch; ++b)
                CHECK_A8W8(a8w8_mx_tile_scales_ab((const uint8_t*)dev_sfa + (size_t)b * args.stride_sfa_batch, M, K / 32,
                                                  dev_ta + b * ta_bytes,
                                                  (const uint8_t*)dev_sfb + (size_t)b * args.stride_sfb_batch, N, K / 32,
                                                  dev_tb + b * tb_bytes, K, nullptr));
            local.scale_mode = A8W8_SCALE_MX_E8M0_TILED;
            local.sfa = dev_ta; local.sfb = dev_tb;
            local.stride_sfa_batch = (int)ta_bytes; local.stride_sfb_batch = (int)tb_bytes;
        }
        if (HARNESS_KIND == 0) CHECK_A8W8(a8w8_gemm_blockscale(&local, nullptr));
        else if (HARNESS_KIND == 1) CHECK_A8W8(a8w8_gemm(&local, nullptr));
        else CHECK_A8W8(a8w8_flatmm(&local, nullptr));
    };

    const int tiles = ((M + 255) / 256) * ((N + 255) / 256);
    printf("Launching GEMM kernel: M=%d, N=%d, K=%d, grid=(%u,%u,%u), block=%d [%s]\n", M, N, K, (unsigned)tiles, 1u,
           (unsigned)batch, 512, a8w8_kernel_name(&args) ? a8w8_kernel_name(&args) : "?");
    launch(0);
    CHECK_HIP(hipDeviceSynchronize());

    if (verify) {
        printf("\nValidating GPU results against CPU reference...\n");
        std::vector<float> host_c(c_elems), host_ref((size_t)M * N);
        if (args.c_dtype == A8W8_C_FP32) {
            CHECK_HIP(hipMemcpy(host_c.data(), dev_c, c_bytes, hipMemcpyDeviceToHost));
        } else {
            std::vector<uint16_t> raw(c_elems);
            CHECK_HIP(hipMemcpy(raw.data(), dev_c, c_bytes, hipMemcpyDeviceToHost));
            for (size_t i = 0; i < c_elems; ++i) host_c[i] = orc_bf16_to_f32(raw[i]);
        }
        bool all_valid = true;
        for (int b = 0; b < batch; ++b) {
            const uint8_t* a = host_a.data() + (size_t)b * M * K;
            const uint8_t* bb = host_b.data() + (size_t)b * N * K;
            if (mode == A8W8_SCALE_MX_E8M0_1x32) {
                orc_gemm_ref_mx(a, bb, sfa_e.data() + (size_t)b * args.stride_sfa_batch,
                                sfb_e.data() + (size_t)b * args.stride_sfb_batch, host_ref.data(), M, N, K, K, K, N,
                                K / 32, K / 32, 0, M, 0);
            } else {
                int gm = 1, gn = 1, gk = K;
                if (mode == A8W8_SCALE_BLOCK_1x128_128x128) { gn = 128; gk = 128; }
                if (mode == A8W8_SCALE_TENSOR) { gm = M; gn = N; }
                orc_gemm_ref(a, bb, sfa_f.data() + (size_t)b * args.stride_sfa_batch,
                             sfb_f.data() + (size_t)b * args.stride_sfb_batch, host_ref.data(), M, N, K, K, K, N,
                             args.stride_sfa, args.stride_sfb, gm, gn, gk, 0, M, 0);
            }
            // the reference's own check is 1e-3 absolute on fp32 output (host.cc:273); bf16 outputs
            // use |C - Cref| <= 1e-2*|Cref| + 1e-2
            const bool valid = args.c_dtype == A8W8_C_FP32
                                   ? valid_vector(host_ref.data(), host_c.data() + (size_t)b * M * N, (size_t)M * N, 0.f, 1e-3f)
                                   : valid_vector(host_ref.data(), host_c.data() + (size_t)b * M * N, (size_t)M * N, 1e-2f, 1e-2f,
                                                  mode == A8W8_SCALE_MX_E8M0_1x32 ? (size_t)M * N / 1000 : 0);
            printf("[GEMM batch %d/%d: %dx%dx%d, block_%dx%dx%d] %s\n", b + 1, batch, M, N, K, 256, 256, 128,
                   valid ? "VALID" : "FAIL");
            all_valid = all_valid && valid;
        }
        printf("\n[Overall] %s\n", all_valid ? "ALL BATCHES VALID" : "SOME BATCHES FAILED");
        if (!all_valid) return 2;
    }

    printf("\n");
    const float avg_time = benchmark(launch, warmup, iters);
    const double flop = 2.0 * M * N * K * batch;
    printf("Kernel Performance: avg_time=%.4f ms, %.2f TFlops\n", avg_time, flop / 1.0e9 / avg_time);
    const double bytes = (double)a_elems + b_elems + c_bytes;
    printf("Roofline: %.1f%% of 5.0 PFLOP/s FP8 MFMA peak, %.1f GB/s of operand+result traffic (%.1f%% of 8 TB/s)\n",
           flop / 1.0e9 / avg_time / 5000.0 * 100.0, bytes / 1.0e6 / avg_time, bytes / 1.0e6 / avg_time / 8000.0 * 100.0);
    printf("\n");
    return 0;
}
