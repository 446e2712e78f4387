// Writes the fixtures hip_fp8_decode.txt and hip_fp8_encode.txt from ROCm's host-side
// hip_fp8.h classes (library code shipped with the toolchain, the same classes the
// reference host harness converts with: __hip_fp8_e4m3 at
// opus_gemm/block_scale_gemm/gemm_a8w8_blockscale_host.cc:29,41,84).
// Build and run on the CPU:
//   hipcc -std=c++17 -O1 --offload-arch=gfx950 gen_hip_fp8_tables.cpp -o /tmp/gen_fp8 && /tmp/gen_fp8 .
#include <hip/hip_fp8.h>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

static uint32_t bits(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
static float fromb(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }

int main(int argc, char** argv) {
    std::string dir = argc > 1 ? argv[1] : ".";
    {   // decode: code, fp32 bits as OCP E4M3, fp32 bits as E4M3 FNUZ
        FILE* f = std::fopen((dir + "/hip_fp8_decode.txt").c_str(), "w");
        std::fprintf(f, "# code ocp_f32_bits fnuz_f32_bits\n");
        for (int c = 0; c < 256; ++c) {
            __hip_fp8_e4m3 o; o.__x = (unsigned char)c;
            __hip_fp8_e4m3_fnuz z; z.__x = (unsigned char)c;
            std::fprintf(f, "%02x %08x %08x\n", c, bits((float)o), bits((float)z));
        }
        std::fclose(f);
    }
    {   // encode: fp32 bits, OCP code, FNUZ code
        std::vector<float> in;
        // every representable magnitude of both dialects, the midpoints between neighbours
        // and the fp32 values one ulp either side of each of them
        for (int dial = 0; dial < 2; ++dial) {
            std::vector<float> vals;
            for (int c = 0; c < 0x7f; ++c) {
                float v;
                if (dial == 0) { __hip_fp8_e4m3 o; o.__x = (unsigned char)c; v = (float)o; }
                else { __hip_fp8_e4m3_fnuz z; z.__x = (unsigned char)c; v = (float)z; }
                vals.push_back(v);
            }
            if (dial == 1) { __hip_fp8_e4m3_fnuz z; z.__x = 0x7f; vals.push_back((float)z); }
            for (size_t i = 0; i < vals.size(); ++i) {
                float pts[2] = {vals[i], i + 1 < vals.size() ? 0.5f * (vals[i] + vals[i + 1]) : vals[i] * 1.0625f};
                for (float p : pts)
                    for (float q : {p, std::nextafterf(p, 1e9f), std::nextafterf(p, -1e9f)})
                        for (float s : {1.0f, -1.0f}) in.push_back(s * q);
            }
        }
        for (float v : {0.0f, -0.0f, 240.0f, 248.0f, 256.0f, 448.0f, 464.0f, 480.0f, 1000.0f, 1e30f, -54.0f,
                        1e-3f, 1e-4f, 1e-9f, 1.17549435e-38f, 1e-40f})
            for (float s : {1.0f, -1.0f}) in.push_back(s * v);
        in.push_back(fromb(0x7f800000u)); in.push_back(fromb(0xff800000u));
        in.push_back(fromb(0x7fc00000u)); in.push_back(fromb(0xffc00000u)); in.push_back(fromb(0x7f800001u));
        uint64_t s = 0x9E3779B97F4A7C15ull;   // splitmix64 stream: random fp32 bit patterns
        for (int i = 0; i < 3000; ++i) {
            s += 0x9E3779B97F4A7C15ull; uint64_t z = s;
            z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull; z = (z ^ (z >> 27)) * 0x94D049BB133111EBull; z ^= z >> 31;
            uint32_t u = (uint32_t)z;
            // keep the exponent in the interesting range 2^-12 .. 2^10
            u = (u & 0x807fffffu) | ((115u + (uint32_t)((z >> 32) % 23)) << 23);
            in.push_back(fromb(u));
        }
        FILE* f = std::fopen((dir + "/hip_fp8_encode.txt").c_str(), "w");
        std::fprintf(f, "# f32_bits ocp_code fnuz_code  (RNE, saturate-to-finite)\n");
        for (float v : in) {
            __hip_fp8_e4m3 o(v);
            __hip_fp8_e4m3_fnuz z(v);
            std::fprintf(f, "%08x %02x %02x\n", bits(v), (unsigned)o.__x, (unsigned)z.__x);
        }
        std::fclose(f);
    }
    return 0;
}
