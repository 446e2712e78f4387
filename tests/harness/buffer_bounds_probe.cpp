// What a raw buffer load returns on gfx950 when the address leaves the descriptor's extent through the
// SCALAR offset.  The GEMM kernels keep one lane offset per operand and move between row groups with the scalar
// offset; they rely on rows past the end of a matrix reading as zero without touching memory.  The instruction-set
// manuals of the family disagree on whether the scalar offset takes part in the range check, so this program
// measures it: the descriptor covers the first 4 KiB of a live, sentinel-filled 1 MiB allocation, so that every
// address used stays inside the allocation whatever the answer, and each case prints how many of the 64 lanes'
// 16-byte loads came back as zeros, as data, or (for the direct-to-LDS form) left LDS untouched.
// Exit status 0 when the range check covers lane offset + scalar offset for both forms of the load.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <vector>

typedef int v4i __attribute__((ext_vector_type(4)));

__global__ void probe(const uint8_t* base, uint32_t extent, int lane_base, int scalar_offset, int* to_regs, int* to_lds)
{
    __shared__ __attribute__((aligned(1024))) char smem[1024];
    const int lane = threadIdx.x;
    for (int i = lane; i < 256; i += 64) ((int*)smem)[i] = 0x11111111;
    __syncthreads();
    __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(base), 0, extent, 0x00020000);
    const v4i v = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rs, lane_base + lane * 16, scalar_offset, 0));
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)smem, 16, lane_base + lane * 16,
                                             scalar_offset, 0, 0);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    for (int e = 0; e < 4; ++e) {
        to_regs[lane * 4 + e] = v[e];
        to_lds[lane * 4 + e] = ((int*)smem)[lane * 4 + e];
    }
}

#define CHECK(call)                                                              \
    do {                                                                         \
        if ((call) != hipSuccess) { fprintf(stderr, "%s failed\n", #call); return 2; } \
    } while (0)

int main()
{
    const size_t bytes = 1 << 20;
    const uint32_t extent = 4096;
    uint8_t* data = nullptr;
    int *regs = nullptr, *lds = nullptr;
    CHECK(hipMalloc(&data, bytes));
    CHECK(hipMalloc(&regs, 1024));
    CHECK(hipMalloc(&lds, 1024));
    CHECK(hipMemset(data, 0xAB, bytes));
    struct Case {
        int lane_base, scalar_offset, want_zero_lanes;
        const char* what;
    };
    const Case cases[] = {
        {0, 0, 0, "inside the extent"},
        {8192, 0, 64, "lane offset past the extent"},
        {0, 8192, 64, "scalar offset past the extent"},
        {0, 4096 - 512, 32, "lane + scalar offset straddles the end"},
        {4096 - 512, 0, 32, "lane offset straddles the end"},
    };
    bool ok = true;
    for (const Case& c : cases) {
        hipLaunchKernelGGL(probe, dim3(1), dim3(64), 0, 0, data, extent, c.lane_base, c.scalar_offset, regs, lds);
        std::vector<int> r(256), l(256);
        CHECK(hipMemcpy(r.data(), regs, 1024, hipMemcpyDeviceToHost));
        CHECK(hipMemcpy(l.data(), lds, 1024, hipMemcpyDeviceToHost));
        int reg_zero = 0, reg_data = 0, lds_zero = 0, lds_data = 0, lds_untouched = 0;
        for (int lane = 0; lane < 64; ++lane) {
            bool rz = true, rd = true, lz = true, ldt = true, lu = true;
            for (int e = 0; e < 4; ++e) {
                rz &= r[lane * 4 + e] == 0;
                rd &= (uint32_t)r[lane * 4 + e] == 0xABABABABu;
                lz &= l[lane * 4 + e] == 0;
                ldt &= (uint32_t)l[lane * 4 + e] == 0xABABABABu;
                lu &= l[lane * 4 + e] == 0x11111111;
            }
            reg_zero += rz; reg_data += rd; lds_zero += lz; lds_data += ldt; lds_untouched += lu;
        }
        const bool pass = reg_zero == c.want_zero_lanes && reg_data == 64 - c.want_zero_lanes &&
                          lds_zero == c.want_zero_lanes && lds_data == 64 - c.want_zero_lanes;
        printf("%-42s lane_base=%d scalar=%d: registers zero=%d data=%d | lds zero=%d data=%d untouched=%d  %s\n", c.what,
               c.lane_base, c.scalar_offset, reg_zero, reg_data, lds_zero, lds_data, lds_untouched, pass ? "ok" : "UNEXPECTED");
        ok = ok && pass;
    }
    printf("%s\n", ok ? "range check covers lane offset + scalar offset: out-of-range loads return zero"
                      : "range check does NOT behave as the kernels assume");
    return ok ? 0 : 1;
}
