// C ABI of libmi355a8w8: argument validation, kernel selection, launches.
#include "../../include/mi355_a8w8.h"

#include <hip/hip_runtime.h>
#include <stdio.h>
#include <string.h>
#include <algorithm>
#include <mutex>
#include <tuple>
#include <utility>

#include "cvt.hpp"
#include "flatmm.hpp"
#include "gemm_general.hpp"
#include "gemm_persist.hpp"
#include "gemm_small.hpp"
#include "gemm_wide.hpp"
#include "hbm_probe.hpp"

using namespace a8w8;

namespace {

// ---------------------------------------------------------------- per-device set-up, done once
// What a device needs before its first launch: its architecture and compute-unit count, and the
// dynamic-LDS limit of every kernel instantiation that uses more than the 64 KiB default.  It runs
// exactly once per device (std::call_once: concurrent first calls from several threads wait for
// it), either from a8w8_init or from the first entry point called with that device current.
constexpr int MAX_DEVICES = 64;
struct DeviceState {
    std::once_flag once;
    int status = A8W8_ERR_NO_DEVICE;
    int num_cus = 0;
};
DeviceState g_dev[MAX_DEVICES];

template <class K>
bool raise_lds_limit(K kern, int bytes)
{
    return hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) == hipSuccess;
}

constexpr int persist_lds_bytes(int mode)
{
    return mode == MODE_MX ? PERSIST_LDS_BYTES_MX : mode == MODE_ROWCOL ? PERSIST_LDS_BYTES_ROWCOL : PERSIST_LDS_BYTES;
}

// LDS stages of the 128 x 64 variant of the 128-tile kernel: as many as fit 160 KiB
constexpr int narrow_stages(int mode) { return mode == MODE_MXT || mode == MODE_F4T ? 5 : 6; }

template <int MODE>
bool raise_lds_limits_of_mode()
{
    bool ok = true;
    if constexpr (MODE == MODE_TENSOR || MODE == MODE_ROWCOL || MODE == MODE_BLOCK || MODE == MODE_MX || MODE == MODE_BF16)
        ok = ok && raise_lds_limit(gemm_a8w8_persist<MODE, C_BF16>, persist_lds_bytes(MODE)) &&
             raise_lds_limit(gemm_a8w8_persist<MODE, C_FP32>, persist_lds_bytes(MODE));
    if constexpr (MODE == MODE_TENSOR || MODE == MODE_ROWCOL || MODE == MODE_MXT || MODE == MODE_BF16 || MODE == MODE_F4T)
        ok = ok && raise_lds_limit(gemm_a8w8_wide<MODE, C_BF16>, wide_lds_bytes(MODE)) &&
             raise_lds_limit(gemm_a8w8_wide<MODE, C_FP32>, wide_lds_bytes(MODE));
    {
        ok = ok && raise_lds_limit(gemm_a8w8_tile128<MODE, C_BF16, 2>, small_lds_bytes(MODE, 2)) &&
             raise_lds_limit(gemm_a8w8_tile128<MODE, C_FP32, 2>, small_lds_bytes(MODE, 2)) &&
             raise_lds_limit(gemm_a8w8_tile128<MODE, C_BF16, 4>, small_lds_bytes(MODE, 4)) &&
             raise_lds_limit(gemm_a8w8_tile128<MODE, C_FP32, 4>, small_lds_bytes(MODE, 4)) &&
             raise_lds_limit(gemm_a8w8_tile128<MODE, C_BF16, narrow_stages(MODE), 64>, small_lds_bytes(MODE, narrow_stages(MODE), 64)) &&
             raise_lds_limit(gemm_a8w8_tile128<MODE, C_FP32, narrow_stages(MODE), 64>, small_lds_bytes(MODE, narrow_stages(MODE), 64));
    }
    return ok;
}

// runs with device `dev` current
void set_up_device(int dev)
{
    DeviceState& d = g_dev[dev];
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) { d.status = A8W8_ERR_NO_DEVICE; return; }
    d.num_cus = prop.multiProcessorCount;
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) { d.status = A8W8_ERR_NO_DEVICE; return; }
    const bool ok = raise_lds_limits_of_mode<MODE_TENSOR>() && raise_lds_limits_of_mode<MODE_ROWCOL>() &&
                    raise_lds_limits_of_mode<MODE_BLOCK>() && raise_lds_limits_of_mode<MODE_MX>() &&
                    raise_lds_limits_of_mode<MODE_MXT>() && raise_lds_limits_of_mode<MODE_BF16>() &&
                    raise_lds_limits_of_mode<MODE_F4T>() && raise_lds_limits_of_mode<MODE_F4>();
    d.status = ok ? A8W8_OK : A8W8_ERR_LAUNCH;
}

// A8W8_OK when the current device is a gfx950 that has been set up (setting it up on first use).
int device_status()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return A8W8_ERR_NO_DEVICE;
    std::call_once(g_dev[dev].once, set_up_device, dev);
    return g_dev[dev].status;
}

// One kernel launch; the status is that of this launch alone (hipLaunchKernel's own return value, not the
// thread's sticky last error, which an earlier unrelated runtime call may have set).
template <class... P, class... A, size_t... I>
int launch_impl(void (*kern)(P...), dim3 grid, dim3 block, unsigned lds, hipStream_t s, std::index_sequence<I...>, A&&... a)
{
    std::tuple<P...> params{static_cast<P>(std::forward<A>(a))...};
    void* ptrs[] = {(void*)&std::get<I>(params)...};
    return hipLaunchKernel((const void*)kern, grid, block, ptrs, lds, s) == hipSuccess ? A8W8_OK : A8W8_ERR_LAUNCH;
}
template <class... P, class... A>
int launch(void (*kern)(P...), dim3 grid, dim3 block, unsigned lds, hipStream_t s, A&&... a)
{
    static_assert(sizeof...(P) == sizeof...(A), "one argument per kernel parameter");
    return launch_impl(kern, grid, block, lds, s, std::index_sequence_for<P...>{}, std::forward<A>(a)...);
}
// a launch in the middle of a sequence: leave with its status if it failed
#define A8W8_LAUNCH_OR_RETURN(...)                       \
    do {                                                 \
        const int st_ = launch(__VA_ARGS__);             \
        if (st_ != A8W8_OK) return st_;                  \
    } while (0)

bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// The two pipelined kernels (and only they) address the 256 rows of a C tile with unsigned 32-bit byte offsets from
// the tile's origin: (255 stride_c + 256) elements of `elem_bytes` must stay below 2^32.  That is stride_c up to
// 4,210,751 for fp32 and 8,421,503 for bf16; the other kernels address C with 64-bit pointers and take any stride.
bool c_tile_fits(long long stride_c, int elem_bytes)
{
    return ((long long)(BM - 1) * stride_c + BN) * elem_bytes < (1ll << 32);
}

// Checks shared by every GEMM entry point (mirrors the reference harness's rejects,
// gemm_a8w8_blockscale_host.cc:175-187, and adds the pointer/stride checks a library needs).
int validate_common(const a8w8_gemm_args* g)
{
    if (!g) return A8W8_ERR_NULL_POINTER;
    if (!g->a || !g->b || !g->c || !g->sfa || !g->sfb) return A8W8_ERR_NULL_POINTER;
    if (g->m <= 0 || g->n <= 0 || g->k <= 0 || g->batch <= 0) return A8W8_ERR_BAD_SHAPE;
    if (g->scale_mode < 0 || g->scale_mode > A8W8_SCALE_MX_E8M0_TILED) return A8W8_ERR_BAD_MODE;
    if (g->c_dtype != A8W8_C_BF16 && g->c_dtype != A8W8_C_FP32) return A8W8_ERR_BAD_MODE;
    if (g->scale_mode == A8W8_SCALE_BLOCK_1x128_128x128 && (g->n % 128 != 0 || g->k % 128 != 0))
        return A8W8_ERR_BAD_GROUP;
    if ((g->scale_mode == A8W8_SCALE_MX_E8M0_1x32 || g->scale_mode == A8W8_SCALE_MX_E8M0_TILED) && g->k % 32 != 0)
        return A8W8_ERR_BAD_GROUP;
    if (g->stride_c < g->n) return A8W8_ERR_BAD_STRIDE;
    if (g->stride_a < g->k) return A8W8_ERR_BAD_STRIDE;
    if (!g->b_preshuffled && g->stride_b < g->k) return A8W8_ERR_BAD_STRIDE;
    if (g->scale_mode == A8W8_SCALE_BLOCK_1x128_128x128 && (g->stride_sfa < g->m || g->stride_sfb < g->k / 128))
        return A8W8_ERR_BAD_STRIDE;
    if (g->scale_mode == A8W8_SCALE_MX_E8M0_1x32 && (g->stride_sfa < g->k / 32 || g->stride_sfb < g->k / 32))
        return A8W8_ERR_BAD_STRIDE;
    if (g->batch > 1 && (g->stride_a_batch < 0 || g->stride_b_batch < 0 || g->stride_c_batch < 0 ||
                         g->stride_sfa_batch < 0 || g->stride_sfb_batch < 0))
        return A8W8_ERR_BAD_STRIDE;
    // the kernels address one batch of A / B with 32-bit byte offsets
    const long long a_span = (long long)(g->m - 1) * g->stride_a + g->k;
    const long long b_span = g->b_preshuffled ? (long long)g->n * g->k : (long long)(g->n - 1) * g->stride_b + g->k;
    if (a_span >= (1ll << 31) || b_span >= (1ll << 31)) return A8W8_ERR_TOO_LARGE;
    if (g->batch > 65535) return A8W8_ERR_TOO_LARGE;
    // ... and the A-side block scales of all K groups, and count 128 x 128 tiles with an int
    if (g->scale_mode == A8W8_SCALE_BLOCK_1x128_128x128 && (long long)(g->k / 128) * g->stride_sfa * 4 >= (1ll << 31))
        return A8W8_ERR_TOO_LARGE;
    if ((long long)((g->m + 127) / 128) * ((g->n + 127) / 128) >= (1ll << 31)) return A8W8_ERR_TOO_LARGE;
    return A8W8_OK;
}

GemmParams make_params(const a8w8_gemm_args* g)
{
    GemmParams p;
    p.a = (const uint8_t*)g->a;
    p.b = (const uint8_t*)g->b;
    p.c = g->c;
    p.sfa = g->sfa;
    p.sfb = g->sfb;
    p.m = g->m; p.n = g->n; p.k = g->k;
    p.lda = g->stride_a; p.ldc = g->stride_c;
    // pre-shuffled B: 16 rows span 16 k bytes and a 128-wide K step two 1 KiB blocks
    p.ldb = g->b_preshuffled ? g->k : g->stride_b;
    p.b_kshift = g->b_preshuffled ? 11 : 7;
    p.a_batch = g->stride_a_batch; p.b_batch = g->stride_b_batch; p.c_batch = g->stride_c_batch;
    p.sfa_batch = g->stride_sfa_batch; p.sfb_batch = g->stride_sfb_batch;
    p.stride_sfa = g->stride_sfa; p.stride_sfb = g->stride_sfb;
    p.tiles_m = (g->m + BM - 1) / BM;
    p.tiles_n = (g->n + BN - 1) / BN;
    return p;
}

// The tiled kernels need whole 128-wide K steps and 16-byte aligned rows in A and B; the MX
// variant also stages its scale bytes with dword-granular loads.
bool tiled_ok(const a8w8_gemm_args* g)
{
    if (g->scale_mode == A8W8_SCALE_MX_E8M0_1x32 &&
        (g->stride_sfa % 4 != 0 || g->stride_sfb % 4 != 0 || ((uintptr_t)g->sfa & 3) || ((uintptr_t)g->sfb & 3) ||
         (g->batch > 1 && (g->stride_sfa_batch % 4 != 0 || g->stride_sfb_batch % 4 != 0))))
        return false;
    if (g->scale_mode == A8W8_SCALE_MX_E8M0_TILED &&
        (!aligned16(g->sfa) || !aligned16(g->sfb) ||
         (g->batch > 1 && (g->stride_sfa_batch % 16 != 0 || g->stride_sfb_batch % 16 != 0))))
        return false;
    return g->k % BK == 0 && g->stride_a % 16 == 0 && g->stride_b % 16 == 0 && aligned16(g->a) && aligned16(g->b) &&
           (g->batch == 1 || (g->stride_a_batch % 16 == 0 && g->stride_b_batch % 16 == 0)) &&
           (long long)((g->m + BM - 1) / BM) * ((g->n + BN - 1) / BN) < (1ll << 31);
}

// B in the a8w8_preshuffle_b layout is read by the MFMA kernels only (the one-thread-per-element kernel reads
// row-major B): whole 16-row groups and 128-wide K steps, aligned pointers.
int validate_shuffled_b(const a8w8_gemm_args* g)
{
    if (!g->b_preshuffled) return A8W8_OK;
    if (g->n % 16 != 0 || g->k % BK != 0) return A8W8_ERR_BAD_GROUP;
    a8w8_gemm_args rows = *g;
    rows.stride_b = g->k;           // what the alignment checks of tiled_ok should see for B
    return tiled_ok(&rows) ? A8W8_OK : A8W8_ERR_MISALIGNED;
}

// The persistent kernel pipelines two K steps ahead and indexes work items with an int.
bool persist_ok(const a8w8_gemm_args* g)
{
    // tiled MX scales come in pairs of K steps (one dword serves two steps)
    if (g->scale_mode == A8W8_SCALE_MX_E8M0_TILED && (g->k / BK) % 2 != 0) return false;
    return g->k >= 2 * BK &&
           (long long)g->batch * ((g->m + BM - 1) / BM) * ((g->n + BN - 1) / BN) < (1ll << 30);
}

// The four-wave kernel walks K in pairs of steps and has the per-tensor, row/col and tiled-MX scale modes.
bool wide_ok(const a8w8_gemm_args* g)
{
    if (g->scale_mode != A8W8_SCALE_TENSOR && g->scale_mode != A8W8_SCALE_ROWCOL && g->scale_mode != A8W8_SCALE_MX_E8M0_TILED)
        return false;
    return persist_ok(g) && (g->k / BK) % 2 == 0;
}

template <int MODE, int CDT>
int launch_general(const GemmParams& p, int batch, hipStream_t stream);

// compute units of the current device (256 before the device has been set up: kernel-name queries on a CPU box)
int num_cus()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return 256;
    return g_dev[dev].num_cus > 0 ? g_dev[dev].num_cus : 256;
}

// 128 x 128 tiles when all of them fit on the chip at once, two workgroups per compute unit: a problem of that
// size leaves 256 x 256 tiles with at most half of the compute units.  Measured on 256 compute units against the
// 256-tile kernels (block / row-col / tiled MX): 2.2x / 1.7x / 1.6x at 64 workgroups, 1.9x / 1.6x / 1.5x at 256,
// +45% / +21% / +15% at 400, +37% / +17% / +9% at 512; beyond that the second round of workgroups costs more than
// the idle compute units did (-9% for row/col at 576).
// (the bound as a switch, for measurement: with 8 instead of 2, 4096 x 7168 x 2048 and 4096^3 take 12-30% longer in every scale mode)
#ifndef A8W8_SMALL_TILES_PER_CU
#define A8W8_SMALL_TILES_PER_CU 2
#endif
#ifndef A8W8_SMALL_DEEP_UP_TO
#define A8W8_SMALL_DEEP_UP_TO 1         // four LDS stages up to this many 128-tiles per compute unit, two stages beyond
#endif
bool small_ok(const a8w8_gemm_args* g)
{
    const bool mxt = g->scale_mode == A8W8_SCALE_MX_E8M0_TILED;
    // tiled MX scales with an odd number of K steps have no 256-tile kernel: any size runs here
    if (mxt && (g->k / BK) % 2 != 0) return true;
    const long long items128 = (long long)g->batch * ((g->m + SM_BM - 1) / SM_BM) * ((g->n + SM_BN - 1) / SM_BN);
    return items128 <= (long long)A8W8_SMALL_TILES_PER_CU * num_cus();
}

// 128 x 64 tiles instead of 128 x 128: when the wide tiles would occupy at most half of the compute units and the K
// loop is long enough for the deeper staging to matter (a problem of a few K steps is bound by launch and store latency,
// which narrower tiles do not change).
#ifndef A8W8_NARROW_MIN_KSTEPS
#define A8W8_NARROW_MIN_KSTEPS 16
#endif
bool narrow_tiles_pay(long long items128, int n, int k)
{
    return 2 * items128 <= num_cus() && n > 64 && k / BK >= A8W8_NARROW_MIN_KSTEPS;
}

template <int MODE, int CDT, int STAGES>
int launch_small_stages(const GemmParams& q, int batch, hipStream_t stream)
{
    dim3 grid((unsigned)(q.tiles_m * q.tiles_n), 1, (unsigned)batch);
    return launch(gemm_a8w8_tile128<MODE, CDT, STAGES>, grid, dim3(SM_THREADS), small_lds_bytes(MODE, STAGES), stream, q);
}

// Up to one workgroup per compute unit: four LDS stages (deep prefetch, one workgroup per compute unit).  More: two
// stages, so that two workgroups share a compute unit and hide each other's waits.
template <int MODE, int CDT>
int launch_small(const GemmParams& p, int batch, hipStream_t stream)
{
    if constexpr (MODE == MODE_TENSOR || MODE == MODE_ROWCOL || MODE == MODE_BLOCK || MODE == MODE_MX || MODE == MODE_MXT ||
                  MODE == MODE_BF16 || MODE == MODE_F4T || MODE == MODE_F4) {
        GemmParams q = p;
        q.tiles_m = (p.m + SM_BM - 1) / SM_BM;
        q.tiles_n = (p.n + SM_BN - 1) / SM_BN;
        const long long items = (long long)q.tiles_m * q.tiles_n * batch;
        if (narrow_tiles_pay(items, p.n, p.k)) {
            // short and wide: 128 x 64 tiles give every compute unit a workgroup, deep staging keeps its share of the
            // weights in flight
            q.tiles_n = (p.n + 63) / 64;
            dim3 grid((unsigned)(q.tiles_m * q.tiles_n), 1, (unsigned)batch);
            constexpr int ST = narrow_stages(MODE);
            return launch(gemm_a8w8_tile128<MODE, CDT, ST, 64>, grid, dim3(SM_THREADS), small_lds_bytes(MODE, ST, 64), stream, q);
        }
        if (items <= (long long)A8W8_SMALL_DEEP_UP_TO * num_cus())
            return launch_small_stages<MODE, CDT, 4>(q, batch, stream);
        return launch_small_stages<MODE, CDT, 2>(q, batch, stream);
    } else {
        return A8W8_ERR_BAD_MODE;
    }
}

template <int MODE, int CDT>
int launch_wide(const GemmParams& p, int batch, hipStream_t stream);

// Persistent pipelined kernel (eight waves): one workgroup per CU walks the (batch, tile) list.
template <int MODE, int CDT>
int launch_persist(const GemmParams& p, int batch, hipStream_t stream)
{
    // tiled MX scales exist on the four-wave kernel only (whatever passes persist_ok with them also passes wide_ok)
    if constexpr (MODE == MODE_MXT) return launch_wide<MODE, CDT>(p, batch, stream);
    else {
    if (!c_tile_fits(p.ldc, CDT == C_BF16 ? 2 : 4)) return A8W8_ERR_TOO_LARGE;
    PersistParams pp;
    pp.g = p;
    pp.batch = batch;
    pp.items = batch * p.tiles_m * p.tiles_n;
    pp.map = make_tile_map(p.tiles_m, p.tiles_n);
    const int cus = num_cus();
    dim3 grid((unsigned)(pp.items < cus ? pp.items : cus), 1, 1);
    return launch(gemm_a8w8_persist<MODE, CDT>, grid, dim3(GEMM_THREADS), persist_lds_bytes(MODE), stream, pp);
    }
}

// Four-wave persistent kernel (one wave per SIMD, 128 x 128 per wave).
template <int MODE, int CDT>
int launch_wide(const GemmParams& p, int batch, hipStream_t stream)
{
    if constexpr (MODE == MODE_TENSOR || MODE == MODE_ROWCOL || MODE == MODE_MXT || MODE == MODE_BF16 || MODE == MODE_F4T) {
        if (!c_tile_fits(p.ldc, CDT == C_BF16 ? 2 : 4)) return A8W8_ERR_TOO_LARGE;
        PersistParams pp;
        pp.g = p;
        pp.batch = batch;
        pp.items = batch * p.tiles_m * p.tiles_n;
        pp.map = make_tile_map(p.tiles_m, p.tiles_n);
        const int cus = num_cus();
        dim3 grid((unsigned)(pp.items < cus ? pp.items : cus), 1, 1);
        return launch(gemm_a8w8_wide<MODE, CDT>, grid, dim3(WIDE_THREADS), wide_lds_bytes(MODE), stream, pp);
    } else {
        return launch_persist<MODE, CDT>(p, batch, stream);
    }
}

template <int MODE, int CDT>
int launch_general(const GemmParams& p, int batch, hipStream_t stream)
{
    dim3 grid((unsigned)((p.n + 15) / 16), (unsigned)((p.m + 15) / 16), (unsigned)batch);
    return launch(gemm_a8w8_general<MODE, CDT>, grid, dim3(256), 0, stream, p);
}


#define A8W8_DISPATCH(FN, mode, cdt, ...)                                                   \
    switch ((mode) * 2 + (cdt)) {                                                           \
        case 0: return FN<MODE_TENSOR, C_BF16>(__VA_ARGS__);                                \
        case 1: return FN<MODE_TENSOR, C_FP32>(__VA_ARGS__);                                \
        case 2: return FN<MODE_ROWCOL, C_BF16>(__VA_ARGS__);                                \
        case 3: return FN<MODE_ROWCOL, C_FP32>(__VA_ARGS__);                                \
        case 4: return FN<MODE_BLOCK, C_BF16>(__VA_ARGS__);                                 \
        case 5: return FN<MODE_BLOCK, C_FP32>(__VA_ARGS__);                                 \
        case 6: return FN<MODE_MX, C_BF16>(__VA_ARGS__);                                    \
        case 7: return FN<MODE_MX, C_FP32>(__VA_ARGS__);                                    \
        case 8: return FN<MODE_MXT, C_BF16>(__VA_ARGS__);                                   \
        case 9: return FN<MODE_MXT, C_FP32>(__VA_ARGS__);                                   \
        default: return A8W8_ERR_BAD_MODE;                                                  \
    }

int dispatch_persist(const a8w8_gemm_args* g, const GemmParams& p, hipStream_t s)
{
    A8W8_DISPATCH(launch_persist, g->scale_mode, g->c_dtype, p, g->batch, s)
}
int dispatch_wide(const a8w8_gemm_args* g, const GemmParams& p, hipStream_t s)
{
    A8W8_DISPATCH(launch_wide, g->scale_mode, g->c_dtype, p, g->batch, s)
}
int dispatch_small(const a8w8_gemm_args* g, const GemmParams& p, hipStream_t s)
{
    A8W8_DISPATCH(launch_small, g->scale_mode, g->c_dtype, p, g->batch, s)
}
int dispatch_general(const a8w8_gemm_args* g, const GemmParams& p, hipStream_t s)
{
    A8W8_DISPATCH(launch_general, g->scale_mode, g->c_dtype, p, g->batch, s)
}

// The flat kernels take up to 128 activation rows: up to four groups of 16 share one pass over the weights, past
// 64 rows two workgroups per group of weight tiles make two passes (the second one from L2).
constexpr int FLAT_MAX_M = 128;

int validate_flat(const a8w8_gemm_args* g)
{
    if (!g) return A8W8_ERR_NULL_POINTER;
    if (!g->b_preshuffled) return A8W8_ERR_BAD_MODE;
    if (g->scale_mode != A8W8_SCALE_ROWCOL && g->scale_mode != A8W8_SCALE_TENSOR && g->scale_mode != A8W8_SCALE_MX_E8M0_TILED &&
        g->scale_mode != A8W8_SCALE_BLOCK_1x128_128x128)
        return A8W8_ERR_BAD_MODE;
    const int st = validate_common(g);
    if (st != A8W8_OK) return st;
    if (g->m > FLAT_MAX_M) return A8W8_ERR_BAD_SHAPE;
    if (g->n % 16 != 0 || g->k % 64 != 0) return A8W8_ERR_BAD_GROUP;
    if (!aligned16(g->a) || !aligned16(g->b) || g->stride_a % 16 != 0) return A8W8_ERR_MISALIGNED;
    if (g->batch > 1 && (g->stride_a_batch % 16 != 0 || g->stride_b_batch % 16 != 0)) return A8W8_ERR_MISALIGNED;
    if (g->scale_mode == A8W8_SCALE_MX_E8M0_TILED &&
        (!aligned16(g->sfa) || !aligned16(g->sfb) || (g->batch > 1 && (g->stride_sfa_batch % 16 != 0 || g->stride_sfb_batch % 16 != 0))))
        return A8W8_ERR_MISALIGNED;
    return A8W8_OK;
}

// Weight tiles (16 rows of B) per workgroup: the activation fragment of a K block is re-used by all of them, but
// the grid shrinks by the same factor: the largest of 4, 2, 1 that still gives every compute unit a workgroup
// (16 x 4096 x 4096: 8.6 us with 4 tiles per workgroup on 64 compute units, 5.4 us with 1 on 256).
template <int NT, int MT, int CDT, int MODE, bool BROW>
int launch_flat_nt(const GemmParams& p, int batch, hipStream_t stream)
{
    const int n_tiles = p.n / 16;
    dim3 grid((unsigned)(((n_tiles + NT - 1) / NT) * ((p.m + 16 * MT - 1) / (16 * MT))), 1, (unsigned)batch);
    return launch(flatmm_a8w8<NT, MT, CDT, MODE, BROW>, grid, dim3(FLAT_THREADS), 0, stream, p);
}

// Up to four groups of 16 activation rows share one pass over the weights; as many weight tiles per workgroup as
// still leave every compute unit a workgroup (every workgroup reads all rows of A once, so more weight tiles per
// workgroup also means fewer reads of A: 16384 x 7168 at M = 48, 30 us with two tiles, 24 us with four).
template <int CDT, int MODE, bool BROW = false>
int launch_flat(const GemmParams& p, int batch, hipStream_t stream)
{
    const long long tiles = (long long)(p.n / 16) * batch;
    const int cus = num_cus();
    // row groups per workgroup: all of them up to four, an even split over two passes beyond
    const int groups = (p.m + 15) / 16, passes = (groups + 3) / 4;
    const int mt = (groups + passes - 1) / passes;
    if (groups > 4 && tiles < 4ll * cus) {
        // too few weight tiles for four per workgroup: two passes would run two tiles per workgroup anyway, and one
        // pass with six or eight row groups on two tiles reads the weights once (8192 x 8192, M = 128: 30 -> 25 us)
        if (groups <= 6) return launch_flat_nt<2, 6, CDT, MODE, BROW>(p, batch, stream);
        // eight groups + scales would spill; with row-major weights their staging does not fit LDS
        if constexpr (MODE != MODE_BLOCK && MODE != MODE_MXT && MODE != MODE_F4T && !BROW)
            return launch_flat_nt<2, 8, CDT, MODE, BROW>(p, batch, stream);
    }
    if (mt == 4) {
        if (tiles >= 4ll * cus) return launch_flat_nt<4, 4, CDT, MODE, BROW>(p, batch, stream);
        return launch_flat_nt<2, 4, CDT, MODE, BROW>(p, batch, stream);
    }
    if (mt == 3) {
        if (tiles >= 4ll * cus) return launch_flat_nt<4, 3, CDT, MODE, BROW>(p, batch, stream);
        return launch_flat_nt<2, 3, CDT, MODE, BROW>(p, batch, stream);
    }
    if (mt == 2) {
        if (tiles >= 4ll * cus) return launch_flat_nt<4, 2, CDT, MODE, BROW>(p, batch, stream);
        return launch_flat_nt<2, 2, CDT, MODE, BROW>(p, batch, stream);
    }
    if (tiles >= 4ll * cus) return launch_flat_nt<4, 1, CDT, MODE, BROW>(p, batch, stream);
    if (tiles >= 2ll * cus) return launch_flat_nt<2, 1, CDT, MODE, BROW>(p, batch, stream);
    return launch_flat_nt<1, 1, CDT, MODE, BROW>(p, batch, stream);
}

// On shuffled weights both the flat GEMM and the MFMA kernels can run a skinny problem; the entry points take the
// one a small cost model calls faster.  Times in microseconds, W = weight bytes, row_bytes = bytes of one weight row:
//   flat:  one pass over the weights at ~6.4 TB/s; every further group of 16 activation rows adds the activation rows
//          that each workgroup reads again for its weight tiles, W / NT bytes at ~21 TB/s (1.4 us on 16384 x 7168), and
//          the scale bytes of MXFP8 about a tenth; a second pass (more than 64 rows over at least four weight tiles
//          per compute unit) reads the weights from L2 and costs 55% more.
//   dense: the 128-tile kernel pulls the weights with one workgroup per 128 weight rows at ~28 GB/s each, or, where
//          128 x 128 tiles would occupy at most half of the compute units, per 64 rows at ~22 GB/s each (its 128 x 64
//          tiles), ~5 TB/s at best over the chip; 20% more at 128 activation rows than at a few.
// Weights of at most 32 MiB always go flat.  Measured on MI355X, shuffled FP8 weights, M = 16 / 32 / 48 / 64 / 80 / 96 /
// 128, flat against dense:
//   16384 x 7168   20 / 21 / 23 / 24 / 35 / 36 / 41  against  30 / 27 / 27 / 28 / 30 / 31 / 33   (MXFP8 about 10% more on both sides)
//   8192 x 8192    13 / 14 / 16 / 18 / 20 / 21 / 26  against  26 / 26 / 26 / 27 / 28 / 29 / 31
//   28672 x 4096   20 / 23 / 25 / 28 / 39 / 41 / 47  against  26 / 26 / 27 / 28 / 29 / 30 / 31
//   4096 x 14336   13 / 19 / 23 / 26 / 31 / 32 / 38  against  41 throughout
// (tests/test_zz_gpu_routing.py times both sides of such cells through a8w8_route_override and checks the choice).
// Row-major weights (a8w8_gemm without b_preshuffled; the flat kernel stages the weight rows through LDS, whole lines
// per load): as fast as shuffled ones unless the rows are a large power of two apart, where the 16 rows of a tile fall
// on the same memory channels -- 16384 x 7168 FP8 M = 16 / 32 / 64: 20 / 21 / 25 us, 8192 x 8192: 17 / 17 / 20 us
// (13 / 14 / 18 shuffled).
int g_route = A8W8_ROUTE_MODEL;      // a8w8_route_override

bool prefer_flat(int m, int n, long long row_bytes, bool scaled_in_loop, double layout_factor = 1.0)
{
    if (g_route != A8W8_ROUTE_MODEL) return g_route == A8W8_ROUTE_FLAT;
    const double w = (double)n * (double)row_bytes;
    if (w <= (double)(32ll << 20)) return true;
    const int groups = (m + 15) / 16, passes = (groups + 3) / 4;
    const int mt = (groups + passes - 1) / passes;
    const int cus = num_cus();
    const int rounds = ((n + 127) / 128 + cus - 1) / cus;
    // one pass over the weights, plus, for every further group of 16 activation rows, the activation rows each
    // workgroup reads again for its NT weight tiles (n * row_bytes / NT bytes from L2) and their MFMAs; nearly twice
    // that where the workgroups do not fit the chip at once
    const long long tiles = n / 16;
    const int nt = tiles >= 4ll * cus ? 4 : tiles >= 2ll * cus ? 2 : 1;
    const double per_group = w / nt / 21.0e6 * (tiles / nt > cus ? 1.9 : 1.0);
    double flat = 1.5 + w / 6.4e6;
    if (groups > 4 && tiles < 4ll * cus && (groups <= 6 || !scaled_in_loop)) {
        flat += per_group * (groups - 1);      // one pass with six or eight row groups (see launch_flat)
    } else {
        flat += per_group * (mt - 1);
        if (passes == 2) flat *= 1.55;      // the second pass reads the weights from L2
    }
    flat *= layout_factor;      // row-major weights: rows staged through LDS, rows a power of two apart share channels
    // (the 128-tile kernel's own choice of tile width, narrow_tiles_pay, for one row of 128-row tiles)
    const bool narrow = narrow_tiles_pay((n + 127) / 128, n, (int)std::min<long long>(row_bytes, 1 << 30));
    const double per_workgroup = narrow ? 64.0 * (double)row_bytes / 22.0e3 : rounds * 128.0 * (double)row_bytes / 28.0e3;
    double dense = 4.0 + std::max(per_workgroup, w / 5.0e6);
    dense *= 1.0 + 0.2 * m / 128.0;
    return flat <= dense;
}

bool prefer_flat_fp8(const a8w8_gemm_args* g)
{
    const bool scaled_in_loop = g->scale_mode == A8W8_SCALE_MX_E8M0_TILED;      // no kernel with eight row groups
    const double layout_factor = g->b_preshuffled ? 1.0 : g->stride_b % 4096 == 0 ? 1.3 : 1.05;
    // (the flat kernel's MX scale bytes, one byte load per weight tile and K pair, cost it about a tenth)
    return prefer_flat(g->m, g->n, g->k, scaled_in_loop, layout_factor * (scaled_in_loop ? 1.1 : 1.0));
}

template <bool BROW>
int launch_flat_fp8_layout(const a8w8_gemm_args* g, hipStream_t s)
{
    const GemmParams p = make_params(g);
    if (g->scale_mode == A8W8_SCALE_MX_E8M0_TILED)
        return g->c_dtype == A8W8_C_BF16 ? launch_flat<C_BF16, MODE_MXT, BROW>(p, g->batch, s) : launch_flat<C_FP32, MODE_MXT, BROW>(p, g->batch, s);
    if (g->scale_mode == A8W8_SCALE_BLOCK_1x128_128x128)
        return g->c_dtype == A8W8_C_BF16 ? launch_flat<C_BF16, MODE_BLOCK, BROW>(p, g->batch, s) : launch_flat<C_FP32, MODE_BLOCK, BROW>(p, g->batch, s);
    const bool tensor = g->scale_mode == A8W8_SCALE_TENSOR;
    if (g->c_dtype == A8W8_C_BF16)
        return tensor ? launch_flat<C_BF16, MODE_TENSOR, BROW>(p, g->batch, s) : launch_flat<C_BF16, MODE_ROWCOL, BROW>(p, g->batch, s);
    return tensor ? launch_flat<C_FP32, MODE_TENSOR, BROW>(p, g->batch, s) : launch_flat<C_FP32, MODE_ROWCOL, BROW>(p, g->batch, s);
}

int launch_flat_fp8(const a8w8_gemm_args* g, hipStream_t s)
{
    return g->b_preshuffled ? launch_flat_fp8_layout<false>(g, s) : launch_flat_fp8_layout<true>(g, s);
}

// A skinny problem on row-major weights that the flat kernel can run (it stages the weight rows through LDS).
bool flat_rowmajor_ok(const a8w8_gemm_args* g)
{
    if (g->b_preshuffled || g->m > FLAT_MAX_M) return false;
    if (g->scale_mode != A8W8_SCALE_ROWCOL && g->scale_mode != A8W8_SCALE_TENSOR && g->scale_mode != A8W8_SCALE_MX_E8M0_TILED &&
        g->scale_mode != A8W8_SCALE_BLOCK_1x128_128x128)
        return false;
    if (g->n % 16 != 0 || g->k % 64 != 0) return false;
    if (!aligned16(g->a) || !aligned16(g->b) || g->stride_a % 16 != 0 || g->stride_b % 16 != 0) return false;
    if (g->batch > 1 && (g->stride_a_batch % 16 != 0 || g->stride_b_batch % 16 != 0)) return false;
    if (g->scale_mode == A8W8_SCALE_MX_E8M0_TILED &&
        (!aligned16(g->sfa) || !aligned16(g->sfb) || (g->batch > 1 && (g->stride_sfa_batch % 16 != 0 || g->stride_sfb_batch % 16 != 0))))
        return false;
    return (long long)(g->n - 1) * g->stride_b + g->k < (1ll << 31);
}

// Whether launch_dense_fp8 (and the bf16 / MXFP4 entry points on their byte views) would take one of the two 256-tile
// kernels: their C tiles must fit 32-bit offsets (c_tile_fits), which the entry points check before any device call.
bool takes_tile256(const a8w8_gemm_args* g)
{
    return tiled_ok(g) && !small_ok(g) && (wide_ok(g) || persist_ok(g));
}
bool c_stride_too_large(const a8w8_gemm_args* g, const a8w8_gemm_args* byte_view)
{
    return takes_tile256(byte_view) && !c_tile_fits(g->stride_c, g->c_dtype == A8W8_C_BF16 ? 2 : 4);
}

int launch_dense_fp8(const a8w8_gemm_args* g, hipStream_t s)
{
    const GemmParams p = make_params(g);
    if (!tiled_ok(g)) return dispatch_general(g, p, s);
    if (small_ok(g)) return dispatch_small(g, p, s);
    if (wide_ok(g)) return dispatch_wide(g, p, s);
    // what is left has a single K step (k = 128) or more work items than the persistent kernels index: the 128-tile
    // kernel runs any number of steps and tiles
    return persist_ok(g) ? dispatch_persist(g, p, s) : dispatch_small(g, p, s);
}

}  // namespace

extern "C" {

int a8w8_gemm(const a8w8_gemm_args* args, void* hip_stream)
{
    const int st = validate_common(args);
    if (st != A8W8_OK) return st;
    a8w8_gemm_args local = *args;
    if (local.b_preshuffled) local.stride_b = local.k;      // stride_b is not read for shuffled weights
    const a8w8_gemm_args* g = &local;
    const int shuf = validate_shuffled_b(g);
    if (shuf != A8W8_OK) return shuf;
    // a skinny problem on shuffled weights: the flat kernel where it is the faster one
    const bool flat = (g->b_preshuffled && validate_flat(g) == A8W8_OK && prefer_flat_fp8(g)) || (flat_rowmajor_ok(g) && prefer_flat_fp8(g));
    if (!flat && c_stride_too_large(g, g)) return A8W8_ERR_TOO_LARGE;
    if (const int ds = device_status(); ds != A8W8_OK) return ds;
    hipStream_t s = (hipStream_t)hip_stream;
    if (flat) return launch_flat_fp8(g, s);
    return launch_dense_fp8(g, s);
}

static int a16w16_flat_impl(const a8w8_gemm_args* g, void* hip_stream, bool allow_dense);

static int a16w16_gemm_impl(const a8w8_gemm_args* g, void* hip_stream, bool allow_flat)
{
    if (!g) return A8W8_ERR_NULL_POINTER;
    // a skinny problem on shuffled weights: the flat kernel where it is the faster one (and can run it)
    if (allow_flat && g->b_preshuffled && g->m > 0 && g->m <= FLAT_MAX_M && prefer_flat(g->m, g->n, 2ll * g->k, false) &&
        a16w16_flat_impl(g, hip_stream, false) == A8W8_OK)
        return A8W8_OK;
    if (!g->a || !g->b || !g->c) return A8W8_ERR_NULL_POINTER;
    if (g->m <= 0 || g->n <= 0 || g->k <= 0 || g->batch <= 0) return A8W8_ERR_BAD_SHAPE;
    if (g->c_dtype != A8W8_C_BF16 && g->c_dtype != A8W8_C_FP32) return A8W8_ERR_BAD_MODE;
    if (g->stride_c < g->n || g->stride_a < g->k || (!g->b_preshuffled && g->stride_b < g->k)) return A8W8_ERR_BAD_STRIDE;
    if (g->batch > 1 && (g->stride_a_batch < 0 || g->stride_b_batch < 0 || g->stride_c_batch < 0)) return A8W8_ERR_BAD_STRIDE;
    const long long a_span = ((long long)(g->m - 1) * g->stride_a + g->k) * 2;
    const long long b_span = (g->b_preshuffled ? (long long)g->n * g->k : (long long)(g->n - 1) * g->stride_b + g->k) * 2;
    if (a_span >= (1ll << 31) || b_span >= (1ll << 31) || g->batch > 65535) return A8W8_ERR_TOO_LARGE;
    // the tiled kernel reads bf16 rows as byte rows of 2k columns
    a8w8_gemm_args bytes = *g;
    bytes.k = g->k * 2;
    bytes.stride_a = g->stride_a * 2; bytes.stride_b = g->b_preshuffled ? bytes.k : g->stride_b * 2;
    bytes.stride_a_batch = g->stride_a_batch * 2; bytes.stride_b_batch = g->stride_b_batch * 2;
    bytes.scale_mode = A8W8_SCALE_TENSOR;
    const bool fits = (long long)g->stride_a_batch * 2 < (1ll << 31) && (long long)g->stride_b_batch * 2 < (1ll << 31);
    const bool flat_rows = fits && flat_rowmajor_ok(&bytes) && prefer_flat(g->m, g->n, bytes.k, false, bytes.stride_b % 4096 == 0 ? 1.3 : 1.05);
    if (!flat_rows && fits && c_stride_too_large(g, &bytes)) return A8W8_ERR_TOO_LARGE;
    if (const int ds = device_status(); ds != A8W8_OK) return ds;
    hipStream_t s = (hipStream_t)hip_stream;
    // a skinny problem on row-major weights: the flat kernel (weight rows staged through LDS) where it is the faster one
    if (flat_rows) {
        GemmParams p = make_params(&bytes);
        p.sfa = p.sfb = nullptr;
        return g->c_dtype == A8W8_C_BF16 ? launch_flat<C_BF16, MODE_BF16, true>(p, g->batch, s)
                                         : launch_flat<C_FP32, MODE_BF16, true>(p, g->batch, s);
    }
    // weights shuffled as bytes (a16w16_flatmm's): MFMA kernels only
    if (g->b_preshuffled && (validate_shuffled_b(&bytes) != A8W8_OK || !fits || !persist_ok(&bytes))) return A8W8_ERR_BAD_GROUP;
    if (fits && tiled_ok(&bytes) && persist_ok(&bytes)) {
        GemmParams p = make_params(&bytes);
        p.sfa = p.sfb = nullptr;
        if (small_ok(&bytes))            // few tiles: 128 x 128 ones
            return g->c_dtype == A8W8_C_BF16 ? launch_small<MODE_BF16, C_BF16>(p, g->batch, s)
                                             : launch_small<MODE_BF16, C_FP32>(p, g->batch, s);
        if ((bytes.k / BK) % 2 == 0)     // an even number of K steps: the four-wave kernel
            return g->c_dtype == A8W8_C_BF16 ? launch_wide<MODE_BF16, C_BF16>(p, g->batch, s)
                                             : launch_wide<MODE_BF16, C_FP32>(p, g->batch, s);
        return g->c_dtype == A8W8_C_BF16 ? launch_persist<MODE_BF16, C_BF16>(p, g->batch, s)
                                         : launch_persist<MODE_BF16, C_FP32>(p, g->batch, s);
    }
    dim3 grid((unsigned)((g->n + 15) / 16), (unsigned)((g->m + 15) / 16), (unsigned)g->batch);
    if (g->c_dtype == A8W8_C_BF16)
        A8W8_LAUNCH_OR_RETURN((gemm_a16w16_general<C_BF16>), grid, dim3(256), 0, s, (const unsigned short*)g->a,
                           (const unsigned short*)g->b, g->c, g->m, g->n, g->k, g->stride_a, g->stride_b, g->stride_c,
                           (long long)g->stride_a_batch, (long long)g->stride_b_batch, (long long)g->stride_c_batch);
    else
        A8W8_LAUNCH_OR_RETURN((gemm_a16w16_general<C_FP32>), grid, dim3(256), 0, s, (const unsigned short*)g->a,
                           (const unsigned short*)g->b, g->c, g->m, g->n, g->k, g->stride_a, g->stride_b, g->stride_c,
                           (long long)g->stride_a_batch, (long long)g->stride_b_batch, (long long)g->stride_c_batch);
    return A8W8_OK;
}

int a16w16_gemm(const a8w8_gemm_args* g, void* hip_stream) { return a16w16_gemm_impl(g, hip_stream, true); }

static int a4w4_flat_impl(const a8w8_gemm_args* g, void* hip_stream, bool allow_dense);

static int a4w4_gemm_impl(const a8w8_gemm_args* g, void* hip_stream, bool allow_flat)
{
    if (!g) return A8W8_ERR_NULL_POINTER;
    // a skinny problem on shuffled weights: the flat kernel where it is the faster one (and can run it)
    if (allow_flat && g->b_preshuffled && g->m > 0 && g->m <= FLAT_MAX_M && prefer_flat(g->m, g->n, g->k / 2, false) &&
        a4w4_flat_impl(g, hip_stream, false) == A8W8_OK)
        return A8W8_OK;
    if (!g->a || !g->b || !g->c || !g->sfa || !g->sfb) return A8W8_ERR_NULL_POINTER;
    if (g->m <= 0 || g->n <= 0 || g->k <= 0 || g->batch <= 0) return A8W8_ERR_BAD_SHAPE;
    if (g->scale_mode != A8W8_SCALE_MX_E8M0_1x32 && g->scale_mode != A8W8_SCALE_MX_E8M0_TILED) return A8W8_ERR_BAD_MODE;
    if (g->c_dtype != A8W8_C_BF16 && g->c_dtype != A8W8_C_FP32) return A8W8_ERR_BAD_MODE;
    if (g->k % 32 != 0) return A8W8_ERR_BAD_GROUP;
    if (g->stride_c < g->n || g->stride_a < g->k || (!g->b_preshuffled && g->stride_b < g->k)) return A8W8_ERR_BAD_STRIDE;
    if ((g->stride_a & 1) || (!g->b_preshuffled && (g->stride_b & 1))) return A8W8_ERR_MISALIGNED;      // rows start on a byte
    const bool tiled = g->scale_mode == A8W8_SCALE_MX_E8M0_TILED;
    if (!tiled && (g->stride_sfa < g->k / 32 || g->stride_sfb < g->k / 32)) return A8W8_ERR_BAD_STRIDE;
    if (g->batch > 1 && ((g->stride_a_batch & 1) || (g->stride_b_batch & 1))) return A8W8_ERR_MISALIGNED;
    if (g->batch > 1 && (g->stride_a_batch < 0 || g->stride_b_batch < 0 || g->stride_c_batch < 0 ||
                         g->stride_sfa_batch < 0 || g->stride_sfb_batch < 0))
        return A8W8_ERR_BAD_STRIDE;
    const long long a_span = ((long long)(g->m - 1) * g->stride_a + g->k) / 2;
    const long long b_span = (g->b_preshuffled ? (long long)g->n * g->k : (long long)(g->n - 1) * g->stride_b + g->k) / 2;
    if (a_span >= (1ll << 31) || b_span >= (1ll << 31) || g->batch > 65535) return A8W8_ERR_TOO_LARGE;
    // the tiled kernel reads packed rows as byte rows of k/2 columns
    a8w8_gemm_args bytes = *g;
    bytes.k = g->k / 2;
    bytes.stride_a = g->stride_a / 2; bytes.stride_b = g->b_preshuffled ? bytes.k : g->stride_b / 2;
    bytes.stride_a_batch = g->stride_a_batch / 2; bytes.stride_b_batch = g->stride_b_batch / 2;
    bytes.scale_mode = A8W8_SCALE_MX_E8M0_TILED;
    const bool flat_rows = tiled && flat_rowmajor_ok(&bytes) && prefer_flat(g->m, g->n, bytes.k, false, bytes.stride_b % 4096 == 0 ? 1.3 : 1.05);
    if (!flat_rows && tiled && g->k % 256 == 0 && c_stride_too_large(g, &bytes)) return A8W8_ERR_TOO_LARGE;
    if (const int ds = device_status(); ds != A8W8_OK) return ds;
    hipStream_t s = (hipStream_t)hip_stream;
    // a skinny problem on row-major weights: the flat kernel where it is the faster one
    if (flat_rows) {
        const GemmParams p = make_params(&bytes);
        return g->c_dtype == A8W8_C_BF16 ? launch_flat<C_BF16, MODE_F4T, true>(p, g->batch, s)
                                         : launch_flat<C_FP32, MODE_F4T, true>(p, g->batch, s);
    }
    // weights shuffled as bytes (a4w4_flatmm's): MFMA kernels only
    if (g->b_preshuffled && (!tiled || g->k % 256 != 0 || validate_shuffled_b(&bytes) != A8W8_OK ||
                             (!small_ok(&bytes) && !persist_ok(&bytes))))
        return A8W8_ERR_BAD_GROUP;
    // row-major scales: the 128-tile kernel at any size (it stages the step's eight scale bytes per row as two dwords:
    // scale rows have to start on dwords)
    if (!tiled && !g->b_preshuffled && g->k % 256 == 0) {
        a8w8_gemm_args rows = bytes;
        rows.scale_mode = A8W8_SCALE_MX_E8M0_1x32;      // what tiled_ok checks the scale strides and pointers against
        if (tiled_ok(&rows) && (long long)((g->m + SM_BM - 1) / SM_BM) * ((g->n + 63) / 64) < (1ll << 31)) {
            const GemmParams p = make_params(&bytes);
            return g->c_dtype == A8W8_C_BF16 ? launch_small<MODE_F4, C_BF16>(p, g->batch, s)
                                             : launch_small<MODE_F4, C_FP32>(p, g->batch, s);
        }
    }
    if (tiled && g->k % 256 == 0 && tiled_ok(&bytes)) {
        const GemmParams p = make_params(&bytes);
        if (small_ok(&bytes))       // few tiles, or an odd number of 128-byte K steps
            return g->c_dtype == A8W8_C_BF16 ? launch_small<MODE_F4T, C_BF16>(p, g->batch, s)
                                             : launch_small<MODE_F4T, C_FP32>(p, g->batch, s);
        if (persist_ok(&bytes))
            return g->c_dtype == A8W8_C_BF16 ? launch_wide<MODE_F4T, C_BF16>(p, g->batch, s)
                                             : launch_wide<MODE_F4T, C_FP32>(p, g->batch, s);
    }
    dim3 grid((unsigned)((g->n + 15) / 16), (unsigned)((g->m + 15) / 16), (unsigned)g->batch);
#define A4W4_GENERAL(CDT, TILED)                                                                                        \
    A8W8_LAUNCH_OR_RETURN((gemm_a4w4_general<CDT, TILED>), grid, dim3(256), 0, s, (const uint8_t*)g->a, (const uint8_t*)g->b, \
                       (const uint8_t*)g->sfa, (const uint8_t*)g->sfb, g->c, g->m, g->n, g->k, g->stride_a / 2,            \
                       g->stride_b / 2, g->stride_c, g->stride_sfa, g->stride_sfb, (long long)g->stride_a_batch / 2,       \
                       (long long)g->stride_b_batch / 2, (long long)g->stride_c_batch, (long long)g->stride_sfa_batch,     \
                       (long long)g->stride_sfb_batch)
    if (g->c_dtype == A8W8_C_BF16) { if (tiled) A4W4_GENERAL(C_BF16, true); else A4W4_GENERAL(C_BF16, false); }
    else { if (tiled) A4W4_GENERAL(C_FP32, true); else A4W4_GENERAL(C_FP32, false); }
#undef A4W4_GENERAL
    return A8W8_OK;
}

int a4w4_gemm(const a8w8_gemm_args* g, void* hip_stream) { return a4w4_gemm_impl(g, hip_stream, true); }

static int a4w4_flat_impl(const a8w8_gemm_args* g, void* hip_stream, bool allow_dense)
{
    if (!g) return A8W8_ERR_NULL_POINTER;
    if (!g->a || !g->b || !g->c || !g->sfa || !g->sfb) return A8W8_ERR_NULL_POINTER;
    if (!g->b_preshuffled || g->scale_mode != A8W8_SCALE_MX_E8M0_TILED) return A8W8_ERR_BAD_MODE;
    if (g->m <= 0 || g->n <= 0 || g->k <= 0 || g->batch <= 0 || g->m > FLAT_MAX_M) return A8W8_ERR_BAD_SHAPE;
    if (g->c_dtype != A8W8_C_BF16 && g->c_dtype != A8W8_C_FP32) return A8W8_ERR_BAD_MODE;
    if (g->n % 16 != 0 || g->k % 128 != 0) return A8W8_ERR_BAD_GROUP;
    if (g->stride_c < g->n || g->stride_a < g->k) return A8W8_ERR_BAD_STRIDE;
    if (g->batch > 1 && (g->stride_a_batch < 0 || g->stride_b_batch < 0 || g->stride_c_batch < 0 ||
                         g->stride_sfa_batch < 0 || g->stride_sfb_batch < 0))
        return A8W8_ERR_BAD_STRIDE;
    if (!aligned16(g->a) || !aligned16(g->b) || !aligned16(g->sfa) || !aligned16(g->sfb) || g->stride_a % 32 != 0)
        return A8W8_ERR_MISALIGNED;
    if (g->batch > 1 && (g->stride_a_batch % 32 != 0 || g->stride_b_batch % 32 != 0 || g->stride_sfa_batch % 16 != 0 ||
                         g->stride_sfb_batch % 16 != 0))
        return A8W8_ERR_MISALIGNED;
    if ((long long)g->n * g->k / 2 >= (1ll << 31) || g->batch > 65535) return A8W8_ERR_TOO_LARGE;
    if (const int ds = device_status(); ds != A8W8_OK) return ds;
    // several groups of 16 rows over weights too large to stay in cache: the MFMA kernels read the same weights
    if (allow_dense && !prefer_flat(g->m, g->n, g->k / 2, false) && a4w4_gemm_impl(g, hip_stream, false) == A8W8_OK)
        return A8W8_OK;
    a8w8_gemm_args bytes = *g;      // packed rows as byte rows of k/2 columns
    bytes.k = g->k / 2;
    bytes.stride_a = g->stride_a / 2; bytes.stride_b = g->k / 2;
    bytes.stride_a_batch = g->stride_a_batch / 2; bytes.stride_b_batch = g->stride_b_batch / 2;
    const GemmParams p = make_params(&bytes);
    hipStream_t s = (hipStream_t)hip_stream;
    return g->c_dtype == A8W8_C_BF16 ? launch_flat<C_BF16, MODE_F4T>(p, g->batch, s) : launch_flat<C_FP32, MODE_F4T>(p, g->batch, s);
}

int a4w4_flatmm(const a8w8_gemm_args* g, void* hip_stream) { return a4w4_flat_impl(g, hip_stream, true); }

// the vectorised quantisers read 16 bytes per lane and write packed words
static bool quant_vec_ok(const float* src, int rows, int k, int ld, const uint8_t* q, int q_align)
{
    return aligned16(src) && ld % 4 == 0 && k % 4 == 0 && ((uintptr_t)q & (uintptr_t)(q_align - 1)) == 0 &&
           (long long)rows * k < (1ll << 31);
}

int a4w4_quantize_mx(const float* src, int rows, int k, int ld, uint8_t* q, uint8_t* scale, int tiled, void* hip_stream)
{
    if (!src || !q || !scale) return A8W8_ERR_NULL_POINTER;
    if (rows <= 0 || k <= 0) return A8W8_ERR_BAD_SHAPE;
    if (k % 32 != 0) return A8W8_ERR_BAD_GROUP;
    if (ld < k) return A8W8_ERR_BAD_STRIDE;
    if (tiled && ((uintptr_t)scale & 3)) return A8W8_ERR_MISALIGNED;
    if (const int ds = device_status(); ds != A8W8_OK) return ds;
    hipStream_t s = (hipStream_t)hip_stream;
    const long long threads = (long long)rows * k;
    if (tiled) {
        if (rows % 64 != 0 || k % 512 != 0) {
            const size_t dwords = mx_tiled_bytes(rows, k) / 4;
            A8W8_LAUNCH_OR_RETURN(mx_tiled_fill_kernel, dim3((unsigned)((dwords + 255) / 256)), dim3(256), 0, s, (uint32_t*)scale, dwords);
        }
        if (quant_vec_ok(src, rows, k, ld, q, 4))
            A8W8_LAUNCH_OR_RETURN(quant_mxfp4_vec_kernel<true>, dim3((unsigned)((threads / 8 + 255) / 256)), dim3(256), 0, s, src, rows, k, ld, q, scale);
        else
            A8W8_LAUNCH_OR_RETURN(quant_mxfp4_kernel<true>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, src, rows, k, ld, q, scale);
    } else {
        if (quant_vec_ok(src, rows, k, ld, q, 4))
            A8W8_LAUNCH_OR_RETURN(quant_mxfp4_vec_kernel<false>, dim3((unsigned)((threads / 8 + 255) / 256)), dim3(256), 0, s, src, rows, k, ld, q, scale);
        else
            A8W8_LAUNCH_OR_RETURN(quant_mxfp4_kernel<false>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, src, rows, k, ld, q, scale);
    }
    return A8W8_OK;
}

static int a16w16_flat_impl(const a8w8_gemm_args* g, void* hip_stream, bool allow_dense)
{
    if (!g) return A8W8_ERR_NULL_POINTER;
    if (!g->a || !g->b || !g->c) return A8W8_ERR_NULL_POINTER;
    if (!g->b_preshuffled) return A8W8_ERR_BAD_MODE;
    if (g->m <= 0 || g->n <= 0 || g->k <= 0 || g->batch <= 0 || g->m > FLAT_MAX_M) return A8W8_ERR_BAD_SHAPE;
    if (g->c_dtype != A8W8_C_BF16 && g->c_dtype != A8W8_C_FP32) return A8W8_ERR_BAD_MODE;
    if (g->n % 16 != 0 || g->k % 32 != 0) return A8W8_ERR_BAD_GROUP;
    if (g->stride_c < g->n || g->stride_a < g->k) return A8W8_ERR_BAD_STRIDE;
    if (!aligned16(g->a) || !aligned16(g->b) || g->stride_a % 8 != 0) return A8W8_ERR_MISALIGNED;
    if (g->batch > 1 && (g->stride_a_batch % 8 != 0 || g->stride_b_batch % 8 != 0)) return A8W8_ERR_MISALIGNED;
    if ((long long)g->n * g->k * 2 >= (1ll << 31) || g->batch > 65535) return A8W8_ERR_TOO_LARGE;
    // batch strides are doubled into byte counts held in an int
    if (g->batch > 1 && ((long long)g->stride_a_batch * 2 >= (1ll << 31) || (long long)g->stride_b_batch * 2 >= (1ll << 31)))
        return A8W8_ERR_TOO_LARGE;
    if (const int ds = device_status(); ds != A8W8_OK) return ds;
    // several groups of 16 rows over weights too large to stay in cache: the MFMA kernels read the same weights
    if (allow_dense && !prefer_flat(g->m, g->n, 2ll * g->k, false) && a16w16_gemm_impl(g, hip_stream, false) == A8W8_OK)
        return A8W8_OK;
    a8w8_gemm_args bytes = *g;      // bf16 rows as byte rows of 2k columns
    bytes.k = g->k * 2;
    bytes.stride_a = g->stride_a * 2; bytes.stride_b = g->k * 2;
    bytes.stride_a_batch = g->stride_a_batch * 2; bytes.stride_b_batch = g->stride_b_batch * 2;
    GemmParams p = make_params(&bytes);
    p.sfa = p.sfb = nullptr;
    hipStream_t s = (hipStream_t)hip_stream;
    return g->c_dtype == A8W8_C_BF16 ? launch_flat<C_BF16, MODE_BF16>(p, g->batch, s)
                                     : launch_flat<C_FP32, MODE_BF16>(p, g->batch, s);
}

int a16w16_flatmm(const a8w8_gemm_args* g, void* hip_stream) { return a16w16_flat_impl(g, hip_stream, true); }

int a8w8_gemm_blockscale(const a8w8_gemm_args* g, void* hip_stream)
{
    if (!g) return A8W8_ERR_NULL_POINTER;
    a8w8_gemm_args local = *g;
    local.scale_mode = A8W8_SCALE_BLOCK_1x128_128x128;
    return a8w8_gemm(&local, hip_stream);
}

int a8w8_flatmm(const a8w8_gemm_args* g, void* hip_stream)
{
    const int st = validate_flat(g);
    if (st != A8W8_OK) return st;
    if (const int ds = device_status(); ds != A8W8_OK) return ds;
    hipStream_t s = (hipStream_t)hip_stream;
    // several groups of 16 rows over weights too large to stay in cache: the MFMA kernels read the same weights
    if (!prefer_flat_fp8(g)) {
        a8w8_gemm_args local = *g;
        local.stride_b = local.k;
        if (validate_shuffled_b(&local) == A8W8_OK) return launch_dense_fp8(&local, s);
    }
    return launch_flat_fp8(g, s);
}

static size_t shuffled_index(int j, int p, int k)
{
    return (((size_t)(j / 16) * (k / 64) + p / 64) * 4 + (p % 64) / 16) * 256 + (size_t)(j % 16) * 16 + p % 16;
}

int a8w8_preshuffle_b(const void* b_host, void* out_host, int n, int k)
{
    if (!b_host || !out_host) return A8W8_ERR_NULL_POINTER;
    if (n <= 0 || k <= 0) return A8W8_ERR_BAD_SHAPE;
    if (n % 16 != 0 || k % 64 != 0) return A8W8_ERR_BAD_GROUP;
    const uint8_t* b = (const uint8_t*)b_host;
    uint8_t* o = (uint8_t*)out_host;
    for (int j = 0; j < n; ++j)
        for (int p = 0; p < k; p += 16) memcpy(o + shuffled_index(j, p, k), b + (size_t)j * k + p, 16);
    return A8W8_OK;
}

int a8w8_unshuffle_b(const void* bshuf_host, void* out_host, int n, int k)
{
    if (!bshuf_host || !out_host) return A8W8_ERR_NULL_POINTER;
    if (n <= 0 || k <= 0) return A8W8_ERR_BAD_SHAPE;
    if (n % 16 != 0 || k % 64 != 0) return A8W8_ERR_BAD_GROUP;
    const uint8_t* s = (const uint8_t*)bshuf_host;
    uint8_t* o = (uint8_t*)out_host;
    for (int j = 0; j < n; ++j)
        for (int p = 0; p < k; p += 16) memcpy(o + (size_t)j * k + p, s + shuffled_index(j, p, k), 16);
    return A8W8_OK;
}

int a8w8_preshuffle_b_device(const void* b_dev, void* out_dev, int n, int k, void* hip_stream)
{
    if (!b_dev || !out_dev) return A8W8_ERR_NULL_POINTER;
    if (n <= 0 || k <= 0) return A8W8_ERR_BAD_SHAPE;
    if (n % 16 != 0 || k % 64 != 0) return A8W8_ERR_BAD_GROUP;
    if (!aligned16(out_dev)) return A8W8_ERR_MISALIGNED;
    if (const int ds = device_status(); ds != A8W8_OK) return ds;
    const long long units = (long long)n * k / 16;
    A8W8_LAUNCH_OR_RETURN(preshuffle_b_kernel, dim3((unsigned)((units + 255) / 256)), dim3(256), 0,
                       (hipStream_t)hip_stream, (const uint8_t*)b_dev, (uint8_t*)out_dev, n, k);
    return A8W8_OK;
}

int a8w8_cvt_f32_to_e4m3(const float* src, uint8_t* dst, size_t n, int dialect, int clamp240, void* hip_stream)
{
    if (dialect != A8W8_E4M3_OCP && dialect != A8W8_E4M3_FNUZ) return A8W8_ERR_BAD_MODE;
    if (n == 0) return A8W8_OK;
    if (!src || !dst) return A8W8_ERR_NULL_POINTER;
    if ((n + 3) / 4 > 0x7fffffffull * 256) return A8W8_ERR_TOO_LARGE;
    if (const int ds = device_status(); ds != A8W8_OK) return ds;
    hipStream_t s = (hipStream_t)hip_stream;
    const dim3 grid((unsigned)(((n + 3) / 4 + 255) / 256)), block(256);
    if (dialect == A8W8_E4M3_OCP)
        return clamp240 ? launch(cvt_f32_to_e4m3_kernel<0, 1>, grid, block, 0, s, src, dst, n)
                        : launch(cvt_f32_to_e4m3_kernel<0, 0>, grid, block, 0, s, src, dst, n);
    return clamp240 ? launch(cvt_f32_to_e4m3_kernel<1, 1>, grid, block, 0, s, src, dst, n)
                    : launch(cvt_f32_to_e4m3_kernel<1, 0>, grid, block, 0, s, src, dst, n);
}

int a8w8_cvt_e4m3_to_f32(const uint8_t* src, float* dst, size_t n, int dialect, void* hip_stream)
{
    if (dialect != A8W8_E4M3_OCP && dialect != A8W8_E4M3_FNUZ) return A8W8_ERR_BAD_MODE;
    if (n == 0) return A8W8_OK;
    if (!src || !dst) return A8W8_ERR_NULL_POINTER;
    if (n > 0x7fffffffull * 256) return A8W8_ERR_TOO_LARGE;
    if (const int ds = device_status(); ds != A8W8_OK) return ds;
    hipStream_t s = (hipStream_t)hip_stream;
    const dim3 grid((unsigned)((n + 255) / 256)), block(256);
    return dialect == A8W8_E4M3_OCP ? launch(cvt_e4m3_to_f32_kernel<0>, grid, block, 0, s, src, dst, n)
                                    : launch(cvt_e4m3_to_f32_kernel<1>, grid, block, 0, s, src, dst, n);
}

int a8w8_quantize(const float* src, int rows, int k, int ld, uint8_t* q, void* scale, int scale_mode, int group_rows,
                  void* hip_stream)
{
    if (!src || !q || !scale) return A8W8_ERR_NULL_POINTER;
    if (rows <= 0 || k <= 0) return A8W8_ERR_BAD_SHAPE;
    if (ld < k) return A8W8_ERR_BAD_STRIDE;
    hipStream_t s = (hipStream_t)hip_stream;
    switch (scale_mode) {
        case A8W8_SCALE_TENSOR: {
            if (const int ds = device_status(); ds != A8W8_OK) return ds;
            const long long total = (long long)rows * k;
            const unsigned grid = (unsigned)(total / 256 + 1 < 4096 ? total / 256 + 1 : 4096);
            A8W8_LAUNCH_OR_RETURN(quant_tensor_clear_kernel, dim3(1), dim3(1), 0, s, (float*)scale);
            if (ld == k && total % 4 == 0 && aligned16(src) && ((uintptr_t)q & 3) == 0) {
                const size_t units = (size_t)(total / 4);
                const unsigned vgrid = (unsigned)(units / 1024 + 1 < 2048 ? units / 1024 + 1 : 2048);
                A8W8_LAUNCH_OR_RETURN(quant_tensor_amax_vec_kernel, dim3(vgrid), dim3(256), 0, s, (const float4*)src, units, (float*)scale);
                A8W8_LAUNCH_OR_RETURN(quant_tensor_apply_vec_kernel, dim3(vgrid), dim3(256), 0, s, (const float4*)src, units, (uint32_t*)q,
                                   (const float*)scale);
            } else {
                A8W8_LAUNCH_OR_RETURN(quant_tensor_amax_kernel, dim3(grid), dim3(256), 0, s, src, rows, k, ld, (float*)scale);
                A8W8_LAUNCH_OR_RETURN(quant_tensor_apply_kernel, dim3(grid), dim3(256), 0, s, src, rows, k, ld, q, (const float*)scale);
            }
            A8W8_LAUNCH_OR_RETURN(quant_tensor_finish_kernel, dim3(1), dim3(1), 0, s, (float*)scale);
            return A8W8_OK;
        }
        case A8W8_SCALE_ROWCOL:
            if (const int ds = device_status(); ds != A8W8_OK) return ds;
            if (quant_vec_ok(src, rows, k, ld, q, 4) && k <= 8192)
                A8W8_LAUNCH_OR_RETURN(quant_rowwise_vec_kernel<true>, dim3((unsigned)rows), dim3(256), 0, s, src, k, ld, q, (float*)scale);
            else if (quant_vec_ok(src, rows, k, ld, q, 4))
                A8W8_LAUNCH_OR_RETURN(quant_rowwise_vec_kernel<false>, dim3((unsigned)rows), dim3(256), 0, s, src, k, ld, q, (float*)scale);
            else
                A8W8_LAUNCH_OR_RETURN(quant_rowwise_kernel, dim3((unsigned)rows), dim3(256), 0, s, src, k, ld, q, (float*)scale);
            return A8W8_OK;
        case A8W8_SCALE_BLOCK_1x128_128x128:
            if (k % 128 != 0) return A8W8_ERR_BAD_GROUP;
            if (group_rows == 1) {
                if (const int ds = device_status(); ds != A8W8_OK) return ds;
                const long long waves = (long long)rows * (k / 128);
                if (quant_vec_ok(src, rows, k, ld, q, 4))
                    A8W8_LAUNCH_OR_RETURN(quant_1x128_vec_kernel, dim3((unsigned)((waves + 8 * QUANT_1X128_GROUPS - 1) / (8 * QUANT_1X128_GROUPS))), dim3(256), 0, s, src, rows, k, ld, q,
                                       (float*)scale);
                else
                    A8W8_LAUNCH_OR_RETURN(quant_1x128_kernel, dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, s, src, rows, k,
                                       ld, q, (float*)scale);
                return A8W8_OK;
            }
            if (group_rows == 128) {
                if (rows % 128 != 0) return A8W8_ERR_BAD_GROUP;
                if (const int ds = device_status(); ds != A8W8_OK) return ds;
                A8W8_LAUNCH_OR_RETURN(quant_128x128_kernel, dim3((unsigned)(k / 128), (unsigned)(rows / 128)), dim3(256), 0,
                                   s, src, k, ld, q, (float*)scale);
                return A8W8_OK;
            }
            return A8W8_ERR_BAD_MODE;
        case A8W8_SCALE_MX_E8M0_1x32: {
            if (k % 32 != 0) return A8W8_ERR_BAD_GROUP;
            if (const int ds = device_status(); ds != A8W8_OK) return ds;
            const long long threads = (long long)rows * k;
            if (quant_vec_ok(src, rows, k, ld, q, 4))
                A8W8_LAUNCH_OR_RETURN(quant_mx_vec_kernel<false>, dim3((unsigned)((threads / (4 * QUANT_MX_CHUNKS) + 255) / 256)), dim3(256), 0, s, src,
                                   rows, k, ld, q, (uint8_t*)scale);
            else
                A8W8_LAUNCH_OR_RETURN(quant_mx_kernel<false>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, src, rows, k,
                                   ld, q, (uint8_t*)scale);
            return A8W8_OK;
        }
        case A8W8_SCALE_MX_E8M0_TILED: {
            if (k % 32 != 0) return A8W8_ERR_BAD_GROUP;
            if (const int ds = device_status(); ds != A8W8_OK) return ds;
            if (((uintptr_t)scale & 3) != 0) return A8W8_ERR_MISALIGNED;
            const long long threads = (long long)rows * k;
            if (rows % 64 != 0 || k % 512 != 0) {   // positions no (row, block) owns: 127 first
                const size_t dwords = mx_tiled_bytes(rows, k) / 4;
                A8W8_LAUNCH_OR_RETURN(mx_tiled_fill_kernel, dim3((unsigned)((dwords + 255) / 256)), dim3(256), 0, s,
                                   (uint32_t*)scale, dwords);
            }
            if (quant_vec_ok(src, rows, k, ld, q, 4))
                A8W8_LAUNCH_OR_RETURN(quant_mx_vec_kernel<true>, dim3((unsigned)((threads / (4 * QUANT_MX_CHUNKS) + 255) / 256)), dim3(256), 0, s, src,
                                   rows, k, ld, q, (uint8_t*)scale);
            else
                A8W8_LAUNCH_OR_RETURN(quant_mx_kernel<true>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, src, rows,
                                   k, ld, q, (uint8_t*)scale);
            return A8W8_OK;
        }
        default:
            return A8W8_ERR_BAD_MODE;
    }
}

int a8w8_mx_tile_scales(const uint8_t* sf, int rows, int k, int stride, uint8_t* out, void* hip_stream)
{
    if (!sf || !out) return A8W8_ERR_NULL_POINTER;
    if (rows <= 0 || k <= 0) return A8W8_ERR_BAD_SHAPE;
    if (k % 32 != 0) return A8W8_ERR_BAD_GROUP;
    if (stride < k / 32) return A8W8_ERR_BAD_STRIDE;
    if (!aligned16(out)) return A8W8_ERR_MISALIGNED;
    if (const int ds = device_status(); ds != A8W8_OK) return ds;
    const size_t units = mx_tiled_bytes(rows, k) >> 10;
    A8W8_LAUNCH_OR_RETURN(mx_tile_scales_kernel, dim3((unsigned)((units + 3) / 4)), dim3(256), 0,
                       (hipStream_t)hip_stream, sf, rows, stride, out, (const uint8_t*)nullptr, 0, 0, (uint8_t*)nullptr, k);
    return A8W8_OK;
}

int a8w8_mx_tile_scales_ab(const uint8_t* sfa, int m, int stride_sfa, uint8_t* out_a, const uint8_t* sfb, int n,
                           int stride_sfb, uint8_t* out_b, int k, void* hip_stream)
{
    if (!sfa || !out_a || !sfb || !out_b) return A8W8_ERR_NULL_POINTER;
    if (m <= 0 || n <= 0 || k <= 0) return A8W8_ERR_BAD_SHAPE;
    if (k % 32 != 0) return A8W8_ERR_BAD_GROUP;
    if (stride_sfa < k / 32 || stride_sfb < k / 32) return A8W8_ERR_BAD_STRIDE;
    if (!aligned16(out_a) || !aligned16(out_b)) return A8W8_ERR_MISALIGNED;
    if (const int ds = device_status(); ds != A8W8_OK) return ds;
    const size_t units0 = mx_tiled_bytes(m, k) >> 10, units1 = mx_tiled_bytes(n, k) >> 10;
    A8W8_LAUNCH_OR_RETURN(mx_tile_scales_kernel, dim3((unsigned)((units0 + units1 + 3) / 4)), dim3(256), 0,
                       (hipStream_t)hip_stream, sfa, m, stride_sfa, out_a, sfb, n, stride_sfb, out_b, k);
    return A8W8_OK;
}

size_t a8w8_mx_tiled_bytes(int rows, int k)
{
    if (rows <= 0 || k <= 0) return 0;
    return mx_tiled_bytes(rows, k);
}

// ------------------------------------------------------------ weight files (host only)
namespace {
const char kWeightMagic[8] = {'A', '8', 'W', '8', 'W', 'G', 'T', 0};

uint64_t fnv1a64(const void* data, size_t n, uint64_t h)
{
    const uint8_t* p = (const uint8_t*)data;
    for (size_t i = 0; i < n; ++i) { h ^= p[i]; h *= 1099511628211ull; }
    return h;
}

int check_header(const a8w8_weight_header& h)
{
    if (memcmp(h.magic, kWeightMagic, 8) != 0 || h.version != 1) return A8W8_ERR_BAD_FILE;
    if (h.n == 0 || h.k == 0 || h.n > (1u << 30) || h.k > (1u << 30)) return A8W8_ERR_BAD_FILE;
    if (h.b_bytes != (uint64_t)h.n * h.k) return A8W8_ERR_BAD_FILE;
    if (h.scale_bytes == 0 || h.scale_bytes != a8w8_weight_scale_bytes((int)h.n, (int)h.k, (int)h.scale_mode))
        return A8W8_ERR_BAD_FILE;
    return A8W8_OK;
}
}  // namespace

size_t a8w8_weight_scale_bytes(int n, int k, int scale_mode)
{
    if (n <= 0 || k <= 0) return 0;
    switch (scale_mode) {
        case A8W8_SCALE_TENSOR: return 4;
        case A8W8_SCALE_ROWCOL: return (size_t)n * 4;
        case A8W8_SCALE_BLOCK_1x128_128x128: return (n % 128 || k % 128) ? 0 : (size_t)(n / 128) * (k / 128) * 4;
        case A8W8_SCALE_MX_E8M0_1x32: return k % 32 ? 0 : (size_t)n * (k / 32);
        case A8W8_SCALE_MX_E8M0_TILED: return k % 32 ? 0 : mx_tiled_bytes(n, k);
        default: return 0;
    }
}

int a8w8_weights_save(const char* path, const void* b_host, const void* scale_host, int n, int k, int b_preshuffled,
                      int scale_mode)
{
    if (!path || !b_host || !scale_host) return A8W8_ERR_NULL_POINTER;
    if (n <= 0 || k <= 0) return A8W8_ERR_BAD_SHAPE;
    if (b_preshuffled && (n % 16 != 0 || k % 64 != 0)) return A8W8_ERR_BAD_GROUP;
    const size_t sbytes = a8w8_weight_scale_bytes(n, k, scale_mode);
    if (sbytes == 0) return scale_mode < 0 || scale_mode > A8W8_SCALE_MX_E8M0_TILED ? A8W8_ERR_BAD_MODE : A8W8_ERR_BAD_GROUP;
    a8w8_weight_header h;
    memset(&h, 0, sizeof h);
    memcpy(h.magic, kWeightMagic, 8);
    h.version = 1;
    h.n = (uint32_t)n; h.k = (uint32_t)k;
    h.b_preshuffled = b_preshuffled ? 1 : 0;
    h.scale_mode = (uint32_t)scale_mode;
    h.b_bytes = (uint64_t)n * k;
    h.scale_bytes = sbytes;
    h.checksum = fnv1a64(scale_host, sbytes, fnv1a64(b_host, (size_t)h.b_bytes, 14695981039346656037ull));
    FILE* f = fopen(path, "wb");
    if (!f) return A8W8_ERR_IO;
    const bool ok = fwrite(&h, sizeof h, 1, f) == 1 && fwrite(b_host, 1, (size_t)h.b_bytes, f) == h.b_bytes &&
                    fwrite(scale_host, 1, sbytes, f) == sbytes;
    return (fclose(f) == 0 && ok) ? A8W8_OK : A8W8_ERR_IO;
}

int a8w8_weights_info(const char* path, a8w8_weight_header* out)
{
    if (!path || !out) return A8W8_ERR_NULL_POINTER;
    FILE* f = fopen(path, "rb");
    if (!f) return A8W8_ERR_IO;
    const size_t got = fread(out, 1, sizeof *out, f);
    fclose(f);
    if (got != sizeof *out) return A8W8_ERR_BAD_FILE;
    return check_header(*out);
}

int a8w8_weights_load(const char* path, void* b_host, size_t b_capacity, void* scale_host, size_t scale_capacity)
{
    if (!path || !b_host || !scale_host) return A8W8_ERR_NULL_POINTER;
    FILE* f = fopen(path, "rb");
    if (!f) return A8W8_ERR_IO;
    a8w8_weight_header h;
    int st = fread(&h, 1, sizeof h, f) == sizeof h ? check_header(h) : A8W8_ERR_BAD_FILE;
    if (st == A8W8_OK && (h.b_bytes > b_capacity || h.scale_bytes > scale_capacity)) st = A8W8_ERR_BAD_STRIDE;
    if (st == A8W8_OK && (fread(b_host, 1, (size_t)h.b_bytes, f) != h.b_bytes ||
                          fread(scale_host, 1, (size_t)h.scale_bytes, f) != h.scale_bytes))
        st = A8W8_ERR_BAD_FILE;
    fclose(f);
    if (st != A8W8_OK) return st;
    const uint64_t sum = fnv1a64(scale_host, (size_t)h.scale_bytes, fnv1a64(b_host, (size_t)h.b_bytes, 14695981039346656037ull));
    return sum == h.checksum ? A8W8_OK : A8W8_ERR_BAD_FILE;
}

const char* a8w8_status_string(int status)
{
    switch (status) {
        case A8W8_OK: return "ok";
        case A8W8_ERR_NULL_POINTER: return "null pointer";
        case A8W8_ERR_BAD_SHAPE: return "m, n, k and batch must be positive (and m <= 128 for the flat GEMMs)";
        case A8W8_ERR_BAD_GROUP: return "m/n/k must be multiples of the scale group (or of the shuffle tile)";
        case A8W8_ERR_BAD_STRIDE: return "a stride is smaller than the extent it spans";
        case A8W8_ERR_MISALIGNED: return "pointer or stride not 16-byte aligned";
        case A8W8_ERR_BAD_MODE: return "unsupported scale mode, output type or layout flag";
        case A8W8_ERR_TOO_LARGE: return "matrix too large for 32-bit offsets";
        case A8W8_ERR_LAUNCH: return "kernel launch failed";
        case A8W8_ERR_NO_DEVICE: return "current device is not gfx950";
        case A8W8_ERR_IO: return "weight file could not be opened, read or written";
        case A8W8_ERR_BAD_FILE: return "not a weight file of this version, truncated, or checksum mismatch";
        default: return "unknown status";
    }
}

const char* a8w8_kernel_name(const a8w8_gemm_args* g)
{
    if (!g) return nullptr;
    // shuffled weights: a8w8_gemm and a8w8_flatmm both pick the flat kernel for skinny problems it runs faster
    a8w8_gemm_args local = *g;
    if (local.b_preshuffled) local.stride_b = local.k;
    g = &local;
    const bool dense_ok = validate_common(g) == A8W8_OK && validate_shuffled_b(g) == A8W8_OK;
    if (g->b_preshuffled && validate_flat(g) == A8W8_OK && (prefer_flat_fp8(g) || !dense_ok)) return "flatmm_a8w8";
    if (dense_ok && flat_rowmajor_ok(g) && prefer_flat_fp8(g)) return "flatmm_a8w8";
    if (!dense_ok) return nullptr;
    if (!tiled_ok(g)) return "gemm_a8w8_general";
    if (small_ok(g)) return "gemm_a8w8_tile128";
    if (wide_ok(g)) return "gemm_a8w8_wide";
    return persist_ok(g) ? "gemm_a8w8_persist" : "gemm_a8w8_tile128";
}

int a8w8_hbm_read_probe(const void* src, size_t bytes, void* sink, void* hip_stream)
{
    if (!src || !sink) return A8W8_ERR_NULL_POINTER;
    if (bytes == 0) return A8W8_ERR_BAD_SHAPE;
    if (bytes % 16 != 0 || !aligned16(src) || ((uintptr_t)sink & 3)) return A8W8_ERR_MISALIGNED;
    if (const int ds = device_status(); ds != A8W8_OK) return ds;
    const size_t n16 = bytes / 16;
    // eight workgroups per compute unit (the best of the grids tried on a 117 MB buffer), fewer for buffers that do not
    // give every thread a load
    const size_t want = (n16 + HBM_PROBE_THREADS - 1) / HBM_PROBE_THREADS;
    const size_t most = (size_t)num_cus() * 8;
    const unsigned grid = (unsigned)(want < most ? want : most);
    return launch(hbm_read_probe_kernel, dim3(grid), dim3(HBM_PROBE_THREADS), 0, (hipStream_t)hip_stream, (const v4i*)src, n16,
                  (int*)sink);
}

int a8w8_route_override(int choice)
{
    if (choice != A8W8_ROUTE_MODEL && choice != A8W8_ROUTE_FLAT && choice != A8W8_ROUTE_DENSE) return A8W8_ERR_BAD_MODE;
    const int before = g_route;
    g_route = choice;
    return before;
}

int a8w8_init(int device)
{
    int current = 0;
    if (hipGetDevice(&current) != hipSuccess) return A8W8_ERR_NO_DEVICE;
    if (device < 0) device = current;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || device >= count || device >= MAX_DEVICES) return A8W8_ERR_NO_DEVICE;
    if (device != current && hipSetDevice(device) != hipSuccess) {
        (void)hipGetLastError();      // the failed switch must not linger as the thread's last error
        return A8W8_ERR_NO_DEVICE;
    }
    const int st = device_status();
    if (device != current) (void)hipSetDevice(current);
    return st;
}

// An ablated build (measurement switches of gemm_wide.hpp) reports a negative version, so that nothing mistakes it
// for the library.
int a8w8_version(void) { return A8W8_ABLATED ? -300 : 300; }

}  // extern "C"
