// Version / status strings and the VALU calibration kernel.
#include "ds_common.h"
#include <atomic>
#include <string>

namespace ds {

// A dependency-free stream of the two instructions one shift-add term costs (v_ashrrev_i32 then
// v_xad_u32) with wave-uniform shift amounts and sign masks, i.e. the instruction mix of
// shift_kernel with nothing else in the way.  16 accumulators x 4 activations = 64 pairs per
// iteration and lane.
__global__ __launch_bounds__(256) void valu_calibrate_kernel(int32_t *sink, int iters, uint32_t seed)
{
    int32_t acc[16][4];
    int32_t xv[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) xv[r] = (int32_t)(threadIdx.x * 2654435761u + r * 40503u + blockIdx.x);
#pragma unroll
    for (int j = 0; j < 16; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[j][r] = j + r;
    uint32_t w = seed;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const uint32_t s = (w >> j) & 31u;
            const int32_t mask = -(int32_t)((w >> (j + 8)) & 1u);
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[j][r] = ((xv[r] >> s) ^ mask) + acc[j][r];
        }
        w = w * 1664525u + 1013904223u;
    }
    int32_t total = 0;
#pragma unroll
    for (int j = 0; j < 16; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) total += acc[j][r];
    sink[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = total;
}

Tune g_tune;

int device_cus()
{
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n > 0) return n;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) n = 256;
    cached[dev].store(n, std::memory_order_relaxed);
    return n;
}

}  // namespace ds

using namespace ds;

DS_EXPORT int ds_test_tune(const char *knob, int value)
{
    if (!knob) {
        g_tune.reset();
        chain_test_knobs(-1, -1);
        return DS_OK;
    }
    const std::string k(knob);
    if (k == "planes") g_tune.planes = value;
    else if (k == "split") g_tune.split = value;
    else if (k == "tile") g_tune.tile = value;
    else if (k == "cu") g_tune.cu = value;
    else if (k == "notail") g_tune.notail = value;
    else if (k == "wide") g_tune.wide = value;
    else if (k == "perm") g_tune.perm = value;
    else if (k == "chain_spin_us") { g_tune.chain_spin_us = value; chain_test_knobs(g_tune.chain_spin_us, g_tune.chain_extra); }
    else if (k == "chain_extra") { g_tune.chain_extra = value; chain_test_knobs(g_tune.chain_spin_us, g_tune.chain_extra); }
    else return DS_EINVAL;
    return DS_OK;
}

__global__ void fast_div_kernel(const uint32_t *n, uint32_t *q, long count, ds::FastDiv f, int uniform_form)
{
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    q[i] = uniform_form ? ds::div_by_uniform(n[i], f) : ds::div_by(n[i], f);
}

DS_EXPORT int ds_test_fast_div(const unsigned int *n, unsigned int *q, long count, unsigned int d, int uniform_form,
                               ds_stream_t stream)
{
    if (count < 0 || d < 1 || (count > 0 && (!n || !q))) return DS_EINVAL;
    if (count == 0) return DS_OK;
    const long blocks = (count + 255) / 256;
    if (blocks > 0x7fffffffL) return DS_ETOOLARGE;
    hipLaunchKernelGGL(fast_div_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, n, q, count,
                       ds::fast_div(d), uniform_form);
    return ds::launch_status();
}

DS_EXPORT int ds_version(void) { return 100; }

DS_EXPORT const char *ds_status_string(int status)
{
    switch (status) {
    case DS_OK: return "ok";
    case DS_EINVAL: return "invalid argument (null pointer, negative or inconsistent size)";
    case DS_EBITS: return "unsupported bits (1..6 supported)";
    case DS_EBASE: return "unsupported base (must be in -31..0)";
    case DS_EWORKSPACE: return "workspace missing or too small";
    case DS_ETOOLARGE: return "tensor too large for 32-bit offsets";
    case DS_ESCRATCH: return "problem needs more than the built-in scratch of the allocation-free entry point";
    default: break;
    }
    if (status <= DS_EHIP) return hipGetErrorString((hipError_t)(DS_EHIP - status));
    return "unknown status";
}

DS_EXPORT int ds_valu_calibrate(int32_t *sink, int blocks, int iters, ds_stream_t stream)
{
    if (!sink || blocks < 1 || iters < 0) return DS_EINVAL;
    hipLaunchKernelGGL(valu_calibrate_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, sink,
                       iters, 0x9E3779B9u);
    return launch_status();
}
