// Machine probes behind the figures that the design of the tile-sparse kernels rests on: what a
// kernel boundary costs, and how fast one compute unit takes bytes in.  Not part of the drop-in
// boundary (declared in et_tuning.h); scpaper-2021_amd/kernel_bench.py --set machine times them.
#include "common.hip.h"
#include "../../include/et_tuning.h"

namespace et {

__global__ void probe_empty_kernel(uint32_t *sink) {
    if (sink == nullptr && threadIdx.x == 12345) *reinterpret_cast<volatile uint32_t *>(sink) = 0;  // never taken
}

// Every workgroup requests `vec_per_thread` 16-byte vectors per thread — all of them before it uses
// the first — from its own region of src (shared == 0), or from the region of the first workgroup of
// its XCD (shared != 0: after the first touch the lines come from that XCD's L2), and adds them up.
template <int V> __global__ __launch_bounds__(1024) void probe_read_kernel(const uint4 *src, size_t vec_per_wg, int shared,
                                                                          uint32_t *sink) {
    const size_t wg = shared ? (blockIdx.x % 8) : blockIdx.x;
    const uint4 *p = src + wg * vec_per_wg;
    uint4 v[V];
#pragma unroll
    for (int k = 0; k < V; k++) v[k] = p[(size_t)k * blockDim.x + threadIdx.x];
    uint32_t s = 0;
#pragma unroll
    for (int k = 0; k < V; k++) s += v[k].x ^ v[k].y ^ v[k].z ^ v[k].w;
    if (s == 0x9e3779b9u) sink[blockIdx.x] = s;  // keeps the loads alive; practically never true
}

}  // namespace et

using namespace et;

extern "C" {

int et_probe_empty(int nwg, int threads, et_stream stream) {
    ET_REQUIRE(nwg > 0 && threads > 0 && threads <= 1024, ET_ERR_INVALID_ARG, "et_probe_empty: nwg=%d threads=%d", nwg, threads);
    probe_empty_kernel<<<nwg, threads, 0, as_stream(stream)>>>(nullptr);
    return check_launch("probe_empty_kernel");
}

int et_probe_read(const void *src, size_t src_bytes, int nwg, int threads, int vec_per_thread, int shared, uint32_t *sink,
                  et_stream stream) {
    ET_REQUIRE(src && sink && nwg > 0 && threads > 0 && threads <= 1024 && threads % 64 == 0, ET_ERR_INVALID_ARG,
               "et_probe_read: bad arguments");
    const size_t vec_per_wg = (size_t)vec_per_thread * threads;
    ET_REQUIRE((size_t)(shared ? 8 : nwg) * vec_per_wg * 16 <= src_bytes, ET_ERR_INVALID_ARG, "et_probe_read: src holds %zu bytes",
               src_bytes);
    const uint4 *s = static_cast<const uint4 *>(src);
    hipStream_t st = as_stream(stream);
    switch (vec_per_thread) {
        case 4: probe_read_kernel<4><<<nwg, threads, 0, st>>>(s, vec_per_wg, shared, sink); break;
        case 8: probe_read_kernel<8><<<nwg, threads, 0, st>>>(s, vec_per_wg, shared, sink); break;
        case 16: probe_read_kernel<16><<<nwg, threads, 0, st>>>(s, vec_per_wg, shared, sink); break;
        case 32: probe_read_kernel<32><<<nwg, threads, 0, st>>>(s, vec_per_wg, shared, sink); break;
        default: return fail(ET_ERR_INVALID_ARG, "et_probe_read: vec_per_thread must be 4, 8, 16 or 32");
    }
    return check_launch("probe_read_kernel");
}

}  // extern "C"
