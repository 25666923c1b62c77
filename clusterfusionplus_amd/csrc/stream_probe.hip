// Bare read probes behind the numbers the design notes quote for "what this part streams at" (a measurement tool, not
// part of the library; built and run by clusterfusionplus_amd/stream_probe.py).
//
//   1. streaming rate and the latency of a dependent memory round trip, by the number of streaming waves per compute
//      unit (4 or 7; an eighth wave times a chain of dependent returning atomics / coherent loads, which is what every
//      hop of a device-wide event or of the attention chain is) and by the load instructions each wave keeps in flight
//      (1 KB each: 8 KB rows, non-temporal 16-byte lane loads, as the weight streams of the layer kernels);
//   2. the same streams with the address of every piece worked out slightly differently (same rows, or rows interleaved
//      with an odd stride, or a contiguous range per wave): how much of the rates of 1. is the exact instruction stream;
//   3. a region read again after a warm-up pass against the same region read cold (another gigabyte read in between):
//      what the 256 MB memory-side cache is worth to a weight stream.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <vector>

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

#define CHECK(e)                                                                             \
    do {                                                                                     \
        hipError_t err_ = (e);                                                               \
        if (err_ != hipSuccess) { printf("HIP error %s at line %d\n", hipGetErrorString(err_), __LINE__); return 1; } \
    } while (0)

// D load instructions in flight per streaming wave, issued in two half batches; `nstream` streaming waves per
// workgroup (one workgroup of eight waves per compute unit); wave 7 times `hops` dependent round trips.
// VARIANT: the same rows for the same waves (pad 0, contiguous 0), but the address of a piece is worked out with a
// run-time choice of the row order in it: rows of the waves interleaved with a stride of waves + pad rows, or a
// contiguous range per wave.
template <int D, bool VARIANT = false>
__global__ __launch_bounds__(512) void k_stream(const u32x4* __restrict__ w, int nrows, int nstream, int* ctr, int hops, float* lat,
                                                unsigned* out, int coherent_load, int pad = 0, int contiguous = 0) {
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    constexpr int HB = D / 2;
    if (wave < nstream) {
        const int gw = blockIdx.x * nstream + wave, nw = gridDim.x * nstream;
        unsigned acc = 0;
        // piece i of this wave: 1 KB, eight consecutive pieces are one 8 KB row; the rows of the waves interleave
        const size_t per = (size_t)(nrows / (nw + pad));
        auto addr = [&](size_t i) {
            size_t row = (i / 8) * nw + gw;
            if (VARIANT) row = contiguous ? (size_t)gw * per + i / 8 : (i / 8) * (size_t)(nw + pad) + gw;
            return w + (row * 8 + i % 8) * 64 + lane;
        };
        const size_t mine = per * 8;
        u32x4 a[HB], b[HB];
#pragma unroll
        for (int u = 0; u < HB; ++u) a[u] = __builtin_nontemporal_load(addr(u));
#pragma unroll
        for (int u = 0; u < HB; ++u) b[u] = __builtin_nontemporal_load(addr(HB + u));
        for (size_t i = 0; i + 2 * D <= mine; i += D) {
#pragma unroll
            for (int u = 0; u < HB; ++u) acc ^= a[u].x ^ a[u].y ^ a[u].z ^ a[u].w;
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < HB; ++u) a[u] = __builtin_nontemporal_load(addr(i + D + u));
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < HB; ++u) acc ^= b[u].x ^ b[u].y ^ b[u].z ^ b[u].w;
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < HB; ++u) b[u] = __builtin_nontemporal_load(addr(i + D + HB + u));
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int u = 0; u < HB; ++u) acc ^= a[u].x ^ a[u].y ^ a[u].z ^ a[u].w ^ b[u].x ^ b[u].y ^ b[u].z ^ b[u].w;
        if (acc == 0x12345678u) out[0] = acc;
    } else if (wave == 7 && hops > 0) {
        long long t = wall_clock64();
        while (wall_clock64() - t < 500) {}      // 5 us at 100 MHz: the streams are up by then
        const int idx = blockIdx.x * hops;
        const long long t0 = wall_clock64();
        int v = 0;
        for (int h = 0; h < hops; ++h) {
            int* p = ctr + (size_t)(idx + h + (v & 0)) * 32;    // a 128-byte line of its own; the address depends on the last value
            if (lane == 0) {
                if (coherent_load) v = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                else v = __hip_atomic_fetch_add(p, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            v = __builtin_amdgcn_readfirstlane(v);
        }
        const long long t1 = wall_clock64();
        if (lane == 0) lat[blockIdx.x] = (float)(t1 - t0) / hops / 100.f;
        if (v == 0x7fffffff) out[1] = v;
    }
}

// whole 8 KB rows, a contiguous range per wave, U rows in flight per wave
template <int U>
__global__ __launch_bounds__(512) void k_rows(const u32x4* __restrict__ p, int nrows, unsigned* out) {
    const int lane = threadIdx.x & 63;
    const int gw = (blockIdx.x * blockDim.x + threadIdx.x) >> 6, nw = (gridDim.x * blockDim.x) >> 6;
    unsigned acc = 0;
    const int r0 = (int)(((long long)gw * nrows) / nw), r1 = (int)(((long long)(gw + 1) * nrows) / nw);
    for (int r = r0; r < r1; r += U) {
        u32x4 v[U][8];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int rr = r + u < r1 ? r + u : r;
            const u32x4* rp = p + (size_t)rr * 512 + lane;
#pragma unroll
            for (int c = 0; c < 8; ++c) v[u][c] = __builtin_nontemporal_load(rp + c * 64);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int c = 0; c < 8; ++c) acc ^= v[u][c].x ^ v[u][c].y ^ v[u][c].z ^ v[u][c].w;
    }
    if (acc == 0x12345678u) out[0] = acc;
}

template <int D, bool VARIANT = false>
int run_stream(const std::vector<u32x4*>& bufs, int& turn, int nrows, int grid, int nstream, int hops, int coherent, int* ctr, float* lat,
               unsigned* out, hipEvent_t e0, hipEvent_t e1, int pad = 0, int contiguous = 0) {
    CHECK(hipMemset(lat, 0, grid * sizeof(float)));
    float best = 1e9f;
    for (int it = 0; it < 6; ++it) {
        CHECK(hipEventRecord(e0));
        hipLaunchKernelGGL((k_stream<D, VARIANT>), dim3(grid), dim3(512), 0, 0, bufs[(turn++) % bufs.size()], nrows, nstream, ctr, hops, lat, out, coherent,
                           pad, contiguous);
        CHECK(hipEventRecord(e1));
        CHECK(hipEventSynchronize(e1));
        float ms = 0.f;
        CHECK(hipEventElapsedTime(&ms, e0, e1));
        if (it > 1 && ms < best) best = ms;
    }
    std::vector<float> hl(grid);
    CHECK(hipMemcpy(hl.data(), lat, grid * sizeof(float), hipMemcpyDeviceToHost));
    double s = 0, mx = 0;
    for (float x : hl) { s += x; if (x > mx) mx = x; }
    const double bytes = (double)(grid * nstream) * (double)((nrows / (grid * nstream + pad)) * 8) * 1024.0;
    if (VARIANT) printf("[%s] ", contiguous ? "contiguous rows per wave" : pad ? "interleaved, stride waves + 1" : "interleaved, stride waves   ");
    printf("%2d loads (KB) in flight per wave, %d streaming waves per compute unit = %3d KB per compute unit: %6.1f us %.2f TB/s", D, nstream,
           D * nstream, best * 1e3, bytes / best / 1e9);
    if (hops > 0) printf(" ; dependent %s: mean %.2f us, slowest compute unit %.2f us", coherent ? "coherent load" : "returning atomic", s / grid, mx);
    printf("\n");
    return 0;
}

int main() {
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    const int grid = prop.multiProcessorCount;
    printf("device: %s, %d compute units\n", prop.name, grid);
    const int nrows = 49152;                      // 8 KB rows: 402 MB per buffer, four buffers in turn (every pass reads HBM-cold data)
    const size_t bytes = (size_t)nrows * 8192;
    std::vector<u32x4*> bufs(4);
    for (auto& b : bufs) { CHECK(hipMalloc(&b, bytes)); CHECK(hipMemset(b, 1, bytes)); }
    unsigned* out; CHECK(hipMalloc(&out, 8));
    int* ctr; CHECK(hipMalloc(&ctr, (size_t)grid * 64 * 128)); CHECK(hipMemset(ctr, 0, (size_t)grid * 64 * 128));
    float* lat; CHECK(hipMalloc(&lat, grid * sizeof(float)));
    hipEvent_t e0, e1; CHECK(hipEventCreate(&e0)); CHECK(hipEventCreate(&e1));
    int turn = 0;
    printf("\n[1] streaming rate of 402 MB (cold) and the latency of a dependent round trip issued beside the streams\n");
    for (int coherent = 0; coherent < 2; ++coherent)
        for (int ns : {4, 7}) {
            if (run_stream<32>(bufs, turn, nrows, grid, ns, 16, coherent, ctr, lat, out, e0, e1)) return 1;
            if (run_stream<16>(bufs, turn, nrows, grid, ns, 16, coherent, ctr, lat, out, e0, e1)) return 1;
            if (run_stream<8>(bufs, turn, nrows, grid, ns, 16, coherent, ctr, lat, out, e0, e1)) return 1;
            if (run_stream<4>(bufs, turn, nrows, grid, ns, 16, coherent, ctr, lat, out, e0, e1)) return 1;
        }
    printf("\n[2] the same without the timing wave\n");
    for (int ns : {4, 7, 8}) {
        if (run_stream<32>(bufs, turn, nrows, grid, ns, 0, 0, ctr, lat, out, e0, e1)) return 1;
        if (run_stream<16>(bufs, turn, nrows, grid, ns, 0, 0, ctr, lat, out, e0, e1)) return 1;
        if (run_stream<8>(bufs, turn, nrows, grid, ns, 0, 0, ctr, lat, out, e0, e1)) return 1;
    }
    printf("\n[4] section [2] with the address arithmetic of the variant kernel (the first line of each group reads exactly the rows of\n"
           "    section [2], wave by wave)\n");
    for (int ns : {4, 7, 8})
        for (int mode = 0; mode < 3; ++mode) {
            const int pad = mode == 1, cont = mode == 2;
            if (run_stream<32, true>(bufs, turn, nrows, grid, ns, 0, 0, ctr, lat, out, e0, e1, pad, cont)) return 1;
            if (run_stream<16, true>(bufs, turn, nrows, grid, ns, 0, 0, ctr, lat, out, e0, e1, pad, cont)) return 1;
            if (run_stream<8, true>(bufs, turn, nrows, grid, ns, 0, 0, ctr, lat, out, e0, e1, pad, cont)) return 1;
        }
    printf("\n[3] a region read again after a warm-up pass, and read cold (1 GB of another buffer read in between); 8 waves per compute unit,\n"
           "    two 8 KB rows in flight per wave\n");
    u32x4 *big, *other;
    const size_t gb = (size_t)1 << 30;
    CHECK(hipMalloc(&big, gb)); CHECK(hipMemset(big, 1, gb));
    CHECK(hipMalloc(&other, gb)); CHECK(hipMemset(other, 2, gb));
    for (int mb : {32, 64, 128, 160, 200, 256, 403}) {
        const size_t nb = (size_t)mb << 20;
        const int rows = (int)(nb / 8192);
        float warm = 0.f, cold = 0.f;
        for (int it = 0; it < 10; ++it) {
            float ms = 0.f;
            hipLaunchKernelGGL((k_rows<2>), dim3(grid), dim3(512), 0, 0, other, (int)(gb / 8192), out);     // evict
            hipLaunchKernelGGL((k_rows<2>), dim3(grid), dim3(512), 0, 0, big, rows, out);                   // warm
            CHECK(hipEventRecord(e0));
            hipLaunchKernelGGL((k_rows<2>), dim3(grid), dim3(512), 0, 0, big, rows, out);
            CHECK(hipEventRecord(e1)); CHECK(hipEventSynchronize(e1)); CHECK(hipEventElapsedTime(&ms, e0, e1));
            warm += ms;
            hipLaunchKernelGGL((k_rows<2>), dim3(grid), dim3(512), 0, 0, other, (int)(gb / 8192), out);     // evict
            CHECK(hipEventRecord(e0));
            hipLaunchKernelGGL((k_rows<2>), dim3(grid), dim3(512), 0, 0, big, rows, out);
            CHECK(hipEventRecord(e1)); CHECK(hipEventSynchronize(e1)); CHECK(hipEventElapsedTime(&ms, e0, e1));
            cold += ms;
        }
        printf("%4d MB: after a warm-up pass %6.1f us %.2f TB/s | cold %6.1f us %.2f TB/s\n", mb, warm * 100, nb / (warm / 10) / 1e9, cold * 100,
               nb / (cold / 10) / 1e9);
    }
    return 0;
}
