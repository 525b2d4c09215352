// Read bandwidth HBM delivers for the access pattern of the decode kernels: 8192 concurrent
// sequential streams (one per (sequence, head, segment) unit), each advanced CHUNK bytes at a
// time by half a wave with 16-byte loads, DEPTH steps in flight per wave, 256 workgroups of 16
// waves (one per CU).  Nothing else runs: this is the ceiling the memory system sets for the
// pattern, to put the decode kernels' code-byte rate against.
//
//     python -m adkv_amd.tools.hbm_streams        (builds this file with hipcc and runs it)
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

template <int BATCH, int DEPTH>
__global__ __launch_bounds__(1024) void k_stream(const uint4* __restrict__ src, uint32_t* out, int nsteps, size_t unit_vecs)
{
    const int wave = blockIdx.x * 16 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int unit = wave * 2 + (lane >> 5);
    const uint4* p = src + (size_t)unit * unit_vecs + (lane & 31);
    uint4 buf[DEPTH][BATCH];
    uint32_t acc = 0;
#pragma unroll
    for (int d = 0; d < DEPTH; d++)
#pragma unroll
        for (int b = 0; b < BATCH; b++) buf[d][b] = p[(size_t)(d * BATCH + b) * 32];
    for (int s = 0; s < nsteps; s += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
#pragma unroll
            for (int b = 0; b < BATCH; b++) acc += buf[d][b].x ^ buf[d][b].y ^ buf[d][b].z ^ buf[d][b].w;
            int nx = s + d + DEPTH;
            nx = nx < nsteps ? nx : nsteps - 1;
#pragma unroll
            for (int b = 0; b < BATCH; b++) buf[d][b] = p[(size_t)(nx * BATCH + b) * 32];
        }
    }
    if (acc == 0x12345678) out[threadIdx.x] = acc;
}

// For comparison: the same 1 GiB read the plain way, every workgroup one contiguous 4 MiB region,
// its 16 waves taking consecutive kilobytes, DEPTH loads in flight per wave.
template <int DEPTH>
__global__ __launch_bounds__(1024) void k_contig(const uint4* __restrict__ src, uint32_t* out, int nsteps)
{
    const uint4* p = src + (size_t)blockIdx.x * nsteps * 1024 + threadIdx.x; // 1024 threads x 16 B = 16 KB per step
    uint4 buf[DEPTH];
    uint32_t acc = 0;
#pragma unroll
    for (int d = 0; d < DEPTH; d++) buf[d] = p[(size_t)d * 1024];
    for (int s = 0; s < nsteps; s += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            acc += buf[d].x ^ buf[d].y ^ buf[d].z ^ buf[d].w;
            int nx = s + d + DEPTH;
            nx = nx < nsteps ? nx : nsteps - 1;
            buf[d] = p[(size_t)nx * 1024];
        }
    }
    if (acc == 0x12345678) out[threadIdx.x] = acc;
}

int main()
{
    const int NWG = 256, NU = NWG * 32;   // 8192 streams
    const size_t LEN = 128 * 1024;        // bytes per stream: one 2048-token segment of 4-bit codes, head dim 128
    const size_t total = NU * LEN;        // 1 GiB, the K codes of the headline shape
    uint4* src;
    uint32_t* out;
    (void)hipMalloc(&src, total + 65536);
    (void)hipMalloc(&out, 4096);
    (void)hipMemset(src, 1, total + 65536);
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    auto run = [&](const char* name, auto kern, int batch) {
        const int nsteps = (int)(LEN / 512 / batch / 24 * 24);
        for (int w = 0; w < 3; w++) hipLaunchKernelGGL(kern, dim3(NWG), dim3(1024), 0, 0, src, out, nsteps, LEN / 16);
        (void)hipEventRecord(e0);
        for (int w = 0; w < 10; w++) hipLaunchKernelGGL(kern, dim3(NWG), dim3(1024), 0, 0, src, out, nsteps, LEN / 16);
        (void)hipEventRecord(e1);
        (void)hipEventSynchronize(e1);
        float ms;
        (void)hipEventElapsedTime(&ms, e0, e1);
        ms /= 10;
        const double bytes = (double)NU * nsteps * batch * 512;
        printf("%-34s %7.1f us  %5.2f TB/s  (%4.1f %% of 8 TB/s)\n", name, ms * 1e3, bytes / (ms * 1e-3) / 1e12,
               bytes / (ms * 1e-3) / 8e10);
    };
    run("512 B per step, 1 step in flight", k_stream<1, 1>, 1);
    run("512 B per step, 2 in flight", k_stream<1, 2>, 1);
    run("512 B per step, 3 in flight", k_stream<1, 3>, 1);
    run("512 B per step, 4 in flight", k_stream<1, 4>, 1);
    run("512 B per step, 8 in flight", k_stream<1, 8>, 1);
    run("1 KB per step, 2 in flight", k_stream<2, 2>, 2);
    run("1 KB per step, 4 in flight", k_stream<2, 4>, 2);
    run("2 KB per step, 2 in flight", k_stream<4, 2>, 4);
    run("2 KB per step, 4 in flight", k_stream<4, 4>, 4);
    auto run_contig = [&](const char* name, auto kern) {
        const int nsteps = (int)(total / NWG / 16384);
        for (int w = 0; w < 3; w++) hipLaunchKernelGGL(kern, dim3(NWG), dim3(1024), 0, 0, src, out, nsteps);
        (void)hipEventRecord(e0);
        for (int w = 0; w < 10; w++) hipLaunchKernelGGL(kern, dim3(NWG), dim3(1024), 0, 0, src, out, nsteps);
        (void)hipEventRecord(e1);
        (void)hipEventSynchronize(e1);
        float ms;
        (void)hipEventElapsedTime(&ms, e0, e1);
        ms /= 10;
        printf("%-34s %7.1f us  %5.2f TB/s  (%4.1f %% of 8 TB/s)\n", name, ms * 1e3, total / (ms * 1e-3) / 1e12,
               total / (ms * 1e-3) / 8e10);
    };
    run_contig("contiguous 4 MiB per workgroup, 2", k_contig<2>);
    run_contig("contiguous 4 MiB per workgroup, 4", k_contig<4>);
    run_contig("contiguous 4 MiB per workgroup, 8", k_contig<8>);
    return 0;
}
