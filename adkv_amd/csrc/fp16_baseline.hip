// fp16-KV decode attention for gfx950: the comparator the ADKV path is measured against (the
// uncompressed cache of tools/memory_comparison_fig.py:46-56; the reference ships no kernel for
// it).  Plain split-K
// flash decoding: K and V are fp16 [B, H, T, 128] and are each read exactly once, so the kernel is
// HBM-bound at 4*B*H*T*D bytes per step.
//
//   pass 1  one workgroup per (head, chunk of CHUNK tokens): logits -> chunk softmax -> P.V partial
//   pass 2  merge the chunks of a head (max / sum / weighted partials)
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/adkv_hip.h"

namespace adkv_fp16 {

typedef _Float16 h1;
typedef _Float16 h2 __attribute__((ext_vector_type(2)));

constexpr int D = 128;
constexpr int CHUNK = 512;
constexpr int BLK = 256;

__device__ __forceinline__ h2 as_h2(uint32_t u) { return __builtin_bit_cast(h2, u); }

// sum over the 16 lanes of a DPP row; every lane gets the total
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v)
{
    return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL,
                                                                      0xF, 0xF, false));
}

__device__ __forceinline__ float row16_allreduce(float v)
{
    v = dpp_add<0xB1>(v);  // quad_perm [1,0,3,2]
    v = dpp_add<0x4E>(v);  // quad_perm [2,3,0,1]
    v = dpp_add<0x141>(v); // row_half_mirror
    v = dpp_add<0x140>(v); // row_mirror
    return v;
}

__global__ __launch_bounds__(BLK) void chunk_kernel(
    const h1 *__restrict__ q, const h1 *__restrict__ K, const h1 *__restrict__ V,
    float *__restrict__ part, int T, int nchunk, float scaling)
{
    __shared__ float logit[CHUNK];
    __shared__ float red[BLK / 64];
    __shared__ float accs[BLK / 16][D + 4];

    const int bx = blockIdx.x / nchunk, ck = blockIdx.x % nchunk;
    const int t0 = ck * CHUNK;
    const int n = min(CHUNK, T - t0);
    const int grp = threadIdx.x >> 4; // token slot 0..15
    const int l16 = threadIdx.x & 15; // 8 channels 8*l16..
    const h1 *Kb = K + ((size_t)bx * T + t0) * D + l16 * 8;
    const h1 *Vb = V + ((size_t)bx * T + t0) * D + l16 * 8;

    const uint4 qq = *reinterpret_cast<const uint4 *>(q + (size_t)bx * D + l16 * 8);
    const h2 q0 = as_h2(qq.x), q1 = as_h2(qq.y), q2 = as_h2(qq.z), q3 = as_h2(qq.w);

    // logits, 16 tokens per pass
    float mx = -INFINITY;
    for (int i = grp; i < n; i += BLK / 16) {
        const uint4 k = *reinterpret_cast<const uint4 *>(Kb + (size_t)i * D);
        float s = __builtin_amdgcn_fdot2(q0, as_h2(k.x), 0.0f, false);
        s = __builtin_amdgcn_fdot2(q1, as_h2(k.y), s, false);
        s = __builtin_amdgcn_fdot2(q2, as_h2(k.z), s, false);
        s = __builtin_amdgcn_fdot2(q3, as_h2(k.w), s, false);
        s = row16_allreduce(s) * scaling;
        if (l16 == 0)
            logit[i] = s;
        mx = fmaxf(mx, s);
    }
    // chunk max
    for (int m = 16; m < 64; m <<= 1)
        mx = fmaxf(mx, __shfl_xor(mx, m, 64));
    if ((threadIdx.x & 63) == 0)
        red[threadIdx.x >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));

    // P.V with unnormalised p = exp(l - mx); each 16-lane group owns every 16th token
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    float lsum = 0.0f;
    for (int i = grp; i < n; i += BLK / 16) {
        const float p = __expf(logit[i] - mx);
        lsum += p;
        const uint4 v = *reinterpret_cast<const uint4 *>(Vb + (size_t)i * D);
        const h2 v0 = as_h2(v.x), v1 = as_h2(v.y), v2 = as_h2(v.z), v3 = as_h2(v.w);
        acc[0] = __builtin_fmaf(p, (float)v0.x, acc[0]);
        acc[1] = __builtin_fmaf(p, (float)v0.y, acc[1]);
        acc[2] = __builtin_fmaf(p, (float)v1.x, acc[2]);
        acc[3] = __builtin_fmaf(p, (float)v1.y, acc[3]);
        acc[4] = __builtin_fmaf(p, (float)v2.x, acc[4]);
        acc[5] = __builtin_fmaf(p, (float)v2.y, acc[5]);
        acc[6] = __builtin_fmaf(p, (float)v3.x, acc[6]);
        acc[7] = __builtin_fmaf(p, (float)v3.y, acc[7]);
    }
#pragma unroll
    for (int c = 0; c < 8; c++)
        accs[grp][l16 * 8 + c] = acc[c];
    if (l16 == 0)
        accs[grp][D] = lsum;
    __syncthreads();
    // fold the 16 token slots
    float *o = part + ((size_t)bx * nchunk + ck) * (D + 2);
    if (threadIdx.x < D + 1) {
        float s = 0.0f;
#pragma unroll
        for (int g = 0; g < BLK / 16; g++)
            s += accs[g][threadIdx.x];
        o[threadIdx.x] = s; // [0..D) partial output, [D] partial sum of p
    }
    if (threadIdx.x == 0)
        o[D + 1] = mx;
}

__global__ __launch_bounds__(D) void merge_kernel(const float *__restrict__ part, h1 *__restrict__ out,
                                                  int nchunk)
{
    const int bx = blockIdx.x, c = threadIdx.x;
    const float *p = part + (size_t)bx * nchunk * (D + 2);
    float mx = -INFINITY;
    for (int k = 0; k < nchunk; k++)
        mx = fmaxf(mx, p[k * (D + 2) + D + 1]);
    float num = 0.0f, den = 0.0f;
    for (int k = 0; k < nchunk; k++) {
        const float w = __expf(p[k * (D + 2) + D + 1] - mx);
        num += w * p[k * (D + 2) + c];
        den += w * p[k * (D + 2) + D];
    }
    out[(size_t)bx * D + c] = (h1)(num / den);
}

} // namespace adkv_fp16

extern "C" {

int64_t adkv_fp16_decode_workspace_bytes(int B, int H, int T)
{
    const int nchunk = (T + adkv_fp16::CHUNK - 1) / adkv_fp16::CHUNK;
    return (int64_t)B * H * nchunk * (adkv_fp16::D + 2) * 4;
}

int adkv_fp16_decode(const void *q, const void *K, const void *V, void *out, void *workspace,
                     int64_t workspace_bytes, int B, int H, int T, int D, float scaling, void *stream)
{
    using namespace adkv_fp16;
    if (!q || !K || !V || !out || !workspace)
        return ADKV_E_NULL;
    if (D != adkv_fp16::D)
        return ADKV_E_DIM;
    if (B <= 0 || H <= 0 || T <= 0)
        return ADKV_E_SHAPE;
    if (workspace_bytes < adkv_fp16_decode_workspace_bytes(B, H, T))
        return ADKV_E_WORKSPACE;
    if (((uintptr_t)q | (uintptr_t)K | (uintptr_t)V) & 15)
        return ADKV_E_ALIGN;
    const int nchunk = (T + CHUNK - 1) / CHUNK;
    hipLaunchKernelGGL(chunk_kernel, dim3((unsigned)((long)B * H * nchunk)), dim3(BLK), 0,
                       (hipStream_t)stream, (const h1 *)q, (const h1 *)K, (const h1 *)V,
                       (float *)workspace, T, nchunk, scaling);
    hipLaunchKernelGGL(merge_kernel, dim3((unsigned)(B * H)), dim3(adkv_fp16::D), 0, (hipStream_t)stream,
                       (const float *)workspace, (h1 *)out, nchunk);
    return hipGetLastError() == hipSuccess ? ADKV_OK : ADKV_E_LAUNCH;
}

} // extern "C"
