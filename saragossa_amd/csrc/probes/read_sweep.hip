// Measurement aid, not part of the library: how fast can ONE launch fetch the 64 MiB of K/V that
// a full-attention layer of BASELINE configs[2] holds at 32768 rows (kv2/hd256 bf16, 16-token
// pages behind a permuted block table), over launch shapes? Ten layers' pools are walked in
// turn (640 MiB, more than the 256 MiB memory-side cache), launches back to back on one
// stream, timed with HIP events, median of seven groups of 100 launches.
// Build: make -C saragossa_amd/csrc probes    Run: saragossa_amd/csrc/probes/bin/read_sweep
#include <hip/hip_runtime.h>
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("err %s line %d\n", hipGetErrorString(e), __LINE__); exit(1);} }while(0)
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

__global__ void empty_k(unsigned *sink) { if (sink == (unsigned *)1) sink[0] = 1; }

// tiny second kernel like the merge: 256 WGs x 256 threads, each thread reads 8 floats far apart, writes one
__global__ __launch_bounds__(256) void merge_like(const float *part, float *out) {
    const int t = threadIdx.x, b = blockIdx.x;
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += part[((size_t)(i * 16 + (t >> 4)) * 4096 + b * 16 + (t & 15))];
    if ((t >> 4) == 0) out[b * 16 + (t & 15)] = s;
}

// WG = (split, kvh); wave w walks pages pb0 + w*DEPTH .. stride WAVES*DEPTH; per page 8 K + 8 V 1-KiB loads
template <int WAVES, int DEPTH, bool NT, bool TABLE>
__global__ __launch_bounds__(WAVES * 64) void read_paged(const u32x4 *kpool, const u32x4 *vpool, const int *table,
                                                         int n_pages, int splits, int kv_heads, float *part) {
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int split = blockIdx.x, kvh = blockIdx.y;
    const int pb0 = (int)(((long)split * n_pages) / splits), pb1 = (int)(((long)(split + 1) * n_pages) / splits);
    unsigned acc = 0;
    const size_t page16 = (size_t)kv_heads * 512;
    for (int pb = pb0 + wave * DEPTH; pb < pb1; pb += WAVES * DEPTH) {
        u32x4 k[DEPTH][8], v[DEPTH][8];
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            int pp = pb + d < pb1 ? pb + d : pb;
            int page = TABLE ? __builtin_amdgcn_readfirstlane(table[pp]) : pp;
            const u32x4 *kp = kpool + page * page16 + kvh * 512 + lane;
            const u32x4 *vp = vpool + page * page16 + kvh * 512 + lane;
#pragma unroll
            for (int i = 0; i < 8; ++i) k[d][i] = NT ? __builtin_nontemporal_load(kp + i * 64) : kp[i * 64];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[d][i] = NT ? __builtin_nontemporal_load(vp + i * 64) : vp[i * 64];
        }
#pragma unroll
        for (int d = 0; d < DEPTH; ++d)
#pragma unroll
            for (int i = 0; i < 8; ++i) acc ^= k[d][i].x ^ k[d][i].w ^ v[d][i].y ^ v[d][i].z;
    }
    // an 8 KiB partial per workgroup like the split kernel's (first 512 threads-worth)
    if (part) {
        const int wg = blockIdx.y * gridDim.x + blockIdx.x;
        float4 pv = make_float4((float)(acc & 255), 1.f, 2.f, 3.f);
        for (int i = threadIdx.x; i < 512; i += WAVES * 64)
            __builtin_nontemporal_store(pv.x, part + ((size_t)wg * 512 + i) * 4);
    } else if (acc == 0x12345678) {
        ((unsigned *)kpool)[0] = acc;
    }
}

template <int UNROLL>
__global__ __launch_bounds__(256) void read_contig(const u32x4 *p, size_t n16, unsigned *sink) {
    size_t i = (size_t)blockIdx.x * 256 * UNROLL + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256 * UNROLL;
    unsigned acc = 0;
    for (; i + (UNROLL - 1) * 256 < n16; i += stride) {
        u32x4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) v[u] = __builtin_nontemporal_load(p + i + u * 256);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (acc == 0x12345678) sink[0] = acc;
}

int main(int argc, char **argv) {
    const int rows = 32768, kv_heads = 2, hd = 256;
    const int n_pages = rows / 16;
    const size_t pool_bytes = (size_t)n_pages * kv_heads * hd * 16 * 2;
    const int NL = 10;
    std::vector<u32x4 *> kp(NL), vp(NL);
    std::vector<int *> tb(NL);
    std::mt19937 rng(1);
    for (int l = 0; l < NL; ++l) {
        CK(hipMalloc(&kp[l], pool_bytes));
        CK(hipMalloc(&vp[l], pool_bytes));
        CK(hipMalloc(&tb[l], n_pages * 4));
        CK(hipMemset(kp[l], 1, pool_bytes));
        CK(hipMemset(vp[l], 2, pool_bytes));
        std::vector<int> t(n_pages);
        for (int i = 0; i < n_pages; ++i) t[i] = i;
        std::shuffle(t.begin(), t.end(), rng);
        CK(hipMemcpy(tb[l], t.data(), n_pages * 4, hipMemcpyHostToDevice));
    }
    unsigned *sink;
    CK(hipMalloc(&sink, 4));
    float *part, *out;
    CK(hipMalloc(&part, (size_t)4096 * 512 * 16));
    CK(hipMalloc(&out, 65536 * 4));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    auto timeit = [&](const char *name, auto launch) {
        for (int w = 0; w < 2; ++w)
            for (int l = 0; l < NL; ++l) launch(l);
        CK(hipDeviceSynchronize());
        std::vector<float> ts;
        for (int r = 0; r < 7; ++r) {
            const int iters = 10;
            CK(hipEventRecord(e0));
            for (int it = 0; it < iters; ++it)
                for (int l = 0; l < NL; ++l) launch(l);
            CK(hipEventRecord(e1));
            CK(hipEventSynchronize(e1));
            float ms;
            CK(hipEventElapsedTime(&ms, e0, e1));
            ts.push_back(ms * 1e3f / (iters * NL));
        }
        std::sort(ts.begin(), ts.end());
        const double us = ts[ts.size() / 2];
        printf("%-52s %7.2f us  %6.0f GB/s  %5.1f %%\n", name, us, 2.0 * pool_bytes / us / 1e3, 2.0 * pool_bytes / us / 1e3 / 80.0);
        fflush(stdout);
    };
    timeit("empty 1x64", [&](int) { hipLaunchKernelGGL(empty_k, dim3(1), dim3(64), 0, 0, sink); });
    timeit("empty 256x512", [&](int) { hipLaunchKernelGGL(empty_k, dim3(256), dim3(512), 0, 0, sink); });
    timeit("merge_like alone", [&](int) { hipLaunchKernelGGL(merge_like, dim3(256), dim3(256), 0, 0, part, out); });
    for (int blocks : {1024, 2048, 4096, 8192}) {
        char nm[96];
        snprintf(nm, 96, "contig nt unroll8 blocks=%d (K then V launch)", blocks);
        timeit(nm, [&](int l) {
            hipLaunchKernelGGL(read_contig<8>, dim3(blocks), dim3(256), 0, 0, kp[l], pool_bytes / 16, sink);
            hipLaunchKernelGGL(read_contig<8>, dim3(blocks), dim3(256), 0, 0, vp[l], pool_bytes / 16, sink);
        });
    }
#define PAGED(W, D, NTV, TB, SPL, PART)                                                                      \
    {                                                                                                        \
        char nm[96];                                                                                         \
        snprintf(nm, 96, "paged waves=%d depth=%d nt=%d table=%d wgs=%d part=%d", W, D, NTV, TB, SPL * 2, PART); \
        timeit(nm, [&](int l) {                                                                              \
            hipLaunchKernelGGL((read_paged<W, D, NTV, TB>), dim3(SPL, kv_heads), dim3(W * 64), 0, 0, kp[l], vp[l], \
                               tb[l], n_pages, SPL, kv_heads, PART ? part : nullptr);                        \
        });                                                                                                  \
    }
    // the decode kernel's own shape first
    PAGED(8, 1, true, true, 128, 0)
    PAGED(8, 1, true, true, 128, 1)
    PAGED(8, 1, false, true, 128, 0)
    PAGED(8, 1, true, false, 128, 0)
    PAGED(8, 2, true, true, 128, 0)
    PAGED(8, 1, true, true, 256, 0)
    PAGED(8, 2, true, true, 256, 0)
    PAGED(8, 1, true, true, 512, 0)
    PAGED(8, 1, true, true, 64, 0)
    PAGED(8, 2, true, true, 64, 0)
    PAGED(8, 4, true, true, 64, 0)
    PAGED(4, 1, true, true, 128, 0)
    PAGED(4, 2, true, true, 128, 0)
    PAGED(4, 4, true, true, 128, 0)
    PAGED(4, 1, true, true, 256, 0)
    PAGED(4, 2, true, true, 256, 0)
    PAGED(4, 4, true, true, 256, 0)
    PAGED(4, 1, true, true, 512, 0)
    PAGED(4, 2, true, true, 512, 0)
    PAGED(4, 1, true, true, 1024, 0)
    PAGED(16, 1, true, true, 128, 0)
    PAGED(16, 2, true, true, 128, 0)
    PAGED(16, 1, true, true, 64, 0)
    PAGED(16, 2, true, true, 64, 0)
    PAGED(16, 4, true, true, 64, 0)
    PAGED(2, 2, true, true, 512, 0)
    PAGED(2, 4, true, true, 512, 0)
    PAGED(2, 2, true, true, 1024, 0)
    // the pair: read with partials + a merge-like second launch
    timeit("pair: paged 8/1 wgs=256 part + merge_like", [&](int l) {
        hipLaunchKernelGGL((read_paged<8, 1, true, true>), dim3(128, kv_heads), dim3(512), 0, 0, kp[l], vp[l], tb[l],
                           n_pages, 128, kv_heads, part);
        hipLaunchKernelGGL(merge_like, dim3(256), dim3(256), 0, 0, part, out);
    });
    timeit("pair: paged 8/1 wgs=256 part + empty", [&](int l) {
        hipLaunchKernelGGL((read_paged<8, 1, true, true>), dim3(128, kv_heads), dim3(512), 0, 0, kp[l], vp[l], tb[l],
                           n_pages, 128, kv_heads, part);
        hipLaunchKernelGGL(empty_k, dim3(1), dim3(64), 0, 0, sink);
    });
    CK(hipDeviceSynchronize());
    return 0;
}
