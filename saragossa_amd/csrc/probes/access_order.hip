// Measurement aid, not part of the library: does the ORDER in which a workgroup asks for its 16
// pages matter to a read-only launch over the K/V of one layer of BASELINE configs[2] (64 MiB)?
// Whole tiles a page at a time (the decode split kernel's pattern), everything up front, K
// tiles plus 1 KiB slices of every V tile per wavefront, with and without extra same-address
// loads. Every variant also writes an 8 KiB partial per workgroup, like the split kernel.
// Build: make -C saragossa_amd/csrc probes    Run: saragossa_amd/csrc/probes/bin/access_order
#include <hip/hip_runtime.h>
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("err %s line %d\n", hipGetErrorString(e), __LINE__); exit(1);} }while(0)
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// MODE 0: wave w reads whole K and V tiles of pages w, w+8 (the split kernel's pattern), one page at a time
// MODE 1: all requests up front: K tiles of pages w, w+8; then the kk=w slice (1 KiB) of V of all 16 pages
// MODE 2: as 1, plus 9 dummy 16-byte loads per wave
// MODE 3: all requests up front, whole tiles: K and V tiles of pages w, w+8 (32 loads in flight)
// MODE 4: as 1 but V slices first then K
template <int MODE>
__global__ __launch_bounds__(512) void rd(const u32x4 *kpool, const u32x4 *vpool, const int *table, int n_pages, int splits, float *part) {
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int split = blockIdx.x, kvh = blockIdx.y;
    const int pb0 = split * 16; // 16 pages per workgroup exactly
    unsigned acc = 0;
    const size_t page16 = (size_t)2 * 512;
    const int ids = table[pb0 + (lane & 15)];
    if (MODE == 0) {
        for (int c = 0; c < 2; ++c) {
            const int page = __builtin_amdgcn_readlane(ids, wave + c * 8);
            const u32x4 *kp = kpool + page * page16 + kvh * 512 + lane;
            const u32x4 *vp = vpool + page * page16 + kvh * 512 + lane;
            u32x4 k[8], v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) k[i] = __builtin_nontemporal_load(kp + i * 64);
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = __builtin_nontemporal_load(vp + i * 64);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc ^= k[i].x ^ v[i].y;
        }
    } else if (MODE == 3) {
        u32x4 k[2][8], v[2][8];
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const int page = __builtin_amdgcn_readlane(ids, wave + c * 8);
            const u32x4 *kp = kpool + page * page16 + kvh * 512 + lane;
            const u32x4 *vp = vpool + page * page16 + kvh * 512 + lane;
#pragma unroll
            for (int i = 0; i < 8; ++i) k[c][i] = __builtin_nontemporal_load(kp + i * 64);
#pragma unroll
            for (int i = 0; i < 8; ++i) v[c][i] = __builtin_nontemporal_load(vp + i * 64);
        }
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int i = 0; i < 8; ++i) acc ^= k[c][i].x ^ v[c][i].y;
    } else {
        u32x4 k[2][8], v[16], d[9];
        if (MODE == 4) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int page = __builtin_amdgcn_readlane(ids, i);
                v[i] = __builtin_nontemporal_load(vpool + page * page16 + kvh * 512 + wave * 64 + lane);
            }
        }
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const int page = __builtin_amdgcn_readlane(ids, wave + c * 8);
            const u32x4 *kp = kpool + page * page16 + kvh * 512 + lane;
#pragma unroll
            for (int i = 0; i < 8; ++i) k[c][i] = __builtin_nontemporal_load(kp + i * 64);
        }
        if (MODE == 2) {
            const int page = __builtin_amdgcn_readlane(ids, 0);
            const u32x4 *dp = vpool + page * page16 + kvh * 512 + wave * 64;
#pragma unroll
            for (int i = 0; i < 9; ++i) d[i] = __builtin_nontemporal_load(dp);
        }
        if (MODE != 4) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int page = __builtin_amdgcn_readlane(ids, i);
                v[i] = __builtin_nontemporal_load(vpool + page * page16 + kvh * 512 + wave * 64 + lane);
            }
        }
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int i = 0; i < 8; ++i) acc ^= k[c][i].x;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc ^= v[i].y;
        if (MODE == 2) {
#pragma unroll
            for (int i = 0; i < 9; ++i) acc ^= d[i].z;
        }
    }
    const int wg = blockIdx.y * gridDim.x + blockIdx.x;
    typedef float f4 __attribute__((ext_vector_type(4)));
    f4 pv = {(float)(acc & 255), 1.f, 2.f, 3.f};
    __builtin_nontemporal_store(pv, (f4 *)part + (size_t)wg * 512 + threadIdx.x);
}

int main() {
    const int rows = 32768, kv_heads = 2, hd = 256, n_pages = rows / 16, NL = 10, splits = 128;
    const size_t pool_bytes = (size_t)n_pages * kv_heads * hd * 16 * 2;
    std::vector<u32x4 *> kp(NL), vp(NL);
    std::vector<int *> tb(NL);
    std::mt19937 rng(1);
    for (int l = 0; l < NL; ++l) {
        CK(hipMalloc(&kp[l], pool_bytes)); CK(hipMalloc(&vp[l], pool_bytes)); CK(hipMalloc(&tb[l], n_pages * 4));
        CK(hipMemset(kp[l], 1, pool_bytes)); CK(hipMemset(vp[l], 2, pool_bytes));
        std::vector<int> t(n_pages);
        for (int i = 0; i < n_pages; ++i) t[i] = i;
        std::shuffle(t.begin(), t.end(), rng);
        CK(hipMemcpy(tb[l], t.data(), n_pages * 4, hipMemcpyHostToDevice));
    }
    float *part;
    CK(hipMalloc(&part, (size_t)256 * 512 * 16));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    auto timeit = [&](const char *name, auto launch) {
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
        printf("%-70s %7.2f us (min %.2f)\n", name, ts[ts.size() / 2], ts[0]);
        fflush(stdout);
    };
#define RUN(M, NAME) timeit(NAME, [&](int l) { hipLaunchKernelGGL(rd<M>, dim3(splits, kv_heads), dim3(512), 0, 0, kp[l], vp[l], tb[l], n_pages, splits, part); });
    RUN(0, "0 whole tiles, a page at a time (split kernel's pattern)")
    RUN(3, "3 whole tiles, both pages up front")
    RUN(1, "1 K tiles of 2 pages + 1 KiB V slices of 16 pages, all up front")
    RUN(2, "2 ... plus 9 dummy loads per wavefront")
    RUN(4, "4 V slices first, then K tiles")
    RUN(0, "0 again")
    CK(hipDeviceSynchronize());
    return 0;
}
