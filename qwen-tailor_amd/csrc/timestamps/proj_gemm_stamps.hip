// Time stamps inside xlds_gemm_kernel (a timeline per workgroup, 100 MHz clock; in_proj [8224 x 1024] on M rows): a stand-alone program that compiles the kernel source with its profiling macro
// defined, runs it on synthetic input and prints the stamps.  Not part of the library.  Build and run (from this directory):
//     hipcc -O3 --offload-arch=gfx950 -std=c++17 -I.. -Xclang -target-feature -Xclang -packed-fp32-ops proj_gemm_stamps.hip -o proj_gemm_stamps
//     ./proj_gemm_stamps [M]
#define QT_XLDS_PROF
#include "../proj_gemv.hip"
#include <cstdio>
#include <vector>
#include <algorithm>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e), __LINE__); exit(1);} } while (0)
int main(int argc, char** argv) {
    const int M = argc > 1 ? atoi(argv[1]) : 64, N = 8224, K = 1024;
    void *W[4], *x, *y; long long* prof;
    for (int i = 0; i < 4; i++) { CK(hipMalloc(&W[i], (size_t)N * K * 2)); CK(hipMemset(W[i], 0x3c, (size_t)N * K * 2)); }
    CK(hipMalloc(&x, (size_t)64 * K * 2)); CK(hipMemset(x, 0x3c, (size_t)64 * K * 2));
    CK(hipMalloc(&y, (size_t)64 * N * 2));
    const int nwg = 600;
    CK(hipMalloc(&prof, (size_t)nwg * 8 * 8));
    CK(hipMemcpyToSymbol(HIP_SYMBOL(xl_prof_buf), &prof, sizeof(prof)));
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    for (int it = 0; it < 6; it++) {
        CK(hipMemset(prof, 0, (size_t)nwg * 8 * 8));
        CK(hipDeviceSynchronize());
        CK(hipEventRecord(e0, 0));
        if (qt_fused_gemv(W[it % 4], x, nullptr, y, M, N, K, 0, 0) != 0) { printf("launch failed\n"); return 1; }
        CK(hipEventRecord(e1, 0)); CK(hipEventSynchronize(e1));
        float ms; CK(hipEventElapsedTime(&ms, e0, e1)); printf("M=%d iter %d: %.1f us\n", M, it, ms * 1e3);
    }
    std::vector<long long> h((size_t)nwg * 8);
    CK(hipMemcpy(h.data(), prof, h.size() * 8, hipMemcpyDeviceToHost));
    long long t0 = -1; int n = 0;
    for (int b = 0; b < nwg; b++) if (h[b * 8]) { n++; if (t0 < 0 || h[b * 8] < t0) t0 = h[b * 8]; }
    printf("%d workgroups; times in us after the first workgroup's start (100 MHz clock): min / median / max\n", n);
    const char* names[6] = {"start", "loads issued", "loads landed", "barrier passed", "mfma done", "stores issued"};
    for (int m = 0; m < 6; m++) {
        std::vector<double> v;
        for (int b = 0; b < nwg; b++) if (h[b * 8] && h[b * 8 + m]) v.push_back((h[b * 8 + m] - t0) / 100.0);
        std::sort(v.begin(), v.end());
        if (!v.empty()) printf("  %-16s %6.2f %6.2f %6.2f\n", names[m], v.front(), v[v.size() / 2], v.back());
    }
    return 0;
}
