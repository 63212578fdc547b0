// Time stamps inside attn_prefill_kernel (shader-clock ticks per phase of a 64-key tile): a stand-alone program that compiles the kernel source with its profiling macro
// defined, runs it on synthetic input and prints the stamps.  Not part of the library.  Build and run (from this directory):
//     hipcc -O3 --offload-arch=gfx950 -std=c++17 -I.. -Xclang -target-feature -Xclang -packed-fp32-ops attn_prefill_stamps.hip -o attn_prefill_stamps
//     ./attn_prefill_stamps [S]
#define QT_ATTN_PREFILL_PROF
#include "../gqa_prefill.hip"
#include <cstdio>
#include <vector>
#include <cstdlib>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e), __LINE__); exit(1);} } while (0)
int main(int argc, char** argv) {
    const int S = argc > 1 ? atoi(argv[1]) : 8192;
    void *q, *K, *V, *o; long long* prof;
    CK(hipMalloc(&q, (size_t)8 * S * 512)); CK(hipMemset(q, 0x3c, (size_t)8 * S * 512));
    CK(hipMalloc(&K, (size_t)2 * S * 512)); CK(hipMemset(K, 0x3c, (size_t)2 * S * 512));
    CK(hipMalloc(&V, (size_t)2 * S * 512)); CK(hipMemset(V, 0x3c, (size_t)2 * S * 512));
    CK(hipMalloc(&o, (size_t)8 * S * 512));
    const int nwg = ((S + 15) / 16) * 2;
    CK(hipMalloc(&prof, (size_t)nwg * 4 * 8 * 8));
    CK(hipMemcpyToSymbol(HIP_SYMBOL(ap_prof_buf), &prof, sizeof(prof)));
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    for (int it = 0; it < 4; it++) {
        CK(hipMemset(prof, 0, (size_t)nwg * 4 * 8 * 8));
        CK(hipEventRecord(e0, 0));
        if (qt_gqa_prefill_causal(q, K, V, o, nullptr, 0, S, S, 0, (long)S * 256, (long)S * 256, 0) != 0) { printf("launch failed\n"); return 1; }
        CK(hipEventRecord(e1, 0)); CK(hipEventSynchronize(e1));
        float ms; CK(hipEventElapsedTime(&ms, e0, e1)); printf("S=%d iter %d: %.1f us\n", S, it, ms * 1e3);
    }
    std::vector<long long> h((size_t)nwg * 4 * 8);
    CK(hipMemcpy(h.data(), prof, h.size() * 8, hipMemcpyDeviceToHost));
    // the workgroup with the most tiles is blockIdx.x = 0 (long rows first), kv head 0
    const int ntiles = (S + 63) / 64;
    for (int w = 0; w < 4; w++) {
        printf("wg 0 wave %d ticks per tile:", w);
        for (int m = 0; m < 7; m++) printf(" %7.0f", (double)h[(size_t)w * 8 + m] / ntiles);
        double tot = 0; for (int m = 0; m < 7; m++) tot += (double)h[(size_t)w * 8 + m];
        printf("  | total/tile %7.0f\n", tot / ntiles);
    }
    printf("marks: 0 = loop top, 1 = vmcnt wait, 2 = barrier (+ tail loads), 3 = mask + first fragments + maxima, 4 = steps, 5 = rescale, 6 = P.V\n");
    return 0;
}
