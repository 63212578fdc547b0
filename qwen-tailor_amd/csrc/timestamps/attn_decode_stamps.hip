// Time stamps inside attn_partial_kernel<M> (a timeline per workgroup, 100 MHz clock; a batch like benchmark config 3 for M = 1, config 4 for M = 4): a stand-alone program that compiles the kernel source with its profiling macro
// defined, runs it on synthetic input and prints the stamps.  Not part of the library.  Build and run (from this directory):
//     hipcc -O3 --offload-arch=gfx950 -std=c++17 -I.. -Xclang -target-feature -Xclang -packed-fp32-ops attn_decode_stamps.hip -o attn_decode_stamps
//     ./attn_decode_stamps [M]
#define QT_ATTN_DECODE_PROF
#include "../gqa_decode.hip"
#include <cstdio>
#include <vector>
#include <algorithm>
#include <random>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e), __LINE__); exit(1);} } while (0)
int main(int argc, char** argv) {
    const int M = argc > 1 ? atoi(argv[1]) : 4, B = 16;
    const int lo = M == 1 ? 512 : 1024, hi = M == 1 ? 32768 : 8192, Lmax = hi + 8;
    std::mt19937 rng(7);
    std::vector<int> pos(B), slots(B);
    long sumL = 0;
    for (int b = 0; b < B; b++) { pos[b] = lo + rng() % (hi - lo); slots[b] = b; sumL += pos[b]; }
    void *Kp, *Vp, *q, *kn, *vn, *out, *ws; int *dpos, *dslots; long long* prof;
    const size_t pool = (size_t)(B + 1) * 2 * Lmax * 512;
    CK(hipMalloc(&Kp, pool)); CK(hipMemset(Kp, 0x3c, pool));
    CK(hipMalloc(&Vp, pool)); CK(hipMemset(Vp, 0x3c, pool));
    CK(hipMalloc(&q, (size_t)B * M * 8 * 512)); CK(hipMemset(q, 0x3c, (size_t)B * M * 8 * 512));
    CK(hipMalloc(&kn, (size_t)B * M * 2 * 512)); CK(hipMemset(kn, 0x3c, (size_t)B * M * 2 * 512));
    CK(hipMalloc(&vn, (size_t)B * M * 2 * 512)); CK(hipMemset(vn, 0x3c, (size_t)B * M * 2 * 512));
    CK(hipMalloc(&out, (size_t)B * M * 8 * 512));
    const long wsb = qt_gqa_attn_workspace_bytes(B, M, Lmax, 1024);
    CK(hipMalloc(&ws, wsb));
    CK(hipMalloc(&dpos, B * 4)); CK(hipMalloc(&dslots, B * 4));
    CK(hipMemcpy(dpos, pos.data(), B * 4, hipMemcpyHostToDevice)); CK(hipMemcpy(dslots, slots.data(), B * 4, hipMemcpyHostToDevice));
    const int nwg = 1024;
    CK(hipMalloc(&prof, (size_t)nwg * 8 * 8));
    CK(hipMemcpyToSymbol(HIP_SYMBOL(ad_prof_buf), &prof, sizeof(prof)));
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    for (int it = 0; it < 5; it++) {
        CK(hipMemset(prof, 0, (size_t)nwg * 8 * 8));
        CK(hipDeviceSynchronize());
        CK(hipEventRecord(e0, 0));
        const int rc = qt_gqa_attn_decode(q, kn, vn, Kp, Vp, dslots, dpos, out, ws, wsb, B, M, Lmax, B + 1, 1024, 0);
        if (rc != 0) { printf("launch failed %d\n", rc); return 1; }
        CK(hipEventRecord(e1, 0)); CK(hipEventSynchronize(e1));
        float ms; CK(hipEventElapsedTime(&ms, e0, e1)); printf("M=%d sumL=%ld (%.1f MB) iter %d: %.1f us\n", M, sumL, sumL * 2048e-6, it, ms * 1e3);
    }
    std::vector<long long> h((size_t)nwg * 8);
    CK(hipMemcpy(h.data(), prof, h.size() * 8, hipMemcpyDeviceToHost));
    long long t0 = -1; int n = 0;
    for (int b = 0; b < nwg; b++) if (h[b * 8]) { n++; if (t0 < 0 || h[b * 8] < t0) t0 = h[b * 8]; }
    printf("%d workgroups; us after the first workgroup's start (last segment visit of each workgroup): min / median / max\n", n);
    const char* names[7] = {"start", "segments built", "first loads issued", "tile loop done", "new keys + append", "wave merge done", "partial stored"};
    for (int m = 0; m < 7; m++) {
        std::vector<double> v;
        for (int b = 0; b < nwg; b++) if (h[b * 8] && h[b * 8 + m]) v.push_back((h[b * 8 + m] - t0) / 100.0);
        std::sort(v.begin(), v.end());
        if (!v.empty()) printf("  %-20s %6.2f %6.2f %6.2f\n", names[m], v.front(), v[v.size() / 2], v.back());
    }
    std::vector<std::pair<double,int>> ends;
    for (int b = 0; b < nwg; b++) if (h[b * 8]) ends.push_back({(h[b * 8 + 6] - t0) / 100.0, b});
    std::sort(ends.begin(), ends.end());
    printf("slowest workgroups: wg, [first loads issued, tile loop done, partial stored] of its last visit\n");
    for (int i = (int)ends.size() - 1; i >= 0 && i >= (int)ends.size() - 14; i--) {
        const int b = ends[i].second;
        printf("  wg %3d: %6.2f %6.2f %6.2f\n", b, (h[b*8+2]-t0)/100.0, (h[b*8+3]-t0)/100.0, (h[b*8+6]-t0)/100.0);
    }
    printf("fastest:\n");
    for (int i = 0; i < 6; i++) { const int b = ends[i].second; printf("  wg %3d: %6.2f %6.2f %6.2f\n", b, (h[b*8+2]-t0)/100.0, (h[b*8+3]-t0)/100.0, (h[b*8+6]-t0)/100.0); }
    return 0;
}
