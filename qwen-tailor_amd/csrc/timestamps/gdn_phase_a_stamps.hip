// Time stamps inside gdn_phase_a_kernel (conv + phase A of the chunked prefill; when workgroups start and end, shader-clock ticks
// between the kernel's marks): a stand-alone program that compiles the kernel source with its profiling macro defined, runs it
// on synthetic input and prints the stamps.  Not part of the library.  Build and run (from this directory):
//     hipcc -O3 --offload-arch=gfx950 -std=c++17 -I.. -Xclang -target-feature -Xclang -packed-fp32-ops gdn_phase_a_stamps.hip -o gdn_phase_a_stamps
//     ./gdn_phase_a_stamps [T]
#define QT_PHASE_A_PROF
#include "../gdn_chunked.hip"
namespace ops_ns {
#include "../gdn_ops.hip"
}
#include <cstdio>
#include <vector>
#include <cstdlib>
#include <cstring>
#include <algorithm>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e), __LINE__); exit(1);} } while (0)
static void fill(void* d, size_t n, float sc, uint32_t seed) {
    std::vector<uint16_t> hb(n); uint32_t st = seed;
    for (size_t i = 0; i < n; i++) { float a = 0; for (int k = 0; k < 12; k++) { st = st * 1664525u + 1013904223u; a += (st >> 8) * (1.0f / 16777216.0f); }
        float v = (a - 6.0f) * sc; uint32_t u; memcpy(&u, &v, 4); hb[i] = (uint16_t)((u + 0x7fffu + ((u >> 16) & 1)) >> 16); }
    CK(hipMemcpy(d, hb.data(), n * 2, hipMemcpyHostToDevice));
}
int main(int argc, char** argv) {
    const int T = argc > 1 ? atoi(argv[1]) : 2048, NC = (T + 63) / 64, NWG = NC * 16;
    void *proj, *cs, *cw, *tab, *ops; float *A, *dt, *U, *gC; long long* prof;
    CK(hipMalloc(&proj, (size_t)T * 8224 * 2)); fill(proj, (size_t)T * 8224, 1.0f, 1);
    CK(hipMalloc(&cs, 3 * 6144 * 2)); fill(cs, 3 * 6144, 1.0f, 2);
    CK(hipMalloc(&cw, 6144 * 8)); fill(cw, 6144 * 4, 0.5f, 3);
    CK(hipMalloc(&tab, SILU_TAB_SIZE * 2));
    CK(hipMalloc(&A, 64)); CK(hipMemset(A, 0, 64)); CK(hipMalloc(&dt, 64)); CK(hipMemset(dt, 0, 64));
    CK(hipMalloc(&ops, qt_gdn_chunk_ops_bytes(T))); CK(hipMalloc(&U, qt_gdn_chunk_u_bytes(T))); CK(hipMalloc(&gC, qt_gdn_chunk_gc_bytes(T)));
    CK(hipMalloc(&prof, (size_t)NWG * 4 * 16 * 8)); CK(hipMemset(prof, 0, (size_t)NWG * 4 * 16 * 8));
    CK(hipMemcpyToSymbol(HIP_SYMBOL(pa_prof_buf), &prof, sizeof(prof)));
    if (ops_ns::qt_silu_table_build(tab, 0) != 0) return 2;
    CK(hipDeviceSynchronize());
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    for (int it = 0; it < 5; it++) {
        CK(hipEventRecord(e0, 0));
        if (qt_gdn_phase_a_conv(proj, cs, cw, tab, A, dt, nullptr, nullptr, nullptr, nullptr, ops, U, gC, T, 0) != 0) { printf("launch failed\n"); return 1; }
        CK(hipEventRecord(e1, 0)); CK(hipEventSynchronize(e1));
        float ms; CK(hipEventElapsedTime(&ms, e0, e1));
        printf("iter %d: %.1f us\n", it, ms * 1e3);
    }
    std::vector<long long> h((size_t)NWG * 4 * 16);
    CK(hipMemcpy(h.data(), prof, h.size() * 8, hipMemcpyDeviceToHost));
    // per-mark deltas (cycles of the s_memtime counter), averaged over workgroups, for wave 0 and wave 3; plus spread of start / end
    long long tmin = 1LL << 62, tmax = 0;
    for (int g = 0; g < NWG; g++) for (int w = 0; w < 4; w++) { tmin = std::min(tmin, h[((size_t)g * 4 + w) * 16 + 14]); tmax = std::max(tmax, h[((size_t)g * 4 + w) * 16 + 15]); }
    printf("wall span first start -> last end: %.2f us\n", (tmax - tmin) * 0.01);
    { std::vector<double> st, en, du; for (int g = 0; g < NWG; g++) { st.push_back((h[((size_t)g * 4) * 16 + 14] - tmin) * 0.01); en.push_back((h[((size_t)g * 4 + 3) * 16 + 15] - tmin) * 0.01); du.push_back(en.back() - st.back()); }
      auto pr = [&](const char* n, std::vector<double> v) { std::sort(v.begin(), v.end()); printf("%s: min %.2f p10 %.2f p50 %.2f p90 %.2f max %.2f us\n", n, v[0], v[v.size() / 10], v[v.size() / 2], v[v.size() * 9 / 10], v.back()); };
      pr("wg start", st); pr("wg end", en); pr("wg duration", du);
      double tk = 0; for (int g = 0; g < NWG; g++) tk += (double)(h[((size_t)g * 4) * 16 + 10] - h[((size_t)g * 4) * 16]); printf("ticks per us: %.0f\n", tk / NWG / (du[du.size() / 2])); }
    for (int w = 0; w < 4; w++) {
        printf("wave %d avg delta per mark:", w);
        for (int m = 1; m <= 10; m++) { double s = 0; for (int g = 0; g < NWG; g++) s += (double)(h[((size_t)g * 4 + w) * 16 + m] - h[((size_t)g * 4 + w) * 16 + m - 1]); printf(" %7.0f", s / NWG); }
        printf("\n");
    }
    return 0;
}
