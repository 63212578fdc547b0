// In-place strided copies between state containers for gfx950: admission of a prefilled sequence into its slot, migration
// between the plain pools and the snapshot pools.  Replaces the Metal kernel blit_{ctype} (qwen35/batch.py:349-372) behind
// batch.blit, which Pools.load / read (batch.py:431-462) and the scheduler's _to_spec / _to_plain (qwen35/serve.py:310-348) use:
//     dst.flat[d0 + y * dstride + i] = src.flat[s0 + y * sstride + i]      for i < n, y < ny
// The copy is pure HBM traffic (n * ny elements read and written once).  Rows whose byte offsets and length are multiples
// of 16 move as 16-byte vectors, a lane per vector, 4 vectors in flight per lane; anything else moves element by element.
#include "qt_common.h"

namespace {

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

// one workgroup copies up to 256 * 4 vectors of one row y; grid = (ceil(nvec / 1024), ny)
__global__ __launch_bounds__(256) void blit_vec_kernel(u32x4* __restrict__ dst, const u32x4* __restrict__ src, long nvec,
                                                       long d0, long s0, long dstride, long sstride) {
    const long y = blockIdx.y;
    u32x4* d = dst + d0 + y * dstride;
    const u32x4* s = src + s0 + y * sstride;
    const long i0 = (long)blockIdx.x * 1024 + threadIdx.x;
    u32x4 v[4];
#pragma unroll
    for (int k = 0; k < 4; k++)
        if (i0 + k * 256 < nvec) v[k] = __builtin_nontemporal_load(s + i0 + k * 256);
#pragma unroll
    for (int k = 0; k < 4; k++)
        if (i0 + k * 256 < nvec) __builtin_nontemporal_store(v[k], d + i0 + k * 256);
}

// Many copies in one launch: a sequence's admission moves 48 separate pieces (18 layers of conv window and recurrent state,
// 6 layers of K and V rows); launched one by one they cost a launch each (about 3 us), far more than their bytes.  The jobs
// travel by value in the kernel arguments; all sizes, offsets and strides are in 16-byte vectors.
struct BlitJob {
    u32x4* dst;
    const u32x4* src;
    long nvec, ny, dstride, sstride;
};
constexpr int MAX_JOBS = 64;           // 64 x 48 bytes of kernel arguments
constexpr int BLIT_WGS_PER_CU = 8;
struct BlitJobs {
    BlitJob job[MAX_JOBS];
    int first_block[MAX_JOBS + 1];     // exclusive prefix of the jobs' (row, 1024-vector block) counts
};
// One flat space of (job, row, 1024-vector block) units of 16 KiB, walked with a grid stride: every workgroup moves the same
// number of units whatever the mix of job sizes, and asks for its next unit's vectors before it stores the current one's.
__global__ __launch_bounds__(256) void blit_batch_kernel(const BlitJobs jobs, int njobs) {
    const int total = jobs.first_block[njobs];
    auto locate = [&](int b, const u32x4*& s, u32x4*& d, long& left) {
        int lo = 0, hi = njobs - 1;                                  // the job that holds unit b (uniform binary search)
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (jobs.first_block[mid] <= b) lo = mid; else hi = mid - 1;
        }
        const BlitJob& j = jobs.job[lo];
        const long r = b - jobs.first_block[lo], blocks_per_row = (j.nvec + 1023) / 1024;
        const long y = r / blocks_per_row, i0 = (r % blocks_per_row) * 1024 + threadIdx.x;
        s = j.src + y * j.sstride + i0;
        d = j.dst + y * j.dstride + i0;
        left = j.nvec - i0;                                          // vectors of the row from this lane's first one on
    };
    int b = blockIdx.x;
    if (b >= total) return;
    const u32x4* s;
    u32x4* d;
    long left;
    locate(b, s, d, left);
    u32x4 v[4];
#pragma unroll
    for (int k = 0; k < 4; k++)
        if (k * 256 < left) v[k] = __builtin_nontemporal_load(s + k * 256);
    while (true) {
        const int nb = b + gridDim.x;
        const u32x4* s2 = nullptr;
        u32x4* d2 = nullptr;
        long left2 = 0;
        u32x4 v2[4];
        if (nb < total) {
            locate(nb, s2, d2, left2);
#pragma unroll
            for (int k = 0; k < 4; k++)
                if (k * 256 < left2) v2[k] = __builtin_nontemporal_load(s2 + k * 256);
        }
#pragma unroll
        for (int k = 0; k < 4; k++)
            if (k * 256 < left) __builtin_nontemporal_store(v[k], d + k * 256);
        if (nb >= total) break;
        b = nb, d = d2, left = left2;
        v[0] = v2[0], v[1] = v2[1], v[2] = v2[2], v[3] = v2[3];
    }
}

template <typename T>
__global__ __launch_bounds__(256) void blit_elem_kernel(T* __restrict__ dst, const T* __restrict__ src, long n, long d0, long s0,
                                                        long dstride, long sstride) {
    const long y = blockIdx.y, i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[d0 + y * dstride + i] = src[s0 + y * sstride + i];
}

}  // namespace

extern "C" {

// elem_size 2 (bf16) or 4 (f32); n, d0, s0, dstride, sstride in elements.  The ranges written must not overlap the ranges read.
int qt_blit(void* dst, const void* src, int elem_size, long n, long d0, long s0, long ny, long dstride, long sstride,
            hipStream_t stream) {
    if (!dst || !src) return QT_ERR_NULL;
    if (elem_size != 2 && elem_size != 4) return QT_ERR_UNSUPPORTED;
    if (n < 0 || ny < 0 || d0 < 0 || s0 < 0 || dstride < 0 || sstride < 0 || ny > 65535) return QT_ERR_DIM;
    if (n == 0 || ny == 0) return QT_OK;
    const long e = elem_size;
    const bool vec = ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15u) == 0 &&
                     ((n * e) | (d0 * e) | (s0 * e) | (dstride * e) | (sstride * e)) % 16 == 0;
    if (vec) {
        const long per = 16 / e, nvec = n / per;
        hipLaunchKernelGGL(blit_vec_kernel, dim3((unsigned)((nvec + 1023) / 1024), (unsigned)ny), dim3(256), 0, stream, (u32x4*)dst,
                           (const u32x4*)src, nvec, d0 / per, s0 / per, dstride / per, sstride / per);
    } else if (elem_size == 2) {
        hipLaunchKernelGGL(blit_elem_kernel<uint16_t>, dim3((unsigned)((n + 255) / 256), (unsigned)ny), dim3(256), 0, stream,
                           (uint16_t*)dst, (const uint16_t*)src, n, d0, s0, dstride, sstride);
    } else {
        hipLaunchKernelGGL(blit_elem_kernel<uint32_t>, dim3((unsigned)((n + 255) / 256), (unsigned)ny), dim3(256), 0, stream,
                           (uint32_t*)dst, (const uint32_t*)src, n, d0, s0, dstride, sstride);
    }
    QT_CHECK_LAUNCH();
    return QT_OK;
}

// `count` copies in one launch per 64 of them.  dst[k] / src[k] are device base pointers (host arrays), meta[7 k .. 7 k + 6] =
// { elem_size, n, d0, s0, ny, dstride, sstride } as for qt_blit (host array).  Every job must be 16-byte granular (pointers,
// n, offsets and strides as bytes); otherwise QT_ERR_ALIGN and nothing is launched.
int qt_blit_batch(void* const* dst, const void* const* src, const long* meta, int count, hipStream_t stream) {
    if (!dst || !src || !meta) return QT_ERR_NULL;
    if (count < 0) return QT_ERR_DIM;
    for (int k = 0; k < count; k++) {
        const long* m = meta + 7 * k;
        const long e = m[0];
        if (!dst[k] || !src[k]) return QT_ERR_NULL;
        if (e != 2 && e != 4) return QT_ERR_UNSUPPORTED;
        for (int i = 1; i < 7; i++)
            if (m[i] < 0) return QT_ERR_DIM;
        if (((reinterpret_cast<uintptr_t>(dst[k]) | reinterpret_cast<uintptr_t>(src[k])) & 15u) ||
            ((m[1] * e) | (m[2] * e) | (m[3] * e) | (m[5] * e) | (m[6] * e)) % 16)
            return QT_ERR_ALIGN;
    }
    for (int k0 = 0; k0 < count; k0 += MAX_JOBS) {
        BlitJobs jobs;
        const int nj = count - k0 < MAX_JOBS ? count - k0 : MAX_JOBS;
        long total = 0;
        for (int k = 0; k < nj; k++) {
            const long* m = meta + 7 * (k0 + k);
            const long per = 16 / m[0];
            BlitJob& j = jobs.job[k];
            j.dst = (u32x4*)dst[k0 + k] + m[2] / per;
            j.src = (const u32x4*)src[k0 + k] + m[3] / per;
            j.nvec = m[1] / per;
            j.ny = m[4];
            j.dstride = m[5] / per;
            j.sstride = m[6] / per;
            jobs.first_block[k] = (int)total;
            total += (j.nvec + 1023) / 1024 * j.ny;
            if (total > 0x7fffffffL) return QT_ERR_DIM;                  // (32 TiB in one call)
        }
        for (int k = nj; k < MAX_JOBS; k++) jobs.job[k] = BlitJob{nullptr, nullptr, 0, 0, 0, 0};
        for (int k = nj; k <= MAX_JOBS; k++) jobs.first_block[k] = (int)total;
        if (total == 0) continue;
        const long wgs = (long)qt::cu_count() * BLIT_WGS_PER_CU;
        hipLaunchKernelGGL(blit_batch_kernel, dim3((unsigned)(total < wgs ? total : wgs)), dim3(256), 0, stream, jobs, nj);
        QT_CHECK_LAUNCH();
    }
    return QT_OK;
}

}  // extern "C"
