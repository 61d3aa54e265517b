// Device side of the growable KV cache: strided row copies and zero fill.
// Reference behaviour being replaced: TensorCache::append's cat + slice_assign
// (fusor-ml/fusor/src/cache/tensor_cache.rs:80-110), which copies the whole cache on every call;
// here an append moves only the new rows.
#include "common.h"
#include "device_utils.h"

namespace fhip {

// One thread per `VB`-byte piece of the innermost (contiguous) dimension.
template <int VB>
__global__ __launch_bounds__(256) void copy_rows_kernel(const char *src, char *dst, int64_t ss0, int64_t ss1,
                                                        int64_t ss2, int64_t ds0, int64_t ds1, int64_t ds2,
                                                        uint32_t n0, uint32_t n1, uint32_t n2, uint32_t pieces,
                                                        bool zero) {
    const int64_t total = (int64_t)n0 * n1 * n2 * pieces;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const uint32_t pc = (uint32_t)(i % pieces);
        int64_t t = i / pieces;
        const uint32_t i2 = (uint32_t)(t % n2);
        t /= n2;
        const uint32_t i1 = (uint32_t)(t % n1);
        const uint32_t i0 = (uint32_t)(t / n1);
        char *d = dst + (i0 * ds0 + i1 * ds1 + i2 * ds2) + (int64_t)pc * VB;
        if (zero) {
            if constexpr (VB == 16) *(uint4_t *)d = uint4_t{0, 0, 0, 0};
            else if constexpr (VB == 4) *(uint32_t *)d = 0;
            else *(uint16_t *)d = 0;
        } else {
            const char *s = src + (i0 * ss0 + i1 * ss1 + i2 * ss2) + (int64_t)pc * VB;
            if constexpr (VB == 16) *(uint4_t *)d = *(const uint4_t *)s;
            else if constexpr (VB == 4) *(uint32_t *)d = *(const uint32_t *)s;
            else *(uint16_t *)d = *(const uint16_t *)s;
        }
    }
}

// Fully strided fallback (innermost stride != 1 on either side): one thread per element.  `zero`: the destination
// elements are cleared and `src` (null then) is never read.
template <typename E>
__global__ __launch_bounds__(256) void copy_elems_kernel(const E *src, E *dst, int64_t ss0, int64_t ss1, int64_t ss2,
                                                         int64_t ss3, int64_t ds0, int64_t ds1, int64_t ds2,
                                                         int64_t ds3, uint32_t n0, uint32_t n1, uint32_t n2,
                                                         uint32_t n3, bool zero) {
    const int64_t total = (int64_t)n0 * n1 * n2 * n3;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const uint32_t i3 = (uint32_t)(i % n3);
        int64_t t = i / n3;
        const uint32_t i2 = (uint32_t)(t % n2);
        t /= n2;
        const uint32_t i1 = (uint32_t)(t % n1);
        const uint32_t i0 = (uint32_t)(t / n1);
        E val = 0;
        if (!zero) val = src[i0 * ss0 + i1 * ss1 + i2 * ss2 + i3 * ss3];
        dst[i0 * ds0 + i1 * ds1 + i2 * ds2 + i3 * ds3] = val;
    }
}

static unsigned grid_for(int64_t total) {
    int64_t b = (total + 255) / 256;
    if (b < 1) b = 1;
    if (b > 65536) b = 65536;
    return (unsigned)b;
}

// strides in ELEMENTS; elem_bytes 2 or 4
static int copy_or_zero(const void *src, const int64_t *ss, void *dst, const int64_t *ds, const uint32_t *shape,
                        int eb, bool zero, hipStream_t stream) {
    const int64_t total_elems = (int64_t)shape[0] * shape[1] * shape[2] * shape[3];
    if (total_elems == 0) return FHIP_OK;
    const bool inner_contig = (shape[3] == 1 || (ds[3] == 1 && (zero || ss[3] == 1)));
    if (inner_contig) {
        const int64_t row_bytes = (int64_t)shape[3] * eb;
        bool v16 = row_bytes % 16 == 0 && ((uintptr_t)dst % 16) == 0 && (zero || ((uintptr_t)src % 16) == 0);
        for (int i = 0; i < 3 && v16; i++) {
            if (shape[i] > 1 && (ds[i] * eb) % 16 != 0) v16 = false;
            if (!zero && shape[i] > 1 && (ss[i] * eb) % 16 != 0) v16 = false;
        }
        const int64_t s0 = zero ? 0 : ss[0] * eb, s1 = zero ? 0 : ss[1] * eb, s2 = zero ? 0 : ss[2] * eb;
        if (v16) {
            const uint32_t pieces = (uint32_t)(row_bytes / 16);
            const int64_t total = (int64_t)shape[0] * shape[1] * shape[2] * pieces;
            hipLaunchKernelGGL(copy_rows_kernel<16>, dim3(grid_for(total)), dim3(256), 0, stream, (const char *)src,
                               (char *)dst, s0, s1, s2, ds[0] * eb, ds[1] * eb, ds[2] * eb, shape[0], shape[1],
                               shape[2], pieces, zero);
        } else if (eb == 4) {
            hipLaunchKernelGGL(copy_rows_kernel<4>, dim3(grid_for(total_elems)), dim3(256), 0, stream,
                               (const char *)src, (char *)dst, s0, s1, s2, ds[0] * eb, ds[1] * eb, ds[2] * eb,
                               shape[0], shape[1], shape[2], shape[3], zero);
        } else {
            hipLaunchKernelGGL(copy_rows_kernel<2>, dim3(grid_for(total_elems)), dim3(256), 0, stream,
                               (const char *)src, (char *)dst, s0, s1, s2, ds[0] * eb, ds[1] * eb, ds[2] * eb,
                               shape[0], shape[1], shape[2], shape[3], zero);
        }
    } else if (eb == 4) {
        hipLaunchKernelGGL(copy_elems_kernel<uint32_t>, dim3(grid_for(total_elems)), dim3(256), 0, stream,
                           (const uint32_t *)src, (uint32_t *)dst, ss[0], ss[1], ss[2], ss[3], ds[0], ds[1], ds[2],
                           ds[3], shape[0], shape[1], shape[2], shape[3], zero);
    } else {
        hipLaunchKernelGGL(copy_elems_kernel<uint16_t>, dim3(grid_for(total_elems)), dim3(256), 0, stream,
                           (const uint16_t *)src, (uint16_t *)dst, ss[0], ss[1], ss[2], ss[3], ds[0], ds[1], ds[2],
                           ds[3], shape[0], shape[1], shape[2], shape[3], zero);
    }
    FHIP_HIP_CHECK(hipGetLastError());
    return FHIP_OK;
}

__global__ __launch_bounds__(256) void fill_zero_kernel(uint32_t *dst, size_t words) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < words; i += (size_t)gridDim.x * 256) dst[i] = 0u;
}

// Zero fill by a kernel (not a memset node), so a caller may record it into a HIP graph.
int launch_fill_zero_bytes(void *dst, size_t bytes, hipStream_t stream) {
    if (bytes == 0) return FHIP_OK;
    if (((uintptr_t)dst & 3) != 0 || (bytes & 3) != 0) {
        set_error("zero fill needs a 4-byte aligned pointer and size");
        return FHIP_ERR_INVALID_ARG;
    }
    const size_t words = bytes / 4;
    hipLaunchKernelGGL(fill_zero_kernel, dim3(grid_for((int64_t)words)), dim3(256), 0, stream, (uint32_t *)dst, words);
    FHIP_HIP_CHECK(hipGetLastError());
    return FHIP_OK;
}

// memset by a kernel: unaligned head and tail byte by byte, the body in 16-byte stores
__global__ __launch_bounds__(256) void fill_bytes_kernel(unsigned char *dst, size_t bytes, unsigned char value, size_t head,
                                                         size_t vecs) {
    const size_t tid = (size_t)blockIdx.x * 256 + threadIdx.x, nthreads = (size_t)gridDim.x * 256;
    const uint32_t w = value * 0x01010101u;
    uint4 *body = (uint4 *)(dst + head);
    for (size_t i = tid; i < vecs; i += nthreads) body[i] = make_uint4(w, w, w, w);
    const size_t tail0 = head + vecs * 16;
    for (size_t i = tid; i < head; i += nthreads) dst[i] = value;
    for (size_t i = tail0 + tid; i < bytes; i += nthreads) dst[i] = value;
}

int launch_fill_bytes(void *dst, int value, size_t bytes, hipStream_t stream) {
    if (bytes == 0) return FHIP_OK;
    size_t head = (16 - ((uintptr_t)dst & 15)) & 15;
    if (head > bytes) head = bytes;
    const size_t vecs = (bytes - head) / 16;
    hipLaunchKernelGGL(fill_bytes_kernel, dim3(grid_for((int64_t)(vecs > 256 ? vecs : 256))), dim3(256), 0, stream,
                       (unsigned char *)dst, bytes, (unsigned char)value, head, vecs);
    FHIP_HIP_CHECK(hipGetLastError());
    return FHIP_OK;
}

int launch_copy_rows(const void *src, const int64_t sstride[4], void *dst, const int64_t dstride[4],
                     const uint32_t shape[4], int elem_bytes, hipStream_t stream) {
    return copy_or_zero(src, sstride, dst, dstride, shape, elem_bytes, false, stream);
}

int launch_fill_zero_rows(void *dst, const int64_t dstride[4], const uint32_t shape[4], int elem_bytes,
                          hipStream_t stream) {
    return copy_or_zero(nullptr, dstride, dst, dstride, shape, elem_bytes, true, stream);
}

}  // namespace fhip
