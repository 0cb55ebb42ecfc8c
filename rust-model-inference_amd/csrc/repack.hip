// Upload-time repacking of GGUF block rows into the HBM tile streams described
// in rmi_internal.h, and the row copier behind fuse_vstack.  A weight arrives in
// chunks of whole tiles: `src` holds the rows from tile `tile0` on, the grid
// covers the tiles of the chunk.
#include "rmi_internal.h"

namespace {

// One workgroup per (tile, octet) of the destination.
__global__ __launch_bounds__(256) void repack_q8_0_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                           uint32_t n_out, uint32_t nb, uint32_t n_oct, uint32_t tile0) {
    const uint32_t tile = tile0 + blockIdx.x / n_oct;
    const uint32_t o = blockIdx.x % n_oct;
    const uint32_t tid = threadIdx.x;
    const uint32_t row0 = tile0 * kTileRows;
    uint8_t *tile_base = dst + size_t(tile) * n_oct * kOctetBytes;
    const size_t row_stride = size_t(nb) * 34;

    if (tid < 64) {
        const uint32_t r = tid >> 3, jj = tid & 7;
        const uint32_t row = tile * kTileRows + r, blk = o * 8 + jj;
        uint16_t d = 0;
        if (row < n_out && blk < nb) {
            const uint8_t *p = src + (row - row0) * row_stride + size_t(blk) * 34;
            d = uint16_t(p[0]) | (uint16_t(p[1]) << 8);
        }
        reinterpret_cast<uint16_t *>(tile_base + size_t(o) * 128 + r * 16)[jj] = d;
    }
    uint8_t *quants = tile_base + size_t(n_oct) * 128;
    for (uint32_t idx = tid; idx < 512; idx += 256) {
        const uint32_t ql = idx >> 8, rem = idx & 255;
        const uint32_t r = rem >> 5, L = (rem >> 2) & 7, j = rem & 3;
        const uint32_t row = tile * kTileRows + r, q = 2 * o + ql, blk = q * 4 + j;
        uint32_t v = 0;
        if (row < n_out && blk < nb) {
            const uint8_t *p = src + (row - row0) * row_stride + size_t(blk) * 34 + 2 + 4 * L;
            v = uint32_t(p[0]) | (uint32_t(p[1]) << 8) | (uint32_t(p[2]) << 16) | (uint32_t(p[3]) << 24);
        }
        reinterpret_cast<uint32_t *>(quants + size_t(q) * 1024 + (r * 8 + L) * 16)[j] = v;
    }
}

// One workgroup per (tile, super-block) of the destination: 288 dwords.
__global__ __launch_bounds__(256) void repack_q4_k_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                           uint32_t n_out, uint32_t n_sb, uint32_t tile0) {
    const uint32_t tile = tile0 + blockIdx.x / n_sb;
    const uint32_t sb = blockIdx.x % n_sb;
    uint32_t *chunk = reinterpret_cast<uint32_t *>(dst + (size_t(tile) * n_sb + sb) * kQ4KSuperBytes);
    for (uint32_t idx = threadIdx.x; idx < 288; idx += 256) {
        uint32_t r, src_dword;
        if (idx < 32) {  // header: d, dmin, 12 scale bytes
            r = idx >> 2;
            src_dword = idx & 3;
        } else {  // quants: (r, L, g) <- nibble bytes 32g + 4L
            const uint32_t k = idx - 32;
            r = k >> 5;
            const uint32_t L = (k >> 2) & 7, g = k & 3;
            src_dword = 4 + 8 * g + L;
        }
        const uint32_t row = tile * kTileRows + r;
        uint32_t v = 0;
        if (row < n_out)
            v = reinterpret_cast<const uint32_t *>(src + (size_t(row - tile0 * kTileRows) * n_sb + sb) * 144)[src_dword];
        chunk[idx] = v;
    }
}

// One workgroup per (tile, super-block) of the destination: 420 dwords.
__global__ __launch_bounds__(256) void repack_q6_k_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                           uint32_t n_out, uint32_t n_sb, uint32_t tile0) {
    const uint32_t tile = tile0 + blockIdx.x / n_sb;
    const uint32_t sb = blockIdx.x % n_sb;
    uint8_t *chunk = dst + (size_t(tile) * n_sb + sb) * kQ6KSuperBytes;
    // the 210-byte source blocks are only 2-byte aligned: move 16-bit units
    for (uint32_t idx = threadIdx.x; idx < 840; idx += 256) {
        uint32_t r, src_half;  // destination 16-bit unit idx <- unit src_half of row r's block
        if (idx < 64) {        // scales
            r = idx >> 3;
            src_half = 96 + (idx & 7);
        } else if (idx < 72) {  // d
            r = idx - 64;
            src_half = 104;
        } else if (idx < 584) {  // ql: (r, L, c) <- bytes 32c + 4L.. ; two units per dword
            const uint32_t k = idx - 72;
            r = k >> 6;
            const uint32_t L = (k >> 3) & 7, c = (k >> 1) & 3, h = k & 1;
            src_half = 16 * c + 2 * L + h;
        } else {  // qh: (r, L, c) <- bytes 128 + 32c + 4L..
            const uint32_t k = idx - 584;
            r = k >> 5;
            const uint32_t L = (k >> 2) & 7, c = (k >> 1) & 1, h = k & 1;
            src_half = 64 + 16 * c + 2 * L + h;
        }
        const uint32_t row = tile * kTileRows + r;
        uint16_t v = 0;
        if (row < n_out)
            v = reinterpret_cast<const uint16_t *>(src + (size_t(row - tile0 * kTileRows) * n_sb + sb) * 210)[src_half];
        reinterpret_cast<uint16_t *>(chunk)[idx] = v;
    }
}

// uint4 index, inside one tile, of piece p of (unit u, row r).
__device__ __forceinline__ uint32_t piece_index(int dtype, uint32_t n_units, uint32_t u, uint32_t r, uint32_t p) {
    if (dtype == RMI_HIP_DTYPE_Q8_0) {
        if (p == 0) return u * 8 + r;
        const uint32_t q = 2 * u + ((p - 1) >> 3), L = (p - 1) & 7;
        return n_units * 8 + q * 64 + r * 8 + L;
    }
    if (dtype == RMI_HIP_DTYPE_Q6_K) {  // 105 uint4 per unit; piece 0 scales, 1..8 ql, 9..12 qh (d is copied apart)
        if (p == 0) return u * 105 + r;
        if (p < 9) return u * 105 + 9 + r * 8 + (p - 1);
        return u * 105 + 73 + r * 4 + (p - 9);
    }
    if (p == 0) return u * 72 + r;
    return u * 72 + 8 + r * 8 + (p - 1);
}

__host__ __device__ __forceinline__ uint32_t pieces_of(int dtype) {
    return dtype == RMI_HIP_DTYPE_Q8_0 ? 17 : (dtype == RMI_HIP_DTYPE_Q6_K ? 13 : 9);
}

__global__ __launch_bounds__(256) void copy_rows_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst,
                                                         int dtype, uint32_t n_rows, uint32_t n_units,
                                                         uint32_t tile_u4, uint32_t dst_row0) {
    const uint32_t pieces = pieces_of(dtype);
    const uint64_t total = uint64_t(n_rows) * n_units * pieces;
    for (uint64_t i = blockIdx.x * uint64_t(blockDim.x) + threadIdx.x; i < total;
         i += uint64_t(gridDim.x) * blockDim.x) {
        const uint32_t p = uint32_t(i % pieces);
        const uint64_t ru = i / pieces;
        const uint32_t u = uint32_t(ru % n_units);
        const uint32_t row = uint32_t(ru / n_units);
        const uint32_t drow = dst_row0 + row;
        const uint4 v = src[size_t(row >> 3) * tile_u4 + piece_index(dtype, n_units, u, row & 7, p)];
        dst[size_t(drow >> 3) * tile_u4 + piece_index(dtype, n_units, u, drow & 7, p)] = v;
        if (dtype == RMI_HIP_DTYPE_Q6_K && p == 0) {  // the row's f16 d: 8 rows share one uint4
            const uint16_t *s16 = reinterpret_cast<const uint16_t *>(src + size_t(row >> 3) * tile_u4 + u * 105 + 8);
            uint16_t *d16 = reinterpret_cast<uint16_t *>(dst + size_t(drow >> 3) * tile_u4 + u * 105 + 8);
            d16[drow & 7] = s16[row & 7];
        }
    }
}

}  // namespace

int rmi_launch_repack_q8_0(const uint8_t *src, rmi_hip_weight *w, uint32_t tile0, uint32_t n_tiles, hipStream_t s) {
    const uint32_t grid = n_tiles * w->n_units;
    if (grid == 0) return RMI_HIP_OK;
    hipLaunchKernelGGL(repack_q8_0_kernel, dim3(grid), dim3(256), 0, s, src, w->data, w->n_out, w->n_in / 32,
                       w->n_units, tile0);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

int rmi_launch_repack_q4_k(const uint8_t *src, rmi_hip_weight *w, uint32_t tile0, uint32_t n_tiles, hipStream_t s) {
    const uint32_t grid = n_tiles * w->n_units;
    if (grid == 0) return RMI_HIP_OK;
    hipLaunchKernelGGL(repack_q4_k_kernel, dim3(grid), dim3(256), 0, s, src, w->data, w->n_out, w->n_units, tile0);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

int rmi_launch_repack_q6_k(const uint8_t *src, rmi_hip_weight *w, uint32_t tile0, uint32_t n_tiles, hipStream_t s) {
    const uint32_t grid = n_tiles * w->n_units;
    if (grid == 0) return RMI_HIP_OK;
    hipLaunchKernelGGL(repack_q6_k_kernel, dim3(grid), dim3(256), 0, s, src, w->data, w->n_out, w->n_units, tile0);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

int rmi_launch_copy_rows(const rmi_hip_weight *src, rmi_hip_weight *dst, uint32_t dst_row0, hipStream_t s) {
    if (src->n_out == 0 || src->n_units == 0) return RMI_HIP_OK;
    if (src->dtype != dst->dtype || src->n_units != dst->n_units || dst_row0 + src->n_out > dst->n_out)
        return rmi_fail(RMI_HIP_E_INVALID, "copy_rows: layouts differ");
    const uint32_t pieces = pieces_of(src->dtype);
    const uint64_t total = uint64_t(src->n_out) * src->n_units * pieces;
    const uint32_t grid = uint32_t(total / 256 + 1 < 65535 ? total / 256 + 1 : 65535);
    hipLaunchKernelGGL(copy_rows_kernel, dim3(grid), dim3(256), 0, s, reinterpret_cast<const uint4 *>(src->data),
                       reinterpret_cast<uint4 *>(dst->data), src->dtype, src->n_out, src->n_units,
                       uint32_t(src->tile_bytes / 16), dst_row0);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}
