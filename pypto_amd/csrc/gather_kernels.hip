// Paged row gather - gfx950 kernel.
//
// Replaces the device side of gather_in_ub / gather_in_l1 (python/pypto/experimental/gather.py:18-84; semantics
// framework/src/interface/interpreter/calculator/calc_torch.cpp:1870-1981):
//   out[j, :size] = src[ page[idx[j] / bs] * bs + idx[j] % bs , :size ]
// for a batch of independent (index row, page-table row) pairs.  The reference's interpreter asserts that every
// logical index lies inside the page table and maps to a row of src; on the device such an entry cannot stop the
// launch, so its output row is written as zeros and, when the caller passed a status word, counted there.
//
// The op is a pure HBM stream: algorithmic bytes per output row = 2 * size * element bytes + the index (4 or 8 bytes).
// One workgroup owns 32 output rows: 32 lanes resolve the rows' physical addresses once (index -> page -> row, two
// dependent loads) into LDS, then all 256 lanes copy the rows in pieces of V bytes (V = 16 when the row width, the
// source pitch and both base addresses allow it), consecutive lanes taking consecutive pieces of a row; every lane
// requests four pieces before it stores the first, so a workgroup has up to 16 KB of reads in flight.
#include "common.h"
#include "kernels.h"
#include "timing.h"

namespace pto {
namespace {

constexpr int GROWS = 32; // output rows per workgroup
constexpr int GUNROLL = 4;

template <int V>
struct Piece;
template <>
struct Piece<16> { typedef u32x4 type; };
template <>
struct Piece<8> { typedef u32x2 type; };
template <>
struct Piece<4> { typedef uint32_t type; };
template <>
struct Piece<2> { typedef uint16_t type; };
template <>
struct Piece<1> { typedef uint8_t type; };

__device__ __forceinline__ int64_t load_index(const void* p, bool is64, int64_t i)
{
    return is64 ? static_cast<const int64_t*>(p)[i] : (int64_t) static_cast<const int32_t*>(p)[i];
}

template <int V>
__global__ __launch_bounds__(256) void paged_gather_kernel(GatherArgs a)
{
    typedef typename Piece<V>::type vec_t;
    __shared__ int64_t s_row[GROWS]; // byte offset of the source row, -1 = no such row
    const int tid = threadIdx.x;
    const int64_t row0 = (int64_t)blockIdx.x * GROWS;
    if (tid < GROWS) {
        const int64_t j = row0 + tid;
        int64_t off = -1;
        if (j < a.rows) {
            const int64_t bi = j / a.k;
            const int64_t idx = load_index(a.indices, a.idx64, j);
            if (idx >= 0 && idx < a.nblk * a.block_size) {
                const int64_t lb = idx / a.block_size;
                const int64_t page = load_index(a.block_table, a.bt64, bi * a.nblk + lb);
                const int64_t r = page * a.block_size + (idx - lb * a.block_size);
                if (page >= 0 && r < a.n_src) off = r * a.src_pitch;
            }
            if (off < 0 && a.status != nullptr) atomicAdd(a.status, 1);
        }
        s_row[tid] = off;
    }
    __syncthreads();
    const int nrows = (int)min((int64_t)GROWS, a.rows - row0);
    const uint32_t pieces = (uint32_t)(a.row_bytes / V); // per row; the host keeps GROWS * pieces below 2^31
    const uint32_t total = (uint32_t)nrows * pieces;
    const uint8_t* src = static_cast<const uint8_t*>(a.src);
    uint8_t* out = static_cast<uint8_t*>(a.out) + row0 * a.row_bytes;
    for (uint32_t base = 0; base < total; base += 256 * GUNROLL) {
        vec_t v[GUNROLL];
        uint32_t dst[GUNROLL];
#pragma unroll
        for (int u = 0; u < GUNROLL; ++u) {
            const uint32_t p = base + u * 256 + tid;
            v[u] = vec_t{};
            dst[u] = 0xffffffffu;
            if (p < total) {
                const uint32_t r = p / pieces, c = p - r * pieces;
                const int64_t off = s_row[r];
                dst[u] = p; // out is row-major with pitch row_bytes: piece p of the workgroup sits at p * V
                if (off >= 0) v[u] = *reinterpret_cast<const vec_t*>(src + off + (int64_t)c * V);
            }
        }
#pragma unroll
        for (int u = 0; u < GUNROLL; ++u)
            // (streaming stores: the output is written once and not read here; kept out of the caches it leaves them to
            // the random row reads - 16.0 -> 15.1 us at 32 x 2048 rows of 656 bytes)
            if (dst[u] != 0xffffffffu) __builtin_nontemporal_store(v[u], reinterpret_cast<vec_t*>(out + (int64_t)dst[u] * V));
    }
}

} // namespace

hipError_t paged_gather_launch(const GatherArgs& a, hipStream_t stream)
{
    if (a.rows == 0 || a.row_bytes == 0) return hipSuccess;
    // widest piece that divides the row, the source pitch and both base addresses
    const uint64_t bits = (uint64_t)a.row_bytes | (uint64_t)a.src_pitch | reinterpret_cast<uint64_t>(a.src) |
                          reinterpret_cast<uint64_t>(a.out);
    int v = 16;
    while (v > 1 && (bits & (uint64_t)(v - 1))) v >>= 1;
    if (a.row_bytes / v > (int64_t)(0x7fffffff / GROWS)) return hipErrorInvalidValue;
    const int64_t groups = (a.rows + GROWS - 1) / GROWS;
    if (groups > 0x7fffffff) return hipErrorInvalidValue;
    const dim3 grid((unsigned)groups), block(256);
    ScopedKernelTimer tm(KID_PAGED_GATHER, stream);
    switch (v) {
        case 16: hipLaunchKernelGGL(paged_gather_kernel<16>, grid, block, 0, stream, a); break;
        case 8: hipLaunchKernelGGL(paged_gather_kernel<8>, grid, block, 0, stream, a); break;
        case 4: hipLaunchKernelGGL(paged_gather_kernel<4>, grid, block, 0, stream, a); break;
        case 2: hipLaunchKernelGGL(paged_gather_kernel<2>, grid, block, 0, stream, a); break;
        default: hipLaunchKernelGGL(paged_gather_kernel<1>, grid, block, 0, stream, a); break;
    }
    return hipGetLastError();
}

} // namespace pto
