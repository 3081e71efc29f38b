// Precompiled device kernels of the "HIP" policy that are not generated per contraction:
// fill / scale (reference util/CudaUtil.cpp:123-140), batched 1x1 / 2x2 / 3x3 inverse, determinant and fused
// inverse+determinant (reference ops/CudaGPUOps.cpp:13-80,108-275), indexed scatter and compressed-row sum-gather
// (reference ops/CudaGPUOps.cpp:83-105,278-302).
//
// Layout: matrices are stored one after the other (9, 4 or 1 doubles each).  A workgroup of 64 lanes (one wavefront,
// so its barriers cost nothing) owns 64 consecutive matrices; it moves their doubles between HBM and LDS with
// unit-stride 16-byte accesses and each lane then works on "its" matrix out of LDS, so HBM only sees full,
// contiguous lines.  The lane stride in LDS is 9 (or 4+1 padded to 5) doubles, which maps the lanes onto distinct
// banks.  1 x 1 "matrices" have a plain streaming kernel of their own (256 lanes, four entries each).
//
// Arithmetic is written term by term in the order of the reference's ops/NativeCPUOps.hpp:38-86 and compiled
// without multiply-add contraction, so results are bit-identical to the host formulas.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdlib>

#include "HipRuntime.hpp"
#include "NonContractionOps.hpp"

#pragma clang fp contract(off)

namespace acro
{

namespace
{

typedef double Double2 __attribute__((ext_vector_type(2)));  // a 16-byte access the compiler keeps whole
typedef int Int2 __attribute__((ext_vector_type(2)));

constexpr int kLanes = 256;    // fill, scale, scatter, gather
constexpr int kMatLanes = 64;  // batched matrices: one wavefront per workgroup, so its barriers are free

// Fill and scale move 16 bytes per lane and write with non-temporal stores (the result is not read again by the
// kernel).  When the buffer starts on an odd multiple of 8 bytes its first entry is handled alone, so that the body
// is 16-byte aligned; that entry and an odd last one go to the lane after the last pair.
__global__ __launch_bounds__(kLanes) void fillKernel(double *__restrict__ d, double value, size_t n)
{
    const size_t head = ((reinterpret_cast<uintptr_t>(d) & 8) != 0 && n > 0) ? 1 : 0;
    const size_t pairs = (n - head) / 2;
    const size_t p = static_cast<size_t>(blockIdx.x) * kLanes + threadIdx.x;
    if (p < pairs) __builtin_nontemporal_store(Double2{value, value}, reinterpret_cast<Double2 *>(d + head) + p);
    if (p == pairs)
    {
        if (head) d[0] = value;
        if ((n - head) & 1) d[n - 1] = value;
    }
}

__global__ __launch_bounds__(kLanes) void scaleKernel(double *__restrict__ d, double factor, size_t n)
{
    const size_t head = ((reinterpret_cast<uintptr_t>(d) & 8) != 0 && n > 0) ? 1 : 0;
    const size_t pairs = (n - head) / 2;
    const size_t p = static_cast<size_t>(blockIdx.x) * kLanes + threadIdx.x;
    if (p < pairs)
    {
        Double2 *q = reinterpret_cast<Double2 *>(d + head) + p;
        const Double2 v = *q;
        __builtin_nontemporal_store(Double2{v.x * factor, v.y * factor}, q);
    }
    if (p == pairs)
    {
        if (head) d[0] *= factor;
        if ((n - head) & 1) d[n - 1] *= factor;
    }
}

template <int M>
struct SmallMatrix;

template <>
struct SmallMatrix<1>
{
    static __device__ double det(const double *A) { return A[0]; }
    static __device__ void inv(double *Ainv, const double *, double det) { Ainv[0] = 1.0 / det; }
};

template <>
struct SmallMatrix<2>
{
    static __device__ double det(const double *A) { return A[0] * A[3] - A[1] * A[2]; }
    static __device__ void inv(double *Ainv, const double *A, double det)
    {
        const double invdet = 1.0 / det;
        Ainv[0] = invdet * A[3];
        Ainv[1] = -invdet * A[1];
        Ainv[2] = -invdet * A[2];
        Ainv[3] = invdet * A[0];
    }
};

template <>
struct SmallMatrix<3>
{
    static __device__ double det(const double *A)
    {
        return A[0] * A[4] * A[8] + A[1] * A[5] * A[6] + A[2] * A[3] * A[7] - A[6] * A[4] * A[2] -
               A[7] * A[5] * A[0] - A[8] * A[3] * A[1];
    }
    // Cofactors over the determinant WITHOUT the final transposition: for a non-symmetric matrix this is the
    // transpose of the inverse, which is what the reference's host and device code both produce.
    static __device__ void inv(double *Ainv, const double *A, double det)
    {
        const double invdet = 1.0 / det;
        Ainv[0] = invdet * (A[4] * A[8] - A[5] * A[7]);
        Ainv[1] = invdet * (A[5] * A[6] - A[3] * A[8]);
        Ainv[2] = invdet * (A[3] * A[7] - A[4] * A[6]);
        Ainv[3] = invdet * (A[2] * A[7] - A[1] * A[8]);
        Ainv[4] = invdet * (A[0] * A[8] - A[2] * A[6]);
        Ainv[5] = invdet * (A[1] * A[6] - A[0] * A[7]);
        Ainv[6] = invdet * (A[1] * A[5] - A[2] * A[4]);
        Ainv[7] = invdet * (A[2] * A[3] - A[0] * A[5]);
        Ainv[8] = invdet * (A[0] * A[4] - A[1] * A[3]);
    }
};

// 1 x 1 "matrices" (ops/NativeCPUOps.hpp:38-44: the determinant is the entry, the inverse its reciprocal): a plain
// stream, four entries per lane in workgroups of kLanes, so that the launch is bound by memory and not by the rate at
// which 64-lane workgroups start (2^25 entries: 113 us either way with one workgroup per 64 entries).
template <bool WANT_INV, bool WANT_DET>
__global__ __launch_bounds__(kLanes) void batchScalarKernel(const double *__restrict__ A, double *__restrict__ Ainv,
                                                            double *__restrict__ Adet, size_t n)
{
    const size_t first = (static_cast<size_t>(blockIdx.x) * kLanes) * 4 + threadIdx.x;
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        const size_t i = first + static_cast<size_t>(j) * kLanes;
        if (i >= n) break;
        const double det = A[i];
        if (WANT_DET) __builtin_nontemporal_store(det, &Adet[i]);
        if (WANT_INV) __builtin_nontemporal_store(1.0 / det, &Ainv[i]);
    }
}

// One workgroup = kMatLanes consecutive matrices.  WANT_INV / WANT_DET select the outputs.
// The matrices of a workgroup are contiguous in memory, so the workgroup copies them to and from LDS as one
// stream of 16-byte pieces (full-rate HBM access), and lane t works on matrix t out of LDS.  For 2x2 the lane
// stride in LDS is padded from 4 to 5 doubles so that lanes fall into distinct banks; 9 and 1 are odd already.
// PAIRS: the matrices and the inverses start at a multiple of 16 bytes and are read and written as pairs of doubles;
// otherwise (a slice at an odd offset, a caller's device buffer) one double at a time.
template <int M, bool WANT_INV, bool WANT_DET, bool PAIRS>
__global__ __launch_bounds__(kMatLanes) void batchMatrixKernel(const double *__restrict__ A, double *__restrict__ Ainv,
                                                            double *__restrict__ Adet, size_t num_mat)
{
    constexpr int MM = M * M;
    constexpr int LS = (MM % 2 == 0) ? MM + 1 : MM;  // odd lane stride in doubles: no LDS bank conflicts
    __shared__ double tile[kMatLanes * LS];

    const size_t first = static_cast<size_t>(blockIdx.x) * kMatLanes;
    const size_t count = (num_mat - first < static_cast<size_t>(kMatLanes)) ? num_mat - first : kMatLanes;
    const int ndbl = static_cast<int>(count) * MM;
    const double *src = A + first * MM;

    // first * MM * 8 bytes is a multiple of 16 (kMatLanes is even), so pairs of doubles are aligned when A is
    for (int i = threadIdx.x; i < ndbl / 2; i += kMatLanes)
    {
        double2 v;
        if (PAIRS)
        {
            // one instruction of the wavefront reads 1 KB of whole lines that nothing reads again: non-temporal (2^22
            // 3 x 3 matrices from HBM: 108.6 -> 101.1 us; workgroups of 128 or 256 lanes and two matrices per lane
            // measured slower with either kind of load)
            const Double2 w = __builtin_nontemporal_load(reinterpret_cast<const Double2 *>(src) + i);
            v.x = w.x;
            v.y = w.y;
        }
        else
        {
            v.x = src[2 * i];
            v.y = src[2 * i + 1];
        }
        if (LS == MM)
        {
            tile[2 * i] = v.x;
            tile[2 * i + 1] = v.y;
        }
        else
        {
            tile[((2 * i) / MM) * LS + ((2 * i) % MM)] = v.x;
            tile[((2 * i + 1) / MM) * LS + ((2 * i + 1) % MM)] = v.y;
        }
    }
    if ((ndbl & 1) && threadIdx.x == 0) tile[((ndbl - 1) / MM) * LS + ((ndbl - 1) % MM)] = src[ndbl - 1];
    __syncthreads();

    double a[MM], r[MM];
    const bool active = threadIdx.x < count;
    if (active)
    {
#pragma unroll
        for (int j = 0; j < MM; ++j) a[j] = tile[threadIdx.x * LS + j];
        const double det = SmallMatrix<M>::det(a);
        if (WANT_DET) __builtin_nontemporal_store(det, &Adet[first + threadIdx.x]);
        if (WANT_INV) SmallMatrix<M>::inv(r, a, det);
    }
    if (WANT_INV)
    {
        __syncthreads();
        if (active)
        {
#pragma unroll
            for (int j = 0; j < MM; ++j) tile[threadIdx.x * LS + j] = r[j];
        }
        __syncthreads();
        double *dst = Ainv + first * MM;
        for (int i = threadIdx.x; i < ndbl / 2; i += kMatLanes)
        {
            double2 v;
            if (LS == MM)
            {
                v.x = tile[2 * i];
                v.y = tile[2 * i + 1];
            }
            else
            {
                v.x = tile[((2 * i) / MM) * LS + ((2 * i) % MM)];
                v.y = tile[((2 * i + 1) / MM) * LS + ((2 * i + 1) % MM)];
            }
            // results stream out and are not read again here: non-temporal, like the generated kernels' outputs; one
            // 16-byte store per lane where the alignment allows, so that one instruction fills its lines
            if (PAIRS)
            {
                __builtin_nontemporal_store(Double2{v.x, v.y}, reinterpret_cast<Double2 *>(dst) + i);
            }
            else
            {
                __builtin_nontemporal_store(v.x, &dst[2 * i]);
                __builtin_nontemporal_store(v.y, &dst[2 * i + 1]);
            }
        }
        if ((ndbl & 1) && threadIdx.x == 0) dst[ndbl - 1] = tile[((ndbl - 1) / MM) * LS + ((ndbl - 1) % MM)];
    }
}

// Consecutive workgroup ids are dealt round-robin to the 8 XCDs, each with an L2 of its own.  The index kernels
// gather through a map with spatial locality (neighbouring range entries touch neighbouring domain entries), so
// within every block of 8 * kXcdRun workgroup ids each XCD is given kXcdRun neighbouring pieces of the work instead
// of every eighth: lines that neighbouring workgroups share are then fetched once, not once per XCD.  The blocks
// keep the workgroups that run at the same time on one narrow window of memory: with one contiguous eighth of
// the whole range per XCD (eight windows far apart) re-launches on cache-resident data ran as fast, but on data
// that comes from HBM the scatter took 55.9 instead of 45.5 us and the sum-gather 65.3 instead of 59.6 us on the
// 64^3-element degree-3 mesh (plain ids: 46.7 and 61.7 us).
constexpr unsigned kXcdRun = 32;

__device__ inline unsigned xcdContiguousBlock()
{
    constexpr unsigned blk = 8 * kXcdRun;
    const unsigned b = blockIdx.x;
    if (b >= gridDim.x / blk * blk) return b;
    return b / blk * blk + (b % 8) * kXcdRun + (b / 8) % kXcdRun;
}

__global__ __launch_bounds__(kLanes) void scatterKernel(double *__restrict__ Aout, const double *__restrict__ Ain,
                                                        const int *__restrict__ M, int range_size)
{
    int i = blockIdx.x * kLanes + threadIdx.x;
    if (i < range_size) Aout[i] = Ain[M[i]];
}

// Two consecutive range entries per access and kScatterPairs accesses per lane, adjacent lanes on adjacent pairs:
// every load of map entries (8 bytes per lane) and every store (16 bytes per lane) of a wavefront covers whole
// lines, and a lane has 2 * kScatterPairs gathers in flight.  The result streams out with non-temporal stores
// (they only pay off when one store instruction fills its lines: with four consecutive entries per lane, i.e. two
// half-covering instructions per line, they were 1.5x slower than ordinary stores).  Needs Aout aligned to 16 and
// M to 8 bytes; an odd last entry goes to the lane after the last pair.
constexpr int kScatterPairs = 2;

__global__ __launch_bounds__(kLanes) void scatterKernel2(double *__restrict__ Aout, const double *__restrict__ Ain,
                                                         const int *__restrict__ M, int range_size)
{
    const int pairs = range_size / 2;
    const int base = xcdContiguousBlock() * (kLanes * kScatterPairs) + threadIdx.x;
    int2 m[kScatterPairs];
#pragma unroll
    for (int u = 0; u < kScatterPairs; ++u)
    {
        const int p = base + u * kLanes;
        // (the map streams through once, in whole lines per load instruction: non-temporal, so that it does not displace
        // the lines of Ain that neighbouring workgroups share; 64^3 hexahedra of degree 3 from HBM: 45.5 -> 41.2 us.  The
        // same hint on the sum-gather's map, whose chunks start anywhere in a line: 55.2 -> 56.5 us, not taken.)
        const Int2 w = p < pairs ? __builtin_nontemporal_load(reinterpret_cast<const Int2 *>(M) + p) : Int2{0, 0};
        m[u] = make_int2(w.x, w.y);
    }
    double a[kScatterPairs][2];
#pragma unroll
    for (int u = 0; u < kScatterPairs; ++u)
    {
        a[u][0] = Ain[m[u].x];
        a[u][1] = Ain[m[u].y];
    }
#pragma unroll
    for (int u = 0; u < kScatterPairs; ++u)
    {
        const int p = base + u * kLanes;
        if (p < pairs) __builtin_nontemporal_store(Double2{a[u][0], a[u][1]}, reinterpret_cast<Double2 *>(Aout) + p);
        if (p == pairs && (range_size & 1)) Aout[range_size - 1] = Ain[M[range_size - 1]];
    }
}

// Row d of the inverse map lists, in increasing range order, the entries that are added into Aout[d]; summing
// them front to back reproduces the sequential host scatter-add bit for bit and needs no atomics.
// A workgroup owns kGatherRows * kLanes consecutive rows.  Their entries are consecutive in the inverse map, so the workgroup
// walks that range in chunks: all lanes gather a chunk into LDS (unit-stride reads of the map, eight gathers in
// flight per lane whatever the row lengths are), then the lane of each row adds the part of its row that lies in
// the chunk, in row order.  Rows are short on average (2.3 entries for a hexahedral mesh) and uneven (1 to 8), so
// one lane walking its own row leaves most of a wavefront's gather slots empty.
// A chunk should hold all entries of the workgroup's rows: every further chunk is another chain of dependent loads (map,
// then values) behind a barrier.  Lines of mesh nodes that lie on element faces have 3.6 entries per row; with 1 024 rows
// and chunks of 2 048 those workgroups took two chunks (64^3 hexahedra of degree 3, tensors that exceed the memory-side
// cache: 59.5 us); 512 rows per chunk of 2 048, or 1 024 per 4 096: 55.2 us; 256 rows: 57.9 us; 2 048 rows: 64 us.
constexpr int kGatherPerLane = 8;
constexpr int kGatherChunk = kGatherPerLane * kLanes;
constexpr int kGatherRows = 2;  // rows per lane

__global__ __launch_bounds__(kLanes) void sumGatherKernel(double *__restrict__ Aout, const double *__restrict__ Ain,
                                                          const int *__restrict__ InvM,
                                                          const int *__restrict__ InvMOff, int domain_size)
{
    __shared__ double vals[kGatherChunk];
    const int d0 = xcdContiguousBlock() * (kLanes * kGatherRows);  // first row of this workgroup
    if (d0 >= domain_size) return;
    const int dEnd = d0 + kLanes * kGatherRows < domain_size ? d0 + kLanes * kGatherRows : domain_size;
    const int first = InvMOff[d0], last = InvMOff[dEnd];
    int rowBegin[kGatherRows], rowEnd[kGatherRows];
    double sum[kGatherRows];
#pragma unroll
    for (int r = 0; r < kGatherRows; ++r)
    {
        const int d = d0 + r * kLanes + threadIdx.x;
        rowBegin[r] = d < domain_size ? InvMOff[d] : 0;
        rowEnd[r] = d < domain_size ? InvMOff[d + 1] : 0;
        sum[r] = 0.0;
    }
    for (int c = first; c < last; c += kGatherChunk)
    {
        const int n = last - c < kGatherChunk ? last - c : kGatherChunk;
        int idx[kGatherPerLane];
        double a[kGatherPerLane];
#pragma unroll
        for (int u = 0; u < kGatherPerLane; ++u)
        {
            const int j = threadIdx.x + u * kLanes;
            idx[u] = j < n ? InvM[c + j] : -1;
        }
#pragma unroll
        for (int u = 0; u < kGatherPerLane; ++u) a[u] = idx[u] >= 0 ? Ain[idx[u]] : 0.0;
#pragma unroll
        for (int u = 0; u < kGatherPerLane; ++u) vals[threadIdx.x + u * kLanes] = a[u];
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kGatherRows; ++r)
        {
            const int lo = rowBegin[r] > c ? rowBegin[r] : c;
            const int hi = rowEnd[r] < c + n ? rowEnd[r] : c + n;
            for (int k = lo; k < hi; ++k) sum[r] += vals[k - c];
        }
        __syncthreads();
    }
#pragma unroll
    for (int r = 0; r < kGatherRows; ++r)
    {
        const int d = d0 + r * kLanes + threadIdx.x;
        if (d < domain_size) __builtin_nontemporal_store(sum[r], &Aout[d]);
    }
}

unsigned gridFor(size_t n)
{
    size_t blocks = (n + kLanes - 1) / kLanes;
    ACROBATIC_ASSERT(blocks <= 0x7fffffffu, "Operand too large for a one-dimensional grid.");
    return static_cast<unsigned>(blocks == 0 ? 1 : blocks);
}

hipStream_t stream()
{
    return static_cast<hipStream_t>(hip::Stream());
}

template <bool WANT_INV, bool WANT_DET>
void launchBatchMatrix(int mdim, const double *A, double *Ainv, double *Adet, size_t num_mat)
{
    const size_t groups = (num_mat + kMatLanes - 1) / kMatLanes;
    ACROBATIC_ASSERT(groups <= 0x7fffffffu, "Operand too large for a one-dimensional grid.");
    const unsigned grid = static_cast<unsigned>(groups == 0 ? 1 : groups);
    const bool pairs = reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(Ainv) % 16 == 0;
#define ACRO_LAUNCH_BATCH_MATRIX(M)                                                                                   \
    if (pairs)                                                                                                        \
        hipLaunchKernelGGL((batchMatrixKernel<M, WANT_INV, WANT_DET, true>), dim3(grid), dim3(kMatLanes), 0, stream(), \
                           A, Ainv, Adet, num_mat);                                                                   \
    else                                                                                                              \
        hipLaunchKernelGGL((batchMatrixKernel<M, WANT_INV, WANT_DET, false>), dim3(grid), dim3(kMatLanes), 0,          \
                           stream(), A, Ainv, Adet, num_mat)
    switch (mdim)
    {
        case 1:
        {
            const size_t blocks = (num_mat + 4 * kLanes - 1) / (4 * kLanes);
            ACROBATIC_ASSERT(blocks <= 0x7fffffffu, "Operand too large for a one-dimensional grid.");
            hipLaunchKernelGGL((batchScalarKernel<WANT_INV, WANT_DET>), dim3(static_cast<unsigned>(blocks == 0 ? 1 : blocks)),
                               dim3(kLanes), 0, stream(), A, Ainv, Adet, num_mat);
            break;
        }
        case 2:
            ACRO_LAUNCH_BATCH_MATRIX(2);
            break;
        case 3:
            ACRO_LAUNCH_BATCH_MATRIX(3);
            break;
        default:
            ACROBATIC_ASSERT(false, "Batched matrix ops support 1x1, 2x2 and 3x3 matrices only.");
    }
#undef ACRO_LAUNCH_BATCH_MATRIX
    ACRO_HIP_CHECK(hipGetLastError());
}

size_t numMatrices(const Tensor &A)
{
    const int m = A.GetDim(A.GetRank() - 1);
    return static_cast<size_t>(A.GetSize()) / (static_cast<size_t>(m) * m);
}

}  // namespace

namespace hip
{

void FillDouble(double *d, double value, size_t n)
{
    hipLaunchKernelGGL(fillKernel, dim3(gridFor(n / 2 + 1)), dim3(kLanes), 0, stream(), d, value, n);
    ACRO_HIP_CHECK(hipGetLastError());
}

void ScaleDouble(double *d, double factor, size_t n)
{
    hipLaunchKernelGGL(scaleKernel, dim3(gridFor(n / 2 + 1)), dim3(kLanes), 0, stream(), d, factor, n);
    ACRO_HIP_CHECK(hipGetLastError());
}

}  // namespace hip

void HipGPUOps::BatchMatrixInverse(Tensor &Ainv, Tensor &A)
{
    launchBatchMatrix<true, false>(A.GetDim(A.GetRank() - 1), A.GetDeviceData(), Ainv.GetDeviceData(), nullptr,
                                   numMatrices(A));
}

void HipGPUOps::BatchMatrixDet(Tensor &Adet, Tensor &A)
{
    launchBatchMatrix<false, true>(A.GetDim(A.GetRank() - 1), A.GetDeviceData(), nullptr, Adet.GetDeviceData(),
                                   numMatrices(A));
}

void HipGPUOps::BatchMatrixInvDet(Tensor &Ainv, Tensor &Adet, Tensor &A)
{
    launchBatchMatrix<true, true>(A.GetDim(A.GetRank() - 1), A.GetDeviceData(), Ainv.GetDeviceData(),
                                  Adet.GetDeviceData(), numMatrices(A));
}

void HipGPUOps::FlatIndexedScatter(Tensor &Aout, Tensor &Ain, IndexMapping &M)
{
    const int n = M.GetRangeSize();
    const bool aligned = reinterpret_cast<uintptr_t>(Aout.GetDeviceData()) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(M.GetMap().GetDeviceData()) % 8 == 0;
    if (aligned)
        hipLaunchKernelGGL(scatterKernel2, dim3(gridFor((static_cast<size_t>(n) / 2 + 1 + kScatterPairs - 1) / kScatterPairs)),
                           dim3(kLanes), 0, stream(), Aout.GetDeviceData(), Ain.GetDeviceData(),
                           M.GetMap().GetDeviceData(), n);
    else
        hipLaunchKernelGGL(scatterKernel, dim3(gridFor(n)), dim3(kLanes), 0, stream(), Aout.GetDeviceData(),
                           Ain.GetDeviceData(), M.GetMap().GetDeviceData(), n);
    ACRO_HIP_CHECK(hipGetLastError());
}

void HipGPUOps::FlatIndexedSumGather(Tensor &Aout, Tensor &Ain, IndexMapping &M)
{
    const int n = M.GetDomainSize();
    hipLaunchKernelGGL(sumGatherKernel, dim3(gridFor((static_cast<size_t>(n) + kGatherRows - 1) / kGatherRows)), dim3(kLanes), 0, stream(), Aout.GetDeviceData(),
                       Ain.GetDeviceData(), M.GetInvMap().GetDeviceData(), M.GetInvMapOffsets().GetDeviceData(), n);
    ACRO_HIP_CHECK(hipGetLastError());
}

}  // namespace acro
