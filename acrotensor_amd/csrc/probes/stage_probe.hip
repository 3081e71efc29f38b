// Measurement program behind one design decision of the generator: whether the stage contractions of the high-order
// operator applies (p=7 diffusion apply: 10 x 8 operators applied along one direction of an 8 x 8 x 8 ... 10 x 10 x 10
// block per element) should run on the FP64 matrix cores.  It runs the two stage shapes of that chain entirely on chip,
// three workgroups of four wavefronts per compute unit as the fused kernel has, once the way the generator emits
// them (a pencil per lane on the vector ALU, operator in scalar registers) and once with v_mfma_f64_16x16x4 (operator
// fragments in registers, rows padded to 16), and prints the time per stage.  Built by the Makefile next to the
// library (acrotensor_amd/lib/stage_probe); no part of the library uses it.
//
// One sum-factorisation stage of the p=7 diffusion apply, T1[q][c] = sum_i B[q][i] X[i][c] (q < 10, i < 8, c < 64 columns),
// repeated on chip (operands and results in LDS, nothing from device memory in the loop): a pencil per lane on the
// vector ALU against v_mfma_f64_16x16x4 with the 10 rows padded to 16.  Also the transposed stage V[i][c] = sum_q B[q][i] Z[q][c]
// (8 rows padded to 16, 10 terms padded to 12, 100 columns padded to 112).
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#define CHECK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("HIP error %s at %d\n", hipGetErrorString(e), __LINE__); exit(1); } } while (0)
typedef double d4 __attribute__((ext_vector_type(4)));
typedef const __attribute__((address_space(4))) double *scalar_ptr;

// ---- forward stage, vector ALU: lane = column, 8 LDS reads, 80 multiply-adds with B in scalar registers, 10 LDS writes
__global__ __launch_bounds__(256) void fwd_valu(const double *__restrict__ Bm, double *__restrict__ out, int reps)
{
    __shared__ double lds[4][8 * 64 + 10 * 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    double *x = lds[wave], *t = lds[wave] + 512;
    for (int i = 0; i < 8; ++i) x[i * 64 + lane] = 0.001 * (lane + i);
    double keep = 0.0;
    for (int rep = 0; rep < reps; ++rep)
    {
        // the operator is read with scalar loads in every repetition, as every phase of the fused kernel does
        const scalar_ptr B = (scalar_ptr)(Bm + __builtin_amdgcn_readfirstlane((rep & 1) * 80));
        double v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = x[i * 64 + lane];
#pragma unroll
        for (int q = 0; q < 10; ++q)
        {
            double s = B[q * 8] * v[0];
#pragma unroll
            for (int i = 1; i < 8; ++i) s += B[q * 8 + i] * v[i];
            t[q * 64 + lane] = s;
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        x[lane] = t[9 * 64 + lane] != 12345.0 ? 0.001 * lane : 1.0;
    }
    keep = t[lane];
    if (keep == 123.456) out[blockIdx.x * 256 + threadIdx.x] = keep;
}


// ---- dependent scalar loads: how long does one take?
__global__ __launch_bounds__(256) void scalar_chain(const double *__restrict__ Bm, double *__restrict__ out, int reps)
{
    const scalar_ptr B = (scalar_ptr)Bm;
    int idx = 0;
    double acc = 0.0;
    for (int rep = 0; rep < reps; ++rep)
    {
        const double v = B[idx];
        acc += v;
        idx = ((int)(v * 0.0) + rep) & 63;   // depends on the loaded value
    }
    if (acc == 123.456) out[blockIdx.x * 256 + threadIdx.x] = acc;
}

// ---- forward stage, matrix cores: first operand = B (16 rows x 4 terms per instruction, rows 10..15 zero), second = X
__global__ __launch_bounds__(256) void fwd_mfma(const double *__restrict__ Bm, double *__restrict__ out, int reps)
{
    __shared__ double lds[4][8 * 64 + 16 * 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 4, c = lane & 15;
    double *x = lds[wave], *t = lds[wave] + 512;
    for (int i = 0; i < 8; ++i) x[i * 64 + lane] = 0.001 * (lane + i);
    // operator fragment: lane holds B[row = c][term = 4 * step + g]
    double bf[2];
    for (int step = 0; step < 2; ++step) bf[step] = c < 10 ? Bm[c * 8 + 4 * step + g] : 0.0;
    double keep = 0.0;
    for (int rep = 0; rep < reps; ++rep)
    {
        d4 acc[4];
#pragma unroll
        for (int tile = 0; tile < 4; ++tile) acc[tile] = d4{0.0, 0.0, 0.0, 0.0};
#pragma unroll
        for (int step = 0; step < 2; ++step)
#pragma unroll
            for (int tile = 0; tile < 4; ++tile)
                acc[tile] = __builtin_amdgcn_mfma_f64_16x16x4f64(bf[step], x[(4 * step + g) * 64 + 16 * tile + c], acc[tile], 0, 0, 0);
        // result register r of a lane: row 4 r + g, column 16 tile + c; rows 10..15 are padding
#pragma unroll
        for (int tile = 0; tile < 4; ++tile)
#pragma unroll
            for (int r = 0; r < 3; ++r)
                if (4 * r + g < 10) t[(4 * r + g) * 64 + 16 * tile + c] = acc[tile][r];
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        x[lane] = t[9 * 64 + lane] != 12345.0 ? 0.001 * lane : 1.0;
    }
    keep = t[lane];
    if (keep == 123.456) out[blockIdx.x * 256 + threadIdx.x] = keep;
}

// ---- transposed stage, vector ALU: 100 columns over two passes of a wavefront (64 + 36 lanes), 10 reads, 80 multiply-adds, 8 writes
__global__ __launch_bounds__(256) void bwd_valu(const double *__restrict__ Bm, double *__restrict__ out, int reps)
{
    __shared__ double lds[4][10 * 100 + 8 * 100];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    double *z = lds[wave], *v = lds[wave] + 1000;
    for (int i = lane; i < 1000; i += 64) z[i] = 0.001 * i;
    for (int rep = 0; rep < reps; ++rep)
    {
        for (int col = lane, pass = 0; col < 100; col += 64, ++pass)
        {
            const scalar_ptr B = (scalar_ptr)(Bm + __builtin_amdgcn_readfirstlane(((rep + pass) & 1) * 80));
            double u[10];
#pragma unroll
            for (int q = 0; q < 10; ++q) u[q] = z[q * 100 + col];
#pragma unroll
            for (int i = 0; i < 8; ++i)
            {
                double s = B[i] * u[0];
#pragma unroll
                for (int q = 1; q < 10; ++q) s += B[q * 8 + i] * u[q];
                v[i * 100 + col] = s;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        z[lane] = v[700 + lane] != 12345.0 ? 0.001 * lane : 1.0;
    }
    const double keep = v[lane];
    if (keep == 123.456) out[blockIdx.x * 256 + threadIdx.x] = keep;
}

// ---- transposed stage, matrix cores: first operand = B transposed (8 rows padded to 16, 10 terms padded to 12), 7 column tiles
__global__ __launch_bounds__(256) void bwd_mfma(const double *__restrict__ Bm, double *__restrict__ out, int reps)
{
    __shared__ double lds[4][12 * 112 + 8 * 112];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 4, c = lane & 15;
    double *z = lds[wave], *v = lds[wave] + 12 * 112;
    for (int i = lane; i < 12 * 112; i += 64) z[i] = (i / 112 < 10) ? 0.001 * i : 0.0;
    double bf[3];
    for (int step = 0; step < 3; ++step) bf[step] = (c < 8 && 4 * step + g < 10) ? Bm[(4 * step + g) * 8 + c] : 0.0;
    for (int rep = 0; rep < reps; ++rep)
    {
        d4 acc[7];
#pragma unroll
        for (int tile = 0; tile < 7; ++tile) acc[tile] = d4{0.0, 0.0, 0.0, 0.0};
#pragma unroll
        for (int step = 0; step < 3; ++step)
#pragma unroll
            for (int tile = 0; tile < 7; ++tile)
                acc[tile] = __builtin_amdgcn_mfma_f64_16x16x4f64(bf[step], z[(4 * step + g) * 112 + 16 * tile + c], acc[tile], 0, 0, 0);
#pragma unroll
        for (int tile = 0; tile < 7; ++tile)
#pragma unroll
            for (int r = 0; r < 2; ++r) v[(4 * r + g) * 112 + 16 * tile + c] = acc[tile][r];
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        z[lane] = v[7 * 112 + lane] != 12345.0 ? 0.001 * lane : 1.0;
    }
    const double keep = v[lane];
    if (keep == 123.456) out[blockIdx.x * 256 + threadIdx.x] = keep;
}

int main()
{
    double *B, *out;
    CHECK(hipMalloc(&B, 160 * 8));
    CHECK(hipMalloc(&out, 1 << 24));
    double hb[160];
    for (int i = 0; i < 160; ++i) hb[i] = 0.01 * (i % 7) - 0.02;
    CHECK(hipMemcpy(B, hb, sizeof hb, hipMemcpyHostToDevice));
    hipEvent_t a, b;
    CHECK(hipEventCreate(&a));
    CHECK(hipEventCreate(&b));
    const int reps = 2000, groups = 256 * 3;  // three workgroups per CU, as the fused kernel has
    auto run = [&](const char *name, auto kernel, double flops_per_stage) {
        hipLaunchKernelGGL(kernel, dim3(groups), dim3(256), 0, 0, B, out, reps);
        CHECK(hipDeviceSynchronize());
        CHECK(hipEventRecord(a));
        hipLaunchKernelGGL(kernel, dim3(groups), dim3(256), 0, 0, B, out, reps);
        CHECK(hipEventRecord(b));
        CHECK(hipEventSynchronize(b));
        float ms;
        CHECK(hipEventElapsedTime(&ms, a, b));
        const double stages = (double)groups * 4 * reps;
        printf("%-44s %8.1f us  %7.2f ns per repetition  %6.2f TFLOP/s useful\n", name, ms * 1e3, ms * 1e6 / reps,
               stages * flops_per_stage / (ms * 1e-3) * 1e-12);
        fflush(stdout);
    };
    run("forward 10x8 . 8x64, vector ALU pencils", fwd_valu, 2.0 * 10 * 8 * 64);
    run("forward 10x8 . 8x64, v_mfma_f64_16x16x4", fwd_mfma, 2.0 * 10 * 8 * 64);
    run("chain of dependent scalar loads (per load)", scalar_chain, 0.0);
    run("transposed 8x10 . 10x100, vector ALU pencils", bwd_valu, 2.0 * 8 * 10 * 100);
    run("transposed 8x10 . 10x100, v_mfma_f64_16x16x4", bwd_mfma, 2.0 * 8 * 10 * 100);
    return 0;
}
