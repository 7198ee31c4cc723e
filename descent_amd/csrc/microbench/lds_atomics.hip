// Rate of LDS read-modify-write instructions on gfx950 with random targets: what the ScatterAdd kernels' choice of
// accumulator type rests on (the per-workgroup sums are kept in double because ds_add_f64 is several times faster
// than ds_add_f32 here).  512 workgroups of 1024 threads; every thread keeps eight (target, value) records in
// registers and applies them 16 times to a 4096-element LDS array, so the time is the LDS pipeline's.
//
//   hipcc --offload-arch=gfx950 -O3 -o /tmp/lds_atomics descent_amd/csrc/microbench/lds_atomics.hip && /tmp/lds_atomics
#include <hip/hip_runtime.h>
#include <cstdio>
#include <vector>
#include <cstdlib>
#define CHECK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e)); return 1; } } while (0)

__device__ __forceinline__ void cas_add(float* p, float v) {
    unsigned int* q = (unsigned int*)p;
    unsigned int old = *q, assumed;
    do {
        assumed = old;
        old = atomicCAS(q, assumed, __float_as_uint(__uint_as_float(assumed) + v));
    } while (old != assumed);
}

template <int MODE>
__global__ __launch_bounds__(1024) void k(const float2* __restrict__ rec, float* __restrict__ out, int rounds) {
    __shared__ double segd[4096];
    float* seg = (float*)segd;
    for (int i = threadIdx.x; i < 4096; i += 1024) segd[i] = 0.0;
    __syncthreads();
    const float2* r = rec + (size_t)blockIdx.x * 8192 + threadIdx.x;
    float2 a[8];
    for (int u = 0; u < 8; ++u) a[u] = r[u * 1024];
    for (int t = 0; t < rounds; ++t) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int at = (__float_as_int(a[u].x) + t * 67) & 4095;
            if (MODE == 0) atomicAdd(&seg[at], a[u].y);
            else if (MODE == 1) atomicAdd((int*)&seg[at], 1);
            else if (MODE == 2) atomicAdd(&segd[at], (double)a[u].y);
            else if (MODE == 3) cas_add(&seg[at], a[u].y);
            else if (MODE == 4) seg[at] += a[u].y;  // racy, rate only
            else if (MODE == 5) { float old = atomicAdd(&seg[at], a[u].y); if (old == 12345.f) seg[0] = 1.f; }
            else if (MODE == 6) atomicMax((int*)&seg[at], __float_as_int(a[u].y));
        }
    }
    __syncthreads();
    double s = 0.0;
    for (int i = threadIdx.x; i < 4096; i += 1024) s += segd[i];
    if (s == 123456.0) out[blockIdx.x] = (float)s;
}

template <int MODE>
int run(const char* name, const float2* rec, float* out, int wgs, int rounds) {
    hipEvent_t a, b;
    CHECK(hipEventCreate(&a)); CHECK(hipEventCreate(&b));
    for (int w = 0; w < 2; ++w) k<MODE><<<wgs, 1024>>>(rec, out, rounds);
    CHECK(hipEventRecord(a));
    for (int w = 0; w < 5; ++w) k<MODE><<<wgs, 1024>>>(rec, out, rounds);
    CHECK(hipEventRecord(b)); CHECK(hipEventSynchronize(b));
    float ms; CHECK(hipEventElapsedTime(&ms, a, b));
    const double ops_per_cu = (double)wgs * 8192.0 * rounds / 256.0;
    printf("%-34s wgs %5d rounds %3d: %9.2f us/launch  %6.3f ns per op per CU\n", name, wgs, rounds, ms * 200.f, ms / 5 * 1e6 / ops_per_cu);
    return 0;
}

int main() {
    const int wgs = 512;
    std::vector<float2> h((size_t)wgs * 8192);
    srand(1);
    for (auto& r : h) { int at = rand() % 4096; r.x = *(float*)&at; r.y = 1.f; }
    float2* rec; float* out;
    CHECK(hipMalloc(&rec, h.size() * 8)); CHECK(hipMalloc(&out, 4 * wgs));
    CHECK(hipMemcpy(rec, h.data(), h.size() * 8, hipMemcpyHostToDevice));
    const int R = 16;
    if (run<4>("plain read-add-write (racy)", rec, out, wgs, R)) return 1;
    if (run<1>("ds_add_u32", rec, out, wgs, R)) return 1;
    if (run<6>("ds_max_i32", rec, out, wgs, R)) return 1;
    if (run<0>("ds_add_f32", rec, out, wgs, R)) return 1;
    if (run<5>("ds_add_rtn_f32", rec, out, wgs, R)) return 1;
    if (run<2>("ds_add_f64", rec, out, wgs, R)) return 1;
    if (run<3>("compare-and-swap loop, f32", rec, out, wgs, R)) return 1;
    return 0;
}
