// Micro-benchmarks behind three design decisions of the signature kernels (MI355X, gfx950).  Stand-alone:
//     hipcc --offload-arch=gfx950 -O3 -munsafe-fp-atomics -Xclang -target-feature -Xclang -packed-fp32-ops \
//           -mllvm -amdgpu-mfma-vgpr-form=1 -o issue_rate pathsig_amd/csrc/microbench/issue_rate.hip && ./issue_rate
//  (1) rate of plain v_fma_f32 against the number of resident waves per SIMD: a wave issues one vector
//      instruction about every six clocks, so the rate of a kernel is set by how many waves its registers allow;
//  (2) v_mfma_f32_4x4x1 alone and interleaved with v_fma_f32: the two do not overlap, so moving the leaf updates
//      of the sweeps to the matrix pipe buys nothing;
//  (3) accumulating into LDS cells: read-add-write against ds_add_f32 (LDS float atomics).
#include <hip/hip_runtime.h>

#include <cstdio>

typedef float v4f __attribute__((ext_vector_type(4)));

// MODE 0: 16 independent FMAs per iteration; 1: 8 MFMAs; 2: 8 MFMAs + 16 FMAs; 3: 8 (MFMA, FMA) pairs
template <int MODE>
__global__ void __launch_bounds__(256) valu_kernel(float *out, int iters, float x) {
    v4f acc[8];
    float f[16];
    for (int i = 0; i < 8; ++i) acc[i] = (v4f){0.f, 0.f, 0.f, 0.f};
    for (int i = 0; i < 16; ++i) f[i] = threadIdx.x * 0.001f + i;
    const float a = x + threadIdx.x, b = x * 2 + threadIdx.x;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            if (MODE == 1 || MODE == 2 || MODE == 3) acc[r] = __builtin_amdgcn_mfma_f32_4x4x1f32(a, b, acc[r], 0, 0, 0);
            if (MODE == 0 || MODE == 2) {
                f[2 * r] = __builtin_fmaf(f[2 * r], a, b);
                f[2 * r + 1] = __builtin_fmaf(f[2 * r + 1], a, b);
            }
            if (MODE == 3) f[r] = __builtin_fmaf(f[r], a, b);
        }
    }
    float s = 0;
    for (int i = 0; i < 8; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    for (int i = 0; i < 16; ++i) s += f[i];
    out[blockIdx.x * 256 + threadIdx.x] = s;
}

template <int MODE>
float time_valu(int waves_per_simd, int iters) {
    float *out;
    const int blocks = 256 * waves_per_simd;  // blocks of four waves: one wave on each SIMD of a CU
    if (hipMalloc(&out, (size_t)blocks * 256 * sizeof(float)) != hipSuccess) return -1.f;
    hipLaunchKernelGGL(valu_kernel<MODE>, dim3(blocks), dim3(256), 0, 0, out, iters / 10, 1.0f);
    (void)hipDeviceSynchronize();
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    (void)hipEventRecord(e0);
    hipLaunchKernelGGL(valu_kernel<MODE>, dim3(blocks), dim3(256), 0, 0, out, iters, 1.0f);
    (void)hipEventRecord(e1);
    (void)hipEventSynchronize(e1);
    float ms = -1.f;
    (void)hipEventElapsedTime(&ms, e0, e1);
    (void)hipFree(out);
    return ms;
}

// MODE 0: read-add-write, 1: atomicAdd (ds_add_f32), 2: plain store; eight cells per iteration, conflict free
template <int MODE>
__global__ void __launch_bounds__(512) lds_kernel(float *out, int iters, const int *offs) {
    __shared__ float slab[8 * 16 * 65];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float *mine = slab + wave * 16 * 65;
    for (int i = lane; i < 16 * 65; i += 64) mine[i] = 0.f;
    int o[8];
    for (int i = 0; i < 8; ++i) o[i] = offs[i] * 65 + lane;  // run-time rows: the compiler cannot tell the cells apart
    float v = lane * 0.5f;
    __syncthreads();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (MODE == 0) mine[o[i]] += v;
            else if (MODE == 1) atomicAdd(&mine[o[i]], v);
            else mine[o[i]] = v;
            v += 1.0f;
        }
    }
    __syncthreads();
    float s = 0;
    for (int i = 0; i < 16; ++i) s += mine[i * 65 + lane];
    out[blockIdx.x * 512 + threadIdx.x] = s;
}

template <int MODE>
float time_lds(int iters, const int *offs) {
    float *out;
    if (hipMalloc(&out, 256 * 512 * sizeof(float)) != hipSuccess) return -1.f;
    hipLaunchKernelGGL(lds_kernel<MODE>, dim3(256), dim3(512), 0, 0, out, iters / 10, offs);
    (void)hipDeviceSynchronize();
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    (void)hipEventRecord(e0);
    hipLaunchKernelGGL(lds_kernel<MODE>, dim3(256), dim3(512), 0, 0, out, iters, offs);
    (void)hipEventRecord(e1);
    (void)hipEventSynchronize(e1);
    float ms = -1.f;
    (void)hipEventElapsedTime(&ms, e0, e1);
    (void)hipFree(out);
    return ms;
}

int main() {
    const int iters = 200000;
    std::printf("(1) plain v_fma_f32, 16 independent per iteration, blocks of 256 threads, w blocks per CU\n");
    for (int w : {2, 1, 2, 3, 4, 6, 8}) {
        const float ms = time_valu<0>(w, iters);
        const double ns = ms * 1e6 / iters / 16 / w;  // per wave-instruction per SIMD, launch spread evenly
        std::printf("    %d waves/SIMD: %8.3f ms  %.3f ns per wave-FMA per SIMD  %.1f TFLOP/s\n", w, ms, ns,
                    2.0 * 64 * 1024 / ns * 1e-3);
    }
    std::printf("(2) v_mfma_f32_4x4x1 (16 blocks) against v_fma_f32, 2 waves/SIMD, time per iteration per SIMD\n");
    const float fma = time_valu<0>(2, iters), mfma = time_valu<1>(2, iters), both = time_valu<2>(2, iters),
                alt = time_valu<3>(2, iters);
    std::printf("    16 FMA: %.1f ns   8 MFMA: %.1f ns   8 MFMA + 16 FMA: %.1f ns (sum of the two: %.1f)   "
                "8 x (MFMA, FMA): %.1f ns\n",
                fma * 1e6 / iters, mfma * 1e6 / iters, both * 1e6 / iters, (fma + mfma) * 1e6 / iters,
                alt * 1e6 / iters);
    std::printf("(3) LDS accumulate, 8 waves per CU, per accumulate per wave\n");
    int host[8] = {3, 7, 1, 12, 5, 9, 14, 0}, *offs;
    if (hipMalloc(&offs, sizeof(host)) != hipSuccess) return 1;
    (void)hipMemcpy(offs, host, sizeof(host), hipMemcpyHostToDevice);
    const int li = 20000;
    std::printf("    read-add-write: %.1f ns   ds_add_f32: %.1f ns   plain store: %.1f ns\n",
                time_lds<0>(li, offs) * 1e6 / li / 8, time_lds<1>(li, offs) * 1e6 / li / 8,
                time_lds<2>(li, offs) * 1e6 / li / 8);
    return 0;
}
