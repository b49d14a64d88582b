// Stand-alone micro-benchmark of instruction issue costs on gfx950 (not part of libspdnn.so): how long a
// SIMD takes per wave instruction in register-only loops, and a CU per LDS read.  The band walk's choice of
// instructions (one v_add_f32 per input where a layer has one power-of-two weight, scalar work kept to
// four instructions per step, the DPP row broadcast in the TILED kernel) rests on these figures.
//   make -C graphchallenge21_amd/csrc issue_rates && graphchallenge21_amd/issue_rates
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>

#define CHECK(x)                                                                       \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) { fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); return 1; } \
    } while (0)

// 16 independent accumulators per lane, 128 loop items per trip; one workgroup of 4 waves per CU and
// `wps` workgroups per CU, i.e. wps waves per SIMD.
template <int MODE>
__global__ __launch_bounds__(256) void valu_loop(float* out, float w, int iters) {
    float a[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) a[i] = threadIdx.x * 0.001f + i;
    const float x = out[threadIdx.x & 7];
    const float wv = w + threadIdx.x;
    const unsigned u = threadIdx.x;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 8; ++r) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                if (MODE == 0) asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(a[i]) : "s"(w), "v"(x));
                else if (MODE == 1) asm volatile("v_mul_f32 %0, %1, %0" : "+v"(a[i]) : "s"(w));
                else if (MODE == 2) asm volatile("v_add_f32 %0, %1, %0" : "+v"(a[i]) : "v"(x));
                else if (MODE == 3) asm volatile("v_add_u32 %0, %1, %0" : "+v"(a[i]) : "v"(x));
                else if (MODE == 4) asm volatile("v_max_f32 %0, %1, %0" : "+v"(a[i]) : "v"(x));
                else if (MODE == 5) asm volatile("v_add_f32 %0, %1, %0\n\ts_add_u32 s20, s20, 1" : "+v"(a[i]) : "v"(x) : "s20", "scc");
                else if (MODE == 6) asm volatile("v_fmac_f32_dpp %0, %1, %2 row_newbcast:5 row_mask:0xf bank_mask:0xf" : "+v"(a[i]) : "v"(wv), "v"(x));
                else if (MODE == 7) { unsigned t; asm volatile("v_add_u32_dpp %0, %1, %2 row_newbcast:3 row_mask:0xf bank_mask:0xf" : "=v"(t) : "v"(u), "v"(u)); a[i] = __uint_as_float(t); }
                else if (MODE == 8) { unsigned s; asm volatile("v_readlane_b32 %0, %1, 5" : "=s"(s) : "v"(u)); asm volatile("v_add_f32 %0, %1, %0" : "+v"(a[i]) : "s"(s)); }
            }
        }
    }
    float s = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) s += a[i];
    if (s == 12345.678f) out[threadIdx.x] = s;
}

// one 16-wave workgroup per CU, every wave reading LDS back to back (four reads in flight)
template <int MODE>
__global__ __launch_bounds__(1024) void lds_loop(float* out, int iters) {
    __shared__ __align__(16) float sm[16384];
    for (int i = threadIdx.x; i < 16384; i += 1024) sm[i] = i;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t base = (uint32_t)(size_t)(__attribute__((address_space(3))) float*)sm;
    if (MODE == 0) base += wave * 64;                     // b128, all lanes one address
    else if (MODE == 1) base += wave * 64;                // b32, all lanes one address
    else if (MODE == 2) base += wave * 1024 + lane * 4;   // b32, consecutive lanes
    else base += wave * 2048 + lane * 16;                 // b128, consecutive lanes
    float acc = 0;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            if (MODE == 0 || MODE == 3) { float4 v; asm volatile("ds_read_b128 %0, %1 offset:%2\n\ts_waitcnt lgkmcnt(4)" : "=v"(v) : "v"(base), "n"(r * 16)); acc += v.x; }
            else { float v; asm volatile("ds_read_b32 %0, %1 offset:%2\n\ts_waitcnt lgkmcnt(4)" : "=v"(v) : "v"(base), "n"(r * 4)); acc += v; }
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)");
    if (acc == 12345.678f) out[threadIdx.x] = acc;
}

template <int MODE> static int time_valu(float* d, int wps, const char* name, double items_per_loop_item) {
    const int iters = 20000;
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    for (int rep = 0; rep < 2; ++rep) {
        CHECK(hipEventRecord(e0));
        hipLaunchKernelGGL(valu_loop<MODE>, dim3(256 * wps), dim3(256), 0, 0, d, 1.0001f, iters);
        CHECK(hipEventRecord(e1));
        CHECK(hipEventSynchronize(e1));
    }
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    printf("  %-44s %d waves/SIMD: %6.2f ns per instruction and SIMD\n", name, wps, ms * 1e6 / ((double)iters * 128 * wps * items_per_loop_item));
    return 0;
}
template <int MODE> static int time_lds(float* d, const char* name) {
    const int iters = 20000;
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    for (int rep = 0; rep < 2; ++rep) {
        CHECK(hipEventRecord(e0));
        hipLaunchKernelGGL(lds_loop<MODE>, dim3(256), dim3(1024), 0, 0, d, iters);
        CHECK(hipEventRecord(e1));
        CHECK(hipEventSynchronize(e1));
    }
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    printf("  %-44s 16 waves/CU:  %6.2f ns per instruction and CU\n", name, ms * 1e6 / ((double)iters * 8 * 16));
    return 0;
}

int main() {
    float* d = nullptr;
    CHECK(hipMalloc(&d, 4096));
    CHECK(hipMemset(d, 0, 4096));
    printf("vector and scalar instructions (register-only loops, one 4-wave workgroup per CU and waves/SIMD):\n");
    for (int wps : {1, 2, 4}) {
        if (time_valu<0>(d, wps, "v_fmac_f32 (scalar weight)", 1)) return 1;
        if (time_valu<1>(d, wps, "v_mul_f32", 1)) return 1;
        if (time_valu<2>(d, wps, "v_add_f32", 1)) return 1;
        if (time_valu<3>(d, wps, "v_add_u32", 1)) return 1;
        if (time_valu<4>(d, wps, "v_max_f32", 1)) return 1;
        if (time_valu<5>(d, wps, "v_add_f32 + s_add_u32 alternating (per pair)", 1)) return 1;
        if (time_valu<6>(d, wps, "v_fmac_f32_dpp row_newbcast", 1)) return 1;
        if (time_valu<7>(d, wps, "v_add_u32_dpp row_newbcast", 1)) return 1;
        if (time_valu<8>(d, wps, "v_readlane_b32 + v_add_f32 (per pair)", 1)) return 1;
    }
    printf("LDS reads:\n");
    if (time_lds<0>(d, "ds_read_b128, all lanes one address")) return 1;
    if (time_lds<1>(d, "ds_read_b32, all lanes one address")) return 1;
    if (time_lds<2>(d, "ds_read_b32, consecutive lanes")) return 1;
    if (time_lds<3>(d, "ds_read_b128, consecutive lanes")) return 1;
    CHECK(hipFree(d));
    return 0;
}
