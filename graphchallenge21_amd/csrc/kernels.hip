// gfx950 (CDNA4, MI355X) kernels of the Sparse DNN inference path.  wave64 only.
//
// All layer kernels share one scheme: a wavefront works on one row block (64*RL feature rows,
// lane i holds rows i*RL..i*RL+RL-1 in registers) and on a run of output neurons; the input
// index and the weight of every multiply-add are wave-uniform and live in scalar registers, so
// the vector ALUs issue nothing but the multiply-adds, the LDS address add and the epilogue.
// Every output keeps ONE accumulator per row and adds its inputs in ascending input index -
// the order of the reference's CPU checker (src/utils/cpu_spmm.h:14-35) - so results are
// bit-identical to it; no reduction tree over the 32 terms anywhere.
//
// Epilogue (fused into every layer kernel, reference all_network.cu:55-60):
//     y = clamp(acc + bias, 0, 32);  store;  row is active iff some y != 0.
#include "kernels.hpp"

#include <algorithm>
#include <climits>
#include <cstdlib>

namespace spdnn {

namespace {

// Start of row block rb of a feature buffer: block rb >> 1 of the half rb & 1.
__device__ __forceinline__ float* block_base(const Feat& f, int rb, size_t block_floats) {
    return ((rb & 1) ? f.half[1] : f.half[0]) + (size_t)(rb >> 1) * block_floats;
}

template <int RL> struct VecOf;
template <> struct VecOf<1> { using type = float; };
template <> struct VecOf<2> { using type = float2; };
template <> struct VecOf<4> { using type = float4; };

// The band walk touches every input and output column once per layer.  On a large batch its loads and
// stores carry the non-temporal hint: the data of one layer is far larger than the caches, and without
// the hint it pushes out what is used again (measured at N=65536, batch 60000: 5.97 -> 5.72 ms per layer
// with loads and stores hinted, 5.95 - 5.96 with only one of the two).  Small launches, whose output the
// next layer still finds in the caches, keep the plain forms (the launcher decides); so do the BLOCK and
// GATHER kernels, which read columns more than once (hinted stores alone: BLOCK at N=1024, batch 60000
// 99.6 -> 101.9 us per layer, GATHER unchanged).
typedef float stream_f4 __attribute__((ext_vector_type(4)));
typedef float stream_f2 __attribute__((ext_vector_type(2)));
template <int RL> __device__ __forceinline__ void store_stream(float* p, const float* a) {
    if (RL == 4) {
        const stream_f4 v = {a[0], a[1], a[2], a[3]};
        __builtin_nontemporal_store(v, reinterpret_cast<stream_f4*>(p));
    } else if (RL == 2) {
        const stream_f2 v = {a[0], a[1]};
        __builtin_nontemporal_store(v, reinterpret_cast<stream_f2*>(p));
    } else {
        __builtin_nontemporal_store(a[0], p);
    }
}
template <int RL> __device__ __forceinline__ void load_stream(const float* p, float* a) {
    if (RL == 4) {
        const stream_f4 v = __builtin_nontemporal_load(reinterpret_cast<const stream_f4*>(p));
        a[0] = v.x; a[1] = v.y; a[2] = v.z; a[3] = v.w;
    } else if (RL == 2) {
        const stream_f2 v = __builtin_nontemporal_load(reinterpret_cast<const stream_f2*>(p));
        a[0] = v.x; a[1] = v.y;
    } else {
        a[0] = __builtin_nontemporal_load(p);
    }
}
template <int RL> __device__ __forceinline__ void vec_to_arr(const typename VecOf<RL>::type& v, float* a);
template <> __device__ __forceinline__ void vec_to_arr<1>(const float& v, float* a) { a[0] = v; }
template <> __device__ __forceinline__ void vec_to_arr<2>(const float2& v, float* a) { a[0] = v.x; a[1] = v.y; }
template <> __device__ __forceinline__ void vec_to_arr<4>(const float4& v, float* a) {
    a[0] = v.x; a[1] = v.y; a[2] = v.z; a[3] = v.w;
}
template <int RL> __device__ __forceinline__ typename VecOf<RL>::type arr_to_vec(const float* a);
template <> __device__ __forceinline__ float arr_to_vec<1>(const float* a) { return a[0]; }
template <> __device__ __forceinline__ float2 arr_to_vec<2>(const float* a) { return make_float2(a[0], a[1]); }
template <> __device__ __forceinline__ float4 arr_to_vec<4>(const float* a) {
    return make_float4(a[0], a[1], a[2], a[3]);
}

// One multiply-add of the accumulation chain.
//   WMODE 0/1: the product is exact (weight is 0 or a power of two), so a fused multiply-add
//              rounds exactly like the reference's multiply followed by add.
//   WMODE 2:   general weights: rounded multiply, then rounded add, as the CPU reference does.
//   WMODE 3:   (band walk, unrolled path) the layer's ONE weight w is 0 or +-2^e: scaling by a power of
//              two commutes with rounding (nothing here comes near the denormal range, see the
//              inspector's fma_ok), so fl(..fl(fl(w x0) + w x1).. + w xk) = w * fl(..fl(x0 + x1).. + xk):
//              the chain is one v_add_f32 per input - issued at twice the rate of v_fmac_f32 /
//              v_mul_f32 on this hardware (measured: 0.95 against 1.72 ns per wave instruction and
//              SIMD) - and the weight enters once, in the epilogue's fma(sum, w, bias), which rounds
//              like the reference's add of the bias because w * sum is exact.
//   WMODE 4:   WMODE 3 for layers in which the two outputs of every pair use the same inputs (groups of
//              identical rows: the run chains of RadiX-Net layers): the two sums are equal, so the pair
//              keeps one accumulator, adds every step without a mask and stores the result twice.
__device__ __forceinline__ float mul_then_add(float acc, float x, float w) {
#pragma clang fp contract(off)
    const float p = x * w;
    return acc + p;
}
// One step of the add-only walk for a pair of outputs: acc0[q] += x[q] if bit `bit` of mask0 is set,
// acc1[q] += x[q] if it is set in mask1 (q = the wave's RL rows per lane).  The bit, sign-extended to 64
// bits by one scalar instruction, becomes the execution mask of the adds (all lanes or none): no select
// per accumulator, no branch.  CALLERS: every lane of the calling wave must be active (wave-uniform control
// flow around the call): the statement ends by setting the mask to all ones, it does not restore what it found
// (saving and restoring would cost two more scalar instructions per step, which the walk cannot afford).
template <int RL> __device__ __forceinline__ void add_pair_if_used(float* acc0, float* acc1, const float* x,
                                                                 uint64_t mask0, uint64_t mask1, int bit);
template <> __device__ __forceinline__ void add_pair_if_used<4>(float* acc0, float* acc1, const float* x,
                                                                uint64_t mask0, uint64_t mask1, int bit) {
    asm volatile(
        "s_bfe_i64 exec, %12, %14\n\t"
        "v_add_f32 %0, %8, %0\n\tv_add_f32 %1, %9, %1\n\tv_add_f32 %2, %10, %2\n\tv_add_f32 %3, %11, %3\n\t"
        "s_bfe_i64 exec, %13, %14\n\t"
        "v_add_f32 %4, %8, %4\n\tv_add_f32 %5, %9, %5\n\tv_add_f32 %6, %10, %6\n\tv_add_f32 %7, %11, %7\n\t"
        "s_mov_b64 exec, -1"
        : "+v"(acc0[0]), "+v"(acc0[1]), "+v"(acc0[2]), "+v"(acc0[3]), "+v"(acc1[0]), "+v"(acc1[1]), "+v"(acc1[2]),
          "+v"(acc1[3])
        : "v"(x[0]), "v"(x[1]), "v"(x[2]), "v"(x[3]), "s"(mask0), "s"(mask1), "n"(0x10000 | bit)
        : "scc");
}
template <> __device__ __forceinline__ void add_pair_if_used<2>(float* acc0, float* acc1, const float* x,
                                                                uint64_t mask0, uint64_t mask1, int bit) {
    asm volatile(
        "s_bfe_i64 exec, %6, %8\n\t"
        "v_add_f32 %0, %4, %0\n\tv_add_f32 %1, %5, %1\n\t"
        "s_bfe_i64 exec, %7, %8\n\t"
        "v_add_f32 %2, %4, %2\n\tv_add_f32 %3, %5, %3\n\t"
        "s_mov_b64 exec, -1"
        : "+v"(acc0[0]), "+v"(acc0[1]), "+v"(acc1[0]), "+v"(acc1[1])
        : "v"(x[0]), "v"(x[1]), "s"(mask0), "s"(mask1), "n"(0x10000 | bit)
        : "scc");
}
template <> __device__ __forceinline__ void add_pair_if_used<1>(float* acc0, float* acc1, const float* x,
                                                                uint64_t mask0, uint64_t mask1, int bit) {
    asm volatile(
        "s_bfe_i64 exec, %3, %5\n\t"
        "v_add_f32 %0, %2, %0\n\t"
        "s_bfe_i64 exec, %4, %5\n\t"
        "v_add_f32 %1, %2, %1\n\t"
        "s_mov_b64 exec, -1"
        : "+v"(acc0[0]), "+v"(acc1[0])
        : "v"(x[0]), "s"(mask0), "s"(mask1), "n"(0x10000 | bit)
        : "scc");
}
// LDS address of a lane's part of ring column `slot byte b of dword`: one scalar bit-field extract and
// one vector shift-add (written out: the compiler's own choice is a shift and a mask on the scalar unit, and
// scalar instructions are what the add-only walk can least afford: measured, each costs a SIMD as much
// issue time as a multiply-add).
template <int SLOT_BITS, int COL_SHIFT>
__device__ __forceinline__ uint32_t ring_address(uint32_t lane_base, uint32_t dword, int b) {
    uint32_t slot, addr;
    asm("s_bfe_u32 %0, %1, %2" : "=s"(slot) : "s"(dword), "n"((SLOT_BITS << 16) | (8 * b)) : "scc");
    asm("v_lshl_add_u32 %0, %1, %2, %3" : "=v"(addr) : "s"(slot), "n"(COL_SHIFT), "v"(lane_base));
    return addr;
}
// add_pair_if_used followed, in the same statement, by the LDS address of a later step's column (ring_address):
// between two separate asm statements the compiler puts a wait state it cannot know to be unnecessary, two
// per step of the walk; within one statement the scalar extract feeds the vector shift-add directly.
template <int RL, int SLOT_BITS, int COL_SHIFT>
__device__ __forceinline__ uint32_t add_pair_if_used_then_address(float* acc0, float* acc1, const float* x, uint64_t mask0,
                                                                  uint64_t mask1, int bit, uint32_t lane_base,
                                                                  uint32_t dword, int b);
#define SPDNN_ADDR_TAIL "s_mov_b64 exec, -1\n\ts_bfe_u32 %[slot], %[dw], %[fld]\n\tv_lshl_add_u32 %[addr], %[slot], %[sh], %[base]"
template <> __device__ __forceinline__ uint32_t add_pair_if_used_then_address<4, 6, 10>(
    float* acc0, float* acc1, const float* x, uint64_t mask0, uint64_t mask1, int bit, uint32_t lane_base, uint32_t dword, int b) {
    uint32_t addr, slot;
    asm volatile(
        "s_bfe_i64 exec, %[m0], %[bit]\n\t"
        "v_add_f32 %[a0], %[x0], %[a0]\n\tv_add_f32 %[a1], %[x1], %[a1]\n\tv_add_f32 %[a2], %[x2], %[a2]\n\tv_add_f32 %[a3], %[x3], %[a3]\n\t"
        "s_bfe_i64 exec, %[m1], %[bit]\n\t"
        "v_add_f32 %[b0], %[x0], %[b0]\n\tv_add_f32 %[b1], %[x1], %[b1]\n\tv_add_f32 %[b2], %[x2], %[b2]\n\tv_add_f32 %[b3], %[x3], %[b3]\n\t"
        SPDNN_ADDR_TAIL
        : [a0] "+v"(acc0[0]), [a1] "+v"(acc0[1]), [a2] "+v"(acc0[2]), [a3] "+v"(acc0[3]), [b0] "+v"(acc1[0]),
          [b1] "+v"(acc1[1]), [b2] "+v"(acc1[2]), [b3] "+v"(acc1[3]), [addr] "=&v"(addr), [slot] "=&s"(slot)
        : [x0] "v"(x[0]), [x1] "v"(x[1]), [x2] "v"(x[2]), [x3] "v"(x[3]), [m0] "s"(mask0), [m1] "s"(mask1),
          [bit] "n"(0x10000 | bit), [dw] "s"(dword), [fld] "n"((6 << 16) | (8 * b)), [sh] "n"(10), [base] "v"(lane_base)
        : "scc");
    return addr;
}
template <> __device__ __forceinline__ uint32_t add_pair_if_used_then_address<2, 6, 9>(
    float* acc0, float* acc1, const float* x, uint64_t mask0, uint64_t mask1, int bit, uint32_t lane_base, uint32_t dword, int b) {
    uint32_t addr, slot;
    asm volatile(
        "s_bfe_i64 exec, %[m0], %[bit]\n\t"
        "v_add_f32 %[a0], %[x0], %[a0]\n\tv_add_f32 %[a1], %[x1], %[a1]\n\t"
        "s_bfe_i64 exec, %[m1], %[bit]\n\t"
        "v_add_f32 %[b0], %[x0], %[b0]\n\tv_add_f32 %[b1], %[x1], %[b1]\n\t"
        SPDNN_ADDR_TAIL
        : [a0] "+v"(acc0[0]), [a1] "+v"(acc0[1]), [b0] "+v"(acc1[0]), [b1] "+v"(acc1[1]), [addr] "=&v"(addr),
          [slot] "=&s"(slot)
        : [x0] "v"(x[0]), [x1] "v"(x[1]), [m0] "s"(mask0), [m1] "s"(mask1), [bit] "n"(0x10000 | bit), [dw] "s"(dword),
          [fld] "n"((6 << 16) | (8 * b)), [sh] "n"(9), [base] "v"(lane_base)
        : "scc");
    return addr;
}
template <> __device__ __forceinline__ uint32_t add_pair_if_used_then_address<1, 6, 8>(
    float* acc0, float* acc1, const float* x, uint64_t mask0, uint64_t mask1, int bit, uint32_t lane_base, uint32_t dword, int b) {
    uint32_t addr, slot;
    asm volatile(
        "s_bfe_i64 exec, %[m0], %[bit]\n\t"
        "v_add_f32 %[a0], %[x0], %[a0]\n\t"
        "s_bfe_i64 exec, %[m1], %[bit]\n\t"
        "v_add_f32 %[b0], %[x0], %[b0]\n\t"
        SPDNN_ADDR_TAIL
        : [a0] "+v"(acc0[0]), [b0] "+v"(acc1[0]), [addr] "=&v"(addr), [slot] "=&s"(slot)
        : [x0] "v"(x[0]), [m0] "s"(mask0), [m1] "s"(mask1), [bit] "n"(0x10000 | bit), [dw] "s"(dword),
          [fld] "n"((6 << 16) | (8 * b)), [sh] "n"(8), [base] "v"(lane_base)
        : "scc");
    return addr;
}
#undef SPDNN_ADDR_TAIL

// twins (both outputs of a pair add every step): RL adds into the one accumulator, then the address of a
// later step's column, in one statement as above
template <int RL, int SLOT_BITS, int COL_SHIFT>
__device__ __forceinline__ uint32_t add_then_address(float* acc, const float* x, uint32_t lane_base, uint32_t dword, int b) {
    static_assert(SLOT_BITS == 6, "64-slot ring");
    uint32_t addr, slot;
    if (RL == 4)
        asm volatile("v_add_f32 %[a0], %[x0], %[a0]\n\tv_add_f32 %[a1], %[x1], %[a1]\n\tv_add_f32 %[a2], %[x2], %[a2]\n\t"
                     "v_add_f32 %[a3], %[x3], %[a3]\n\ts_bfe_u32 %[slot], %[dw], %[fld]\n\tv_lshl_add_u32 %[addr], %[slot], %[sh], %[base]"
                     : [a0] "+v"(acc[0]), [a1] "+v"(acc[1]), [a2] "+v"(acc[2]), [a3] "+v"(acc[3]), [addr] "=&v"(addr), [slot] "=&s"(slot)
                     : [x0] "v"(x[0]), [x1] "v"(x[1]), [x2] "v"(x[2]), [x3] "v"(x[3]), [dw] "s"(dword),
                       [fld] "n"((6 << 16) | (8 * b)), [sh] "n"(COL_SHIFT), [base] "v"(lane_base)
                     : "scc");
    else if (RL == 2)
        asm volatile("v_add_f32 %[a0], %[x0], %[a0]\n\tv_add_f32 %[a1], %[x1], %[a1]\n\t"
                     "s_bfe_u32 %[slot], %[dw], %[fld]\n\tv_lshl_add_u32 %[addr], %[slot], %[sh], %[base]"
                     : [a0] "+v"(acc[0]), [a1] "+v"(acc[1]), [addr] "=&v"(addr), [slot] "=&s"(slot)
                     : [x0] "v"(x[0]), [x1] "v"(x[1]), [dw] "s"(dword), [fld] "n"((6 << 16) | (8 * b)), [sh] "n"(COL_SHIFT),
                       [base] "v"(lane_base)
                     : "scc");
    else
        asm volatile("v_add_f32 %[a0], %[x0], %[a0]\n\t"
                     "s_bfe_u32 %[slot], %[dw], %[fld]\n\tv_lshl_add_u32 %[addr], %[slot], %[sh], %[base]"
                     : [a0] "+v"(acc[0]), [addr] "=&v"(addr), [slot] "=&s"(slot)
                     : [x0] "v"(x[0]), [dw] "s"(dword), [fld] "n"((6 << 16) | (8 * b)), [sh] "n"(COL_SHIFT), [base] "v"(lane_base)
                     : "scc");
    return addr;
}

// RL floats from an LDS byte address
template <int RL> __device__ __forceinline__ void lds_read(uint32_t lds_address, float* x) {
    typedef float vec_t __attribute__((ext_vector_type(RL)));
    const vec_t v = *(const __attribute__((address_space(3))) vec_t*)(size_t)lds_address;
#pragma unroll
    for (int q = 0; q < RL; ++q) x[q] = v[q];
}
template <> __device__ __forceinline__ void lds_read<1>(uint32_t lds_address, float* x) {
    x[0] = *(const __attribute__((address_space(3))) float*)(size_t)lds_address;
}
template <int WMODE> __device__ __forceinline__ float mac(float acc, float x, float w) {
    if (WMODE == 2) return mul_then_add(acc, x, w);
    return __builtin_fmaf(x, w, acc);
}

// Running "largest output so far" of a row.  Outputs are clamped to [0, clamp], so comparing the
// bit patterns as signed integers orders them like the floats (one v_max_i32, no NaN handling).
__device__ __forceinline__ float nz_merge(float nz, float y) {
    return __int_as_float(max(__float_as_int(nz), __float_as_int(y)));
}

// Row stamps and row counts.  At its end a layer kernel writes `stamp` (the number of its launch)
// into active[row] of every row with a nonzero output: plain stores - all workgroups that work on
// a row block store the same value, so no order among them matters.  How many rows a layer left
// active is counted by the kernel of the NEXT layer: at its start the first workgroup of every row
// block looks at the block's 64*RL stamps anyway (for pruning) and adds the number of rows that
// carry the previous launch's stamp to that layer's counter, one atomic add per row block.
// (Counting while stamping needs an atomic exchange per row and workgroup to find out who is
// first; exchanges on one address are served one after the other, and on a small batch they took
// longer than the layer itself.)
__device__ __forceinline__ void count_newly(int newly, int32_t* __restrict__ count_out) {
    newly += __shfl_down(newly, 32, 64);
    newly += __shfl_down(newly, 16, 64);
    newly += __shfl_down(newly, 8, 64);
    newly += __shfl_down(newly, 4, 64);
    newly += __shfl_down(newly, 2, 64);
    newly += __shfl_down(newly, 1, 64);
    if ((threadIdx.x & 63) == 0 && newly > 0) atomicAdd(count_out, newly);
}

// one wave, lane = RL rows starting at row0
template <int RL>
__device__ __forceinline__ void stamp_rows(const float* nz, int32_t* __restrict__ active, size_t row0, int stamp) {
#pragma unroll
    for (int q = 0; q < RL; ++q)
        if (nz[q] > 0.0f) active[row0 + q] = stamp;
}

// a workgroup of NW waves that all worked on the same 64*RL rows (block_row0 = first row): the
// waves' results are merged through LDS (free after the last barrier of the band walk) and every
// row is stamped by one thread.  count_out (may be nullptr) is for a workgroup that is the only
// one to work on its row block: it then also counts the rows it stamps.  Contains a barrier; the
// caller must put another one before the LDS is written again.
template <int RL, int NW>
__device__ __forceinline__ void stamp_rows_workgroup(const float* nz, unsigned char* smem,
                                                     int32_t* __restrict__ active, size_t block_row0, int stamp,
                                                     int32_t* __restrict__ count_out) {
    constexpr int RB = 64 * RL;
    float* s = reinterpret_cast<float*>(smem);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int q = 0; q < RL; ++q) s[wave * RB + lane * RL + q] = nz[q];
    __syncthreads();
    int newly = 0;
    for (int r = threadIdx.x; r < RB; r += NW * 64) {
        float m = s[r];
#pragma unroll
        for (int w = 1; w < NW; ++w) m = nz_merge(m, s[w * RB + r]);
        if (m > 0.0f) {
            active[block_row0 + r] = stamp;
            ++newly;
        }
    }
    if (count_out) count_newly(newly, count_out);
}

// see Publish: the first workgroup of the launch hands the previous launch's counts to the host
__device__ __forceinline__ void publish_counts(const Publish& p) {
    if (p.n > 0 && blockIdx.x == 0 && blockIdx.y == 0) {
        for (int i = threadIdx.x; i < p.n; i += blockDim.x) p.dst[i] = p.src[i];
        __threadfence_system();  // the host polls this memory while the kernel is still running
    }
}

// Start of a layer kernel (every wave of the workgroup calls it; lane = RL rows from row0, so a
// wave sees its whole row block).  prev_stamp is the stamp of the layer before (0 = none valid).
// Rows that carry it were left active by that layer; so were rows that already carry this
// launch's stamp (another workgroup was faster: with bias <= 0 only a row that was active can be
// active again).  The number of such rows does not depend on when a wave looks.
//  - counter (wave 0 of the row block's first workgroup) adds it to count_prev, if given;
//  - with check_dead the return value says that the row block has no active row, i.e. that its
//    outputs are all zero and the workgroup can leave (uniform over the workgroup; has a barrier).
template <int RL>
__device__ __forceinline__ bool enter_row_block(const int32_t* active, size_t row0, int prev_stamp, int stamp,
                                                int check_dead, int32_t* __restrict__ count_prev, bool counter) {
    if (prev_stamp == 0) return false;
    const bool counts = counter && count_prev != nullptr;
    if (!check_dead && !counts) return false;
    int alive = 0;
#pragma unroll
    for (int q = 0; q < RL; ++q) {
        const int a = active[row0 + q];
        alive += (int)__popcll(__ballot((a == prev_stamp || a == stamp) ? 1 : 0));
    }
    if (counts && (threadIdx.x & 63) == 0 && alive > 0) atomicAdd(count_prev, alive);
    if (!check_dead) return false;
    // (the result is the same for every thread; said explicitly, the branch on it is a scalar one)
    return __builtin_amdgcn_readfirstlane(__syncthreads_or(alive)) == 0;
}


// One input column (64 lanes x 16 bytes) straight from global memory into an LDS column slot,
// without passing through vector registers: lane i's 16 bytes land at lds_col + 16 i, which is
// the layout of a 256-row column.  The transfer is counted like any vector memory load.
// TRACKED: through the compiler's builtin.  Once the compiler knows of a direct-to-LDS load in a kernel
// it no longer counts LDS reads down (lgkmcnt(1), (2)) but waits for all of them (lgkmcnt(0)) wherever
// a wave needs one, which merges the band walk's waits into one per two steps.  Measured at the headline
// shape in one process: the multiply-add walk is faster that way (5.47 against 5.58 ms per layer), the
// add-only walk (WMODE 3) with counted waits (5.16 against 5.22 ms).
// Not TRACKED: as text the compiler does not look into; the callers order these loads by hand
// (wait_vector_memory() and a barrier before any wave reads the slot).  M0 (the LDS base of such a
// load) is the compiler's to manage and is put back.
template <int STREAM, int TRACKED = 1>
__device__ __forceinline__ void column_to_lds(const float* gsrc_lane, unsigned char* lds_col) {
    if (TRACKED) {
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)gsrc_lane,
                                         (__attribute__((address_space(3))) void*)lds_col, 16, 0, STREAM ? 2 : 0);
        return;
    }
    const uint32_t lds_off = (uint32_t)(size_t)((__attribute__((address_space(3))) unsigned char*)lds_col);
    uint32_t m0_saved;
    if (STREAM)
        asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, off nt\n\ts_mov_b32 m0, %0"
                     : "=&s"(m0_saved) : "s"(lds_off), "v"(gsrc_lane) : "memory");
    else
        asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, off\n\ts_mov_b32 m0, %0"
                     : "=&s"(m0_saved) : "s"(lds_off), "v"(gsrc_lane) : "memory");
}
// s_waitcnt vmcnt(0) (the other counters left alone: expcnt 7, lgkmcnt 15 in the gfx9 encoding), as
// the instruction itself rather than inline text, so that the compiler's own bookkeeping of
// outstanding direct-to-LDS loads sees it too.
__device__ __forceinline__ void wait_vector_memory() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0x0F70);
    asm volatile("" ::: "memory");
}
// Workgroup barrier of the band walk.  With columns sent straight into the ring the waves wait for
// their transfers themselves (wait_vector_memory) BEFORE they store their outputs; the fence of
// __syncthreads() would wait on the vector memory counter again behind those stores, i.e. for the
// stores' acknowledgement, once per chunk.  The bare barrier only orders the LDS traffic.
template <int DMA> __device__ __forceinline__ void ring_barrier() {
    if (DMA) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else __syncthreads();
}

__device__ __forceinline__ float relu_clamp(float y, float clampv) {
    // median(y, 0, clamp): 0 below 0, clamp above clamp, y in between (inputs are finite).
    return __builtin_amdgcn_fmed3f(y, 0.0f, clampv);
}

// ------------------------------------------------------------------------------------------
// BAND kernel ("row-succ" / tiled variant).
//
// The inspector has relabelled the layer so that the output at band position v reads input
// columns at positions no further back than `halo` before the 16-aligned group of v and no later
// than the end of that group (mod N): a circulant band, where v reads v-K+1 .. v (halo K-1), or a
// chain of 16-output groups that each read the input runs of the two groups before them and
// their own (halo 32).  A workgroup takes one row block and one
// segment [vb, ve) of band positions and walks it in chunks of T = NW*OPW outputs.  The input
// columns live in an LDS ring of RING column slots (slot = position mod RING, RING | N): while
// the waves compute chunk c from the ring, the T columns of chunk c+1 are already in flight
// from HBM into registers and are dropped into the ring afterwards, so every input column is
// read from HBM once per segment (plus the halo columns at the segment start) and the loads
// overlap the arithmetic.  Needs 2*T + halo <= RING, T a multiple of 16.
//
// Outputs are computed in PAIRS of neighbouring band positions (2u, 2u+1).  Every output adds its
// inputs in ascending input index, so the inputs two outputs share come in the same order in
// both: the inspector merges the two lists into one list of `steps` steps (K+1 for a circulant
// band, K inside a group of a chain), and a wave reads each step's column from the ring ONCE and
// feeds it to both accumulators - half the LDS reads and address arithmetic of one list per
// output.  A step an output does not use enters it with weight 0 (adding an exact zero).
//
// Per pair the scalar unit streams a record of 16 dwords: two 64-bit use masks (output 0, output 1),
// then the steps' one-byte ring selectors; unless the layer has one exact value also two weights per
// step (72 floats per pair).  How a step enters the accumulators depends on the weight mode (see mac
// above): a multiply-add with the step's weight, or - one power-of-two weight per layer - a plain
// add under the output's use bit, the weight applied once in the epilogue.  The output column is written to the physical column the NEXT layer wants it in (dst),
// RB*4 contiguous bytes.
// ------------------------------------------------------------------------------------------
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_const_u4(const __attribute__((address_space(4))) uint32_t* p) {
    const u32x4_t v = *(const __attribute__((address_space(4))) u32x4_t*)p;
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ float4 load_const_f4(const __attribute__((address_space(4))) float* p) {
    const f32x4_t v = *(const __attribute__((address_space(4))) f32x4_t*)p;
    return make_float4(v.x, v.y, v.z, v.w);
}

// RBL: rows per block of the LAYOUT (floats between two columns); larger than the 64*RL rows the
// workgroup handles when it works on a part of a row block (yin / yout then point at that part).
template <int RL, int NW, int OPW, int RING, int WMODE, int KT, int DMA, int RBL = 64 * RL>
__device__ __forceinline__ void band_walk_body(
    const float* __restrict__ yin, float* __restrict__ yout, const uint32_t* __restrict__ pairs_g,
    const float* __restrict__ pw_g, const int32_t* __restrict__ dst_g, int N, int steps, int halo,
    int vb, int ve, float wu, float bias, float clampv, unsigned char* smem, float* nz, int stream) {
    using V = typename VecOf<RL>::type;
    // The plan arrays never change while a kernel runs: read through the constant address space they
    // come by the scalar unit also where the pointers themselves were loaded from memory (the layer
    // table of the fused chain), instead of by vector loads with the selection arithmetic on the
    // vector ALUs.
    const __attribute__((address_space(4))) uint32_t* pairs = (const __attribute__((address_space(4))) uint32_t*)pairs_g;
    const __attribute__((address_space(4))) float* pw = (const __attribute__((address_space(4))) float*)pw_g;
    const __attribute__((address_space(4))) int32_t* dst = (const __attribute__((address_space(4))) int32_t*)dst_g;
    constexpr int T = NW * OPW;
    constexpr int PPW = OPW / 2;  // pairs per wave and chunk
    constexpr int RB = 64 * RL;
    constexpr int COLB = RB * 4;
    static_assert(2 * T + 32 <= RING && T % 16 == 0, "ring too small for a halo of 32 columns");
    static_assert((RING & (RING - 1)) == 0 && RING <= 256, "ring must be a power of two <= 256");
    static_assert(OPW % 2 == 0, "outputs are computed in pairs");
    static_assert(KT == 0 || KT == 36, "KT is 36 (32 entries per output: at least 32 steps) or 0 (fewer: groups of four steps)");
    constexpr bool WSTREAM = WMODE == 1 || WMODE == 2;   // weights come per step from the plan

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int loff = lane * RL;
    const unsigned char* lane_smem = smem + loff * 4;
    const uint32_t lane_base = (uint32_t)(size_t)((const __attribute__((address_space(3))) unsigned char*)lane_smem);
    constexpr int SLOT_BITS = RING == 256 ? 8 : RING == 128 ? 7 : RING == 64 ? 6 : RING == 32 ? 5 : 4;
    constexpr int COL_SHIFT = RL == 4 ? 10 : RL == 2 ? 9 : 8;
    static_assert((1 << SLOT_BITS) == RING && (1 << COL_SHIFT) == COLB, "ring geometry");
    // the layer's one weight as scalar bits: a step's effective weight (wu or 0) is then picked by
    // integer ops on the scalar unit and feeds the multiply-add as a scalar operand
    const uint32_t wu_bits = (uint32_t)__builtin_amdgcn_readfirstlane((int)__float_as_uint(wu));

    // prologue: halo (columns before the segment, wrapping below 0) + first chunk
    static_assert(DMA == 0 || RL == 4, "direct loads into the ring move 16 bytes per lane");
    for (int c = wave; c < halo + T; c += NW) {
        const int p = vb - halo + c;
        if (p < ve) {
            const int g = p < 0 ? p + N : p;
            if (DMA) {
                unsigned char* slot = smem + (size_t)(p & (RING - 1)) * COLB;
                if (stream) column_to_lds<1, (WMODE < 3)>(yin + (size_t)g * RBL + loff, slot);
                else column_to_lds<0, (WMODE < 3)>(yin + (size_t)g * RBL + loff, slot);
                continue;
            }
            float x[RL];
            if (stream) load_stream<RL>(yin + (size_t)g * RBL + loff, x);
            else vec_to_arr<RL>(*reinterpret_cast<const V*>(yin + (size_t)g * RBL + loff), x);
            *reinterpret_cast<V*>(smem + (size_t)(p & (RING - 1)) * COLB + loff * 4) = arr_to_vec<RL>(x);
        }
    }
    if (DMA) wait_vector_memory();
    ring_barrier<DMA>();

    const int last_pair = (ve - 1) >> 1;
    for (int cb = vb; cb < ve; cb += T) {
        // columns of the next chunk: issue the HBM loads now, park them in registers (past the
        // segment end the last column is loaded again and never stored) - or, DMA, send them
        // straight into the ring slots no wave reads during this chunk
        float pf[OPW][RL];
#pragma unroll
        for (int i = 0; i < OPW; ++i) {
            const int p = min(cb + T + wave + i * NW, ve - 1);
            if (DMA) {
                unsigned char* slot = smem + (size_t)((cb + T + wave + i * NW) & (RING - 1)) * COLB;
                if (stream) column_to_lds<1, (WMODE < 3)>(yin + (size_t)p * RBL + loff, slot);
                else column_to_lds<0, (WMODE < 3)>(yin + (size_t)p * RBL + loff, slot);
            } else if (stream) load_stream<RL>(yin + (size_t)p * RBL + loff, pf[i]);
            else vec_to_arr<RL>(*reinterpret_cast<const V*>(yin + (size_t)p * RBL + loff), pf[i]);
        }

        int pr[PPW];
        float acc[PPW][2][RL];
#pragma unroll
        for (int i = 0; i < PPW; ++i) {
            pr[i] = min((cb >> 1) + wave + i * NW, last_pair);
#pragma unroll
            for (int q = 0; q < RL; ++q) acc[i][0][q] = acc[i][1][q] = 0.0f;
        }

        {
            // The whole pair record (masks + 36 selectors) sits in scalar registers up front.  The
            // LDS read of step s+2 is issued before the arithmetic of step s, so a wave always has
            // reads in flight while its multiply-adds issue.  KT = 36 (32 entries per output): the first 32
            // steps run unconditionally, steps 32..35 only if steps > 32.  KT = 0 (fewer entries): the steps
            // run in groups of four as far as `steps` reaches (the padding steps of the last group carry
            // use bits and weights 0).
            uint4 mk[PPW], sa[PPW], sb[PPW];
            uint32_t sc[PPW];
            const __attribute__((address_space(4))) float* wp[PPW];
            float4 w_cur[PPW][2];
#pragma unroll
            for (int i = 0; i < PPW; ++i) {
                const __attribute__((address_space(4))) uint32_t* rec = pairs + (size_t)pr[i] * 16;
                mk[i] = load_const_u4(rec);
                sa[i] = load_const_u4(rec + 4);
                sb[i] = load_const_u4(rec + 8);
                sc[i] = pairs[(size_t)pr[i] * 16 + 12];
                if (WSTREAM) {
                    wp[i] = pw + (size_t)pr[i] * 72;
                    w_cur[i][0] = load_const_f4(wp[i]);
                    w_cur[i][1] = load_const_f4(wp[i] + 4);
                }
            }
            uint64_t use0[PPW], use1[PPW];   // the use masks of output 0 / 1 as 64-bit scalars (WMODE 3)
#pragma unroll
            for (int i = 0; i < PPW; ++i) {
                use0[i] = (uint64_t)mk[i].x | ((uint64_t)mk[i].y << 32);
                use1[i] = (uint64_t)mk[i].z | ((uint64_t)mk[i].w << 32);
            }
            float xb[3][PPW][RL];
            float4 w_nxt[PPW][2];
#define SPDNN_SLOT(i, e)                                                                              \
    (((((e) >> 2) == 0 ? sa[i].x : ((e) >> 2) == 1 ? sa[i].y : ((e) >> 2) == 2 ? sa[i].z                \
       : ((e) >> 2) == 3 ? sa[i].w : ((e) >> 2) == 4 ? sb[i].x : ((e) >> 2) == 5 ? sb[i].y              \
       : ((e) >> 2) == 6 ? sb[i].z : ((e) >> 2) == 7 ? sb[i].w : sc[i]) >> (8 * ((e) & 3))) & (RING - 1))
#define SPDNN_SLOT_DWORD(i, e)                                                                        \
    (((e) >> 2) == 0 ? sa[i].x : ((e) >> 2) == 1 ? sa[i].y : ((e) >> 2) == 2 ? sa[i].z                  \
     : ((e) >> 2) == 3 ? sa[i].w : ((e) >> 2) == 4 ? sb[i].x : ((e) >> 2) == 5 ? sb[i].y                \
     : ((e) >> 2) == 6 ? sb[i].z : ((e) >> 2) == 7 ? sb[i].w : sc[i])
#define SPDNN_READ_COLUMN(i, e, x)                                                                    \
    do {                                                                                              \
        if (WMODE >= 3) lds_read<RL>(col_addr[(e) % 3][i], x);                                         \
        else vec_to_arr<RL>(*reinterpret_cast<const V*>(lane_smem + (size_t)SPDNN_SLOT(i, e) * COLB), x);     \
    } while (0)
            // WMODE 3: the LDS address of step e's column, worked out one iteration before its read is issued
            // (steps 0 .. 2 here, step s + 3 in the same statement as the adds of step s)
            uint32_t col_addr[3][PPW];
            if (WMODE >= 3) {
#pragma unroll
                for (int e = 0; e < 3; ++e)
#pragma unroll
                    for (int i = 0; i < PPW; ++i)
                        col_addr[e][i] = ring_address<SLOT_BITS, COL_SHIFT>(lane_base, SPDNN_SLOT_DWORD(i, e), e & 3);
            }
#define SPDNN_STEP_LIVE(e) (KT == 36 ? ((e) < 32 || (e) < steps) : (((e) & ~3) < steps))
#define SPDNN_USED(i, o, e) (((((e) < 32) ? ((o) ? mk[i].z : mk[i].x) : ((o) ? mk[i].w : mk[i].y)) >> ((e) & 31)) & 1u)
#pragma unroll
            for (int e = 0; e < 2; ++e)
#pragma unroll
                for (int i = 0; i < PPW; ++i)
                    SPDNN_READ_COLUMN(i, e, xb[e][i]);
#pragma unroll
            for (int st = 0; st < 36; ++st) {
                if (st + 2 < 36 && SPDNN_STEP_LIVE(st + 2)) {
#pragma unroll
                    for (int i = 0; i < PPW; ++i)
                        SPDNN_READ_COLUMN(i, st + 2, xb[(st + 2) % 3][i]);
                }
                if (WSTREAM && (st & 3) == 0 && st + 4 < 36) {  // two weights per step, four steps per trip
#pragma unroll
                    for (int i = 0; i < PPW; ++i) {
                        w_nxt[i][0] = load_const_f4(wp[i] + 4 * ((st >> 2) * 2 + 2));
                        w_nxt[i][1] = load_const_f4(wp[i] + 4 * ((st >> 2) * 2 + 3));
                    }
                }
                if (WMODE == 4) {
                    // twins: both outputs of the pair add every step - one accumulator, no masks
                    if (SPDNN_STEP_LIVE(st)) {
#pragma unroll
                        for (int i = 0; i < PPW; ++i) {
                            if (st + 3 < 36)
                                col_addr[st % 3][i] = add_then_address<RL, SLOT_BITS, COL_SHIFT>(
                                    acc[i][0], xb[st % 3][i], lane_base, SPDNN_SLOT_DWORD(i, st + 3), (st + 3) & 3);
                            else
#pragma unroll
                                for (int q = 0; q < RL; ++q) acc[i][0][q] += xb[st % 3][i][q];
                        }
                    }
                } else if (WMODE == 3) {
                    // (add_pair_if_used* set the execution mask and put it back to ALL ONES: every lane of the wave
                    // is active here - the walk's control flow is wave-uniform - and it must stay that way)
                    if (SPDNN_STEP_LIVE(st)) {
#pragma unroll
                        for (int i = 0; i < PPW; ++i) {
                            if (st + 3 < 36)
                                col_addr[st % 3][i] = add_pair_if_used_then_address<RL, SLOT_BITS, COL_SHIFT>(
                                    acc[i][0], acc[i][1], xb[st % 3][i], use0[i], use1[i], st, lane_base,
                                    SPDNN_SLOT_DWORD(i, st + 3), (st + 3) & 3);
                            else
                                add_pair_if_used<RL>(acc[i][0], acc[i][1], xb[st % 3][i], use0[i], use1[i], st);
                        }
                    }
                } else if (SPDNN_STEP_LIVE(st)) {
#pragma unroll
                    for (int i = 0; i < PPW; ++i) {
                        float w0, w1;
                        if (WSTREAM) {
                            const float4 wq = w_cur[i][(st >> 1) & 1];
                            w0 = (st & 1) ? wq.z : wq.x;
                            w1 = (st & 1) ? wq.w : wq.y;
                        } else {
                            w0 = __uint_as_float(wu_bits & (0u - SPDNN_USED(i, 0, st)));
                            w1 = __uint_as_float(wu_bits & (0u - SPDNN_USED(i, 1, st)));
                        }
#pragma unroll
                        for (int q = 0; q < RL; ++q) {
                            acc[i][0][q] = mac<WMODE>(acc[i][0][q], xb[st % 3][i][q], w0);
                            acc[i][1][q] = mac<WMODE>(acc[i][1][q], xb[st % 3][i][q], w1);
                        }
                    }
                }
                if (WSTREAM && (st & 3) == 3 && st + 1 < 36) {
#pragma unroll
                    for (int i = 0; i < PPW; ++i) {
                        w_cur[i][0] = w_nxt[i][0];
                        w_cur[i][1] = w_nxt[i][1];
                    }
                }
                // pin this step's arithmetic before the reads of later steps: without it the
                // compiler issues all reads of every pair first and spills
#pragma unroll
                for (int i = 0; i < PPW; ++i)
#pragma unroll
                    for (int q = 0; q < RL; ++q) {
                        asm volatile("" : "+v"(acc[i][0][q]) : : "memory");
                        asm volatile("" : "+v"(acc[i][1][q]) : : "memory");
                    }
            }
#undef SPDNN_SLOT
#undef SPDNN_SLOT_DWORD
#undef SPDNN_READ_COLUMN
#undef SPDNN_USED
#undef SPDNN_STEP_LIVE
        }

        // The parked columns go into ring slots no wave reads during this chunk - BEFORE the outputs
        // are stored: loads and stores share one counter on this hardware, so waiting for the parked
        // loads after the stores were issued would also wait for the stores to be acknowledged.
        // The write is unconditional: past the segment end it drops a copy of the last column into a
        // slot nobody reads any more, and every path has then waited for the parked loads here, so
        // that nothing downstream needs to wait on the memory counter again.
        if (DMA) {
            wait_vector_memory();  // the columns sent to the ring at the top of the chunk (and older stores)
        } else {
#pragma unroll
            for (int i = 0; i < OPW; ++i) {
                const int p = cb + T + wave + i * NW;
                *reinterpret_cast<V*>(smem + (size_t)(p & (RING - 1)) * COLB + loff * 4) = arr_to_vec<RL>(pf[i]);
            }
        }
        asm volatile("" ::: "memory");
#pragma unroll
        for (int i = 0; i < PPW; ++i) {
            const int v0 = cb + 2 * (wave + i * NW);
            if (v0 + 1 < ve) {
                // both outputs of the pair (the usual case: segments end at even positions)
                float y0[RL], y1[RL];
#pragma unroll
                for (int q = 0; q < RL; ++q) {
                    y0[q] = relu_clamp(WMODE >= 3 ? __builtin_fmaf(acc[i][0][q], wu, bias) : acc[i][0][q] + bias, clampv);
                    y1[q] = WMODE == 4 ? y0[q] : relu_clamp(WMODE == 3 ? __builtin_fmaf(acc[i][1][q], wu, bias) : acc[i][1][q] + bias, clampv);
                    nz[q] = nz_merge(nz[q], nz_merge(y0[q], y1[q]));   // one three-way maximum
                }
                const int d0 = dst[v0], d1 = dst[v0 + 1];
                if (stream) {
                    store_stream<RL>(yout + (size_t)d0 * RBL + loff, y0);
                    store_stream<RL>(yout + (size_t)d1 * RBL + loff, y1);
                } else {
                    *reinterpret_cast<V*>(yout + (size_t)d0 * RBL + loff) = arr_to_vec<RL>(y0);
                    *reinterpret_cast<V*>(yout + (size_t)d1 * RBL + loff) = arr_to_vec<RL>(y1);
                }
            } else if (v0 < ve) {
                float y[RL];
#pragma unroll
                for (int q = 0; q < RL; ++q) {
                    y[q] = relu_clamp(WMODE >= 3 ? __builtin_fmaf(acc[i][0][q], wu, bias) : acc[i][0][q] + bias, clampv);
                    nz[q] = nz_merge(nz[q], y[q]);
                }
                *reinterpret_cast<V*>(yout + (size_t)dst[v0] * RBL + loff) = arr_to_vec<RL>(y);
            }
        }

        ring_barrier<DMA>();
    }
}

template <int RL, int NW, int OPW, int RING, int WMODE, int KT, int DMA>
__global__ __launch_bounds__(NW * 64) void band_walk_kernel(
    Feat yin_all, Feat yout_all, const uint32_t* __restrict__ pairs,
    const float* __restrict__ pw, const int32_t* __restrict__ dst, int32_t* __restrict__ active,
    int32_t* __restrict__ count_prev, int N, int steps, int halo, int seglen, int stamp, int prev_stamp,
    int check_dead, float wu, float bias, float clampv, Publish pub, int nblk, int stream,
    const int32_t* __restrict__ frontier, int frontier_layer) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int RB = 64 * RL;
    publish_counts(pub);
    if ((int)blockIdx.x >= nblk) return;  // padding of the grid's x extent (see the launcher)
    // finishing a persistent launch that gave up: this row block has the layer behind it already
    if (frontier != nullptr && frontier[blockIdx.x] > frontier_layer) return;
    // row blocks vary fastest (measured: launching the segments of one row block together
    // instead is slower on live data and reads more from HBM)
    const int rb = blockIdx.x;
    const int vb = blockIdx.y * seglen;
    const int ve = min(N, vb + seglen);
    const size_t blkf = (size_t)N * RB;
    if (enter_row_block<RL>(active, (size_t)rb * RB + (threadIdx.x & 63) * RL, prev_stamp, stamp, check_dead, count_prev,
                            blockIdx.y == 0 && threadIdx.x < 64))
        return;
    float nz[RL];
#pragma unroll
    for (int q = 0; q < RL; ++q) nz[q] = 0.0f;
    band_walk_body<RL, NW, OPW, RING, WMODE, KT, DMA>(block_base(yin_all, rb, blkf), block_base(yout_all, rb, blkf), pairs,
                                                 pw, dst, N, steps, halo, vb, ve, wu, bias, clampv, smem, nz, stream);
    stamp_rows_workgroup<RL, NW>(nz, smem, active, (size_t)rb * RB, stamp, nullptr);
}

// ------------------------------------------------------------------------------------------
// Fused pair ("fused" variant with the intermediate tile in LDS): two consecutive BAND layers A
// and B, where A writes its outputs exactly where B's band reads them (dst of A = identity), run
// in ONE launch and the activations between them never leave the CU.  The reference fuses the same
// way: a tile of the last layer's outputs, the tile of the layer before sized to cover its halo,
// the intermediate kept in shared memory (src/microbenchmark/fuse.cu:16-110, tile recurrence
// :226-248; the analysis that says which inputs a tile needs is src/fuse/fuse.h:13-53).
//
// A workgroup of 16 waves takes one row block (256 rows) and a segment [vb, ve) of B's band
// positions.  Waves 0-7 walk layer A over positions [vb-32, ve) - B's halo of up to 32 positions is
// computed again by the workgroup of the segment before, the price of not sharing tiles between
// workgroups - from a 64-slot LDS ring fed straight from HBM, and drop their outputs, after the
// epilogue, into a second 64-slot ring.  Waves 8-15 walk layer B over [vb, ve) three chunks behind,
// reading the second ring and storing to HBM.  One barrier per chunk of 16 positions; at step s
// layer A writes ring positions [vb-32+16s, vb-16+16s) while layer B reads [vb-80+16s, vb-32+16s):
// 64 consecutive positions, so no slot is written while it is read.
// HBM traffic per pair of layers: one read and one write of the feature block (plus A's halo of
// 64 columns per segment) instead of two of each.
// ------------------------------------------------------------------------------------------
struct PairSide {
    float wu;
    int halo;
    int steps;
};

// The 2 x 4 x steps multiply-adds of one output pair for a lane's four rows, inputs from an LDS ring
// (16-dword pair records: two 64-bit use masks, 36 one-byte ring selectors; weights per step and
// output unless WMODE is 0).  The LDS read of step s+2 is issued before the arithmetic of step s.
template <int WMODE>
__device__ __forceinline__ void pair_accumulate(const unsigned char* lane_ring, const uint32_t* __restrict__ pairs,
                                                const float* __restrict__ pw, int pr, int steps, uint32_t wu_bits,
                                                float (&acc)[2][4]) {
    const uint4* rec = reinterpret_cast<const uint4*>(pairs + (size_t)pr * 16);
    uint4 mk = rec[0], sa = rec[1], sb = rec[2];
    uint32_t sc = pairs[(size_t)pr * 16 + 12];
    if (WMODE == 3) {
        // the record is the same for every lane; the add-only walk hands its words to the scalar unit as
        // they are, so say so where the compiler has not seen it (free where it has)
        auto uni = [](uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); };
        mk = make_uint4(uni(mk.x), uni(mk.y), uni(mk.z), uni(mk.w));
        sa = make_uint4(uni(sa.x), uni(sa.y), uni(sa.z), uni(sa.w));
        sb = make_uint4(uni(sb.x), uni(sb.y), uni(sb.z), uni(sb.w));
        sc = uni(sc);
    }
    const float4* wp = nullptr;
    float4 w_cur[2], w_nxt[2];
    constexpr bool WSTREAM = WMODE == 1 || WMODE == 2;   // weights come per step from the plan
    const uint32_t lane_base = (uint32_t)(size_t)((const __attribute__((address_space(3))) unsigned char*)lane_ring);
    const uint64_t use0 = (uint64_t)mk.x | ((uint64_t)mk.y << 32), use1 = (uint64_t)mk.z | ((uint64_t)mk.w << 32);
    if (WSTREAM) {
        wp = reinterpret_cast<const float4*>(pw + (size_t)pr * 72);
        w_cur[0] = wp[0];
        w_cur[1] = wp[1];
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) acc[0][q] = acc[1][q] = 0.0f;
    float xb[3][4];
#define SPDNN_PSLOT(e)                                                                                   \
    (((((e) >> 2) == 0 ? sa.x : ((e) >> 2) == 1 ? sa.y : ((e) >> 2) == 2 ? sa.z : ((e) >> 2) == 3 ? sa.w  \
       : ((e) >> 2) == 4 ? sb.x : ((e) >> 2) == 5 ? sb.y : ((e) >> 2) == 6 ? sb.z : ((e) >> 2) == 7 ? sb.w : sc) >> (8 * ((e) & 3))) & 63u)
#define SPDNN_PSLOT_DWORD(e)                                                                             \
    (((e) >> 2) == 0 ? sa.x : ((e) >> 2) == 1 ? sa.y : ((e) >> 2) == 2 ? sa.z : ((e) >> 2) == 3 ? sa.w    \
     : ((e) >> 2) == 4 ? sb.x : ((e) >> 2) == 5 ? sb.y : ((e) >> 2) == 6 ? sb.z : ((e) >> 2) == 7 ? sb.w : sc)
#define SPDNN_PREAD(e, x)                                                                                \
    do {                                                                                                 \
        if (WMODE == 3) lds_read<4>(col_addr[(e) % 3], x);                                                \
        else vec_to_arr<4>(*reinterpret_cast<const float4*>(lane_ring + (size_t)SPDNN_PSLOT(e) * 1024), x); \
    } while (0)
    uint32_t col_addr[3];   // WMODE 3: LDS address of step e's column, worked out one iteration before its read
    if (WMODE == 3) {
#pragma unroll
        for (int e = 0; e < 3; ++e) col_addr[e] = ring_address<6, 10>(lane_base, SPDNN_PSLOT_DWORD(e), e & 3);
    }
#define SPDNN_PUSED(o, e) (((((e) < 32) ? ((o) ? mk.z : mk.x) : ((o) ? mk.w : mk.y)) >> ((e) & 31)) & 1u)
#pragma unroll
    for (int e = 0; e < 2; ++e)
        SPDNN_PREAD(e, xb[e]);
#pragma unroll
    for (int st = 0; st < 36; ++st) {
        if (st + 2 < 36 && (st + 2 < 32 || st + 2 < steps))
            SPDNN_PREAD(st + 2, xb[(st + 2) % 3]);
        if (WSTREAM && (st & 3) == 0 && st + 4 < 36) {
            w_nxt[0] = wp[(st >> 2) * 2 + 2];
            w_nxt[1] = wp[(st >> 2) * 2 + 3];
        }
        if (WMODE == 3) {
            // (as in the band walk: the callee leaves the execution mask at all ones, which is what it is here - the
            // branches around this code are wave-uniform - and must stay)
            if (st < 32 || st < steps) {
                if (st + 3 < 36)
                    col_addr[st % 3] = add_pair_if_used_then_address<4, 6, 10>(acc[0], acc[1], xb[st % 3], use0, use1, st, lane_base,
                                                                               SPDNN_PSLOT_DWORD(st + 3), (st + 3) & 3);
                else
                    add_pair_if_used<4>(acc[0], acc[1], xb[st % 3], use0, use1, st);
            }
        } else if (st < 32 || st < steps) {
            float w0, w1;
            if (WSTREAM) {
                const float4 wq = w_cur[(st >> 1) & 1];
                w0 = (st & 1) ? wq.z : wq.x;
                w1 = (st & 1) ? wq.w : wq.y;
            } else {
                w0 = __uint_as_float(wu_bits & (0u - SPDNN_PUSED(0, st)));
                w1 = __uint_as_float(wu_bits & (0u - SPDNN_PUSED(1, st)));
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                acc[0][q] = mac<WMODE>(acc[0][q], xb[st % 3][q], w0);
                acc[1][q] = mac<WMODE>(acc[1][q], xb[st % 3][q], w1);
            }
        }
        if (WSTREAM && (st & 3) == 3 && st + 1 < 36) {
            w_cur[0] = w_nxt[0];
            w_cur[1] = w_nxt[1];
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {   // keeps the reads of later steps behind this step's arithmetic
            asm volatile("" : "+v"(acc[0][q]) : : "memory");
            asm volatile("" : "+v"(acc[1][q]) : : "memory");
        }
    }
#undef SPDNN_PSLOT
#undef SPDNN_PSLOT_DWORD
#undef SPDNN_PREAD
#undef SPDNN_PUSED
}

template <int WMODE>
__global__ __launch_bounds__(1024) void band_pair_kernel(
    Feat yin_all, Feat yout_all, const uint32_t* __restrict__ pairs_a, const float* __restrict__ pw_a,
    const uint32_t* __restrict__ pairs_b, const float* __restrict__ pw_b, PairSide A, PairSide B,
    const int32_t* __restrict__ dst,
    int32_t* __restrict__ active, int32_t* __restrict__ active_mid, int32_t* __restrict__ count_prev, int N,
    int seglen, int stamp_a, int stamp_b, int prev_stamp, int check_dead, float bias, float clampv, Publish pub,
    int nblk, int stream) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int RB = 256, COLB = 1024, T = 16;
    unsigned char* ring_a = smem;                 // inputs of layer A, 64 column slots
    unsigned char* ring_b = smem + 64 * COLB;     // outputs of layer A = inputs of layer B
    publish_counts(pub);
    if ((int)blockIdx.x >= nblk) return;
    const int rb = blockIdx.x;
    const int vb = blockIdx.y * seglen;
    const int ve = min(N, vb + seglen);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int role = wave >> 3, w = wave & 7;     // role 0: layer A, role 1: layer B
    const int loff = lane * 4;
    if (enter_row_block<4>(active, (size_t)rb * RB + loff, prev_stamp, stamp_b, check_dead, count_prev,
                           blockIdx.y == 0 && threadIdx.x < 64))
        return;
    const size_t blkf = (size_t)N * RB;
    const float* __restrict__ yin = block_base(yin_all, rb, blkf);
    float* __restrict__ yout = block_base(yout_all, rb, blkf);
    const int nb = (ve - vb) / T;                 // chunks of layer B (segments are whole chunks)
    const int na = nb + 2;                        // chunks of layer A: B's halo of 32 positions first
    const int va0 = vb - 32;                      // first position layer A computes (may be negative: wraps)
    float nz[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    const uint32_t wu_bits = (uint32_t)__builtin_amdgcn_readfirstlane((int)__float_as_uint(role ? B.wu : A.wu));
    const float wu = __uint_as_float(wu_bits);   // the layer's one weight (WMODE 0 and 3)

    if (role == 0) {
        // layer A's halo and first chunk
        for (int c = w; c < A.halo + T; c += 8) {
            const int p = va0 - A.halo + c;
            const int g = p < 0 ? p + N : p;
            unsigned char* slot = ring_a + (size_t)(p & 63) * COLB;
            if (stream) column_to_lds<1, WMODE != 3>(yin + (size_t)g * RB + loff, slot);
            else column_to_lds<0, WMODE != 3>(yin + (size_t)g * RB + loff, slot);
        }
        wait_vector_memory();
    }
    ring_barrier<1>();

    for (int s = 0; s < nb + 3; ++s) {
        if (role == 0) {
            if (s < na) {
                const int cb = va0 + s * T;
                if (s + 1 < na) {
#pragma unroll
                    for (int i = 0; i < 2; ++i) {
                        const int p = cb + T + w + i * 8;
                        const int g = p < 0 ? p + N : p;
                        unsigned char* slot = ring_a + (size_t)(p & 63) * COLB;
                        if (stream) column_to_lds<1, WMODE != 3>(yin + (size_t)g * RB + loff, slot);
                        else column_to_lds<0, WMODE != 3>(yin + (size_t)g * RB + loff, slot);
                    }
                }
                const int v0 = cb + 2 * w;
                const int pr = (v0 < 0 ? v0 + N : v0) >> 1;
                float acc[2][4];
                pair_accumulate<WMODE>(ring_a + loff * 4, pairs_a, pw_a, pr, A.steps, wu_bits, acc);
                float y0[4], y1[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    y0[q] = relu_clamp(WMODE == 3 ? __builtin_fmaf(acc[0][q], wu, bias) : acc[0][q] + bias, clampv);
                    y1[q] = relu_clamp(WMODE == 3 ? __builtin_fmaf(acc[1][q], wu, bias) : acc[1][q] + bias, clampv);
                    nz[q] = nz_merge(nz[q], nz_merge(y0[q], y1[q]));
                }
                *reinterpret_cast<float4*>(ring_b + (size_t)(v0 & 63) * COLB + loff * 4) = arr_to_vec<4>(y0);
                *reinterpret_cast<float4*>(ring_b + (size_t)((v0 + 1) & 63) * COLB + loff * 4) = arr_to_vec<4>(y1);
                wait_vector_memory();   // the next chunk's columns are in ring A
            }
        } else if (s >= 3) {
            const int v0 = vb + (s - 3) * T + 2 * w;
            float acc[2][4];
            pair_accumulate<WMODE>(ring_b + loff * 4, pairs_b, pw_b, v0 >> 1, B.steps, wu_bits, acc);
            float y0[4], y1[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                y0[q] = relu_clamp(WMODE == 3 ? __builtin_fmaf(acc[0][q], wu, bias) : acc[0][q] + bias, clampv);
                y1[q] = relu_clamp(WMODE == 3 ? __builtin_fmaf(acc[1][q], wu, bias) : acc[1][q] + bias, clampv);
                nz[q] = nz_merge(nz[q], nz_merge(y0[q], y1[q]));
            }
            const int d0 = dst[v0], d1 = dst[v0 + 1];
            if (stream) {
                store_stream<4>(yout + (size_t)d0 * RB + loff, y0);
                store_stream<4>(yout + (size_t)d1 * RB + loff, y1);
            } else {
                *reinterpret_cast<float4*>(yout + (size_t)d0 * RB + loff) = arr_to_vec<4>(y0);
                *reinterpret_cast<float4*>(yout + (size_t)d1 * RB + loff) = arr_to_vec<4>(y1);
            }
        }
        ring_barrier<1>();
    }

    // row stamps: layer A's into active_mid, layer B's into active (the rings are free now)
    float* sm = reinterpret_cast<float*>(smem);
#pragma unroll
    for (int q = 0; q < 4; ++q) sm[wave * RB + loff + q] = nz[q];
    __syncthreads();
    if (threadIdx.x < 2 * RB) {
        const int which = threadIdx.x >> 8, r = threadIdx.x & 255;
        float m = sm[(which * 8) * RB + r];
#pragma unroll
        for (int k = 1; k < 8; ++k) m = nz_merge(m, sm[(which * 8 + k) * RB + r]);
        if (m > 0.0f) {
            if (which) active[(size_t)rb * RB + r] = stamp_b;
            else active_mid[(size_t)rb * RB + r] = stamp_a;
        }
    }
}

// rows of [0, rows) that carry `stamp`: the count of a layer whose stamps no later launch looks at
__global__ __launch_bounds__(256) void count_stamped_kernel(const int32_t* __restrict__ stamps, int rows, int stamp,
                                                            int32_t* __restrict__ count_out) {
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    const int hit = (r < rows && stamps[r] == stamp) ? 1 : 0;
    const int n = (int)__popcll(__ballot(hit));
    if ((threadIdx.x & 63) == 0 && n > 0) atomicAdd(count_out, n);
}

// ------------------------------------------------------------------------------------------
// GATHER kernel (general CSR / ELL): any sparsity pattern, any row length.  Each wave takes
// OPG consecutive outputs of one row block and reads every input column straight from
// global memory (L2), RB*4 contiguous bytes per read.  No reuse beyond the caches: this is the
// fallback for layers the inspector cannot relabel into a band.
// ------------------------------------------------------------------------------------------
template <int RL, int WMODE>
__global__ __launch_bounds__(256) void gather_kernel(
    Feat yin_all, Feat yout_all, const int32_t* __restrict__ cols,
    const int32_t* __restrict__ rowlen, const float* __restrict__ wv, const int32_t* __restrict__ dst,
    int32_t* __restrict__ active, int32_t* __restrict__ count_prev, int N, int kmax, int opg, int stamp,
    int prev_stamp, int check_dead, float bias, float clampv, Publish pub) {
    using V = typename VecOf<RL>::type;
    constexpr int RB = 64 * RL;
    publish_counts(pub);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int rb = blockIdx.x;
    if (enter_row_block<RL>(active, (size_t)rb * RB + lane * RL, prev_stamp, stamp, check_dead, count_prev,
                            blockIdx.y == 0 && wave == 0))
        return;
    const float* __restrict__ yin = block_base(yin_all, rb, (size_t)N * RB);
    float* __restrict__ yout = block_base(yout_all, rb, (size_t)N * RB);
    const int loff = lane * RL;
    const int j0 = (blockIdx.y * 4 + wave) * opg;
    const int j1 = min(N, j0 + opg);

    float nz[RL];
#pragma unroll
    for (int q = 0; q < RL; ++q) nz[q] = 0.0f;

    for (int j = j0; j < j1; ++j) {
        const int cnt = rowlen[j];
        // Four entries per trip, their four columns requested together (one entry after the other every trip is a
        // scalar load, then a column load, then the arithmetic, each waiting for the one before).  Rows are padded to a
        // multiple of four entries with (column 0, weight +0): x * (+0) added to an accumulator that started at +0
        // changes nothing.  The next trip's entries are requested before this trip's arithmetic.
        const __attribute__((address_space(4))) uint32_t* cp = (const __attribute__((address_space(4))) uint32_t*)(cols + (size_t)j * kmax);
        const __attribute__((address_space(4))) float* wp = (const __attribute__((address_space(4))) float*)(wv + (size_t)j * kmax);
        float acc[RL];
#pragma unroll
        for (int q = 0; q < RL; ++q) acc[q] = 0.0f;
        uint4 c4 = make_uint4(0u, 0u, 0u, 0u);
        float4 w4 = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (cnt > 0) { c4 = load_const_u4(cp); w4 = load_const_f4(wp); }
        for (int m = 0; m < cnt; m += 4) {
            const uint4 c = c4;
            const float4 w = w4;
            V xv[4];
            xv[0] = *reinterpret_cast<const V*>(yin + (size_t)c.x * RB + loff);
            xv[1] = *reinterpret_cast<const V*>(yin + (size_t)c.y * RB + loff);
            xv[2] = *reinterpret_cast<const V*>(yin + (size_t)c.z * RB + loff);
            xv[3] = *reinterpret_cast<const V*>(yin + (size_t)c.w * RB + loff);
            if (m + 4 < cnt) { c4 = load_const_u4(cp + m + 4); w4 = load_const_f4(wp + m + 4); }
            const float ws[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float x[RL];
                vec_to_arr<RL>(xv[e], x);
#pragma unroll
                for (int q = 0; q < RL; ++q) acc[q] = mac<WMODE>(acc[q], x[q], ws[e]);
            }
        }
        float y[RL];
#pragma unroll
        for (int q = 0; q < RL; ++q) {
            y[q] = relu_clamp(acc[q] + bias, clampv);
            nz[q] = nz_merge(nz[q], y[q]);
        }
        *reinterpret_cast<V*>(yout + (size_t)dst[j] * RB + loff) = arr_to_vec<RL>(y);
    }
    stamp_rows<RL>(nz, active, (size_t)rb * RB + loff, stamp);
}

// ------------------------------------------------------------------------------------------
// TILED kernel (general class with reuse): a workgroup of 16 waves takes 64 feature rows (lane =
// row: a quarter of a 256-row block) and a tile of 1024 outputs, 64 per wave, whose accumulators
// stay in registers.  The tile's input columns (the union over its outputs, ascending) pass through
// LDS in panels of 512 columns x 256 bytes, fed straight from global memory; every column is read
// once per tile, whatever the number of outputs that use it.  Per panel a wave works through
// `rounds` rounds of 2 entries per output.  An entry is an LDS byte offset and a weight; streaming
// 8 bytes per multiply-add through the scalar cache does not work (every access misses, and the
// cache serves few misses at a time: measured 0.69 ms per layer of 1024 neurons where the plain
// gather takes 0.45), so the entry blocks (1 KiB per round and wave) go through LDS too, into a
// per-wave ring.  Four reads put a round's block into registers (lane j of every 16-lane row holds
// the entries of outputs j, 16 + j, 32 + j, 48 + j) and the DPP row broadcast hands an entry's offset
// and weight to all lanes inside the add and the multiply that use them.  (Reading the entries back
// pair by pair with broadcast LDS reads - all lanes the same address - took half an LDS instruction
// more per entry: 0.266 against 0.239 ms per layer of 1024 neurons.)
// Accumulation in ascending input index: panels ascend, entries inside a panel ascend; padding
// entries carry weight -0 and add an exact zero.
// ------------------------------------------------------------------------------------------
// 64 lanes x 16 bytes from global memory into 1 KiB of LDS, issued in a form the compiler does not
// follow: it puts a wait for ALL vector memory traffic in front of any LDS read that might touch
// the destination of a direct-to-LDS load it knows of, which here would be the very next read (the
// other half of the wave's entry ring).  The caller waits itself (wait_vector_memory).
__device__ __forceinline__ void block_to_lds_untracked(const float* gsrc_lane, unsigned char* lds_block) {
    const uint32_t lds_off = (uint32_t)(size_t)((__attribute__((address_space(3))) unsigned char*)lds_block);
    uint32_t m0_saved;   // M0 (the LDS base of such a load) is the compiler's to manage: put it back
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, off\n\ts_mov_b32 m0, %0"
                 : "=&s"(m0_saved)
                 : "s"(lds_off), "v"(gsrc_lane)
                 : "memory");
}

// The value lane j of every 16-lane row holds, in all lanes of that row (DPP row_newbcast: the
// compiler folds the move into the instruction that uses it).
__device__ __forceinline__ uint32_t row_lane(uint32_t v, int j) {
    switch (j) {
#define SPDNN_ROW_LANE(J) case J: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x150 + J, 0xf, 0xf, true);
        SPDNN_ROW_LANE(0) SPDNN_ROW_LANE(1) SPDNN_ROW_LANE(2) SPDNN_ROW_LANE(3) SPDNN_ROW_LANE(4) SPDNN_ROW_LANE(5)
        SPDNN_ROW_LANE(6) SPDNN_ROW_LANE(7) SPDNN_ROW_LANE(8) SPDNN_ROW_LANE(9) SPDNN_ROW_LANE(10) SPDNN_ROW_LANE(11)
        SPDNN_ROW_LANE(12) SPDNN_ROW_LANE(13) SPDNN_ROW_LANE(14) SPDNN_ROW_LANE(15)
#undef SPDNN_ROW_LANE
    }
    return v;
}

template <int WMODE>
__global__ __launch_bounds__(1024) void tiled_kernel(
    Feat yin_all, Feat yout_all, const int32_t* __restrict__ cols, const int32_t* __restrict__ hdr,
    const uint32_t* __restrict__ ent, const int32_t* __restrict__ dst, int32_t* __restrict__ active,
    int32_t* __restrict__ count_prev, int N, int ntiles, int rl, int stamp, int prev_stamp, int check_dead,
    float bias, float clampv, Publish pub) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int PANEL_BYTES = 512 * 256;   // then 16 waves x 2 entry blocks of 1 KiB
    publish_counts(pub);
    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int RB = 64 * rl;
    // Which (64 rows, tile) this workgroup takes.  The tiles of one set of rows read much the same input columns
    // (for layers without structure: all of them), so they should run at the same time behind the same L2:
    // workgroups go to the 8 XCDs round robin by number, so the tiles of row set sb get the numbers
    // sb % 8 + 8 * (tile + ntiles * (sb / 8)) - consecutive workgroups of one XCD.  (Row sets beyond the last
    // whole eight: tile after tile.)
    const int nsb = (int)gridDim.x / ntiles, nsb8 = nsb / 8 * 8;
    int sb, t;
    if ((int)blockIdx.x < nsb8 * ntiles) {
        const int x = (int)blockIdx.x % 8, k = (int)blockIdx.x / 8;
        t = k % ntiles;
        sb = (k / ntiles) * 8 + x;
    } else {
        const int rem = (int)blockIdx.x - nsb8 * ntiles;
        sb = nsb8 + rem / ntiles;
        t = rem % ntiles;
    }
    const int rb = sb / rl, q = sb - rb * rl;
    const size_t row = (size_t)rb * RB + q * 64 + lane;
    if (prev_stamp != 0 && (check_dead || (count_prev != nullptr && t == 0))) {
        // Only a row block without ANY active row may be skipped (the kernels of the other classes
        // decide per row block too, and expect the dead rows of a live block to hold zeros, which
        // computing them gives); the count is taken per 64 rows.  Every wave reads the same stamps,
        // so the whole workgroup takes the same way.
        int alive_block = 0, alive_own = 0;
        for (int i = 0; i < rl; ++i) {
            const int a = active[(size_t)rb * RB + i * 64 + lane];
            const int c = (int)__popcll(__ballot((a == prev_stamp || a == stamp) ? 1 : 0));
            alive_block += c;
            if (i == q) alive_own = c;
        }
        if (count_prev != nullptr && t == 0 && threadIdx.x == 0 && alive_own > 0) atomicAdd(count_prev, alive_own);
        if (check_dead && alive_block == 0) return;
    }
    const float* __restrict__ yin = block_base(yin_all, rb, (size_t)N * RB) + q * 64 + lane;
    float* __restrict__ yout = block_base(yout_all, rb, (size_t)N * RB) + q * 64 + lane;
    const int gp0 = hdr[2 * t], np = hdr[2 * t + 1];
    const int32_t* __restrict__ wave_hdr = hdr + 2 * ntiles;
    unsigned char* ring = smem + PANEL_BYTES + w * 2048;          // this wave's two entry blocks
    const unsigned char* lane_panel = smem + lane * 4;

    float acc[64];
#pragma unroll
    for (int o = 0; o < 64; ++o) acc[o] = 0.0f;

    for (int p = 0; p < np; ++p) {
        // the panel's columns, 32 per wave (every wave has finished the panel before: barrier below).  Four
        // columns per instruction: a column is 64 rows x 4 bytes = the 16-byte parts of 16 lanes, so each
        // quarter of the wave brings its own column and the four land in consecutive slots.
        const int32_t* pc = cols + (size_t)(gp0 + p) * 512;
        {
            const float* quarter_src = yin - lane + (lane & 15) * 4;   // (yin points at this lane's row)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int sl0 = w * 32 + i * 4;
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void*)(quarter_src + (size_t)pc[sl0 + (lane >> 4)] * RB),
                    (__attribute__((address_space(3))) void*)(smem + sl0 * 256), 16, 0, 0);
            }
        }
        const int rounds = wave_hdr[((size_t)(gp0 + p) * 16 + w) * 2];
        const float* blk = reinterpret_cast<const float*>(ent) + (size_t)wave_hdr[((size_t)(gp0 + p) * 16 + w) * 2 + 1] * 256;
        if (rounds > 0) {
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(blk + lane * 4),
                                             (__attribute__((address_space(3))) void*)ring, 16, 0, 0);
        }
        wait_vector_memory();
        ring_barrier<1>();
        {
            // A round's entry block, [output][2](LDS offset of the column, weight), goes into registers with four
            // reads: lane j of each of the wave's four 16-lane rows takes the 16 bytes of output 16 g + j, g = 0 .. 3
            // (the rows read the same addresses).  An entry's offset and weight then come to all lanes of a row
            // through the DPP row broadcast of the add and the multiply that use them: one LDS instruction per
            // entry (the column) instead of one and a half.
            const uint32_t ent_base = (uint32_t)(size_t)((__attribute__((address_space(3))) unsigned char*)ring) + (lane & 15) * 16;
            const uint32_t panel_base = (uint32_t)(size_t)((__attribute__((address_space(3))) const unsigned char*)lane_panel);
            float mg[4][4];
            if (rounds > 0) {
#pragma unroll
                for (int g = 0; g < 4; ++g) lds_read<4>(ent_base + g * 256, mg[g]);
            }
            for (int r = 0; r < rounds; ++r) {
                if (r + 1 < rounds) {
                    // the block is in registers: the next round's comes into the same kilobyte
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    block_to_lds_untracked(blk + (size_t)(r + 1) * 256 + lane * 4, ring);
                }
                // units of two outputs (four entries), the columns of the next unit in flight during the arithmetic (two
                // units ahead measures the same)
                float x[2][4];
#define SPDNN_TILE_READ(u, buf)                                                                                 \
    do {                                                                                                        \
        _Pragma("unroll") for (int e = 0; e < 4; ++e) {                                                         \
            const int o = (u) * 2 + (e >> 1);                                                                   \
            const uint32_t off = row_lane(__float_as_uint(mg[o >> 4][(e & 1) * 2]), o & 15);                    \
            lds_read<1>(off + panel_base, &x[buf][e]);                                                          \
        }                                                                                                       \
    } while (0)
                SPDNN_TILE_READ(0, 0);
#pragma unroll 32
                for (int u = 0; u < 32; ++u) {
                    if (u + 1 < 32) SPDNN_TILE_READ(u + 1, (u + 1) & 1);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int o = u * 2 + (e >> 1);
                        const float wgt = __uint_as_float(row_lane(__float_as_uint(mg[o >> 4][(e & 1) * 2 + 1]), o & 15));
                        acc[o] = mac<WMODE>(acc[o], x[u & 1][e], wgt);
                    }
                    // pins the unit's arithmetic here: left alone the compiler gathers all reads of the round first
                    asm volatile("" : "+v"(acc[u * 2]), "+v"(acc[u * 2 + 1]) : : "memory");
                    __builtin_amdgcn_sched_barrier(0);
                }
#undef SPDNN_TILE_READ
                if (r + 1 < rounds) {
                    wait_vector_memory();   // the next entry block has arrived
#pragma unroll
                    for (int g = 0; g < 4; ++g) lds_read<4>(ent_base + g * 256, mg[g]);
                }
            }
        }
        ring_barrier<1>();          // every wave is done with the panel
    }

    float nz = 0.0f;
#pragma unroll
    for (int o = 0; o < 64; ++o) {
        const int d = dst[(size_t)t * 1024 + w * 64 + o];
        if (d >= 0) {
            const float y = relu_clamp(acc[o] + bias, clampv);
            nz = nz_merge(nz, y);
            yout[(size_t)d * RB] = y;
        }
    }
    float* sm = reinterpret_cast<float*>(smem);
    sm[w * 64 + lane] = nz;
    __syncthreads();
    if (threadIdx.x < 64) {
        float m = sm[lane];
#pragma unroll
        for (int k = 1; k < 16; ++k) m = nz_merge(m, sm[k * 64 + lane]);
        if (m > 0.0f) active[row] = stamp;
    }
}

// Lanes in groups of P (4, 2 or 1) neighbours.  group_turn: the value of the lane i places down in the group (lane j
// takes from lane (j - i) mod P); group_lane_value: the value of lane r of the group.  i and r are constants after
// unrolling (DPP quad permutations).
template <int P> __device__ __forceinline__ uint32_t group_turn_u32(uint32_t v, int i) {
    if constexpr (P == 4) {
        switch (i & 3) {
            case 1: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x93, 0xf, 0xf, true);   // quad_perm [3,0,1,2]
            case 2: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4e, 0xf, 0xf, true);   // quad_perm [2,3,0,1]
            case 3: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x39, 0xf, 0xf, true);   // quad_perm [1,2,3,0]
            default: return v;
        }
    } else if constexpr (P == 2) {
        return (i & 1) ? (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xb1, 0xf, 0xf, true) : v;  // quad_perm [1,0,3,2]
    } else {
        return v;
    }
}
template <int P> __device__ __forceinline__ float4 group_turn(const float4& v, int i) {
    float4 o;
    o.x = __uint_as_float(group_turn_u32<P>(__float_as_uint(v.x), i));
    o.y = __uint_as_float(group_turn_u32<P>(__float_as_uint(v.y), i));
    o.z = __uint_as_float(group_turn_u32<P>(__float_as_uint(v.z), i));
    o.w = __uint_as_float(group_turn_u32<P>(__float_as_uint(v.w), i));
    return o;
}
template <int P> __device__ __forceinline__ uint32_t group_lane_value(uint32_t v, int r) {
    if constexpr (P == 4) {
        switch (r & 3) {
            case 0: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x00, 0xf, 0xf, true);
            case 1: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x55, 0xf, 0xf, true);
            case 2: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xaa, 0xf, 0xf, true);
            default: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xff, 0xf, 0xf, true);
        }
    } else if constexpr (P == 2) {
        return (r & 1) ? (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xf5, 0xf, 0xf, true)    // quad_perm [1,1,3,3]
                       : (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xa0, 0xf, 0xf, true);   // quad_perm [0,0,2,2]
    } else {
        return v;
    }
}

// ------------------------------------------------------------------------------------------
// ROWTILE kernel (the other form of a TILED layer): the transposed assignment.  A workgroup of 1024
// threads stages R feature rows - all N columns of them - in LDS, laid out [column][row], and thread
// t computes whole outputs (slots t, t + 1024, ...) for those R rows, the rows in registers.  A lane
// walks its own entry list (input column, weight: 8 bytes from memory, entry-major so that the lanes
// of a wave read neighbouring words, the next entry requested under the arithmetic) and reads the
// column's R rows with R/4 16-byte LDS reads, so an LDS instruction serves four multiply-adds
// instead of one; lanes of a wave differ only in the number of entries, and the slots are ordered by
// length.  No panels, so no padding per panel: with the tiles two fifths of the entry slots are
// padding on layers of 1..24 random inputs, here a fourteenth.  Lane l reads the four-row parts of
// a column in the order l, l + 1, ... (mod R/4) - all lanes at the same part would meet in the same
// banks - and so holds the rows in a rotated order, which only its stores and its alive bits need to
// know.  Accumulation: ascending input index per output, as everywhere.
//
// Measured at N=1024, batch 60000, 1..24 random inputs per output, per layer: 156 us where the tiles take 228
// (166 before the lanes traded parts for the stores); with parts of the kernel switched off, then: nothing but
// the launch 25 us, rows in 40, arithmetic (with its entry reads: 105 KB per row set from L2) 51, rows out 55 -
// the phases add up.  Two other forms were built and
// measured no faster, and are gone: one workgroup per CU that stays and takes row set after row set with two LDS
// buffers, its entries requested a group ahead (192 us), and the same with the entry lists held in registers
// for the whole launch and the rows brought straight into LDS (169 us: its arithmetic is hidden entirely, and
// rows in and out alone take those 169 us - 64-byte pieces both ways, a third of the memory's rate).
// ------------------------------------------------------------------------------------------
struct RowtileArgs {
    Feat yin, yout;
    const uint32_t* ent;
    const int32_t* len;
    const int32_t* dst;
    int32_t* active;
    int32_t* count_prev;
    int N, kmax, rl, stamp, prev_stamp, check_dead;
    float bias, clampv;
    Publish pub;
};

template <int R, int WMODE, bool PAIRS>
__global__ __launch_bounds__(1024) void rowtile_kernel(RowtileArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int sh_alive;
    constexpr int PARTS = R / 4;
    publish_counts(a.pub);
    const int t = (int)threadIdx.x, lane = t & 63;
    const int RB = 64 * a.rl;
    // every XCD takes a contiguous eighth of the rows (see block_resident_kernel)
    const unsigned nwg = gridDim.x;
    const unsigned wg = (nwg % 8u) == 0u ? (blockIdx.x % 8u) * (nwg / 8u) + blockIdx.x / 8u : blockIdx.x;
    const size_t row0 = (size_t)wg * R;
    const int rb = (int)(row0 / (size_t)RB), rin = (int)(row0 - (size_t)rb * RB);
    if (a.prev_stamp != 0 && (a.check_dead || (a.count_prev != nullptr && rin == 0))) {
        // the rows the layer before left active in this row block: counted by the block's first workgroup; a row
        // block without any is skipped (as by the other per-layer kernels)
        const int st = t < RB ? a.active[(size_t)rb * RB + t] : 0;
        const bool alive = t < RB && (st == a.prev_stamp || st == a.stamp);
        const int n_alive = (int)__popcll(__ballot(alive ? 1 : 0));
        if (a.count_prev != nullptr && rin == 0 && lane == 0 && n_alive > 0) atomicAdd(a.count_prev, n_alive);
        if (a.check_dead && __builtin_amdgcn_readfirstlane(__syncthreads_or(alive ? 1 : 0)) == 0) return;
    }
    const size_t blkf = (size_t)a.N * RB;
    // A slot's length, output column and first entries are requested ahead - for the first slot before the rows come
    // in, for a later one under the slot before it - and kept as they come: requested where they are needed they are
    // two round trips to L2 in a row that the whole workgroup waits for.  (Entries 0 and 1 exist for every slot: the
    // lists are padded to four entries and more.)
    typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
    using GB = const __attribute__((address_space(1))) unsigned char*;
    const GB entb = (GB)a.ent;
    const uint32_t estride = (uint32_t)a.N * 8u;   // bytes from a slot's entry k to its entry k + 1
    int n_in_next, d_next;
    u32x2 e0_next, e1_next;
    auto request_slot = [&](int slot0) {
        const int slot = slot0 + t;
        const int sq = slot < a.N ? slot : 0;
        n_in_next = a.len[sq];
        d_next = a.dst[sq];
        e0_next = *reinterpret_cast<const __attribute__((address_space(1))) u32x2*>(entb + (uint32_t)sq * 8u);
        e1_next = *reinterpret_cast<const __attribute__((address_space(1))) u32x2*>(entb + ((uint32_t)sq * 8u + estride));
    };
    request_slot(0);
    {
        // (half by half: indexing the halves of a Feat inside the argument struct would put the struct into scratch memory)
        const float* __restrict__ gin = ((rb & 1) ? a.yin.half[1] : a.yin.half[0]) + (size_t)(rb >> 1) * blkf + rin;
        const int total = a.N * PARTS;
        for (int base = t; base < total; base += 4096) {
            float4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int idx = min(base + u * 1024, total - 1);   // (a lane past the end reads the last piece again and drops it)
                const int col = idx / PARTS, part = idx - col * PARTS;
                v[u] = *reinterpret_cast<const float4*>(gin + (size_t)col * RB + part * 4);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int idx = base + u * 1024;
                if (idx < total) *reinterpret_cast<float4*>(smem + (size_t)idx * 16) = v[u];
            }
        }
    }
    if (t == 0) sh_alive = 0;
    __syncthreads();
    float* __restrict__ gout = ((rb & 1) ? a.yout.half[1] : a.yout.half[0]) + (size_t)(rb >> 1) * blkf + rin;
    // this lane's order of the four-row parts of a column, as byte offsets
    uint32_t poff[PARTS];
#pragma unroll
    for (int i = 0; i < PARTS; ++i) poff[i] = (uint32_t)(((i + lane) & (PARTS - 1)) * 16);
    unsigned bits = 0;   // rows of this workgroup that one of this lane's outputs left nonzero
    for (int slot0 = 0; slot0 < a.N; slot0 += 1024) {
        const int slot = slot0 + t;
        const bool have = slot < a.N;
        const int n_in = have ? n_in_next : 0;
        const int d = have ? d_next : -1;
        const u32x2 e0_first = e0_next, e1_first = e1_next;
        if (slot0 + 1024 < a.N) request_slot(slot0 + 1024);
        // the slots are ordered by length, longest first: the wave's first lane has the most entries
        const int n_wave = __builtin_amdgcn_readfirstlane(n_in);
        float acc[R];
#pragma unroll
        for (int i = 0; i < R; ++i) acc[i] = 0.0f;
        if constexpr (!PAIRS) {
            // (one entry at a time where two workgroups fit a CU - 16 rows of up to 1280 neurons: with two entries the
            // sixteen more registers for the second column leave it one - N=1024, batch 60000: 170 against 156 us per layer)
            uint32_t eoff = (uint32_t)(have ? slot : 0) * 8u;
            u32x2 e = e0_first;
            for (int k = 0; k < n_wave; ++k) {
                const u32x2 cur = e;
                eoff += estride;
                // (lanes with fewer entries read the zero padding behind their lists: the array has kmax rows)
                if (k + 1 < n_wave) e = *reinterpret_cast<const __attribute__((address_space(1))) u32x2*>(entb + eoff);
                if (k < n_in) {
                    const float w = __uint_as_float(cur.y);
                    const uint32_t colb = cur.x * (uint32_t)(R * 4);
#pragma unroll
                    for (int i = 0; i < PARTS; ++i) {
                        const float4 x = *reinterpret_cast<const float4*>(smem + (colb + poff[i]));
                        acc[i * 4 + 0] = mac<WMODE>(acc[i * 4 + 0], x.x, w);
                        acc[i * 4 + 1] = mac<WMODE>(acc[i * 4 + 1], x.y, w);
                        acc[i * 4 + 2] = mac<WMODE>(acc[i * 4 + 2], x.z, w);
                        acc[i * 4 + 3] = mac<WMODE>(acc[i * 4 + 3], x.w, w);
                    }
                }
            }
        } else {
            // Two entries at a time, the next two requested under the arithmetic.  No test of k against the lane's own
            // length: behind a list the array holds (column 0, weight +0), and adding x * (+0) to an accumulator that
            // started at +0 changes nothing (it can never be -0).
            uint32_t eoff = (uint32_t)(have ? slot : 0) * 8u;
            u32x2 e0 = e0_first, e1 = e1_first;
            for (int k = 0; k < n_wave; k += 2) {
                const u32x2 c0 = e0, c1 = e1;
                eoff += 2u * estride;
                if (k + 2 < n_wave) {
                    e0 = *reinterpret_cast<const __attribute__((address_space(1))) u32x2*>(entb + eoff);
                    e1 = *reinterpret_cast<const __attribute__((address_space(1))) u32x2*>(entb + (eoff + estride));
                }
                const float w0 = __uint_as_float(c0.y), w1 = __uint_as_float(c1.y);
                const uint32_t colb0 = c0.x * (uint32_t)(R * 4), colb1 = c1.x * (uint32_t)(R * 4);
                float4 x0[PARTS], x1[PARTS];
#pragma unroll
                for (int i = 0; i < PARTS; ++i) x0[i] = *reinterpret_cast<const float4*>(smem + (colb0 + poff[i]));
#pragma unroll
                for (int i = 0; i < PARTS; ++i) x1[i] = *reinterpret_cast<const float4*>(smem + (colb1 + poff[i]));
#pragma unroll
                for (int i = 0; i < PARTS; ++i) {
                    acc[i * 4 + 0] = mac<WMODE>(acc[i * 4 + 0], x0[i].x, w0);
                    acc[i * 4 + 1] = mac<WMODE>(acc[i * 4 + 1], x0[i].y, w0);
                    acc[i * 4 + 2] = mac<WMODE>(acc[i * 4 + 2], x0[i].z, w0);
                    acc[i * 4 + 3] = mac<WMODE>(acc[i * 4 + 3], x0[i].w, w0);
                }
#pragma unroll
                for (int i = 0; i < PARTS; ++i) {
                    acc[i * 4 + 0] = mac<WMODE>(acc[i * 4 + 0], x1[i].x, w1);
                    acc[i * 4 + 1] = mac<WMODE>(acc[i * 4 + 1], x1[i].y, w1);
                    acc[i * 4 + 2] = mac<WMODE>(acc[i * 4 + 2], x1[i].z, w1);
                    acc[i * 4 + 3] = mac<WMODE>(acc[i * 4 + 3], x1[i].w, w1);
                }
            }
        }
        float4 y[PARTS];
#pragma unroll
        for (int i = 0; i < PARTS; ++i) {
            y[i].x = relu_clamp(acc[i * 4 + 0] + a.bias, a.clampv);
            y[i].y = relu_clamp(acc[i * 4 + 1] + a.bias, a.clampv);
            y[i].z = relu_clamp(acc[i * 4 + 2] + a.bias, a.clampv);
            y[i].w = relu_clamp(acc[i * 4 + 3] + a.bias, a.clampv);
            const unsigned nzb = (y[i].x > 0.0f ? 1u : 0u) | (y[i].y > 0.0f ? 2u : 0u) | (y[i].z > 0.0f ? 4u : 0u) | (y[i].w > 0.0f ? 8u : 0u);
            if (d >= 0) bits |= nzb << (poff[i] >> 2);
        }
        // Stores.  A lane has the R rows of ITS output: written as they are, every 16 bytes are a request of their own
        // to L2 (neighbouring lanes write columns a KiB apart), and the requests, not the bytes, bound the stores
        // (N=1024, batch 60000: 15.4 million write requests per layer, 55 us).  So the PARTS lanes of a group trade
        // parts first - lane j of the group ends up with part j of every output of the group - and each store
        // instruction writes, group by group, one output's R rows as one contiguous piece.
        // y[i] of lane s is part (i + s) mod PARTS of output s; turned by i lanes it arrives at lane j = (s + i) mod
        // PARTS as part j of output s = (j - i) mod PARTS.
        const int j = lane & (PARTS - 1);
        float4 z[PARTS];
#pragma unroll
        for (int r = 0; r < PARTS; ++r) z[r] = y[0];
#pragma unroll
        for (int i = 0; i < PARTS; ++i) {
            const float4 c = group_turn<PARTS>(y[i], i);
#pragma unroll
            for (int r = 0; r < PARTS; ++r)
                if (j == ((r + i) & (PARTS - 1))) z[r] = c;
        }
#pragma unroll
        for (int r = 0; r < PARTS; ++r) {
            const int dr = (int)group_lane_value<PARTS>((uint32_t)d, r);
            // (plain stores and loads: with the non-temporal hint on both the layer takes the same time)
            if (dr >= 0) *reinterpret_cast<float4*>(reinterpret_cast<unsigned char*>(gout + (size_t)dr * RB) + j * 16) = z[r];
        }
    }
    unsigned wave_bits = 0;
#pragma unroll
    for (int b = 0; b < R; ++b)
        if (__ballot((bits >> b) & 1u) != 0ull) wave_bits |= 1u << b;
    if (lane == 0 && wave_bits != 0) atomicOr(&sh_alive, (int)wave_bits);
    __syncthreads();
    if (t < R && ((sh_alive >> t) & 1)) a.active[row0 + t] = a.stamp;
}

// ------------------------------------------------------------------------------------------
// BLOCK kernel: groups of up to 16 outputs that read the same (up to 32) input columns - the
// structure of the challenge's RadiX-Net layers.  A wave loads the shared columns of a group once
// into registers (32 x RB*4 bytes) and every output of the group reuses them: no LDS, register
// operands only, one multiply-add per VALU instruction.  The accumulation order (ascending input
// index) is the same for every output of a group, so the code is fully unrolled.
// ------------------------------------------------------------------------------------------
// groups [g0, g1) of one row block for one wave; nz collects the rows' largest outputs
template <int RL, int WMODE, bool FULL>
__device__ __forceinline__ void block_body(const float* __restrict__ yin, float* __restrict__ yout,
                                           const int32_t* __restrict__ grp_cols, const int32_t* __restrict__ grp_cnt,
                                           const float* __restrict__ wv, const int32_t* __restrict__ dst, int g0, int g1,
                                           int loff, float wu, float bias, float clampv, float* nz) {
    using V = typename VecOf<RL>::type;
    constexpr int RB = 64 * RL;
    for (int g = g0; g < g1; ++g) {
        const int S = FULL ? 32 : grp_cnt[g];
        const int32_t* cp = grp_cols + (size_t)g * 32;
        float x[32][RL];
#pragma unroll
        for (int m = 0; m < 32; ++m) {
            if (FULL || m < S) {
                vec_to_arr<RL>(*reinterpret_cast<const V*>(yin + (size_t)cp[m] * RB + loff), x[m]);
            } else {
#pragma unroll
                for (int q = 0; q < RL; ++q) x[m][q] = 0.0f;
            }
        }
#pragma unroll 1
        for (int o = 0; o < 16; ++o) {
            const int d = dst[(size_t)g * 16 + o];
            if (d < 0) break;  // groups are filled from the front
            const float* wp = WMODE ? wv + ((size_t)g * 16 + o) * 32 : nullptr;
            float acc[RL];
#pragma unroll
            for (int q = 0; q < RL; ++q) acc[q] = 0.0f;
#pragma unroll
            for (int m = 0; m < 32; ++m) {
                if (FULL || m < S) {
                    const float w = WMODE ? wp[m] : wu;
#pragma unroll
                    for (int q = 0; q < RL; ++q) acc[q] = mac<WMODE>(acc[q], x[m][q], w);
                }
            }
            float y[RL];
#pragma unroll
            for (int q = 0; q < RL; ++q) {
                y[q] = relu_clamp(acc[q] + bias, clampv);
                nz[q] = nz_merge(nz[q], y[q]);
            }
            *reinterpret_cast<V*>(yout + (size_t)d * RB + loff) = arr_to_vec<RL>(y);
        }
    }
}

template <int RL, int WMODE, bool FULL>
__global__ __launch_bounds__(256) void block_kernel(
    Feat yin_all, Feat yout_all, const int32_t* __restrict__ grp_cols,
    const int32_t* __restrict__ grp_cnt, const float* __restrict__ wv, const int32_t* __restrict__ dst,
    int32_t* __restrict__ active, int32_t* __restrict__ count_prev, int N, int ngroups, int gpw, int stamp,
    int prev_stamp, int check_dead, float wu, float bias, float clampv, Publish pub,
    const int32_t* __restrict__ frontier, int frontier_layer) {
    constexpr int RB = 64 * RL;
    publish_counts(pub);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int rb = blockIdx.x;
    // finishing a persistent launch that gave up: this row block has the layer behind it already
    if (frontier != nullptr && frontier[rb] > frontier_layer) return;
    if (enter_row_block<RL>(active, (size_t)rb * RB + lane * RL, prev_stamp, stamp, check_dead, count_prev,
                            blockIdx.y == 0 && wave == 0))
        return;
    const float* __restrict__ yin = block_base(yin_all, rb, (size_t)N * RB);
    float* __restrict__ yout = block_base(yout_all, rb, (size_t)N * RB);
    const int loff = lane * RL;
    const int g0 = (blockIdx.y * 4 + wave) * gpw;
    const int g1 = min(ngroups, g0 + gpw);
    float nz[RL];
#pragma unroll
    for (int q = 0; q < RL; ++q) nz[q] = 0.0f;
    block_body<RL, WMODE, FULL>(yin, yout, grp_cols, grp_cnt, wv, dst, g0, g1, loff, wu, bias, clampv, nz);
    stamp_rows<RL>(nz, active, (size_t)rb * RB + loff, stamp);
}

// ------------------------------------------------------------------------------------------
// Persistent launches: several layers of one kind per launch, a dependency per row block between
// the layers (see PersistLaunch).  The reference's loop synchronises the whole device and the
// host once per layer (src/microbenchmark/all_network.cu:333-519, the wait at :453).
// ------------------------------------------------------------------------------------------
struct PersistArgs {
    const LayerDesc* table;
    int nlayers;
    Feat first_in, buf_a, buf_c;
    int32_t* active;
    int32_t* done;
    int done_stride;
    PersistCtl* ctl;
    const PersistCtl* prev_ctl;
    int prev_units;
    int32_t* abort;
    int32_t* host_word;
    int N, nblk, nseg, seglen, total_units, nq, light;
    int stamp0, prev_stamp, check_dead;
    long long wait_limit;
    float bias, clampv;
    int stream;
    Publish pub;
};

// number of the XCD (accelerator die) this wave runs on, from the hardware
__device__ __forceinline__ int xcc_id() {
    uint32_t x;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(x));
    return (int)(x & 7u);
}
__device__ __forceinline__ int load_agent(const int32_t* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// the launch gives up: every workgroup leaves at its next look at `abort`
__device__ __forceinline__ void persist_give_up(const PersistArgs& a) {
    __hip_atomic_store(a.abort, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Start of a persistent kernel: a launch does not start on the ruins of another (uniform result).
__device__ __forceinline__ bool persist_may_start(const PersistArgs& a) {
    int bad = 0;
    if (threadIdx.x == 0) {
        if (load_agent(a.abort) != 0) bad = 1;
        else if (a.prev_ctl != nullptr && load_agent(&a.prev_ctl->units_done) != a.prev_units) {
            persist_give_up(a);
            bad = 1;
        }
    }
    return __builtin_amdgcn_readfirstlane(__syncthreads_or(bad)) == 0;
}

// One thread waits until *cnt >= target; 0 = there, 1 = the launch has given up (here, after wait_limit
// ticks of the 100 MHz clock, or elsewhere).
__device__ __forceinline__ int persist_wait(const PersistArgs& a, const int32_t* cnt, int target) {
    long long t0 = -1;
    for (;;) {
        if (load_agent(cnt) >= target) break;
        if (load_agent(a.abort) != 0) return 1;
        const long long now = (long long)wall_clock64();
        if (t0 < 0) t0 = now;
        if (now - t0 >= a.wait_limit) {
            persist_give_up(a);
            return 1;
        }
        __builtin_amdgcn_s_sleep(1);
    }
    return 0;
}

// After the wait (every wave, behind the barrier that follows it): the writers ran on other CUs, so what this CU's
// L1 holds of the buffer is stale - it may have read the same lines two layers earlier.  Every wave invalidates for
// itself, in front of its own loads: an invalidate issued by one wave orders that wave's loads only.  At device
// scope (buffer_inv sc1), also where writer and reader share an XCD and its L2: the workgroup-scope form (buffer_inv
// sc0) leaves the L1 as it is outside threadgroup-split mode - seen as wrong results (different from run to run) on
// a network of 256 neurons in 64-row blocks, three layers per launch, whose buffers stay in L1 from layer to layer;
// wider layers push their lines out of the 32 KiB by themselves and never showed it.  The invalidate costs the
// launches that are persistent by default nothing measurable (N=1024, batch 60000: 99.5 against 99.8 us per layer).
__device__ __forceinline__ void persist_acquire(const PersistArgs&) {
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}

// Entry j of the layer table through the constant address space: the table never changes while a kernel
// runs, and read this way its words come by the scalar unit and stay in scalar registers - the band walk
// hands them to the scalar unit as they are (pair records, selectors).
__device__ __forceinline__ LayerDesc load_layer_desc(const LayerDesc* table, int j) {
    constexpr int W = (int)(sizeof(LayerDesc) / 4);
    static_assert(sizeof(LayerDesc) % 4 == 0, "layer table entries are whole dwords");
    const __attribute__((address_space(4))) uint32_t* p = (const __attribute__((address_space(4))) uint32_t*)(table + j);
    union { LayerDesc d; uint32_t w[W]; } u;
#pragma unroll
    for (int i = 0; i < W; ++i) u.w[i] = p[i];
    return u.d;
}

// The unit loop.  body(rb, sg, lay, in, out, stamp, prev_stamp) runs one unit; the whole workgroup enters
// it with the same arguments.
//
// One thread (thread 0) does everything between two units in ONE place, right before the barrier at the top of
// the loop: it counts the unit that has just finished, claims the next one and waits for that unit's row block.  (With a single-thread region at the bottom of the loop and another at its top - two regions of
// the same thread on either side of the back edge - the compiler let the other lanes of that wave run ahead into
// the next iteration's barrier.)  The wait for the wave's LDS traffic in front of that barrier is written out
// (ring_barrier): the barrier alone does not order thread 0's LDS writes before the other waves' reads, and the
// compiler leaves the wait of __syncthreads() out there (seen in the generated code, and in rare units whose
// waves disagreed on the unit).
template <int RL, class Body>
__device__ __forceinline__ void persist_loop(const PersistArgs& a, Body body) {
    __shared__ int sh_unit, sh_gone;
    constexpr int RB = 64 * RL;
    publish_counts(a.pub);
    const int q = a.nq > 1 ? xcc_id() : 0;
    const int nrb_q = a.nq > 1 ? (q < a.nblk ? (a.nblk - q + 7) / 8 : 0) : a.nblk;
    const int per_layer = nrb_q * a.nseg;
    const int total_q = per_layer * a.nlayers;
    const size_t blkf = (size_t)a.N * RB;
    // (pointer by pointer: a choice between whole structs would keep the kernel's arguments in scratch memory)
    const bool in_a = a.first_in.half[0] == a.buf_a.half[0];   // the launch's first layer reads buffer A, so it writes C
    float* const out0_h0 = in_a ? a.buf_c.half[0] : a.buf_a.half[0];
    float* const out0_h1 = in_a ? a.buf_c.half[1] : a.buf_a.half[1];
    float* const out1_h0 = in_a ? a.buf_a.half[0] : a.buf_c.half[0];
    float* const out1_h1 = in_a ? a.buf_a.half[1] : a.buf_c.half[1];
    // where unit u's row block counts its finished units, and what unit u waits for (thread 0)
    auto counter_of = [&](int u) -> int32_t* {
        const int j = u / per_layer, rem = u - j * per_layer, ri = rem / a.nseg;
        return a.done + (size_t)j * a.done_stride + (a.nq > 1 ? q + 8 * ri : ri);
    };
    auto wait_for = [&](int u) -> int {
        if (u >= total_q || u < per_layer) return 0;   // no such unit, or a unit of the launch's first layer
        return persist_wait(a, counter_of(u) - a.done_stride, a.nseg);
    };
    if (persist_may_start(a)) {
        if (threadIdx.x == 0) {
            const int first = __hip_atomic_fetch_add(&a.ctl->head[q], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            sh_unit = first;
            sh_gone = wait_for(first);
        }
        for (;;) {
            ring_barrier<1>();
            const int u = __builtin_amdgcn_readfirstlane(sh_unit);
            if (u >= total_q || __builtin_amdgcn_readfirstlane(sh_gone) != 0) break;
            const int j = u / per_layer, rem = u - j * per_layer, ri = rem / a.nseg, sg = rem - ri * a.nseg;
            const int rb = a.nq > 1 ? q + 8 * ri : ri;
            if (j > 0) persist_acquire(a);
            const LayerDesc lay = load_layer_desc(a.table, j);
            const int stamp = a.stamp0 + j;
            const int prev_stamp = j > 0 ? stamp - 1 : a.prev_stamp;
            const float* const in_h0 = j == 0 ? a.first_in.half[0] : ((j & 1) ? out0_h0 : out1_h0);
            const float* const in_h1 = j == 0 ? a.first_in.half[1] : ((j & 1) ? out0_h1 : out1_h1);
            float* const out_h0 = (j & 1) ? out1_h0 : out0_h0;
            float* const out_h1 = (j & 1) ? out1_h1 : out0_h1;
            const size_t boff = (size_t)(rb >> 1) * blkf;   // row block rb is block rb >> 1 of half rb & 1
            body(rb, sg, lay, ((rb & 1) ? in_h1 : in_h0) + boff, ((rb & 1) ? out_h1 : out_h0) + boff, stamp, prev_stamp);
            wait_vector_memory();   // this wave's stores have arrived in L2
            ring_barrier<1>();      // ... every wave's have, and every thread has read sh_unit / sh_gone
            if (threadIdx.x == 0) {
                if (!(a.light & 2)) {
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");   // the XCD's L2 writes back what it holds ...
                    wait_vector_memory();   // ... and has done so before the count goes up (said explicitly: with no load or
                                            // store of its own outstanding the compiler leaves the fence's wait out)
                }
                __hip_atomic_fetch_add(counter_of(u), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_fetch_add(&a.ctl->units_done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                // (claimed here, not a unit ahead under the arithmetic: a unit held by a busy workgroup while others
                // idle costs more than the atomic's round trip - 21.8 against 18.2 us per layer at N=1024, batch 6000)
                const int next = __hip_atomic_fetch_add(&a.ctl->head[q], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                sh_unit = next;
                sh_gone = wait_for(next);
            }
        }
    }
    // The last workgroup to leave tells the host: the unit total if every unit was run, -2 if the launch gave up.
    if (threadIdx.x == 0) {
        wait_vector_memory();   // this thread's counts have been made
        const int left = __hip_atomic_fetch_add(&a.ctl->exited, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (left == (int)gridDim.x - 1) {
            const int done = load_agent(&a.ctl->units_done);
            __hip_atomic_store(a.host_word, (done == a.total_units && load_agent(a.abort) == 0) ? done : -2, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_SYSTEM);
        }
    }
}

template <int RL, int WMODE, int KT, int DMA>
__global__ __launch_bounds__(512) void band_persist_kernel(PersistArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int RB = 64 * RL;
    persist_loop<RL>(a, [&](int rb, int sg, const LayerDesc& lay, const float* yin, float* yout, int stamp, int prev_stamp) __attribute__((always_inline)) {
        if (enter_row_block<RL>(a.active, (size_t)rb * RB + (threadIdx.x & 63) * RL, prev_stamp, stamp, a.check_dead,
                                nullptr, false))
            return;
        const int vb = sg * a.seglen, ve = min(a.N, vb + a.seglen);
        float nz[RL];
#pragma unroll
        for (int x = 0; x < RL; ++x) nz[x] = 0.0f;
        band_walk_body<RL, 8, 2, 64, WMODE, KT, DMA>(yin, yout, lay.pairs, lay.pw, lay.dst, a.N, lay.steps, lay.halo, vb, ve,
                                                     lay.wu, a.bias, a.clampv, smem, nz, a.stream);
        // (one store per row through LDS: with every wave stamping its rows itself - 8 times the stores on the
        // row block's 1 KiB of stamps from every unit of the block - a small layer took 0.5 - 1.5 us longer)
        stamp_rows_workgroup<RL, 8>(nz, smem, a.active, (size_t)rb * RB, stamp, nullptr);
    });
}

// unit = 4 waves x seglen groups of one row block
template <int RL, int WMODE, bool FULL>
__global__ __launch_bounds__(256) void block_persist_kernel(PersistArgs a) {
    constexpr int RB = 64 * RL;
    persist_loop<RL>(a, [&](int rb, int sg, const LayerDesc& lay, const float* yin, float* yout, int stamp, int prev_stamp) __attribute__((always_inline)) {
        const int lane = threadIdx.x & 63;
        const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
        if (enter_row_block<RL>(a.active, (size_t)rb * RB + lane * RL, prev_stamp, stamp, a.check_dead, nullptr, false))
            return;
        const int g0 = (sg * 4 + wave) * a.seglen, g1 = min(lay.ngroups, g0 + a.seglen);
        float nz[RL];
#pragma unroll
        for (int x = 0; x < RL; ++x) nz[x] = 0.0f;
        block_body<RL, WMODE, FULL>(yin, yout, lay.blk_cols, lay.blk_cnt, lay.blk_wv, lay.blk_dst, g0, g1, lane * RL, lay.wu,
                                    a.bias, a.clampv, nz);
        stamp_rows<RL>(nz, a.active, (size_t)rb * RB + lane * RL, stamp);
    });
}

// ------------------------------------------------------------------------------------------
// Resident launch: rows never interact, so a workgroup can keep a handful of feature rows in LDS and
// take them through many layers with no other workgroup to wait for - the only traffic to memory is
// the rows coming in, the rows going out and the layers' index lists (from L2).  What makes it pay
// is the BLOCK structure (RadiX-Net layers): the 16 outputs of a group read the same 32 columns and,
// under the layer's one exact weight, are equal, so a (group, row) item costs 32 LDS reads and 16
// LDS writes; a layer without that structure would need 32 reads per output, and LDS would then be no
// faster than the per-layer kernels' memory.  (The reference fuses two layers this way for one tile,
// src/microbenchmark/fuse.cu:16-110; its loop over the other layers goes through memory and the
// host, all_network.cu:333-519.)
//
// A workgroup of 1024 threads owns R consecutive rows of one row block (R = 16 for up to 1024 neurons,
// 4 for up to 4096: two buffers of N x R floats in LDS, laid out [column][row]) and
// thread t the item (group t / R, row t % R).  The R lanes of a group hold the group's 32 column
// offsets and 16 output columns between them (32/R and 16/R registers each, read from memory in one
// coalesced piece, a layer ahead) and hand them round by DPP (16-lane row broadcast for R = 16, quad
// broadcast for R = 4).  Accumulation as in block_body: ascending input index, multiply-add by the one exact
// weight, bias last.  One barrier per layer.  Rows are stamped with the last layer that left them
// nonzero (the per-layer counts are taken from the stamps behind the launch); once all R rows are
// zero and the bias is not positive the workgroup stops and stores zeros.
// ------------------------------------------------------------------------------------------
struct ResidentArgs {
    const LayerDesc* table;
    int nlayers;
    Feat first_in, buf_a, buf_c;
    int32_t* active;
    int N, ngroups, rl;
    int stamp0, prev_stamp, check_dead;
    float bias, clampv;
    Publish pub;
    // QUAD form: the arrays of the launch's first layer; those of layer j lie j * quad_stride bytes further on
    const uint32_t* quad_col;
    const float* quad_w;
    const int32_t* quad_dst;
    long long quad_stride;
};

// the value register k / R of the lane with row index k % R of this lane's group holds (k a constant after unrolling)
template <int R, int NREG> __device__ __forceinline__ uint32_t group_lane(const uint32_t (&v)[NREG], int k) {
    if constexpr (R == 16) {
        return row_lane(v[k >> 4], k & 15);
    } else if constexpr (R == 4) {
        const int x = (int)v[k >> 2];
        switch (k & 3) {
            case 0: return (uint32_t)__builtin_amdgcn_update_dpp(0, x, 0x00, 0xf, 0xf, true);
            case 1: return (uint32_t)__builtin_amdgcn_update_dpp(0, x, 0x55, 0xf, 0xf, true);
            case 2: return (uint32_t)__builtin_amdgcn_update_dpp(0, x, 0xaa, 0xf, 0xf, true);
            default: return (uint32_t)__builtin_amdgcn_update_dpp(0, x, 0xff, 0xf, 0xf, true);
        }
    } else {
        static_assert(R == 16 || R == 4, "rows per workgroup: 16 or 4");
        return 0;
    }
}

template <int R, bool FULL>
__global__ __launch_bounds__(1024) void block_resident_kernel(ResidentArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int sh_alive[3];
    constexpr int LOG_R = R == 16 ? 4 : 2;
    constexpr int NC = 32 / R, ND = 16 / R;    // index registers per lane
    constexpr int VW = 4;                      // floats per memory access of a column's rows
    constexpr int PARTS = R / VW;
    using V = typename VecOf<VW>::type;
    publish_counts(a.pub);
    const int t = (int)threadIdx.x, lane = t & 63, nthr = (int)blockDim.x;   // (ngroups * R threads, rounded up to whole waves)
    const int RB = 64 * a.rl;
    // Workgroups go to the 8 XCDs round robin by number; a 64-byte piece of a column holds the rows of 16 / R
    // workgroups, which should find it in ONE L2: every XCD takes a contiguous eighth of the rows.
    const unsigned nwg = gridDim.x;
    const unsigned wg = (nwg % 8u) == 0u ? (blockIdx.x % 8u) * (nwg / 8u) + blockIdx.x / 8u : blockIdx.x;
    const size_t row0 = (size_t)wg * R;
    const int rb = (int)(row0 / (size_t)RB), rin = (int)(row0 - (size_t)rb * RB);
    if (a.check_dead && a.prev_stamp != 0) {   // a row block without an active row is skipped, as by the per-layer kernels
        int alive = 0;
        for (int i = t; i < RB; i += nthr) alive |= (a.active[(size_t)rb * RB + i] == a.prev_stamp) ? 1 : 0;
        if (__syncthreads_or(alive) == 0) return;
    }
    const size_t blkf = (size_t)a.N * RB;
    // two buffers of N + 1 columns x R rows; column N takes the stores of lanes without an output
    const uint32_t buf_bytes = (uint32_t)(a.N + 1) * R * 4;
    unsigned char* const buf0 = smem;
    unsigned char* const buf1 = smem + buf_bytes;
    {
        // (four loads in flight per thread: a workgroup has nothing else to do while its rows come in)
        const float* __restrict__ gin = block_base(a.first_in, rb, blkf) + rin;
        const int total = a.N * PARTS;
        for (int base = t; base < total; base += 4 * nthr) {
            V v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int idx = min(base + u * nthr, total - 1);   // (a lane past the end reads the last piece again and drops it)
                const int col = idx / PARTS, part = idx - col * PARTS;
                v[u] = *reinterpret_cast<const V*>(gin + (size_t)col * RB + part * VW);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int idx = base + u * nthr;
                const int col = idx / PARTS, part = idx - col * PARTS;
                if (idx < total) *reinterpret_cast<V*>(buf0 + ((size_t)col * R + part * VW) * 4) = v[u];
            }
        }
    }
    if (t < 3) sh_alive[t] = 0;
    const int g = t >> LOG_R, r = t & (R - 1);
    const bool item = g < a.ngroups;
    const int gq = item ? g : 0;               // (lanes without an item go through the motions of group 0 and store to column N)
    // the group's input columns and its outputs' columns, spread over the group's lanes: requested a layer ahead and
    // kept as they come (arithmetic on a requested value would make the wave wait for the load then and there - all 16
    // waves at once, at the top of every layer); turned into byte offsets inside a buffer when their layer begins
    int32_t c_next[NC], d_next[ND];
    int cnt_next = 32;
    auto request_indices = [&](int j) {
        const LayerDesc lay = load_layer_desc(a.table, j);
        // (the pointers come out of the table: said to be global memory, or the loads become flat ones)
        using GI = const __attribute__((address_space(1))) int32_t*;
        const GI cols = (GI)lay.blk_cols, dsts = (GI)lay.blk_dst, cnts = (GI)lay.blk_cnt;
#pragma unroll
        for (int i = 0; i < NC; ++i) c_next[i] = cols[(size_t)gq * 32 + i * R + r];
#pragma unroll
        for (int i = 0; i < ND; ++i) d_next[i] = dsts[(size_t)gq * 16 + i * R + r];
        if (!FULL) cnt_next = cnts[gq];
    };
    request_indices(0);
    int last_alive = -1;
    bool all_dead = false;
    int done_layers = 0;
    ring_barrier<1>();
    for (int j = 0; j < a.nlayers; ++j) {
        const unsigned char* const in = ((j & 1) ? buf1 : buf0) + r * 4;
        unsigned char* const out = ((j & 1) ? buf0 : buf1) + r * 4;
        const float wu = load_layer_desc(a.table, j).wu;
        uint32_t cb[NC], db[ND];
#pragma unroll
        for (int i = 0; i < NC; ++i) cb[i] = (uint32_t)c_next[i] * (uint32_t)(R * 4);
#pragma unroll
        for (int i = 0; i < ND; ++i) db[i] = (uint32_t)((item && d_next[i] >= 0) ? d_next[i] : a.N) * (uint32_t)(R * 4);
        const int cnt = cnt_next;
        if (j + 1 < a.nlayers) request_indices(j + 1);   // in flight under this layer's arithmetic
        float x[32];
#pragma unroll
        for (int k = 0; k < 32; ++k) x[k] = *reinterpret_cast<const float*>(in + group_lane<R, NC>(cb, k));
        float acc = 0.0f;
#pragma unroll
        for (int k = 0; k < 32; ++k)
            if (FULL || k < cnt) acc = mac<0>(acc, x[k], wu);
        const float y = relu_clamp(acc + a.bias, a.clampv);
#pragma unroll
        for (int o = 0; o < 16; ++o) *reinterpret_cast<float*>(out + group_lane<R, ND>(db, o)) = y;
        unsigned long long m = __ballot((item && y > 0.0f) ? 1 : 0);
#pragma unroll
        for (int sft = R; sft < 64; sft <<= 1) m |= m >> sft;
        const int bits = (int)(m & ((1ull << R) - 1ull));
        if (lane == 0 && bits != 0) atomicOr(&sh_alive[j % 3], bits);
        ring_barrier<1>();
        const int mask = sh_alive[j % 3];
        if (t == 0) sh_alive[(j + 2) % 3] = 0;
        if (t < R && ((mask >> t) & 1)) last_alive = j;
        done_layers = j + 1;
        if (mask == 0 && a.bias <= 0.0f) { all_dead = true; break; }   // zero rows stay zero
    }
    // the launch's last layer writes the work buffer the layer before it did not (layer 0: the one it did not read)
    const bool in_a = a.first_in.half[0] == a.buf_a.half[0];
    const bool to_c = in_a == ((a.nlayers & 1) != 0);
    float* const o_h0 = to_c ? a.buf_c.half[0] : a.buf_a.half[0];
    float* const o_h1 = to_c ? a.buf_c.half[1] : a.buf_a.half[1];
    float* __restrict__ gout = ((rb & 1) ? o_h1 : o_h0) + (size_t)(rb >> 1) * blkf + rin;
    const unsigned char* const fin = (done_layers & 1) ? buf1 : buf0;
    for (int idx = t; idx < a.N * PARTS; idx += nthr) {
        const int col = idx / PARTS, part = idx - col * PARTS;
        V v;
        if (all_dead) v = V{};
        else v = *reinterpret_cast<const V*>(fin + ((size_t)col * R + part * VW) * 4);
        *reinterpret_cast<V*>(gout + (size_t)col * RB + part * VW) = v;
    }
    if (t < R && last_alive >= 0) a.active[row0 + t] = a.stamp0 + last_alive;
}

// The resident launch of TILED layers: block_resident_kernel's frame (R rows of a workgroup in LDS through all layers
// of the launch, two buffers, one barrier per layer, rows stamped with the last layer that left them nonzero, a
// workgroup whose rows are all zero stops) around rowtile_kernel's arithmetic (thread t computes whole outputs - slots
// t, t + 1024, ... - from its own entry list, 16-byte LDS reads of a column's rows in a lane-rotated order).  The
// outputs go to the other LDS buffer as they are (a lane writes its parts where they belong), so of a layer's time
// in rowtile_kernel - the launch, the rows in, the rows out - only the arithmetic is left.
template <int R, int WMODE>
__global__ __launch_bounds__(1024) void rowtile_resident_kernel(ResidentArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int sh_alive[3];
    constexpr int PARTS = R / 4;
    typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
    using GB = const __attribute__((address_space(1))) unsigned char*;
    using GI = const __attribute__((address_space(1))) int32_t*;
    publish_counts(a.pub);
    const int t = (int)threadIdx.x, lane = t & 63;
    const int RB = 64 * a.rl;
    const unsigned nwg = gridDim.x;
    const unsigned wg = (nwg % 8u) == 0u ? (blockIdx.x % 8u) * (nwg / 8u) + blockIdx.x / 8u : blockIdx.x;
    const size_t row0 = (size_t)wg * R;
    const int rb = (int)(row0 / (size_t)RB), rin = (int)(row0 - (size_t)rb * RB);
    if (a.check_dead && a.prev_stamp != 0) {   // a row block without an active row is skipped, as by the per-layer kernels
        int alive = 0;
        for (int i = t; i < RB; i += 1024) alive |= (a.active[(size_t)rb * RB + i] == a.prev_stamp) ? 1 : 0;
        if (__syncthreads_or(alive) == 0) return;
    }
    const size_t blkf = (size_t)a.N * RB;
    const uint32_t buf_bytes = (uint32_t)a.N * R * 4;
    const int total = a.N * PARTS;
    {
        const float* __restrict__ gin = ((rb & 1) ? a.first_in.half[1] : a.first_in.half[0]) + (size_t)(rb >> 1) * blkf + rin;
        for (int base = t; base < total; base += 4096) {
            float4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int idx = min(base + u * 1024, total - 1);   // (a lane past the end reads the last piece again and drops it)
                const int col = idx / PARTS, part = idx - col * PARTS;
                v[u] = *reinterpret_cast<const float4*>(gin + (size_t)col * RB + part * 4);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int idx = base + u * 1024;
                if (idx < total) *reinterpret_cast<float4*>(smem + (size_t)idx * 16) = v[u];
            }
        }
    }
    if (t < 3) sh_alive[t] = 0;
    uint32_t poff[PARTS];   // this lane's order of the four-row parts of a column, as byte offsets
#pragma unroll
    for (int i = 0; i < PARTS; ++i) poff[i] = (uint32_t)(((i + lane) & (PARTS - 1)) * 16);
    const uint32_t estride = (uint32_t)a.N * 8u;
    // A slot's length, output column and first two entries are requested one slot ahead - for a layer's first slot:
    // a layer ahead - and kept as they come: a request made where its value is needed is a round trip to L2 that all 16
    // waves of the workgroup make at once, right behind the barrier (three of them in a row, a third of a layer).
    // (Entries 0 and 1 exist for every slot: the lists are padded to four entries and more.)
    int n_in_next, d_next;
    u32x2 e0_next, e1_next;
    auto request_slot = [&](const LayerDesc& lay, int slot0) {
        const int slot = slot0 + t;
        const bool have = slot < a.N;
        const GB entb = (GB)lay.rt_ent;
        const uint32_t eoff = (uint32_t)(have ? slot : 0) * 8u;
        n_in_next = ((GI)lay.rt_len)[have ? slot : 0];
        d_next = ((GI)lay.rt_dst)[have ? slot : 0];
        e0_next = *reinterpret_cast<const __attribute__((address_space(1))) u32x2*>(entb + eoff);
        e1_next = *reinterpret_cast<const __attribute__((address_space(1))) u32x2*>(entb + (eoff + estride));
    };
    LayerDesc lay_next = load_layer_desc(a.table, 0);
    request_slot(lay_next, 0);
    int last_alive = -1;
    bool all_dead = false;
    int done_layers = 0;
    __syncthreads();
    for (int j = 0; j < a.nlayers; ++j) {
        const unsigned char* const in = smem + ((j & 1) ? buf_bytes : 0u);
        unsigned char* const out = smem + ((j & 1) ? 0u : buf_bytes);
        const LayerDesc lay = lay_next;
        if (j + 1 < a.nlayers) lay_next = load_layer_desc(a.table, j + 1);
        const GB entb = (GB)lay.rt_ent;
        unsigned bits = 0;   // rows that one of this lane's outputs left nonzero
        for (int slot0 = 0; slot0 < a.N; slot0 += 1024) {
            const int slot = slot0 + t;
            const bool have = slot < a.N;
            const int n_in = have ? n_in_next : 0;
            const int d = have ? d_next : -1;
            u32x2 e0 = e0_next, e1 = e1_next;
            if (slot0 + 1024 < a.N) request_slot(lay, slot0 + 1024);
            else if (j + 1 < a.nlayers) request_slot(lay_next, 0);
            const int n_wave = __builtin_amdgcn_readfirstlane(n_in);   // slots are ordered by length: the wave's first lane has the most
            float acc[R];
#pragma unroll
            for (int i = 0; i < R; ++i) acc[i] = 0.0f;
            // Two entries at a time, the next two requested under the arithmetic: one workgroup per CU leaves a SIMD
            // four waves, so a wave has to keep eight LDS reads of its own in flight.  No test of k against the lane's
            // own length: behind a list the array holds (column 0, weight +0), and adding x * (+0) to an accumulator
            // that started at +0 changes nothing (it can never be -0).
            uint32_t eoff = (uint32_t)(have ? slot : 0) * 8u;
            for (int k = 0; k < n_wave; k += 2) {
                const u32x2 c0 = e0, c1 = e1;
                eoff += 2u * estride;
                if (k + 2 < n_wave) {
                    e0 = *reinterpret_cast<const __attribute__((address_space(1))) u32x2*>(entb + eoff);
                    e1 = *reinterpret_cast<const __attribute__((address_space(1))) u32x2*>(entb + (eoff + estride));
                }
                const float w0 = __uint_as_float(c0.y), w1 = __uint_as_float(c1.y);
                const uint32_t colb0 = c0.x * (uint32_t)(R * 4), colb1 = c1.x * (uint32_t)(R * 4);
                float4 x0[PARTS], x1[PARTS];
#pragma unroll
                for (int i = 0; i < PARTS; ++i) x0[i] = *reinterpret_cast<const float4*>(in + (colb0 + poff[i]));
#pragma unroll
                for (int i = 0; i < PARTS; ++i) x1[i] = *reinterpret_cast<const float4*>(in + (colb1 + poff[i]));
#pragma unroll
                for (int i = 0; i < PARTS; ++i) {
                    acc[i * 4 + 0] = mac<WMODE>(acc[i * 4 + 0], x0[i].x, w0);
                    acc[i * 4 + 1] = mac<WMODE>(acc[i * 4 + 1], x0[i].y, w0);
                    acc[i * 4 + 2] = mac<WMODE>(acc[i * 4 + 2], x0[i].z, w0);
                    acc[i * 4 + 3] = mac<WMODE>(acc[i * 4 + 3], x0[i].w, w0);
                }
#pragma unroll
                for (int i = 0; i < PARTS; ++i) {
                    acc[i * 4 + 0] = mac<WMODE>(acc[i * 4 + 0], x1[i].x, w1);
                    acc[i * 4 + 1] = mac<WMODE>(acc[i * 4 + 1], x1[i].y, w1);
                    acc[i * 4 + 2] = mac<WMODE>(acc[i * 4 + 2], x1[i].z, w1);
                    acc[i * 4 + 3] = mac<WMODE>(acc[i * 4 + 3], x1[i].w, w1);
                }
            }
#pragma unroll
            for (int i = 0; i < PARTS; ++i) {
                float4 y;
                y.x = relu_clamp(acc[i * 4 + 0] + a.bias, a.clampv);
                y.y = relu_clamp(acc[i * 4 + 1] + a.bias, a.clampv);
                y.z = relu_clamp(acc[i * 4 + 2] + a.bias, a.clampv);
                y.w = relu_clamp(acc[i * 4 + 3] + a.bias, a.clampv);
                const unsigned nzb = (y.x > 0.0f ? 1u : 0u) | (y.y > 0.0f ? 2u : 0u) | (y.z > 0.0f ? 4u : 0u) | (y.w > 0.0f ? 8u : 0u);
                if (d >= 0) {
                    bits |= nzb << (poff[i] >> 2);
                    *reinterpret_cast<float4*>(out + ((uint32_t)d * (uint32_t)(R * 4) + poff[i])) = y;
                }
            }
        }
        unsigned wave_bits = 0;
#pragma unroll
        for (int b = 0; b < R; ++b)
            if (__ballot((bits >> b) & 1u) != 0ull) wave_bits |= 1u << b;
        if (lane == 0 && wave_bits != 0) atomicOr(&sh_alive[j % 3], (int)wave_bits);
        __syncthreads();
        const int mask = sh_alive[j % 3];
        if (t == 0) sh_alive[(j + 2) % 3] = 0;
        if (t < R && ((mask >> t) & 1)) last_alive = j;
        done_layers = j + 1;
        if (mask == 0 && a.bias <= 0.0f) { all_dead = true; break; }   // zero rows stay zero
    }
    // the launch's last layer writes the work buffer the layer before it did not (layer 0: the one it did not read)
    const bool in_a = a.first_in.half[0] == a.buf_a.half[0];
    const bool to_c = in_a == ((a.nlayers & 1) != 0);
    float* const o_h0 = to_c ? a.buf_c.half[0] : a.buf_a.half[0];
    float* const o_h1 = to_c ? a.buf_c.half[1] : a.buf_a.half[1];
    float* __restrict__ gout = ((rb & 1) ? o_h1 : o_h0) + (size_t)(rb >> 1) * blkf + rin;
    const unsigned char* const fin = smem + ((done_layers & 1) ? buf_bytes : 0u);
    for (int idx = t; idx < total; idx += 1024) {
        const int col = idx / PARTS, part = idx - col * PARTS;
        float4 v;
        if (all_dead) v = float4{0.0f, 0.0f, 0.0f, 0.0f};
        else v = *reinterpret_cast<const float4*>(fin + (size_t)idx * 16);
        *reinterpret_cast<float4*>(gout + (size_t)col * RB + part * 4) = v;
    }
    if (t < R && last_alive >= 0) a.active[row0 + t] = a.stamp0 + last_alive;
}

// The resident launch of BAND layers in their QUAD form (up to 1024 neurons, any weights): the frame of the two kernels
// above - 16 rows of a workgroup in LDS through all layers of the launch, two buffers laid out [column][row], one barrier per
// layer, rows stamped with the last layer that left them nonzero, a workgroup whose rows are all zero stops - around an
// arithmetic that shares LDS reads between neighbouring outputs of the band.  The workgroup has N threads; thread t
// belongs to quad t / 4 (band positions 4c .. 4c+3) and computes those four outputs for rows 4 (t % 4) .. + 3.  The four
// outputs add their inputs in ascending input index, so their lists are one merged list of steps (K + 3 for a
// circulant band of K entries): per step ONE 16-byte LDS read - the column's four rows - feeds 16 multiply-adds, a
// step an output does not use entering it with weight 0 (an exact zero added).  The plan stream of a quad - per group
// of four steps the four columns (as byte offsets) and 4 x 4 weights - is spread over the quad's four lanes: lane k holds
// the column of step k and the four outputs' weights of step k.  The columns are handed round by DPP quad permutations
// inside the address adds.  The weights go through LDS: each wave owns a KiB behind the two row buffers, 64 bytes per
// quad; lane k writes its 16 bytes there behind the last read of the group before (the LDS operations of one wave run
// in order, so no barrier is needed) and every lane of the quad reads a step's 16 bytes back, one step ahead of its
// use - a broadcast - so that the 16 multiply-adds of a step have all three operands in the lane's own registers.
// (Handing the weights round by DPP instead costs 4 moves per step in front of dependent multiply-adds, a tenth of the
// layer's time more.)  The groups are requested two ahead of the arithmetic, the first two of the next layer before
// this layer's barrier.
template <int K> __device__ __forceinline__ uint32_t quad_lane(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, K * 0x55, 0xf, 0xf, true);
}
// One step of a quad: acc[o][q] += x[q] * w[o], o, q = 0..3, all operands registers of the lane itself (a v_fmac_f32 on
// three vector registers issues in 0.95 - 1.1 ns per wave and SIMD, one with a DPP or scalar operand in 1.75 ns).  Ends
// with a barrier to the compiler's reordering of memory accesses: the LDS reads of later steps are issued before the
// step's arithmetic and stay there.
template <int WMODE> __device__ __forceinline__ void quad_step(float (&acc)[4][4], const float4& x, const float4& w) {
    const float wo[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int o = 0; o < 4; ++o) {
        acc[o][0] = mac<WMODE>(acc[o][0], x.x, wo[o]);
        acc[o][1] = mac<WMODE>(acc[o][1], x.y, wo[o]);
        acc[o][2] = mac<WMODE>(acc[o][2], x.z, wo[o]);
        acc[o][3] = mac<WMODE>(acc[o][3], x.w, wo[o]);
    }
#pragma unroll
    for (int o = 0; o < 4; ++o)
#pragma unroll
        for (int q = 0; q < 4; ++q) asm volatile("" : "+v"(acc[o][q]) : : "memory");
}
// the value lane k of this lane's quad holds (k a constant after unrolling)
__device__ __forceinline__ uint32_t quad_lane_of(uint32_t v, int k) {
    switch (k & 3) {
        case 0: return quad_lane<0>(v);
        case 1: return quad_lane<1>(v);
        case 2: return quad_lane<2>(v);
        default: return quad_lane<3>(v);
    }
}
template <int NG, int WMODE>   // NG: groups of four steps per quad (9: bands of 32 entries), 0: as the launch says
__global__ __launch_bounds__(1024) void band_resident_kernel(ResidentArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int sh_alive[3];
    __shared__ int sh_last[16];
    constexpr int R = 16, PARTS = 4;
    using GU = const __attribute__((address_space(1))) uint32_t*;
    using GW = const __attribute__((address_space(1))) f32x4_t*;
    using GI = const __attribute__((address_space(1))) int32_t*;
    publish_counts(a.pub);
    const int t = (int)threadIdx.x, lane = t & 63, nthr = a.N;   // (launched with N threads)
    const int RB = 64 * a.rl;
    const unsigned nwg = gridDim.x;
    const unsigned wg = (nwg % 8u) == 0u ? (blockIdx.x % 8u) * (nwg / 8u) + blockIdx.x / 8u : blockIdx.x;
    const size_t row0 = (size_t)wg * R;
    const int rb = (int)(row0 / (size_t)RB), rin = (int)(row0 - (size_t)rb * RB);
    if (a.check_dead && a.prev_stamp != 0) {   // a row block without an active row is skipped, as by the per-layer kernels
        int alive = 0;
        for (int i = t; i < RB; i += nthr) alive |= (a.active[(size_t)rb * RB + i] == a.prev_stamp) ? 1 : 0;
        if (__syncthreads_or(alive) == 0) return;
    }
    const size_t blkf = (size_t)a.N * RB;
    const uint32_t buf_bytes = (uint32_t)a.N * R * 4;
    const int total = a.N * PARTS;
    {
        const float* __restrict__ gin = ((rb & 1) ? a.first_in.half[1] : a.first_in.half[0]) + (size_t)(rb >> 1) * blkf + rin;
        // N * 4 pieces (a column's rows in four parts) over N threads: four loads each, all in flight together
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int idx = t + u * nthr;
            const int col = idx / PARTS, part = idx - col * PARTS;
            v[u] = *reinterpret_cast<const float4*>(gin + (size_t)col * RB + part * 4);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) *reinterpret_cast<float4*>(smem + (size_t)(t + u * nthr) * 16) = v[u];
    }
    if (t < 3) sh_alive[t] = 0;
    if (t < R) sh_last[t] = -1;
    const int rq = t & 3;
    const uint32_t lane_off = (uint32_t)rq * 16u;
    // the wave's own KiB behind the two row buffers, this lane's quad's 64 bytes of it
    unsigned char* const wslot = smem + 2u * buf_bytes + (uint32_t)(t >> 6) * 1024u + (uint32_t)((t & 63) >> 2) * 64u;
    const int ng = NG ? NG : a.ngroups;
    // this lane's place in a quad's plan stream: group gi lies 4 lanes further on
    const size_t qoff = (size_t)(t >> 2) * (size_t)ng * 4 + (size_t)rq;
    uint32_t c_first[2], d_first;
    f32x4_t w_first[2];
    // (no layer table here: a table entry read at the top of a layer - a scalar load, then the loads that need its
    // pointers - would be waited for by every wave of the workgroup at once, right behind the barrier: 2.8 us of a 7 us layer)
    using GB = const __attribute__((address_space(1))) unsigned char*;
    const GB col_base = (GB)a.quad_col + qoff * 4, w_base = (GB)a.quad_w + qoff * 16, dst_base = (GB)a.quad_dst + (size_t)t * 4;
    auto request_first = [&](int j) {
        const GU colp = (GU)(col_base + (long long)j * a.quad_stride);
        const GW wp = (GW)(w_base + (long long)j * a.quad_stride);
        c_first[0] = colp[0];
        w_first[0] = wp[0];
        c_first[1] = colp[ng > 1 ? 4 : 0];
        w_first[1] = wp[ng > 1 ? 4 : 0];
        d_first = (uint32_t)(*(GI)(dst_base + (long long)j * a.quad_stride));   // (used as it comes: arithmetic on it here would wait for the load)
    };
    request_first(0);
    int last_nz[4] = {-1, -1, -1, -1};
    bool all_dead = false;
    int done_layers = 0;
    __syncthreads();
    for (int j = 0; j < a.nlayers; ++j) {
        const unsigned char* const in = smem + ((j & 1) ? buf_bytes : 0u);
        unsigned char* const out = smem + ((j & 1) ? 0u : buf_bytes);
        const GU colp = (GU)(col_base + (long long)j * a.quad_stride);
        const GW wp = (GW)(w_base + (long long)j * a.quad_stride);
        uint32_t cr[3];
        f32x4_t wr[3];
        cr[0] = c_first[0]; cr[1] = c_first[1];
        wr[0] = w_first[0]; wr[1] = w_first[1];
        const uint32_t dcol = d_first * (uint32_t)(R * 4);
        if (j + 1 < a.nlayers) request_first(j + 1);   // in flight under this layer's arithmetic
        float acc[4][4];
#pragma unroll
        for (int o = 0; o < 4; ++o)
#pragma unroll
            for (int q = 0; q < 4; ++q) acc[o][q] = 0.0f;
        // step e = 4 gi + k: the LDS read of step e + 3 is issued before the arithmetic of step e (the waves of a workgroup
        // leave the barrier together: a wave that waited for each read right after issuing it would wait when all others do).
        // The weights of a group of four steps go through the wave's own 1 KiB of LDS: lane k of a quad has requested the
        // four outputs' weights of step k, writes them behind the last read of the group before (one wave's LDS
        // instructions run in order: no barrier), and every lane of the quad reads a step's four weights back, one
        // step ahead - all sixteen multiply-adds of a step then take their operands from the lane's own registers.
        const int nsteps = 4 * ng;
        float4 xb[4];
        float4 wq[2];
        xb[0] = *reinterpret_cast<const float4*>(in + (quad_lane<0>(cr[0]) + lane_off));
        xb[1] = *reinterpret_cast<const float4*>(in + (quad_lane<1>(cr[0]) + lane_off));
        xb[2] = *reinterpret_cast<const float4*>(in + (quad_lane<2>(cr[0]) + lane_off));
        *reinterpret_cast<f32x4_t*>(wslot + lane_off) = wr[0];
        wq[0] = *reinterpret_cast<const float4*>(wslot);
#pragma unroll
        for (int e = 0; e < 36; ++e) {
            if (e < nsteps) {
                const int gi = e >> 2;
                if ((e & 3) == 0 && e + 8 < 36 && e + 8 < nsteps) {   // the plan stream: two groups ahead
                    cr[(gi + 2) % 3] = colp[(gi + 2) * 4];
                    wr[(gi + 2) % 3] = wp[(gi + 2) * 4];
                }
                if (e + 3 < 36 && e + 3 < nsteps)
                    xb[(e + 3) % 4] = *reinterpret_cast<const float4*>(in + (quad_lane_of(cr[((e + 3) >> 2) % 3], e + 3) + lane_off));
                if (e + 1 < 36 && e + 1 < nsteps) {
                    if ((e & 3) == 3) *reinterpret_cast<f32x4_t*>(wslot + lane_off) = wr[(gi + 1) % 3];   // the next group's weights
                    wq[(e + 1) & 1] = *reinterpret_cast<const float4*>(wslot + ((e + 1) & 3) * 16);
                }
                quad_step<WMODE>(acc, xb[e % 4], wq[e & 1]);
            }
        }
        // (outputs are clamped to [0, clamp]: the largest of a row's four is positive exactly when one of them is nonzero)
        float y[4][4];
#pragma unroll
        for (int o = 0; o < 4; ++o) {
#pragma unroll
            for (int q = 0; q < 4; ++q) y[o][q] = relu_clamp(acc[o][q] + a.bias, a.clampv);
        }
        *reinterpret_cast<float4*>(out + (quad_lane<0>(dcol) + lane_off)) = float4{y[0][0], y[0][1], y[0][2], y[0][3]};
        *reinterpret_cast<float4*>(out + (quad_lane<1>(dcol) + lane_off)) = float4{y[1][0], y[1][1], y[1][2], y[1][3]};
        *reinterpret_cast<float4*>(out + (quad_lane<2>(dcol) + lane_off)) = float4{y[2][0], y[2][1], y[2][2], y[2][3]};
        *reinterpret_cast<float4*>(out + (quad_lane<3>(dcol) + lane_off)) = float4{y[3][0], y[3][1], y[3][2], y[3][3]};
        float top = 0.0f;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float m = __builtin_fmaxf(__builtin_fmaxf(__builtin_fmaxf(y[0][q], y[1][q]), y[2][q]), y[3][q]);
            if (m > 0.0f) last_nz[q] = j;   // this lane's outputs left row 4 rq + q nonzero
            top = __builtin_fmaxf(top, m);
        }
        // the workgroup goes on while one of its rows is nonzero: a flag per layer, the rows' own last layers are put
        // together once, behind the loop
        if (__ballot(top > 0.0f ? 1 : 0) != 0ull && lane == 0) sh_alive[j % 3] = 1;
        __syncthreads();
        const int some = sh_alive[j % 3];
        if (t == 0) sh_alive[(j + 2) % 3] = 0;
        done_layers = j + 1;
        if (some == 0 && a.bias <= 0.0f) { all_dead = true; break; }   // zero rows stay zero
    }
    // the last layer that left each of the 16 rows nonzero: the largest over the lanes that hold the row's outputs
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        int v = last_nz[q];
#pragma unroll
        for (int sft = 4; sft < 64; sft <<= 1) v = max(v, __shfl_xor(v, sft, 64));
        if (lane < 4 && v >= 0) atomicMax(&sh_last[lane * 4 + q], v);
    }
    __syncthreads();
    const int last_alive = t < R ? sh_last[t] : -1;
    // the launch's last layer writes the work buffer the layer before it did not (layer 0: the one it did not read)
    const bool in_a = a.first_in.half[0] == a.buf_a.half[0];
    const bool to_c = in_a == ((a.nlayers & 1) != 0);
    float* const o_h0 = to_c ? a.buf_c.half[0] : a.buf_a.half[0];
    float* const o_h1 = to_c ? a.buf_c.half[1] : a.buf_a.half[1];
    float* __restrict__ gout = ((rb & 1) ? o_h1 : o_h0) + (size_t)(rb >> 1) * blkf + rin;
    const unsigned char* const fin = smem + ((done_layers & 1) ? buf_bytes : 0u);
    for (int idx = t; idx < total; idx += nthr) {
        const int col = idx / PARTS, part = idx - col * PARTS;
        float4 v;
        if (all_dead) v = float4{0.0f, 0.0f, 0.0f, 0.0f};
        else v = *reinterpret_cast<const float4*>(fin + (size_t)idx * 16);
        *reinterpret_cast<float4*>(gout + (size_t)col * RB + part * 4) = v;
    }
    if (t < R && last_alive >= 0) a.active[row0 + t] = a.stamp0 + last_alive;
}

// counts[i] = rows whose stamp is at least stamp_lo + i (see launch_count_stamp_range).  Every workgroup takes a
// share of the rows: a histogram in LDS (per wave one atomic per distinct value), sums from the top, and - where the
// launch has several workgroups - the sums added to `partial` (n words, zero when the launch starts).  The workgroup
// that finishes last (a ticket in partial[kCountTicket]) hands the totals over and leaves partial zero again.
constexpr int kCountTicket = 8192;   // words of `partial` in front of the ticket: the largest n
__global__ __launch_bounds__(1024) void count_stamp_range_kernel(const int32_t* __restrict__ stamps, int rows, int stamp_lo,
                                                                 int n, int32_t* __restrict__ counts_dev,
                                                                 int32_t* __restrict__ counts_host, int32_t* __restrict__ partial) {
    extern __shared__ int hist[];
    __shared__ int sh_last;
    for (int i = threadIdx.x; i < n; i += 1024) hist[i] = 0;
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const int per = (((rows + (int)gridDim.x - 1) / (int)gridDim.x) + 1023) & ~1023;   // rows per workgroup: whole trips of 1024
    const int r_begin = (int)blockIdx.x * per, r_end = min(rows, r_begin + per);
    for (int r0 = r_begin; r0 < r_end; r0 += 1024) {
        const int r = r0 + (int)threadIdx.x;
        int d = r < r_end ? stamps[r] - stamp_lo : -1;
        if (d >= n) d = n - 1;
        unsigned long long todo = __ballot(d >= 0 ? 1 : 0);
        while (todo) {
            const int first = (int)__ffsll((long long)todo) - 1;
            const int v = __shfl(d, first, 64);
            const unsigned long long same = __ballot(d == v ? 1 : 0);
            if (lane == first) atomicAdd(&hist[v], (int)__popcll(same));
            todo &= ~same;
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int acc = 0;
        for (int i = n - 1; i >= 0; --i) { acc += hist[i]; hist[i] = acc; }
    }
    __syncthreads();
    if (gridDim.x > 1) {
        for (int i = threadIdx.x; i < n; i += 1024)
            if (hist[i] != 0) atomicAdd(&partial[i], hist[i]);
        __threadfence();
        __syncthreads();
        if (threadIdx.x == 0) sh_last = atomicAdd(&partial[kCountTicket], 1) == (int)gridDim.x - 1 ? 1 : 0;
        __syncthreads();
        if (!sh_last) return;
        __threadfence();
        for (int i = threadIdx.x; i < n; i += 1024) hist[i] = atomicExch(&partial[i], 0);
        if (threadIdx.x == 0) atomicExch(&partial[kCountTicket], 0);
    }
    for (int i = threadIdx.x; i < n; i += 1024) {
        if (counts_dev) counts_dev[i] = hist[i];
        if (counts_host) __hip_atomic_store(counts_host + i, hist[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
}

// ------------------------------------------------------------------------------------------
// Active-row scan.  Workgroup b (1024 threads) owns the tile of rows [1024 b, 1024 b + 1024),
// thread = row, so all reads are coalesced.  Its survivors go behind those of the tiles before
// it; how many those are it counts itself (the flags of at most 58 earlier tiles, 8 bytes a row
// from L2 - cheaper than a second launch or a chain of workgroups waiting for each other).
// Inside the tile a survivor's place comes from the wave's ballot and an LDS sum over the 16
// waves.  Stable: survivors keep their order, as the reference's host loop does
// (all_network.cu:455-463).  The last workgroup writes the total.
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void scan_active_kernel(
    const int32_t* __restrict__ active, const int32_t* __restrict__ gid, int rows, int stamp,
    int32_t* __restrict__ count, int32_t* __restrict__ alive_src, int32_t* __restrict__ alive_gid) {
    __shared__ int wave_tot[16];
    __shared__ int wave_before[16];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int tile = blockIdx.x;
    // survivors among this wave's 64 rows of every earlier tile (eight tiles' loads in flight at a time: one after the
    // other the loop is as long as 58 round trips to L2)
    int mine = 0;
#pragma unroll 8
    for (int t = 0; t < tile; ++t) {
        const int r = t * 1024 + (int)threadIdx.x;  // < rows: an earlier tile is a full one
        const int st = active[r], gd = gid[r];   // (both loaded whatever the first says: a load behind a test is a round trip of its own)
        mine += ((st == stamp) & (gd >= 0)) ? 1 : 0;
    }
    int before = mine;
#pragma unroll
    for (int sft = 1; sft < 64; sft <<= 1) before += __shfl_xor(before, sft, 64);
    const int r = tile * 1024 + (int)threadIdx.x;
    const int g = r < rows ? gid[r] : -1;
    const bool alive = r < rows && g >= 0 && active[r] == stamp;
    const unsigned long long mask = __ballot(alive ? 1 : 0);
    if (lane == 0) {
        wave_tot[wave] = (int)__popcll(mask);
        wave_before[wave] = before;
    }
    __syncthreads();
    int base = 0, total = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
        base += wave_before[w];
        total += wave_before[w] + wave_tot[w];
        if (w < wave) base += wave_tot[w];
    }
    if (alive) {
        const int k = base + (int)__popcll(mask & ((1ull << lane) - 1ull));
        alive_src[k] = r;
        alive_gid[k] = g;
    }
    if (tile == (int)gridDim.x - 1 && threadIdx.x == 0) count[0] = total;
}

// Repack survivors into dense row blocks.  Thread = destination row slot; loops over a chunk of
// columns.  Reads are 4-byte gathers (one per surviving row and column), writes are coalesced.
template <int RL>
__global__ __launch_bounds__(64 * RL) void repack_kernel(
    Feat src, Feat dstb, const int32_t* __restrict__ count,
    const int32_t* __restrict__ alive_src, const int32_t* __restrict__ alive_gid,
    int32_t* __restrict__ gid_out, int N, int cols_per_wg) {
    constexpr int RB = 64 * RL;
    const int nb = blockIdx.y;
    const int slot = nb * RB + threadIdx.x;
    const int cnt = count[0];
    const bool live = slot < cnt;
    const int srow = live ? alive_src[slot] : 0;
    const float* sp = block_base(src, srow / RB, (size_t)N * RB) + (srow % RB);
    float* dp = block_base(dstb, nb, (size_t)N * RB) + threadIdx.x;
    const int c0 = blockIdx.x * cols_per_wg;
    const int c1 = min(N, c0 + cols_per_wg);
    for (int c = c0; c < c1; ++c) {
        const float x = live ? sp[(size_t)c * RB] : 0.0f;
        dp[(size_t)c * RB] = x;
    }
    if (blockIdx.x == 0) gid_out[slot] = live ? alive_gid[slot] : -1;
}

// ------------------------------------------------------------------------------------------
// Features
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ uint64_t sm64(uint64_t x) {
    uint64_t z = x + 0x9E3779B97F4A7C15ULL;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

// Seeded Bernoulli rows: element (row, c) = hi32(sm64(rk(row) + c)) < thr(row) ? 1 : 0, where
// rk and thr depend on the seed and the row only.  Thread = row; a workgroup covers one row
// block and a chunk of physical columns.
template <int RL>
__global__ __launch_bounds__(64 * RL) void synth_features_kernel(
    Feat y, const int32_t* __restrict__ col_of_phys, int N, int batch, int cols_per_wg,
    uint64_t kf, uint64_t lo, uint64_t span) {
    constexpr int RB = 64 * RL;
    const int rb = blockIdx.y;
    const long long row = (long long)rb * RB + threadIdx.x;
    const bool real = row < batch;
    const uint64_t rk = sm64(kf + (uint64_t)row);
    const uint64_t a = sm64(rk + 0xFFFFFFFF00000000ULL) >> 32;
    uint64_t thr = lo + ((a * span) >> 32);
    if (thr > 0xFFFFFFFFULL) thr = 0xFFFFFFFFULL;
    const int c0 = blockIdx.x * cols_per_wg;
    const int c1 = min(N, c0 + cols_per_wg);
    float* yp = block_base(y, rb, (size_t)N * RB) + threadIdx.x;
    for (int pc = c0; pc < c1; ++pc) {
        const int n = col_of_phys[pc];
        const uint32_t e = (uint32_t)(sm64(rk + (uint64_t)n) >> 32);
        yp[(size_t)pc * RB] = (real && e < (uint32_t)thr) ? 1.0f : 0.0f;
    }
}

// Row-major chunk -> row-block layout, 32 columns x RB rows per workgroup through an LDS tile.
template <int RL>
__global__ __launch_bounds__(256) void pack_rows_kernel(
    const float* __restrict__ rowmajor, Feat y, const int32_t* __restrict__ phys_of_col,
    int N, long long row0, int nrows, int32_t* __restrict__ nonfinite) {
    constexpr int RB = 64 * RL;
    __shared__ float tile[RB][33];
    const int n0 = blockIdx.x * 32;
    const int lb = blockIdx.y;  // row block inside the chunk
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    bool bad = false, tiny = false;
    for (int rr = ty; rr < RB; rr += 8) {
        const int lr = lb * RB + rr;
        float x = 0.0f;
        if (lr < nrows && n0 + tx < N) x = rowmajor[(size_t)lr * N + n0 + tx];
        if (!(fabsf(x) <= 1.2676506e30f)) bad = true;  // NaN, infinity or beyond 2^100
        // below 2^-100 a product with a power-of-two weight may underflow, where a fused
        // multiply-add no longer rounds like multiply-then-add
        if (x != 0.0f && fabsf(x) < 7.888609e-31f) tiny = true;
        tile[rr][tx] = x;
    }
    if (bad) nonfinite[0] = 1;
    if (tiny) nonfinite[1] = 1;
    __syncthreads();
    float* yp = block_base(y, (int)(row0 / RB) + lb, (size_t)N * RB);
    for (int idx = threadIdx.x; idx < 32 * RB; idx += 256) {
        const int c = idx / RB, r = idx % RB;
        if (n0 + c < N) yp[(size_t)phys_of_col[n0 + c] * RB + r] = tile[r][c];
    }
}

__global__ void unpack_rows_kernel(Feat y, const int32_t* __restrict__ phys_of_col,
                                   const int32_t* __restrict__ phys_rows, int N, int RB,
                                   const int32_t* __restrict__ active, int stamp, float* __restrict__ rowmajor) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= N) return;
    const int pr = phys_rows[blockIdx.y];
    float x = 0.0f;
    // a row that the last layer did not stamp is all zero by definition (its block may have been
    // skipped, leaving stale data in the buffer)
    if (pr >= 0 && (stamp == 0 || active[pr] == stamp)) {
        const int pc = phys_of_col ? phys_of_col[n] : n;
        x = block_base(y, pr / RB, (size_t)N * RB)[(size_t)pc * RB + (pr % RB)];
    }
    rowmajor[(size_t)blockIdx.y * N + n] = x;
}

// Row lookup on the device (for callers that cannot allocate): where[g] = physical row that carries
// global id g, -1 for a row that is not carried any more.  fill first, then scatter.
__global__ void fill_i32_kernel(int32_t* __restrict__ p, int n, int32_t v) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}
__global__ void scatter_where_kernel(const int32_t* __restrict__ gid, int carried, int batch, int32_t* __restrict__ where) {
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= carried) return;
    const int g = gid[r];
    if (g >= 0 && g < batch) where[g] = r;
}
__global__ void lookup_rows_kernel(const int32_t* __restrict__ ids, int n, const int32_t* __restrict__ where,
                                   int32_t* __restrict__ phys) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) phys[i] = where[ids[i]];
}

__global__ void iota_gid_kernel(int32_t* gid, int rows, int batch) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < rows) gid[i] = i < batch ? i : -1;
}

// Streaming write into two buffers at once: even workgroups fill p, odd workgroups fill q.
__global__ __launch_bounds__(256) void zero_pair_kernel(float4* __restrict__ p, float4* __restrict__ q, long long n4) {
    float4* d = (blockIdx.x & 1) ? q : p;
    long long i = (long long)(blockIdx.x >> 1) * blockDim.x + threadIdx.x;
    const long long stride = (long long)(gridDim.x >> 1) * blockDim.x;
    for (; i < n4; i += stride) d[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
}

// Copy of two buffers at once: even workgroups copy p0 -> q0, odd workgroups p1 -> q1 (the access
// pattern of a layer kernel over feature buffers whose halves lie in two memory regions).
__global__ __launch_bounds__(256) void copy_pair_kernel(const stream_f4* __restrict__ p0, stream_f4* __restrict__ q0,
                                                        const stream_f4* __restrict__ p1, stream_f4* __restrict__ q1,
                                                        long long n4) {
    const stream_f4* s = (blockIdx.x & 1) ? p1 : p0;
    stream_f4* d = (blockIdx.x & 1) ? q1 : q0;
    long long i = (long long)(blockIdx.x >> 1) * blockDim.x + threadIdx.x;
    const long long stride = (long long)(gridDim.x >> 1) * blockDim.x;
    for (; i < n4; i += stride) __builtin_nontemporal_store(__builtin_nontemporal_load(&s[i]), &d[i]);
}

__global__ __launch_bounds__(256) void copy_f4_kernel(const float4* __restrict__ src, float4* __restrict__ dst,
                                                      long long n4) {
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (; i < n4; i += stride) dst[i] = src[i];
}

// Segment lengths for the band walk, best first: multiples of the chunk T.  More segments fill the
// CUs more evenly, fewer segments load fewer halo columns; score both.  `slots` is the number of
// workgroups resident at once (CUs x workgroups per CU).
int rank_seglens(int N, int K, int T, int nblk, int slots, int* out, int max_out) {
    const int nchunks = (N + T - 1) / T;
    double best[8];
    int n = 0;
    if (max_out > 8) max_out = 8;
    int last_nseg = -1;
    for (int cps = nchunks; cps >= 1; --cps) {  // chunks per segment
        const int nseg = (nchunks + cps - 1) / cps;
        if (nseg > 65535) break;
        if (nseg == last_nseg) continue;  // same grid as a longer segment: keep the balanced one below
        last_nseg = nseg;
        const int cps_bal = (nchunks + nseg - 1) / nseg;  // spread the chunks evenly over nseg segments
        const long long wgs = (long long)nblk * nseg;
        const long long rounds = (wgs + slots - 1) / slots;
        const double fill = (double)wgs / (double)(rounds * slots);
        const double halo = 1.0 / (1.0 + 0.25 * (double)(K - 1) / (double)(cps_bal * T));
        const double score = fill * halo;
        int pos = n;
        while (pos > 0 && score > best[pos - 1] + 1e-9) --pos;
        if (pos >= max_out) continue;
        const int stop = n < max_out ? n : max_out - 1;
        for (int i = stop; i > pos; --i) { best[i] = best[i - 1]; out[i] = out[i - 1]; }
        best[pos] = score;
        out[pos] = cps_bal * T;
        if (n < max_out) ++n;
    }
    return n;
}

// the fill/halo model of rank_seglens for one segment length
double seglen_score(int N, int K, int T, int nblk, int slots, int seglen) {
    const int nseg = (N + seglen - 1) / seglen;
    const long long wgs = (long long)nblk * nseg;
    const long long rounds = (wgs + slots - 1) / slots;
    const double fill = (double)wgs / (double)(rounds * slots);
    return fill / (1.0 + 0.25 * (double)(K - 1) / (double)seglen);
}

template <int RL, int NW, int OPW, int RING, int WMODE, int KT, int DMA>
hipError_t launch_band_inst(const BandLaunch& a, hipStream_t s) {
    constexpr int T = NW * OPW;
    constexpr size_t lds = (size_t)RING * 64 * RL * 4;
    auto kern = band_walk_kernel<RL, NW, OPW, RING, WMODE, KT, DMA>;
    // once per instantiation; a function-local static is initialised by one thread only
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (attr != hipSuccess) return attr;
    int seglen = a.seglen;
    if (seglen <= 0 || (seglen % T) != 0) {
        if (rank_seglens(a.N, a.K, T, a.nblk, a.n_cu > 0 ? a.n_cu : 256, &seglen, 1) < 1) return hipErrorInvalidValue;
    }
    const int nseg = (a.N + seglen - 1) / seglen;
    if (nseg > 65535) return hipErrorInvalidValue;
    // Workgroups go to the 8 XCDs round robin by their linear number (row blocks fastest).  With a
    // grid whose x extent is a multiple of 8 every segment of a row block runs on the same XCD, and
    // what one layer writes is still in that XCD's L2 (4 MiB) when the next layer reads it.  Where
    // the row blocks of an XCD fit that L2 with their input and output, the x extent is therefore
    // padded (the padding workgroups leave at once).  Measured at N=1024: 5 - 7 row blocks 12.3 -
    // 13.3 us per layer without, 9.5 - 10.1 us with the padding; one or two row blocks, or data beyond
    // the L2, are slower with it.
    const size_t block_bytes = (size_t)a.N * 64 * RL * 4;
    const bool pad = a.nblk >= 3 && (a.nblk & 7) != 0 && (size_t)((a.nblk + 7) / 8) * block_bytes * 2 <= ((size_t)4 << 20);
    const int gx = pad ? (a.nblk + 7) / 8 * 8 : a.nblk;
    // Input and output of the launch together beyond what stays in the caches from one layer to the next: the
    // columns are hinted as touched once (see store_stream).  Measured cross-over (N=1024 ... 16384): around
    // 64 - 128 MiB; below it the next layer still finds this layer's output on chip and the hint costs up to 15 %.
    const int stream = (long long)a.nblk * (long long)block_bytes * 2 >= a.stream_min_bytes ? 1 : 0;
    dim3 grid(gx, nseg), block(NW * 64);
    hipLaunchKernelGGL(kern, grid, block, lds, s, a.yin, a.yout, a.pairs, a.pw, a.dst, a.active, a.count_prev,
                       a.N, a.steps, a.halo, seglen, a.stamp, a.prev_stamp, a.check_dead, a.wu, a.bias, a.clampv, a.publish,
                       a.nblk, stream, a.frontier, a.frontier_layer);
    return hipGetLastError();
}

template <int RL, int NW, int OPW, int RING, int DMA>
hipError_t launch_band_rl(const BandLaunch& a, hipStream_t s) {
    if (band_unrolled(a.K, a.steps, a.stride)) {
        switch (a.wmode) {
            case 0:
                if (a.add_only && a.twins) return launch_band_inst<RL, NW, OPW, RING, 4, 36, DMA>(a, s);
                if (a.add_only) return launch_band_inst<RL, NW, OPW, RING, 3, 36, DMA>(a, s);
                return launch_band_inst<RL, NW, OPW, RING, 0, 36, DMA>(a, s);
            case 1: return launch_band_inst<RL, NW, OPW, RING, 1, 36, DMA>(a, s);
            default: return launch_band_inst<RL, NW, OPW, RING, 2, 36, DMA>(a, s);
        }
    }
    switch (a.wmode) {
        case 0:
            if (a.add_only) return launch_band_inst<RL, NW, OPW, RING, 3, 0, DMA>(a, s);
            return launch_band_inst<RL, NW, OPW, RING, 0, 0, DMA>(a, s);
        case 1: return launch_band_inst<RL, NW, OPW, RING, 1, 0, DMA>(a, s);
        default: return launch_band_inst<RL, NW, OPW, RING, 2, 0, DMA>(a, s);
    }
}

}  // namespace

// 32 entries per output (KT = 36: the first 32 steps of a pair run unconditionally); with fewer entries
// the same walk runs its steps in groups of four as far as they reach (KT = 0)
bool band_unrolled(int K, int steps, int stride) { return K == 32 && steps <= 36 && stride == 16; }

// Tile shape of the band walk, the same for every row-block size: 8 waves x 2 outputs (one pair) per
// chunk and a 64-slot ring - 64 KiB of LDS and two workgroups per CU for 256-row blocks (whose load /
// compute / barrier phases interleave), 32 and 16 KiB and four workgroups per CU (the wave limit)
// for 128- and 64-row blocks.  Measured at N=65536: 256-row blocks 6.0 ms per layer, 128-row blocks
// 6.6 ms (8.8 ms with one 16-wave workgroup and a 256-slot ring per CU).
// Variants of the band walk (BandLaunch.shape, BandLaunch.direct_lds): for 256-row blocks the next chunk's
// columns go straight from HBM into the LDS ring (shape 0 with direct_lds), or are parked in registers and
// written to the ring after the arithmetic (shape 1, or direct_lds off; the only form for smaller row
// blocks).  The run-time selection used to try both; measured one after the other on live data, per layer:
// N=1024 102.9 against 107.0 us, N=4096 337.9 against 352 - 380, N=16384 1280 against 1291, N=65536 and batch
// 6000 within the noise - straight into LDS is never the slower one, so it is the one form the selection
// uses and only the segment length is left to it.
int band_shape_count(int rl, int direct_lds) { (void)rl; (void)direct_lds; return 1; }

int band_chunk_outputs(int rl, int shape) {
    (void)rl; (void)shape;
    return 16;
}

int band_workgroups_per_cu(int rl, int shape) {
    (void)shape;
    return rl == 4 ? 2 : 4;
}

int band_seglen_candidates(int N, int K, int nblk, int rl, int shape, int n_cu, int* out, int max_out) {
    // the two best-ranked by the fill/halo model, then a geometric ladder of segment counts
    // (those the model does not rule out): shorter segments mean more, smaller workgroups, which
    // often balances and streams better than the model predicts - the caller measures
    const int T = band_chunk_outputs(rl, shape);
    const int slots = n_cu * band_workgroups_per_cu(rl, shape);
    int n = rank_seglens(N, K, T, nblk, slots, out, max_out < 2 ? max_out : 2);
    if (n < 1) return 0;
    const double floor_score = 0.6 * seglen_score(N, K, T, nblk, slots, out[0]);  // not worth a trial below this
    const int nchunks = (N + T - 1) / T;
    static const int ladder[] = {1, 2, 4, 8, 16, 24, 32, 48, 64, 96, 128, 192, 256, 384, 512};
    for (int nseg : ladder) {
        if (n >= max_out) break;
        const int cps = (nchunks + nseg - 1) / nseg;
        // at least four chunks per workgroup - unless even that leaves most of the chip idle
        // (few row blocks): then single-chunk workgroups, which finish soonest, are candidates too
        const bool starved = (long long)nblk * ((nchunks + 3) / 4) < 2LL * slots;
        if (cps < (starved ? 1 : 4) && nseg > 1) break;
        const int len = cps * T;
        bool dup = seglen_score(N, K, T, nblk, slots, len) < floor_score;
        for (int i = 0; i < n; ++i) dup |= out[i] == len;
        if (!dup) out[n++] = len;
    }
    return n;
}

double band_seglen_score(int N, int K, int nblk, int rl, int shape, int n_cu, int seglen) {
    if (seglen <= 0) return 0.0;
    return seglen_score(N, K, band_chunk_outputs(rl, shape), nblk, n_cu * band_workgroups_per_cu(rl, shape), seglen);
}

hipError_t launch_band(const BandLaunch& a, hipStream_t s) {
    // host-side shape checks: what the kernel and its grid assume
    if (a.N <= 0 || (a.N % 256) != 0 || a.K < 4 || a.K > 32 || (a.K % 4) != 0 || a.nblk <= 0 ||
        a.halo < a.K - 1 || a.halo > 32 || a.halo >= a.N || a.steps < a.K || a.steps > 36 || a.stride != 16 ||
        !a.yin || !a.yout || !a.pairs || !a.dst || !a.active || (a.wmode != 0 && !a.pw))
        return hipErrorInvalidValue;
    BandLaunch b = a;
    b.n_cu = (a.n_cu > 0 ? a.n_cu : 256) * band_workgroups_per_cu(a.rl, a.shape);
    if (b.seglen > 0) b.seglen -= b.seglen % band_chunk_outputs(a.rl, a.shape);  // whole chunks; 0 = heuristic
    switch (a.rl) {
        case 4:
            return (a.direct_lds && a.shape != 1) ? launch_band_rl<4, 8, 2, 64, 1>(b, s)
                                                  : launch_band_rl<4, 8, 2, 64, 0>(b, s);
        case 2: return launch_band_rl<2, 8, 2, 64, 0>(b, s);
        case 1: return launch_band_rl<1, 8, 2, 64, 0>(b, s);
        default: return hipErrorInvalidValue;
    }
}

namespace {
// what a persistent launch is cut into: positions (band walk) or groups (BLOCK) per unit, units per
// row block and layer, queues
struct PersistShape { int seglen, nseg, nq, grid, total; };

PersistShape persist_shape(const PersistLaunch& a) {
    PersistShape p{};
    const int slots_cu = a.block_form ? 8 : band_workgroups_per_cu(a.rl, 0);
    const int slots = (a.n_cu > 0 ? a.n_cu : 256) * slots_cu;
    p.nq = (a.xcd_queues && a.nblk >= 1) ? 8 : 1;
    // row blocks that work side by side: all of them, or those of the fullest queue
    const int nrb = p.nq > 1 ? (a.nblk + 7) / 8 : a.nblk;
    const int slots_q = p.nq > 1 ? std::max(1, slots / 8) : slots;
    if (a.block_form) {
        // pieces of 4 waves x seglen groups; one group per wave where the batch is small
        const int ngroups = a.ngroups;
        const int pieces = (ngroups + 3) / 4;
        int nseg = std::min(pieces, std::max(1, (slots_q + nrb - 1) / nrb));
        int gpw = (pieces + nseg - 1) / nseg;
        if (gpw > 8) gpw = 8;
        if (a.seglen > 0) gpw = a.seglen;
        p.seglen = gpw;
        p.nseg = (pieces + gpw - 1) / gpw;
    } else {
        const int T = band_chunk_outputs(a.rl, 0);
        const int nchunks = (a.N + T - 1) / T;
        // enough units per layer to give every resident workgroup one, as long as a unit keeps a chunk;
        // long units are cut at 64 chunks so that the launch's tail stays short
        int nseg = std::min(nchunks, std::max(1, (slots_q + nrb - 1) / nrb));
        int cps = (nchunks + nseg - 1) / nseg;
        if (cps > 64) cps = 64;
        if (a.seglen > 0) cps = std::max(1, a.seglen / T);
        p.seglen = cps * T;
        p.nseg = (nchunks + cps - 1) / cps;
    }
    p.total = a.nblk * p.nseg * a.nlayers;
    const long long per_layer_q = (long long)nrb * p.nseg;
    p.grid = (int)std::min<long long>(slots, per_layer_q * p.nq);
    if (p.grid < p.nq) p.grid = p.nq;
    return p;
}

PersistArgs persist_args(const PersistLaunch& a, const PersistShape& p) {
    PersistArgs k{};
    k.table = a.table; k.nlayers = a.nlayers; k.first_in = a.first_in; k.buf_a = a.buf_a; k.buf_c = a.buf_c;
    k.active = a.active; k.done = a.done; k.done_stride = a.done_stride; k.ctl = a.ctl; k.prev_ctl = a.prev_ctl;
    k.prev_units = a.prev_units; k.abort = a.abort; k.host_word = a.host_word;
    k.N = a.N; k.nblk = a.nblk; k.nseg = p.nseg; k.seglen = p.seglen; k.total_units = p.total; k.nq = p.nq;
    // light_sync (per-XCD queues only): the writer waits for its stores and leaves the L2 write-back out (bit 1)
    k.light = (p.nq > 1 && a.light_sync) ? 2 : 0;
    k.stamp0 = a.stamp0; k.prev_stamp = a.prev_stamp; k.check_dead = a.check_dead; k.wait_limit = a.wait_limit;
    k.bias = a.bias; k.clampv = a.clampv;
    k.stream = (long long)a.nblk * (long long)a.N * 64 * a.rl * 4 * 2 >= a.stream_min_bytes ? 1 : 0;
    k.pub = a.publish;
    return k;
}

template <int RL, int WMODE, int KT, int DMA>
hipError_t launch_persist_band_dma(const PersistLaunch& a, hipStream_t s) {
    constexpr size_t lds = (size_t)64 * 64 * RL * 4;
    auto kern = band_persist_kernel<RL, WMODE, KT, DMA>;
    // once per instantiation; a function-local static is initialised by one thread only
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (attr != hipSuccess) return attr;
    const PersistShape p = persist_shape(a);
    hipLaunchKernelGGL(kern, dim3(p.grid), dim3(512), lds, s, persist_args(a, p));
    return hipGetLastError();
}
// (256-row blocks: the next chunk's columns straight into the LDS ring, as in the per-layer launches)
template <int RL, int WMODE, int KT>
hipError_t launch_persist_band_inst(const PersistLaunch& a, hipStream_t s) {
    if constexpr (RL == 4) {
        if (a.direct_lds) return launch_persist_band_dma<RL, WMODE, KT, 1>(a, s);
    }
    return launch_persist_band_dma<RL, WMODE, KT, 0>(a, s);
}
template <int RL>
hipError_t launch_persist_band_rl(const PersistLaunch& a, hipStream_t s) {
    if (a.unrolled) {
        switch (a.wmode) {
            case 0:
                if (a.add_only && a.twins) return launch_persist_band_inst<RL, 4, 36>(a, s);
                if (a.add_only) return launch_persist_band_inst<RL, 3, 36>(a, s);
                return launch_persist_band_inst<RL, 0, 36>(a, s);
            case 1: return launch_persist_band_inst<RL, 1, 36>(a, s);
            default: return launch_persist_band_inst<RL, 2, 36>(a, s);
        }
    }
    switch (a.wmode) {
        case 0:
            if (a.add_only) return launch_persist_band_inst<RL, 3, 0>(a, s);
            return launch_persist_band_inst<RL, 0, 0>(a, s);
        case 1: return launch_persist_band_inst<RL, 1, 0>(a, s);
        default: return launch_persist_band_inst<RL, 2, 0>(a, s);
    }
}
template <int RL, int WMODE, bool FULL>
hipError_t launch_persist_block_inst(const PersistLaunch& a, hipStream_t s) {
    const PersistShape p = persist_shape(a);
    hipLaunchKernelGGL((block_persist_kernel<RL, WMODE, FULL>), dim3(p.grid), dim3(256), 0, s, persist_args(a, p));
    return hipGetLastError();
}
template <int RL>
hipError_t launch_persist_block_rl(const PersistLaunch& a, hipStream_t s) {
    switch (a.wmode) {
        case 0: return a.full ? launch_persist_block_inst<RL, 0, true>(a, s) : launch_persist_block_inst<RL, 0, false>(a, s);
        case 1: return a.full ? launch_persist_block_inst<RL, 1, true>(a, s) : launch_persist_block_inst<RL, 1, false>(a, s);
        default: return a.full ? launch_persist_block_inst<RL, 2, true>(a, s) : launch_persist_block_inst<RL, 2, false>(a, s);
    }
}
}  // namespace

int persist_units(const PersistLaunch& a) { return persist_shape(a).total; }

hipError_t launch_persist(const PersistLaunch& a, hipStream_t s) {
    // host-side shape checks: what the kernels and the unit numbering assume
    if (a.N <= 0 || a.nblk <= 0 || a.nlayers < 1 || !a.table || !a.first_in || !a.buf_a || !a.buf_c || a.buf_a == a.buf_c ||
        !a.active || !a.done || a.done_stride < a.nblk || !a.ctl || !a.abort || !a.host_word || a.wait_limit < 0)
        return hipErrorInvalidValue;
    if (a.block_form) {
        if (a.ngroups <= 0) return hipErrorInvalidValue;
    } else if ((a.N % 256) != 0 || a.K < 4 || a.K > 32 || (a.K % 4) != 0) {
        return hipErrorInvalidValue;
    }
    if ((long long)a.nblk * persist_shape(a).nseg * a.nlayers > (long long)INT_MAX / 2) return hipErrorInvalidValue;
    switch (a.rl) {
        case 4: return a.block_form ? launch_persist_block_rl<4>(a, s) : launch_persist_band_rl<4>(a, s);
        case 2: return a.block_form ? launch_persist_block_rl<2>(a, s) : launch_persist_band_rl<2>(a, s);
        case 1: return a.block_form ? launch_persist_block_rl<1>(a, s) : launch_persist_band_rl<1>(a, s);
        default: return hipErrorInvalidValue;
    }
}

int resident_rows_per_workgroup(int N, int ngroups) {
    if (N <= 0 || ngroups <= 0) return 0;
    // (2 and 1 rows per workgroup - 8192 and 16384 neurons - run, but every workgroup then reads a layer's whole
    // index lists for very few rows: measured half as fast as the per-layer kernels, so they are not offered)
    for (int R : {16, 4})
        if ((long long)(N + 1) * R * 8 <= 136 * 1024 && (long long)ngroups * R <= 1024) return R;
    return 0;
}

template <int R>
static hipError_t launch_block_resident_r(const ResidentLaunch& a, hipStream_t s) {
    ResidentArgs k{};
    k.table = a.table; k.nlayers = a.nlayers; k.first_in = a.first_in; k.buf_a = a.buf_a; k.buf_c = a.buf_c; k.active = a.active;
    k.N = a.N; k.ngroups = a.ngroups; k.rl = a.rl; k.stamp0 = a.stamp0; k.prev_stamp = a.prev_stamp; k.check_dead = a.check_dead;
    k.bias = a.bias; k.clampv = a.clampv; k.pub = a.publish;
    const size_t lds = (size_t)(a.N + 1) * R * 8;
    dim3 grid((unsigned)(a.rows / R)), block((unsigned)((a.ngroups * R + 63) / 64 * 64));
#define SPDNN_RESIDENT(FULL)                                                                                              \
    do {                                                                                                                  \
        static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(block_resident_kernel<R, FULL>), \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, 136 * 1024);       \
        if (attr != hipSuccess) return attr;                                                                              \
        hipLaunchKernelGGL((block_resident_kernel<R, FULL>), grid, block, lds, s, k);                                     \
    } while (0)
    if (a.full) SPDNN_RESIDENT(true); else SPDNN_RESIDENT(false);
#undef SPDNN_RESIDENT
    return hipGetLastError();
}

hipError_t launch_block_resident(const ResidentLaunch& a, hipStream_t s) {
    // host-side shape checks: what the kernel's item numbering and its two LDS buffers assume
    if (a.N <= 0 || a.nlayers < 1 || !a.table || !a.first_in || !a.buf_a || !a.buf_c || a.buf_a == a.buf_c || !a.active ||
        a.ngroups <= 0 || a.rows <= 0 || (a.rl != 1 && a.rl != 2 && a.rl != 4) || (a.rows % (64 * a.rl)) != 0)
        return hipErrorInvalidValue;
    const int R = resident_rows_per_workgroup(a.N, a.ngroups);
    if (R == 0 || (64 * a.rl) % R != 0 || (long long)a.rows / R > 0x7fffffffll) return hipErrorInvalidValue;
    return R == 16 ? launch_block_resident_r<16>(a, s) : launch_block_resident_r<4>(a, s);
}

int rowtile_resident_rows(int N) {
    if (N <= 0) return 0;
    if (N <= 1024) return 16;   // two buffers of N x R floats: up to 128 KiB
    if (N <= 2048) return 8;
    if (N <= 4096) return 4;
    return 0;
}

template <int R>
static hipError_t launch_rowtile_resident_r(const ResidentLaunch& a, int wmode, hipStream_t s) {
    ResidentArgs k{};
    k.table = a.table; k.nlayers = a.nlayers; k.first_in = a.first_in; k.buf_a = a.buf_a; k.buf_c = a.buf_c; k.active = a.active;
    k.N = a.N; k.ngroups = 0; k.rl = a.rl; k.stamp0 = a.stamp0; k.prev_stamp = a.prev_stamp; k.check_dead = a.check_dead;
    k.bias = a.bias; k.clampv = a.clampv; k.pub = a.publish;
    const size_t lds = (size_t)a.N * R * 8;
    dim3 grid((unsigned)(a.rows / R)), block(1024);
#define SPDNN_RT_RESIDENT(WM)                                                                                               \
    do {                                                                                                                    \
        static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(rowtile_resident_kernel<R, WM>),   \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);        \
        if (attr != hipSuccess) return attr;                                                                                \
        hipLaunchKernelGGL((rowtile_resident_kernel<R, WM>), grid, block, lds, s, k);                                       \
    } while (0)
    if (wmode != 2) SPDNN_RT_RESIDENT(1); else SPDNN_RT_RESIDENT(2);
#undef SPDNN_RT_RESIDENT
    return hipGetLastError();
}

hipError_t launch_rowtile_resident(const ResidentLaunch& a, int wmode, hipStream_t s) {
    // host-side shape checks: what the kernel's two LDS buffers and its row numbering assume
    if (a.N <= 0 || a.nlayers < 1 || !a.table || !a.first_in || !a.buf_a || !a.buf_c || a.buf_a == a.buf_c || !a.active ||
        a.rows <= 0 || (a.rl != 1 && a.rl != 2 && a.rl != 4) || (a.rows % (64 * a.rl)) != 0)
        return hipErrorInvalidValue;
    const int R = rowtile_resident_rows(a.N);
    if (R == 0 || (64 * a.rl) % R != 0 || (size_t)a.N * R * 8 > 128 * 1024 || (long long)a.rows / R > 0x7fffffffll) return hipErrorInvalidValue;
    switch (R) {
        case 16: return launch_rowtile_resident_r<16>(a, wmode, s);
        case 8: return launch_rowtile_resident_r<8>(a, wmode, s);
        default: return launch_rowtile_resident_r<4>(a, wmode, s);
    }
}

int band_resident_rows(int N) {
    // N threads (a quad of band positions x four of the 16 rows each), two buffers of N x 16 floats
    return (N >= 256 && N <= 1024 && (N % 256) == 0) ? 16 : 0;
}

hipError_t launch_band_resident(const ResidentLaunch& a, int wmode, hipStream_t s) {
    // host-side shape checks: what the kernel's two LDS buffers, its thread numbering and its plan stream assume
    if (a.nlayers < 1 || !a.quad_col || !a.quad_w || !a.quad_dst || (a.quad_stride % 16) != 0 || !a.first_in || !a.buf_a || !a.buf_c ||
        a.buf_a == a.buf_c || !a.active || a.rows <= 0 || (a.rl != 1 && a.rl != 2 && a.rl != 4) || (a.rows % (64 * a.rl)) != 0 ||
        band_resident_rows(a.N) != 16 || a.ngroups < 1 || a.ngroups > 9)
        return hipErrorInvalidValue;
    ResidentArgs k{};
    k.table = a.table; k.nlayers = a.nlayers; k.first_in = a.first_in; k.buf_a = a.buf_a; k.buf_c = a.buf_c; k.active = a.active;
    k.N = a.N; k.ngroups = a.ngroups; k.rl = a.rl; k.stamp0 = a.stamp0; k.prev_stamp = a.prev_stamp; k.check_dead = a.check_dead;
    k.bias = a.bias; k.clampv = a.clampv; k.pub = a.publish;
    k.quad_col = a.quad_col; k.quad_w = a.quad_w; k.quad_dst = a.quad_dst; k.quad_stride = a.quad_stride;
    const size_t lds = (size_t)a.N * 16 * 8 + (size_t)(a.N / 64) * 1024;   // two row buffers, then a KiB per wave for the weights
    dim3 grid((unsigned)(a.rows / 16)), block((unsigned)a.N);
#define SPDNN_BAND_RESIDENT(NG, WM)                                                                                         \
    do {                                                                                                                    \
        static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(band_resident_kernel<NG, WM>),     \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, 144 * 1024);        \
        if (attr != hipSuccess) return attr;                                                                                \
        hipLaunchKernelGGL((band_resident_kernel<NG, WM>), grid, block, lds, s, k);                                         \
    } while (0)
    if (wmode != 2) {
        if (a.ngroups == 9) SPDNN_BAND_RESIDENT(9, 1); else SPDNN_BAND_RESIDENT(0, 1);
    } else {
        if (a.ngroups == 9) SPDNN_BAND_RESIDENT(9, 2); else SPDNN_BAND_RESIDENT(0, 2);
    }
#undef SPDNN_BAND_RESIDENT
    return hipGetLastError();
}

int count_stamp_partial_words() { return kCountTicket + 1; }

hipError_t launch_count_stamp_range(const int32_t* stamps, int rows, int stamp_lo, int n, int32_t* counts_dev,
                                    int32_t* counts_host, int32_t* partial, hipStream_t s) {
    if (!stamps || rows <= 0 || n < 1 || n > kCountTicket || (!counts_dev && !counts_host)) return hipErrorInvalidValue;
    // a workgroup per 4096 rows, 32 at most; a single one without the partial sums' buffer
    const int nwg = partial ? std::max(1, std::min(32, rows / 4096)) : 1;
    hipLaunchKernelGGL(count_stamp_range_kernel, dim3((unsigned)nwg), dim3(1024), (size_t)n * 4, s, stamps, rows, stamp_lo, n,
                       counts_dev, counts_host, partial);
    return hipGetLastError();
}

int band_pair_seglen(int N, int nblk, int n_cu) {
    // one workgroup per CU (128 KiB of LDS); a segment of c chunks costs c + 3 steps
    const int slots = n_cu > 0 ? n_cu : 256;
    const int nchunks = N / 16;
    int best_len = N;
    double best = -1.0;
    for (int nseg = 1; nseg <= nchunks / 8 && nseg <= 65535; ++nseg) {
        const int cps = (nchunks + nseg - 1) / nseg;
        if ((nchunks + cps - 1) / cps != nseg) continue;
        const long long wgs = (long long)nblk * nseg;
        const long long rounds = (wgs + slots - 1) / slots;
        const double score = (double)wgs / (double)(rounds * slots) * (double)cps / (double)(cps + 3);
        if (score > best + 1e-9) { best = score; best_len = cps * 16; }
    }
    return best_len;
}

hipError_t launch_band_pair(const PairLaunch& a, hipStream_t s) {
    if (a.N < 256 || (a.N % 256) != 0 || a.nblk <= 0 || a.rl != 4 || !a.yin || !a.yout || !a.pairs_a || !a.pairs_b ||
        !a.dst || !a.active || !a.active_mid || a.halo_a < 0 || a.halo_a > 32 || a.halo_b < 0 || a.halo_b > 32 ||
        a.steps_a < 32 || a.steps_a > 36 || a.steps_b < 32 || a.steps_b > 36 || (a.wmode != 0 && (!a.pw_a || !a.pw_b)))
        return hipErrorInvalidValue;
    int seglen = a.seglen > 0 ? a.seglen - a.seglen % 16 : 0;
    if (seglen <= 0) seglen = band_pair_seglen(a.N, a.nblk, a.n_cu);
    const int nseg = (a.N + seglen - 1) / seglen;
    if (nseg > 65535) return hipErrorInvalidValue;
    constexpr size_t lds = 128 * 1024;
    PairSide A{a.wu_a, a.halo_a, a.steps_a}, B{a.wu_b, a.halo_b, a.steps_b};
    const int stream = (long long)a.nblk * (long long)a.N * 1024 * 2 >= a.stream_min_bytes ? 1 : 0;
    dim3 grid(a.nblk, nseg), block(1024);
#define SPDNN_PAIR(WM)                                                                                              \
    do {                                                                                                            \
        static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(band_pair_kernel<WM>),     \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);  \
        if (attr != hipSuccess) return attr;                                                                        \
        hipLaunchKernelGGL(band_pair_kernel<WM>, grid, block, lds, s, a.yin, a.yout, a.pairs_a, a.pw_a, a.pairs_b,  \
                           a.pw_b, A, B, a.dst, a.active,                                                           \
                           a.active_mid, a.count_prev, a.N, seglen, a.stamp_a, a.stamp_b, a.prev_stamp, a.check_dead, \
                           a.bias, a.clampv, a.publish, a.nblk, stream);                                            \
    } while (0)
    switch (a.wmode) {
        case 0: if (a.add_only) SPDNN_PAIR(3); else SPDNN_PAIR(0); break;
        case 1: SPDNN_PAIR(1); break;
        default: SPDNN_PAIR(2); break;
    }
#undef SPDNN_PAIR
    return hipGetLastError();
}

hipError_t launch_count_stamped(const int32_t* stamps, int rows, int stamp, int32_t* count_out, hipStream_t s) {
    if (rows <= 0 || !stamps || !count_out) return hipErrorInvalidValue;
    hipLaunchKernelGGL(count_stamped_kernel, dim3((rows + 255) / 256), dim3(256), 0, s, stamps, rows, stamp, count_out);
    return hipGetLastError();
}

hipError_t launch_gather(const GatherLaunch& a, hipStream_t s) {
    // (kmax: the rows' stride in cols and wv, a multiple of four - the kernel takes four entries per trip)
    if (a.N <= 0 || a.kmax < 0 || (a.kmax % 4) != 0 || a.nblk <= 0 || !a.yin || !a.yout || !a.cols || !a.rowlen || !a.wv ||
        !a.dst || !a.active)
        return hipErrorInvalidValue;
    const int opg = 8;
    dim3 grid(a.nblk, (a.N + 4 * opg - 1) / (4 * opg)), block(256);
    if (grid.y > 65535) return hipErrorInvalidValue;
#define SPDNN_GATHER(RLv, WM)                                                                         \
    hipLaunchKernelGGL((gather_kernel<RLv, WM>), grid, block, 0, s, a.yin, a.yout, a.cols, a.rowlen,  \
                       a.wv, a.dst, a.active, a.count_prev, a.N, a.kmax, opg, a.stamp, a.prev_stamp, a.check_dead, a.bias, a.clampv, \
                       a.publish)
    const bool exact = a.wmode != 2;
    switch (a.rl) {
        case 4: if (exact) SPDNN_GATHER(4, 1); else SPDNN_GATHER(4, 2); break;
        case 2: if (exact) SPDNN_GATHER(2, 1); else SPDNN_GATHER(2, 2); break;
        case 1: if (exact) SPDNN_GATHER(1, 1); else SPDNN_GATHER(1, 2); break;
        default: return hipErrorInvalidValue;
    }
#undef SPDNN_GATHER
    return hipGetLastError();
}

hipError_t launch_tiled(const TiledLaunch& a, hipStream_t s) {
    if (a.N <= 0 || a.ntiles <= 0 || a.ntiles > 65535 || a.nblk <= 0 || a.rl < 1 || a.rl > 4 || !a.yin || !a.yout ||
        !a.cols || !a.hdr || !a.ent || !a.dst || !a.active)
        return hipErrorInvalidValue;
    constexpr size_t lds = 512 * 256 + 16 * 2048;   // one panel and the waves' entry rings: all 160 KiB of a CU
    if ((long long)a.nblk * a.rl * a.ntiles > 0x7fffffffll) return hipErrorInvalidValue;
    dim3 grid((unsigned)(a.nblk * a.rl * a.ntiles)), block(1024);
#define SPDNN_TILED(WM)                                                                                          \
    do {                                                                                                         \
        static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(tiled_kernel<WM>),      \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
        if (attr != hipSuccess) return attr;                                                                     \
        hipLaunchKernelGGL((tiled_kernel<WM>), grid, block, lds, s, a.yin, a.yout, a.cols, a.hdr, a.ent, a.dst,  \
                           a.active, a.count_prev, a.N, a.ntiles, a.rl, a.stamp, a.prev_stamp, a.check_dead,     \
                           a.bias, a.clampv, a.publish);                                                         \
    } while (0)
    if (a.wmode != 2) SPDNN_TILED(1); else SPDNN_TILED(2);
#undef SPDNN_TILED
    return hipGetLastError();
}

int rowtile_rows_per_workgroup(int N) {
    if (N <= 0) return 0;
    if (N <= 2048) return 16;   // N x 64 bytes of LDS: up to 128 KiB
    if (N <= 4096) return 8;
    if (N <= 8192) return 4;
    return 0;
}

template <int R>
static hipError_t launch_rowtile_r(const RowtileLaunch& a, hipStream_t s) {
    RowtileArgs k{};
    k.yin = a.yin; k.yout = a.yout; k.ent = a.ent; k.len = a.len; k.dst = a.dst; k.active = a.active; k.count_prev = a.count_prev;
    k.N = a.N; k.kmax = a.kpad; k.rl = a.rl; k.stamp = a.stamp; k.prev_stamp = a.prev_stamp; k.check_dead = a.check_dead;
    k.bias = a.bias; k.clampv = a.clampv; k.pub = a.publish;
    const size_t lds = (size_t)a.N * R * 4;
    dim3 grid((unsigned)(a.rows / R)), block(1024);
#define SPDNN_ROWTILE(WM, PAIRS)                                                                                        \
    do {                                                                                                                \
        static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(rowtile_kernel<R, WM, PAIRS>), \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);    \
        if (attr != hipSuccess) return attr;                                                                            \
        hipLaunchKernelGGL((rowtile_kernel<R, WM, PAIRS>), grid, block, lds, s, k);                                     \
    } while (0)
    // two entries per step where a CU holds one workgroup anyway (more than half of its LDS)
    if (R == 16 && lds <= 80 * 1024) {
        if (a.wmode != 2) SPDNN_ROWTILE(1, false); else SPDNN_ROWTILE(2, false);
    } else {
        if (a.wmode != 2) SPDNN_ROWTILE(1, true); else SPDNN_ROWTILE(2, true);
    }
#undef SPDNN_ROWTILE
    return hipGetLastError();
}

hipError_t launch_rowtile(const RowtileLaunch& a, hipStream_t s) {
    // host-side shape checks: what the kernel's LDS buffer and its row numbering assume
    if (a.N <= 0 || a.kpad < 1 || !a.yin || !a.yout || !a.ent || !a.len || !a.dst || !a.active || a.rows <= 0 ||
        (a.rl != 1 && a.rl != 2 && a.rl != 4) || (a.rows % (64 * a.rl)) != 0)
        return hipErrorInvalidValue;
    const int R = rowtile_rows_per_workgroup(a.N);
    if (R == 0 || (64 * a.rl) % R != 0 || (size_t)a.N * R * 4 > 128 * 1024) return hipErrorInvalidValue;
    switch (R) {
        case 16: return launch_rowtile_r<16>(a, s);
        case 8: return launch_rowtile_r<8>(a, s);
        default: return launch_rowtile_r<4>(a, s);
    }
}

hipError_t launch_block(const BlockLaunch& a, hipStream_t s) {
    if (a.N <= 0 || a.ngroups <= 0 || a.nblk <= 0 || !a.yin || !a.yout || !a.cols || !a.cnt || !a.dst ||
        !a.active || (a.wmode != 0 && !a.wv))
        return hipErrorInvalidValue;
    // groups per wave: enough workgroups to fill the chip several times over, but long enough
    // runs per wave to amortise the launch
    int gpw = 8;
    while (gpw > 1 && (long long)a.nblk * ((a.ngroups + 4 * gpw - 1) / (4 * gpw)) < 2048) gpw >>= 1;
    dim3 grid(a.nblk, (a.ngroups + 4 * gpw - 1) / (4 * gpw)), block(256);
    if (grid.y > 65535) return hipErrorInvalidValue;
#define SPDNN_BLOCK(RLv, WM, FL)                                                                          \
    hipLaunchKernelGGL((block_kernel<RLv, WM, FL>), grid, block, 0, s, a.yin, a.yout, a.cols, a.cnt, a.wv, \
                       a.dst, a.active, a.count_prev, a.N, a.ngroups, gpw, a.stamp, a.prev_stamp, a.check_dead, a.wu, \
                       a.bias, a.clampv, a.publish, a.frontier, a.frontier_layer)
#define SPDNN_BLOCK_WM(RLv)                                                                 \
    switch (a.wmode) {                                                                      \
        case 0: if (a.full) SPDNN_BLOCK(RLv, 0, true); else SPDNN_BLOCK(RLv, 0, false); break; \
        case 1: if (a.full) SPDNN_BLOCK(RLv, 1, true); else SPDNN_BLOCK(RLv, 1, false); break; \
        default: if (a.full) SPDNN_BLOCK(RLv, 2, true); else SPDNN_BLOCK(RLv, 2, false); break; \
    }
    switch (a.rl) {
        case 4: SPDNN_BLOCK_WM(4); break;
        case 2: SPDNN_BLOCK_WM(2); break;
        case 1: SPDNN_BLOCK_WM(1); break;
        default: return hipErrorInvalidValue;
    }
#undef SPDNN_BLOCK_WM
#undef SPDNN_BLOCK
    return hipGetLastError();
}

hipError_t launch_scan_active(const int32_t* active, const int32_t* gid, int rows, int stamp, int32_t* count,
                              int32_t* alive_src, int32_t* alive_gid, hipStream_t s) {
    if (rows < 0 || !active || !gid || !count || !alive_src || !alive_gid) return hipErrorInvalidValue;
    hipLaunchKernelGGL(scan_active_kernel, dim3(std::max(1, (rows + 1023) / 1024)), dim3(1024), 0, s, active, gid, rows,
                       stamp, count, alive_src, alive_gid);
    return hipGetLastError();
}

hipError_t launch_repack(const Feat& src, const Feat& dst, const int32_t* count, const int32_t* alive_src,
                         const int32_t* alive_gid, int32_t* gid_out, int N, int rl, int dst_blocks,
                         hipStream_t s) {
    if (dst_blocks <= 0 || dst_blocks > 65535 || N <= 0) return hipErrorInvalidValue;
    // 64 columns per workgroup where that still makes a couple of thousand workgroups, fewer columns where few row
    // blocks survive (N=1024, 8 blocks: 128 workgroups of 64 columns took 55 us)
    int cpw = 64;
    while (cpw > 8 && (long long)((N + cpw - 1) / cpw) * dst_blocks < 2048) cpw /= 2;
    dim3 grid((N + cpw - 1) / cpw, dst_blocks);
    switch (rl) {
        case 4: hipLaunchKernelGGL(repack_kernel<4>, grid, dim3(256), 0, s, src, dst, count, alive_src, alive_gid, gid_out, N, cpw); break;
        case 2: hipLaunchKernelGGL(repack_kernel<2>, grid, dim3(128), 0, s, src, dst, count, alive_src, alive_gid, gid_out, N, cpw); break;
        case 1: hipLaunchKernelGGL(repack_kernel<1>, grid, dim3(64), 0, s, src, dst, count, alive_src, alive_gid, gid_out, N, cpw); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_synth_features(const Feat& y, const int32_t* col_of_phys, int N, int batch, int nblk, int rl,
                                 uint64_t seed, float dmin, float dmax, hipStream_t s) {
    if (nblk <= 0 || nblk > 65535 || N <= 0) return hipErrorInvalidValue;
    // host side of the generator definition: keys and the density range as 32.32 fixed point
    auto h = [](uint64_t x) {
        uint64_t z = x + 0x9E3779B97F4A7C15ULL;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
        return z ^ (z >> 31);
    };
    const uint64_t kf = h(seed ^ 0x46454154ULL);
    const uint64_t lo = (uint64_t)((double)dmin * 4294967296.0);
    const uint64_t span = (uint64_t)(((double)dmax - (double)dmin) * 4294967296.0);
    const int cpw = 64;
    dim3 grid((N + cpw - 1) / cpw, nblk);
    switch (rl) {
        case 4: hipLaunchKernelGGL(synth_features_kernel<4>, grid, dim3(256), 0, s, y, col_of_phys, N, batch, cpw, kf, lo, span); break;
        case 2: hipLaunchKernelGGL(synth_features_kernel<2>, grid, dim3(128), 0, s, y, col_of_phys, N, batch, cpw, kf, lo, span); break;
        case 1: hipLaunchKernelGGL(synth_features_kernel<1>, grid, dim3(64), 0, s, y, col_of_phys, N, batch, cpw, kf, lo, span); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_pack_rows(const float* rowmajor, const Feat& y, const int32_t* phys_of_col, int N, int64_t row0,
                            int nrows, int rl, int32_t* nonfinite, hipStream_t s) {
    const int RB = 64 * rl;
    if (nrows <= 0 || N <= 0 || (row0 % RB) != 0) return hipErrorInvalidValue;
    const int nb = (nrows + RB - 1) / RB;
    if (nb > 65535) return hipErrorInvalidValue;
    dim3 grid((N + 31) / 32, nb);
    switch (rl) {
        case 4: hipLaunchKernelGGL(pack_rows_kernel<4>, grid, dim3(256), 0, s, rowmajor, y, phys_of_col, N, (long long)row0, nrows, nonfinite); break;
        case 2: hipLaunchKernelGGL(pack_rows_kernel<2>, grid, dim3(256), 0, s, rowmajor, y, phys_of_col, N, (long long)row0, nrows, nonfinite); break;
        case 1: hipLaunchKernelGGL(pack_rows_kernel<1>, grid, dim3(256), 0, s, rowmajor, y, phys_of_col, N, (long long)row0, nrows, nonfinite); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_unpack_rows(const Feat& y, const int32_t* phys_of_col, const int32_t* phys_rows, int nreq,
                              int N, int rl, const int32_t* active, int stamp, float* rowmajor, hipStream_t s) {
    if (nreq <= 0 || nreq > 65535 || N <= 0) return hipErrorInvalidValue;
    dim3 grid((N + 255) / 256, nreq);
    hipLaunchKernelGGL(unpack_rows_kernel, grid, dim3(256), 0, s, y, phys_of_col, phys_rows, N, 64 * rl, active,
                       stamp, rowmajor);
    return hipGetLastError();
}

hipError_t launch_row_table(const int32_t* gid, int carried, int batch, int32_t* where, hipStream_t s) {
    if (batch <= 0 || carried < 0 || !where || (carried > 0 && !gid)) return hipErrorInvalidValue;
    hipLaunchKernelGGL(fill_i32_kernel, dim3((batch + 255) / 256), dim3(256), 0, s, where, batch, -1);
    if (carried > 0)
        hipLaunchKernelGGL(scatter_where_kernel, dim3((carried + 255) / 256), dim3(256), 0, s, gid, carried, batch, where);
    return hipGetLastError();
}

hipError_t launch_lookup_rows(const int32_t* ids, int n, const int32_t* where, int32_t* phys, hipStream_t s) {
    if (n <= 0 || !ids || !where || !phys) return hipErrorInvalidValue;
    hipLaunchKernelGGL(lookup_rows_kernel, dim3((n + 255) / 256), dim3(256), 0, s, ids, n, where, phys);
    return hipGetLastError();
}

hipError_t launch_iota_gid(int32_t* gid, int rows, int batch, hipStream_t s) {
    if (rows <= 0) return hipSuccess;
    hipLaunchKernelGGL(iota_gid_kernel, dim3((rows + 255) / 256), dim3(256), 0, s, gid, rows, batch);
    return hipGetLastError();
}

hipError_t launch_zero_pair(float* p, float* q, int64_t n_floats_each, hipStream_t s) {
    if (n_floats_each <= 0 || (n_floats_each % 4) != 0 || !p || !q) return hipErrorInvalidValue;
    hipLaunchKernelGGL(zero_pair_kernel, dim3(65536), dim3(256), 0, s, reinterpret_cast<float4*>(p),
                       reinterpret_cast<float4*>(q), (long long)(n_floats_each / 4));
    return hipGetLastError();
}

hipError_t launch_copy_pair(const Feat& src, const Feat& dst, int64_t n_floats_each, hipStream_t s) {
    if (n_floats_each <= 0 || (n_floats_each % 4) != 0 || !src || !dst || !src.half[1] || !dst.half[1])
        return hipErrorInvalidValue;
    hipLaunchKernelGGL(copy_pair_kernel, dim3(65536), dim3(256), 0, s, reinterpret_cast<const stream_f4*>(src.half[0]),
                       reinterpret_cast<stream_f4*>(dst.half[0]), reinterpret_cast<const stream_f4*>(src.half[1]),
                       reinterpret_cast<stream_f4*>(dst.half[1]), (long long)(n_floats_each / 4));
    return hipGetLastError();
}

hipError_t launch_copy_f4(const float* src, float* dst, int64_t n_floats, hipStream_t s) {
    if (n_floats <= 0 || (n_floats % 4) != 0) return hipErrorInvalidValue;
    hipLaunchKernelGGL(copy_f4_kernel, dim3(65536), dim3(256), 0, s, reinterpret_cast<const float4*>(src),
                       reinterpret_cast<float4*>(dst), (long long)(n_floats / 4));
    return hipGetLastError();
}

}  // namespace spdnn
