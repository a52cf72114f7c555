// Measurement aids of bench.py, built into their own library (libmi355_bench_probes.so). Nothing here is a product path and the
// product library does not contain or load any of it: these kernels tell what the machine sustains - a read-only stream in the
// shapes the decode kernels use, and a register-only matrix-core loop - so that the product kernels can be priced against it.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) uint8_t lds_u8;
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr uint32_t kStage = 9216;      // bytes per stage: what one wave of the decode sweeps moves per step (64 rows x 144 bytes)

__device__ __forceinline__ void copy16(const void* src, uint32_t lds_at) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_at), "v"(src) : "memory", "m0");
}
template <int N> __device__ __forceinline__ void wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory"); }

// A one-wave workgroup streams `stages` stages of 9,216 bytes.
//  MODE 0: global_load_dwordx4 into registers, contiguous (lane l reads 16 bytes at 1024 i + 16 l of the stage), DEPTH stages requested ahead.
//  MODE 1: global_load_lds_dwordx4 into a ring of DEPTH LDS slots, contiguous; every lane reads its 144 bytes of a landed slot back.
//  MODE 2: as 1, but a stage is one 144-byte block of each of 64 rows that lie row_bytes apart (the Q4_K super-block sweep:
//          piece j of the stage is piece j % 9 of row j / 9), stage b = block b of the rows.
// sink receives one word per wave (the xor of everything read), so nothing is optimised away.
template <int MODE, int DEPTH>
__global__ __launch_bounds__(64) void read_stream_kernel(const uint8_t* src, uint64_t wave_bytes, uint32_t stages, uint32_t row_bytes, uint32_t* sink) {
    __shared__ __attribute__((aligned(16))) uint8_t ring[MODE == 0 ? 16 : DEPTH * kStage];
    const uint32_t lane = threadIdx.x;
    const uint8_t* base = src + static_cast<uint64_t>(blockIdx.x) * wave_bytes;
    u32x4 acc = {0U, 0U, 0U, 0U};
    if constexpr (MODE == 0) {
        u32x4 v[DEPTH][9];
#pragma unroll
        for (int d = 0; d < DEPTH - 1; ++d)
            if (static_cast<uint32_t>(d) < stages)
#pragma unroll
                for (int i = 0; i < 9; ++i) v[d][i] = *reinterpret_cast<const u32x4*>(base + static_cast<uint64_t>(d) * kStage + 1024U * i + 16U * lane);
        for (uint32_t s0 = 0; s0 < stages; s0 += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) {
                const uint32_t s = s0 + d, ahead = s + DEPTH - 1U;
                if (s < stages) {
                    if (ahead < stages)
#pragma unroll
                        for (int i = 0; i < 9; ++i)
                            v[(d + DEPTH - 1) % DEPTH][i] = *reinterpret_cast<const u32x4*>(base + static_cast<uint64_t>(ahead) * kStage + 1024U * i + 16U * lane);
#pragma unroll
                    for (int i = 0; i < 9; ++i) acc ^= v[d][i];
                }
            }
        }
    } else {
        const uint32_t ring_at = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_u8*)ring));
        const uint8_t* piece[9];
#pragma unroll
        for (uint32_t i = 0; i < 9U; ++i) {
            const uint32_t j = i * 64U + lane;
            if constexpr (MODE == 1) piece[i] = base + 16U * j;
            else { const uint32_t r = j / 9U, c = j - 9U * r; piece[i] = base + static_cast<uint64_t>(r) * row_bytes + 16U * c; }
        }
        const uint32_t step = MODE == 1 ? kStage : 144U;
        auto start = [&](uint32_t slot) {
#pragma unroll
            for (uint32_t i = 0; i < 9U; ++i) { copy16(piece[i], ring_at + slot * kStage + 1024U * i); piece[i] += step; }
        };
#pragma unroll
        for (int d = 0; d < DEPTH - 1; ++d)
            if (static_cast<uint32_t>(d) < stages) start(d);
        for (uint32_t s0 = 0; s0 < stages; s0 += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) {
                const uint32_t s = s0 + d;
                if (s < stages) {
                    const uint32_t last = s + DEPTH - 1U < stages ? s + DEPTH - 1U : stages, ahead = last - 1U - s;
                    if (ahead == 0) wait_vm<0>();
                    else if (ahead == 1) wait_vm<9>();
                    else if (ahead == 2) wait_vm<18>();
                    else wait_vm<27>();
                    if (s + DEPTH - 1U < stages) start((d + DEPTH - 1) % DEPTH);
                    const u32x4* mine = reinterpret_cast<const u32x4*>(ring + d * kStage + lane * 144U);
#pragma unroll
                    for (int i = 0; i < 9; ++i) acc ^= mine[i];
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");       // the slot is read before a later copy may land in it
                }
            }
        }
    }
    uint32_t x = acc.x ^ acc.y ^ acc.z ^ acc.w;
    for (int d = 32; d; d >>= 1) x ^= __shfl_xor(x, d);
    if (lane == 0) sink[blockIdx.x] = x;
}

// Every wave of a 512-thread workgroup (two waves per SIMD) runs iterations x 4 independent v_mfma_f32_32x32x16_f16 on operands that
// stay in registers. random_operands != 0 fills them with pseudo-random halves (weights in the range of the prefill's sc * q
// operands): the sustained rate then falls with the switching power, which is the ceiling a real product has.
__global__ __launch_bounds__(512) void mfma_f16_kernel(uint32_t iterations, uint32_t random_operands, float* sink) {
    floatx16 acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[i][j] = 0.0F;
    half8 a, b;
    uint32_t state = (threadIdx.x + blockIdx.x * 977U) * 2654435761U;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        state = state * 1664525U + 1013904223U;
        a[j] = random_operands ? static_cast<_Float16>(static_cast<float>(state >> 22)) : static_cast<_Float16>(1.0F);
        state = state * 1664525U + 1013904223U;
        b[j] = random_operands ? static_cast<_Float16>((static_cast<float>(state >> 16) - 32768.0F) * (1.0F / 8192.0F)) : static_cast<_Float16>(1.0F);
    }
    for (uint32_t it = 0; it < iterations; ++it) {
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i], 0, 0, 0);
        asm volatile("" : "+v"(a), "+v"(b));                  // the operands stay what they are; the loop is not folded
    }
    float s = 0.0F;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) s += acc[i][j];
    sink[blockIdx.x * 512U + threadIdx.x] = s;
}

template <int MODE>
int32_t launch_read(int depth, uint32_t waves, const uint8_t* src, uint64_t wave_bytes, uint32_t stages, uint32_t row_bytes, uint32_t* sink, hipStream_t st) {
    switch (depth) {
    case 2: read_stream_kernel<MODE, 2><<<waves, 64, 0, st>>>(src, wave_bytes, stages, row_bytes, sink); break;
    case 3: read_stream_kernel<MODE, 3><<<waves, 64, 0, st>>>(src, wave_bytes, stages, row_bytes, sink); break;
    case 4: read_stream_kernel<MODE, 4><<<waves, 64, 0, st>>>(src, wave_bytes, stages, row_bytes, sink); break;
    default: return -1;
    }
    return hipGetLastError() == hipSuccess ? 0 : -3;
}

}  // namespace

extern "C" {

// src: waves x stages x 9,216 bytes, 16-byte aligned (mode 2: every wave owns 64 rows of `stages` 144-byte blocks, back to back).
// sink: one word per wave. Returns 0, -1 (arguments) or -3 (launch).
int32_t bench_probe_read_stream(const void* src, uint32_t waves, uint32_t stages, uint32_t mode, uint32_t depth, uint32_t* sink, void* stream) {
    if (!src || !sink || waves == 0 || stages == 0 || mode > 2U || (reinterpret_cast<uintptr_t>(src) & 15U)) return -1;
    const uint64_t wave_bytes = static_cast<uint64_t>(stages) * kStage;
    const uint8_t* s = static_cast<const uint8_t*>(src);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (mode == 0) return launch_read<0>(static_cast<int>(depth), waves, s, wave_bytes, stages, 0U, sink, st);
    if (mode == 1) return launch_read<1>(static_cast<int>(depth), waves, s, wave_bytes, stages, 0U, sink, st);
    return launch_read<2>(static_cast<int>(depth), waves, s, wave_bytes, stages, stages * 144U, sink, st);
}

// sink: at least 512 floats per compute unit; *flops = the launch's matrix-core FLOPs.
int32_t bench_probe_mfma_f16(uint32_t iterations, uint32_t random_operands, float* sink, uint64_t sink_floats, uint64_t* flops, void* stream) {
    int device = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&device) != hipSuccess || hipGetDeviceProperties(&prop, device) != hipSuccess) return -3;
    const uint32_t blocks = static_cast<uint32_t>(prop.multiProcessorCount);
    if (!sink || !flops || sink_floats < 512ULL * blocks || iterations == 0) return -1;
    mfma_f16_kernel<<<blocks, 512, 0, static_cast<hipStream_t>(stream)>>>(iterations, random_operands, sink);
    if (hipGetLastError() != hipSuccess) return -3;
    *flops = 2ULL * 32U * 32U * 16U * 4U * iterations * 8ULL * blocks;
    return 0;
}

}  // extern "C"
