// Instruction-rate probes for gfx950: what one wave64 vector instruction costs a SIMD, alone, beside another kind, in a
// dependent chain, and beside a running int8 MFMA.  These are the figures the forward kernels' vector-pipe bound is priced
// with.  Stand-alone program (no library code): built by `python -m int_flashattention_amd.build` into ./bench_rate_probe,
// run as `./bench_rate_probe` on the GPU; prints one table per question, a few seconds in all.
//
// Method: single-wave workgroups whose LDS allocation fixes how many of them share a SIMD (36 KiB -> 4 per CU = 1 wave per
// SIMD, 18 KiB -> 2, 9.5 KiB -> 4); the grid fills the chip exactly once; every lane runs `iters` trips of a loop body of
// 64 inline-assembly instructions (8 groups of 8, an optional MFMA in front of each group) on `NCH` registers in rotation
// (16 = independent neighbours, 1 = every instruction depends on the one before).  Reported: launch time by HIP events /
// (trips x instructions one SIMD executed) = SIMD time per instruction, in ns.
#include <hip/hip_runtime.h>
#include <cstdio>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

enum Kind { ADD, MUL, FMA, MOV, SUB_INLINE, ADD_SGPR, CVT_I32, MAX3, MAX, CVT_PK_U8, CVT_PK_F16, PK_MUL_F16, PK_ADD_F16,
            CVT_U16_SDWA, DOT2, PERM, FMA_MIX, LDEXP, XOR, LSHL, EXP, RCP, FMA_F16, NKIND };
static const char* kind_name[NKIND] = {"v_add_f32", "v_mul_f32", "v_fma_f32", "v_mov_b32", "v_sub_f32 (inline constant)",
    "v_add_f32 (SGPR operand)", "v_cvt_f32_i32", "v_max3_f32", "v_max_f32", "v_cvt_pk_u8_f32", "v_cvt_pk_f16_f32", "v_pk_mul_f16",
    "v_pk_add_f16", "v_cvt_u16_f16 (SDWA byte write)", "v_dot2_f32_f16", "v_perm_b32", "v_fma_mix_f32", "v_ldexp_f32", "v_xor_b32",
    "v_lshlrev_b32", "v_exp_f32", "v_rcp_f32", "v_fma_f16"};

template <int K> __device__ __forceinline__ void emit(float& x, float a, float b) {
    if (K == ADD) asm volatile("v_add_f32 %0, %0, %1" : "+v"(x) : "v"(a), "v"(b));
    if (K == MUL) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x) : "v"(a), "v"(b));
    if (K == FMA) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x) : "v"(a), "v"(b));
    if (K == MOV) asm volatile("v_mov_b32 %0, %1" : "+v"(x) : "v"(a), "v"(b));
    if (K == SUB_INLINE) asm volatile("v_sub_f32 %0, 0.15915494, %0" : "+v"(x) : "v"(a), "v"(b));
    if (K == ADD_SGPR) asm volatile("v_add_f32 %0, s4, %0" : "+v"(x) : "v"(a), "v"(b) : "s4");
    if (K == CVT_I32) asm volatile("v_cvt_f32_i32 %0, %0" : "+v"(x) : "v"(a), "v"(b));
    if (K == MAX3) asm volatile("v_max3_f32 %0, %0, %1, %2" : "+v"(x) : "v"(a), "v"(b));
    if (K == MAX) asm volatile("v_max_f32 %0, %0, %1" : "+v"(x) : "v"(a), "v"(b));
    if (K == CVT_PK_U8) asm volatile("v_cvt_pk_u8_f32 %0, %1, 1, %0" : "+v"(x) : "v"(a), "v"(b));
    if (K == CVT_PK_F16) asm volatile("v_cvt_pk_f16_f32 %0, %0, %1" : "+v"(x) : "v"(a), "v"(b));
    if (K == PK_MUL_F16) asm volatile("v_pk_mul_f16 %0, %0, %1" : "+v"(x) : "v"(a), "v"(b));
    if (K == PK_ADD_F16) asm volatile("v_pk_add_f16 %0, %0, %1" : "+v"(x) : "v"(a), "v"(b));
    if (K == CVT_U16_SDWA) asm volatile("v_cvt_u16_f16_sdwa %0, %1 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_1" : "+v"(x) : "v"(a), "v"(b));
    if (K == DOT2) asm volatile("v_dot2_f32_f16 %0, %1, %2, %0" : "+v"(x) : "v"(a), "v"(b));
    if (K == PERM) asm volatile("v_perm_b32 %0, %0, %1, %2" : "+v"(x) : "v"(a), "v"(b));
    if (K == FMA_MIX) asm volatile("v_fma_mix_f32 %0, %0, %1, %2" : "+v"(x) : "v"(a), "v"(b));
    if (K == LDEXP) asm volatile("v_ldexp_f32 %0, %0, %1" : "+v"(x) : "v"(a), "v"(b));
    if (K == XOR) asm volatile("v_xor_b32 %0, %0, %1" : "+v"(x) : "v"(a), "v"(b));
    if (K == LSHL) asm volatile("v_lshlrev_b32 %0, 1, %0" : "+v"(x) : "v"(a), "v"(b));
    if (K == EXP) asm volatile("v_exp_f32 %0, %0" : "+v"(x) : "v"(a), "v"(b));
    if (K == RCP) asm volatile("v_rcp_f32 %0, %0" : "+v"(x) : "v"(a), "v"(b));
    if (K == FMA_F16) asm volatile("v_fma_f16 %0, %0, %1, %2" : "+v"(x) : "v"(a), "v"(b));
}

// Loop body: 8 x [optional MFMA, NV instructions alternating between kinds KA and KB] on NCH registers in rotation.
template <int KA, int KB, int MF, int NV, int NCH, int LDSB>
__global__ void __launch_bounds__(64) probe(float* out, int iters) {
    __shared__ char pad[LDSB];
    pad[threadIdx.x] = 0;
    v4i fa = (v4i){(int)threadIdx.x, 1, 2, 3}, fb = (v4i){7, (int)threadIdx.x, 5, 6};
    v16i acc[4];
    for (int j = 0; j < 4; ++j)
        for (int r = 0; r < 16; ++r) acc[j][r] = 0;
    float x[16];
    for (int i = 0; i < 16; ++i) x[i] = threadIdx.x * 0.001f + i * 0.01f;
    const float a = 0.999f + threadIdx.x * 1e-6f, b = 1e-3f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            if (MF) acc[m & 3] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, fb, acc[m & 3], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                float& r = x[(m * NV + v) % NCH];
                if (v & 1) emit<KB>(r, a, b); else emit<KA>(r, a, b);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    float s = 0;
    for (int j = 0; j < 4; ++j)
        for (int r = 0; r < 16; ++r) s += (float)acc[j][r];
    for (int i = 0; i < 16; ++i) s += x[i];
    out[blockIdx.x * 64 + threadIdx.x] = s + pad[threadIdx.x];
}

static float* g_out;
// SIMD time of one loop trip (8 groups), in ns, at WPS waves per SIMD
template <int KA, int KB, int MF, int NV, int NCH, int WPS> float trip_ns() {
    constexpr int LDSB = WPS == 1 ? 36 * 1024 : (WPS == 2 ? 18 * 1024 : 9 * 1024 + 512);
    const int iters = 6000, grid = 256 * 4 * WPS;
    hipLaunchKernelGGL((probe<KA, KB, MF, NV, NCH, LDSB>), dim3(grid), dim3(64), 0, 0, g_out, 10);
    (void)hipDeviceSynchronize();
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0); (void)hipEventCreate(&e1);
    (void)hipEventRecord(e0);
    hipLaunchKernelGGL((probe<KA, KB, MF, NV, NCH, LDSB>), dim3(grid), dim3(64), 0, 0, g_out, iters);
    (void)hipEventRecord(e1); (void)hipEventSynchronize(e1);
    float ms = 0;
    (void)hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
    return ms * 1e6f / iters / WPS;      // per wave's trip, as seen by the SIMD
}

template <int K> void alone() {
    printf("  %-34s %6.2f %6.2f %6.2f\n", kind_name[K], trip_ns<K, K, 0, 8, 16, 1>() / 64, trip_ns<K, K, 0, 8, 16, 2>() / 64,
           trip_ns<K, K, 0, 8, 16, 4>() / 64);
}
template <int KA, int KB> void pair() {
    printf("  %-34s + %-28s %6.2f   (alone: %5.2f + %5.2f)\n", kind_name[KA], kind_name[KB], trip_ns<KA, KB, 0, 8, 16, 2>() / 32,
           trip_ns<KA, KA, 0, 8, 16, 2>() / 64, trip_ns<KB, KB, 0, 8, 16, 2>() / 64);
}
template <int K> void chain() {
    printf("  %-34s 1 wave: %5.2f %5.2f %5.2f %5.2f   2 waves: %5.2f %5.2f %5.2f %5.2f\n", kind_name[K],
           trip_ns<K, K, 0, 8, 1, 1>() / 64, trip_ns<K, K, 0, 8, 2, 1>() / 64, trip_ns<K, K, 0, 8, 4, 1>() / 64, trip_ns<K, K, 0, 8, 16, 1>() / 64,
           trip_ns<K, K, 0, 8, 1, 2>() / 64, trip_ns<K, K, 0, 8, 2, 2>() / 64, trip_ns<K, K, 0, 8, 4, 2>() / 64, trip_ns<K, K, 0, 8, 16, 2>() / 64);
}
template <int K, int NV> void beside_mfma() {
    const float with = trip_ns<K, K, 1, NV, 16, 2>() / 8, without = trip_ns<K, K, 0, NV, 16, 2>() / 8;
    printf("  %2d x %-30s with the MFMA %6.2f, without %6.2f: the MFMA adds %5.2f\n", NV, kind_name[K], with, without, with - without);
}

int main() {
    if (hipMalloc(&g_out, 256 * 16 * 64 * 4) != hipSuccess) { printf("no GPU\n"); return 1; }
    printf("A. one kind, 64 independent instructions per trip: SIMD ns per instruction at 1 / 2 / 4 waves per SIMD\n");
    alone<ADD>(); alone<MUL>(); alone<FMA>(); alone<MOV>(); alone<SUB_INLINE>(); alone<ADD_SGPR>(); alone<CVT_I32>(); alone<MAX3>();
    alone<MAX>(); alone<CVT_PK_U8>(); alone<CVT_PK_F16>(); alone<PK_MUL_F16>(); alone<PK_ADD_F16>(); alone<CVT_U16_SDWA>(); alone<DOT2>();
    alone<PERM>(); alone<FMA_MIX>(); alone<LDEXP>(); alone<XOR>(); alone<LSHL>(); alone<EXP>(); alone<RCP>(); alone<FMA_F16>();
    printf("B. two kinds alternating, two waves per SIMD: SIMD ns per PAIR\n");
    pair<CVT_I32, ADD>(); pair<CVT_I32, FMA>(); pair<MAX3, MUL>(); pair<CVT_PK_U8, ADD>(); pair<CVT_I32, CVT_PK_U8>(); pair<ADD, MUL>();
    pair<EXP, ADD>(); pair<EXP, FMA>(); pair<EXP, CVT_I32>();
    printf("C. dependent chains: 64 instructions per trip on 1 / 2 / 4 / 16 registers in rotation, SIMD ns per instruction\n");
    chain<ADD>(); chain<FMA>(); chain<CVT_I32>(); chain<EXP>();
    printf("D. v_mfma_i32_32x32x32_i8 (four independent accumulators) with N vector instructions behind each, two waves per SIMD:\n"
           "   SIMD ns per (MFMA + N instructions) of one wave; the MFMA alone: %.2f\n", trip_ns<ADD, ADD, 1, 0, 16, 2>() / 8);
    beside_mfma<CVT_I32, 8>(); beside_mfma<CVT_I32, 16>(); beside_mfma<CVT_PK_U8, 8>(); beside_mfma<CVT_PK_U8, 16>(); beside_mfma<MAX3, 8>();
    beside_mfma<MAX3, 16>(); beside_mfma<EXP, 4>(); beside_mfma<EXP, 8>(); beside_mfma<FMA, 8>(); beside_mfma<FMA, 16>(); beside_mfma<ADD, 8>();
    beside_mfma<ADD, 16>(); beside_mfma<MUL, 8>(); beside_mfma<MUL, 16>();
    return 0;
}
