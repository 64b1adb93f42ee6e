// Issue rate of single vector instructions on gfx950: each kernel runs ITER x 64 copies of one instruction on 8
// independent registers, with 1, 2 or 4 wavefronts on every SIMD; prints cycles per wavefront-instruction per SIMD.
// A measuring tool for the kernels' cost estimates, not part of the library:  make microbench && microbench/valu_rate
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdint>
#define REP8(X) X(0) X(1) X(2) X(3) X(4) X(5) X(6) X(7)
#define REP64(X) REP8(X) REP8(X) REP8(X) REP8(X) REP8(X) REP8(X) REP8(X) REP8(X)
constexpr int ITER = 2000;

#define KERNEL(name, ASMSTR)                                                              \
__global__ __launch_bounds__(256) void name(float *out, float seed) {                     \
    float a0 = seed, a1 = seed + 1, a2 = seed + 2, a3 = seed + 3, a4 = seed + 4, a5 = seed + 5, a6 = seed + 6, a7 = seed + 7; \
    float b = seed * 0.5f, c = seed * 0.25f;                                              \
    for (int it = 0; it < ITER; ++it) {                                                   \
        asm volatile(ASMSTR : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(a4), "+v"(a5), "+v"(a6), "+v"(a7) : "v"(b), "v"(c)); \
    }                                                                                     \
    out[blockIdx.x * blockDim.x + threadIdx.x] = a0 + a1 + a2 + a3 + a4 + a5 + a6 + a7;    \
}
#define I8(OP) OP("%0") OP("%1") OP("%2") OP("%3") OP("%4") OP("%5") OP("%6") OP("%7")
#define I64(OP) I8(OP) I8(OP) I8(OP) I8(OP) I8(OP) I8(OP) I8(OP) I8(OP)

#define OP_FMA(r) "v_fma_f32 " r ", %8, %9, " r "\n"
#define OP_FMAMIX(r) "v_fma_mix_f32 " r ", %8, %9, " r " op_sel_hi:[1,1,0]\n"
#define OP_FMAMIXLO(r) "v_fma_mixlo_f16 " r ", %8, %9, " r " op_sel_hi:[1,1,0]\n"
#define OP_DOT2C(r) "v_dot2c_f32_f16 " r ", %8, %9\n"
#define OP_DOT2(r) "v_dot2_f32_f16 " r ", %8, %9, " r "\n"
#define OP_PKADD(r) "v_pk_add_f16 " r ", %8, " r "\n"
#define OP_PKFMA(r) "v_pk_fma_f16 " r ", %8, %9, " r "\n"
#define OP_AND(r) "v_and_b32 " r ", %8, " r "\n"
#define OP_ADD(r) "v_add_f32 " r ", %8, " r "\n"
#define OP_EXP(r) "v_exp_f32 " r ", " r "\n"
#define OP_CVT(r) "v_cvt_f32_f16 " r ", " r "\n"
#define OP_CVTH(r) "v_cvt_f16_f32 " r ", " r "\n"
#define OP_DPPADD(r) "v_add_f32_dpp " r ", " r ", " r " quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n"
#define OP_MIN3(r) "v_min3_f32 " r ", %8, %9, " r "\n"
#define OP_PERM(r) "v_perm_b32 " r ", %8, " r ", %9\n"
#define OP_PKMAX(r) "v_pk_max_f16 " r ", %8, " r "\n"
#define OP_PKMUL(r) "v_pk_mul_f16 " r ", %8, " r "\n"
#define OP_MAD(r) "v_mad_f32 " r ", %8, %9, " r "\n"
#define OP_FMAC(r) "v_fmac_f32 " r ", %8, %9\n"

#define OP_PACK(r) "v_pack_b32_f16 " r ", %8, " r " op_sel:[1,1,0]\n"
#define OP_PACKLO(r) "v_pack_b32_f16 " r ", %8, " r "\n"
#define OP_BFI(r) "v_bfi_b32 " r ", %8, %9, " r "\n"
#define OP_ALIGNBIT(r) "v_alignbit_b32 " r ", %8, " r ", 16\n"
#define OP_LSHLOR(r) "v_lshl_or_b32 " r ", %8, 16, " r "\n"
#define OP_ANDOR(r) "v_and_or_b32 " r ", %8, %9, " r "\n"
#define OP_MOV(r) "v_mov_b32 " r ", %8\n"
#define OP_LSHR(r) "v_lshrrev_b32 " r ", 16, " r "\n"
#define OP_SUBF16(r) "v_sub_f16 " r ", %8, " r "\n"
#define OP_MAXF16(r) "v_max_f16 " r ", %8, " r "\n"
#define OP_PKMINU16(r) "v_pk_min_u16 " r ", %8, " r "\n"
#define OP_PKSUBU16(r) "v_pk_sub_u16 " r ", %8, " r "\n"
#define OP_ADD3(r) "v_add3_u32 " r ", %8, %9, " r "\n"
#define OP_XOR(r) "v_xor_b32 " r ", %8, " r "\n"
#define OP_MED3(r) "v_med3_f32 " r ", %8, %9, " r "\n"
#define OP_FMAMIX32(r) "v_fma_mix_f32 " r ", %8, %9, " r " op_sel_hi:[1,0,0]\n"
KERNEL(k_fma, I64(OP_FMA))
KERNEL(k_fmac, I64(OP_FMAC))
KERNEL(k_fmamix, I64(OP_FMAMIX))
KERNEL(k_fmamixlo, I64(OP_FMAMIXLO))
KERNEL(k_dot2c, I64(OP_DOT2C))
KERNEL(k_dot2, I64(OP_DOT2))
KERNEL(k_pkadd, I64(OP_PKADD))
KERNEL(k_pkfma, I64(OP_PKFMA))
KERNEL(k_pkmax, I64(OP_PKMAX))
KERNEL(k_and, I64(OP_AND))
KERNEL(k_add, I64(OP_ADD))
KERNEL(k_exp, I64(OP_EXP))
KERNEL(k_cvt, I64(OP_CVT))
KERNEL(k_cvth, I64(OP_CVTH))
KERNEL(k_dppadd, I64(OP_DPPADD))
KERNEL(k_min3, I64(OP_MIN3))
KERNEL(k_perm, I64(OP_PERM))

KERNEL(k_pack, I64(OP_PACK))
KERNEL(k_packlo, I64(OP_PACKLO))
KERNEL(k_bfi, I64(OP_BFI))
KERNEL(k_alignbit, I64(OP_ALIGNBIT))
KERNEL(k_lshlor, I64(OP_LSHLOR))
KERNEL(k_andor, I64(OP_ANDOR))
KERNEL(k_mov, I64(OP_MOV))
KERNEL(k_lshr, I64(OP_LSHR))
KERNEL(k_subf16, I64(OP_SUBF16))
KERNEL(k_maxf16, I64(OP_MAXF16))
KERNEL(k_pkminu16, I64(OP_PKMINU16))
KERNEL(k_pksubu16, I64(OP_PKSUBU16))
KERNEL(k_add3, I64(OP_ADD3))
KERNEL(k_xor, I64(OP_XOR))
KERNEL(k_med3, I64(OP_MED3))
KERNEL(k_fmamix32, I64(OP_FMAMIX32))
template <typename K> void run(const char *name, K k, float *d, int waves_per_simd) {
    const int blocks = 256 * waves_per_simd;   // 256 CUs x (4 waves per block = 1 per SIMD) x waves_per_simd
    hipEvent_t e0, e1; (void)hipEventCreate(&e0); (void)hipEventCreate(&e1);
    hipLaunchKernelGGL(k, dim3(blocks), dim3(256), 0, 0, d, 1.0f);
    (void)hipDeviceSynchronize();
    (void)hipEventRecord(e0);
    hipLaunchKernelGGL(k, dim3(blocks), dim3(256), 0, 0, d, 1.0f);
    (void)hipEventRecord(e1); (void)hipEventSynchronize(e1);
    float ms; (void)hipEventElapsedTime(&ms, e0, e1);
    const double inst_per_simd = (double)ITER * 64 * waves_per_simd;
    printf("%-12s waves/simd %d: %8.3f ms  -> %6.2f ns per wave-instruction per SIMD (x2.27 GHz = %5.2f cycles)\n", name, waves_per_simd, ms,
           ms * 1e6 / inst_per_simd, ms * 1e6 / inst_per_simd * 2.27);
}
int main() {
    float *d; (void)hipMalloc(&d, 256 * 8 * 256 * sizeof(float));
    for (int w : {1, 2, 4}) {
        run("fma_f32", k_fma, d, w); run("fmac_f32", k_fmac, d, w); run("fma_mix", k_fmamix, d, w); run("fma_mixlo", k_fmamixlo, d, w);
        run("dot2c", k_dot2c, d, w); run("dot2", k_dot2, d, w); run("pk_add_f16", k_pkadd, d, w); run("pk_fma_f16", k_pkfma, d, w);
        run("pk_max_f16", k_pkmax, d, w); run("and_b32", k_and, d, w); run("add_f32", k_add, d, w); run("exp_f32", k_exp, d, w);
        run("cvt_f32_f16", k_cvt, d, w); run("cvt_f16_f32", k_cvth, d, w); run("add_dpp", k_dppadd, d, w); run("min3", k_min3, d, w);
        run("perm_b32", k_perm, d, w);
        run("pack_hi", k_pack, d, w); run("pack_lo", k_packlo, d, w); run("bfi", k_bfi, d, w); run("alignbit", k_alignbit, d, w);
        run("lshl_or", k_lshlor, d, w); run("and_or", k_andor, d, w); run("mov", k_mov, d, w); run("lshr", k_lshr, d, w);
        run("sub_f16", k_subf16, d, w); run("max_f16", k_maxf16, d, w); run("pk_min_u16", k_pkminu16, d, w); run("pk_sub_u16", k_pksubu16, d, w);
        run("add3_u32", k_add3, d, w); run("xor", k_xor, d, w); run("med3_f32", k_med3, d, w); run("fma_mix f16*f32", k_fmamix32, d, w);
    }
    return 0;
}
