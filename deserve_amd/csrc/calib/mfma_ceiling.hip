// Measurement aid, not part of the KV path: what the matrix pipeline of the chip sustains
// on the operand bits it is given, and what is left of that once the loop also reads its
// operands from LDS and computes a softmax - the denominators against which the prefill
// attention kernel's rate is read.  Built into libdskv_calib.so, loaded by bench.py only.
//
// One workgroup = 8 waves (two per SIMD), as the prefill kernel.  Per iteration a wave
// issues the 16 v_mfma_f32_32x32x16 of one 32-token block of that kernel: 8 for a 32x32
// score tile over head_dim 128, 8 for the 32 x 128 output tile over 32 tokens.
//   level 0: the MFMAs alone, operands held in registers (loaded once from `operands`)
//   level 1: + the operand traffic of the block: 8 ds_read_b128 (K rows) and 16
//            ds_read_b64_tr_b16 (V, transposed) per iteration, from LDS filled from `operands`
//   level 2: + the softmax of the block: 16 exponentials, packing to 16-bit, row sum,
//            running maximum; the packed probabilities are the B operand of the output MFMAs
// The caller fills `operands` (N(0, 1) or constants): the instruction stream is the same,
// only the bits differ.
#include "../kv_tile.h"

namespace dskv {

constexpr int kCalibWaves = 8;
constexpr int kCalibRegion = 1088;                 // the prefill kernel's LDS region pitch
constexpr int kCalibStage = 8 * kCalibRegion;      // one 32-token block of K or V rows

template <int LEVEL>
__global__ __launch_bounds__(64 * kCalibWaves) void mfma_ceiling_kernel(
    const uint16_t *__restrict__ operands, float *__restrict__ sink, int iters, float scale_log2)
{
    typedef Elt<DSKV_BF16> E;
    __shared__ __align__(16) char k_stage[4][kCalibStage];
    __shared__ __align__(16) char v_stage[4][kCalibStage];
    const int lane = threadIdx.x & 63;
    const int h = lane >> 5, r = lane & 31, g = lane >> 4, c = lane & 15;
    // operands: 16 x 16 bytes per thread, distinct per thread
    const u32x4 *mine = reinterpret_cast<const u32x4 *>(operands) + (long)threadIdx.x * 16;
    u32x4 ka[8], qb[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        ka[i] = mine[i];
        qb[i] = mine[8 + i];
    }
    if (LEVEL >= 1) {
        // fill the eight stages from the same data (every byte written once)
        char *lds = &k_stage[0][0];
        for (int off = threadIdx.x * 16; off < 8 * kCalibStage; off += 64 * kCalibWaves * 16)
            *reinterpret_cast<u32x4 *>(lds + off) = mine[(off >> 4) & 15];
        __syncthreads();
    }
    f32x16 acc[4], s_acc;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[i][v] = 0.f;
    float m_run = -1.0e4f, l_run = 0.f;
    u32x4 pb[2] = {qb[0], qb[1]};
    const int k_lane_off = (r >> 2) * kCalibRegion + h * 64 + (r & 3) * 16;
    const int v_lane_off = h * kCalibRegion + (2 * (g & 1) + ((c & 3) >> 1)) * 64 + (c >> 2) * 16 + (c & 1) * 8;
    for (int it = 0; it < iters; it++) {
        u32x4 va[4][2];
        if (LEVEL >= 1) {
            asm volatile("" ::: "memory");   // the reads belong to this iteration
            const char *kst = k_stage[it & 3] + k_lane_off;
#pragma unroll
            for (int ks = 0; ks < 8; ks++) ka[ks] = *reinterpret_cast<const u32x4 *>(kst + ks * 128);
            const char *vst = v_stage[(it + 3) & 3] + v_lane_off;
#pragma unroll
            for (int dt = 0; dt < 4; dt++)
#pragma unroll
                for (int ks = 0; ks < 2; ks++) {
                    const char *vp = vst + ks * 4 * kCalibRegion + dt * 256;
                    const u32x2 lo = read_transposed(vp), hi = read_transposed(vp + 2 * kCalibRegion);
                    va[dt][ks] = u32x4{lo.x, lo.y, hi.x, hi.y};
                }
        } else {
#pragma unroll
            for (int dt = 0; dt < 4; dt++)
#pragma unroll
                for (int ks = 0; ks < 2; ks++) va[dt][ks] = ka[2 * dt + ks];
        }
#pragma unroll
        for (int v = 0; v < 16; v++) s_acc[v] = 0.f;
#pragma unroll
        for (int ks = 0; ks < 8; ks++) s_acc = E::mfma_32x32(ka[ks], qb[ks], s_acc);
        const u32x4 pb0 = pb[0], pb1 = pb[1];
#pragma unroll
        for (int dt = 0; dt < 4; dt++) {
            acc[dt] = E::mfma_32x32(va[dt][0], pb0, acc[dt]);
            acc[dt] = E::mfma_32x32(va[dt][1], pb1, acc[dt]);
        }
        if (LEVEL >= 2) {
            float p[16], p_sum = 0.f;
            float m = fmaxf(fmaxf(s_acc[0], s_acc[1]), s_acc[2]);
#pragma unroll
            for (int v = 3; v < 15; v += 2) m = fmaxf(fmaxf(m, s_acc[v]), s_acc[v + 1]);
            m = fmaxf(m, s_acc[15]);
            float other = m;
            swap_halves32(m, other);
            m_run = fmaxf(m_run, fmaxf(m, other) * scale_log2 - 1.0e4f);   // never raised: no rescale branch
#pragma unroll
            for (int v = 0; v < 16; v++) {
                p[v] = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[v], scale_log2, -m_run - 1.0e4f));
                p_sum += p[v];
            }
            l_run += p_sum;
#pragma unroll
            for (int ks = 0; ks < 2; ks++)
                pb[ks] = u32x4{E::pack2(p[8 * ks], p[8 * ks + 1]), E::pack2(p[8 * ks + 2], p[8 * ks + 3]),
                               E::pack2(p[8 * ks + 4], p[8 * ks + 5]), E::pack2(p[8 * ks + 6], p[8 * ks + 7])};
        } else {
            // keep the score tile alive without vector work
            asm volatile("" ::"v"(s_acc));
        }
    }
    float out = l_run + m_run;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) out += acc[i][v];
    sink[(long)blockIdx.x * blockDim.x + threadIdx.x] = out;
}

}  // namespace dskv

// operands: 64 * 8 * 256 bytes (one workgroup's worth, shared by all workgroups); sink:
// workgroups * 512 floats.  Returns 0, -1 for bad arguments, or a hipError_t.
extern "C" int dskv_calib_mfma_loop(const void *operands, float *sink, int level, int workgroups,
                                    int iters, float scale_log2, void *stream)
{
    using namespace dskv;
    if (!operands || !sink || level < 0 || level > 2 || workgroups <= 0 || iters <= 0) return -1;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)workgroups), block(64 * kCalibWaves);
    if (level == 0)
        hipLaunchKernelGGL(mfma_ceiling_kernel<0>, grid, block, 0, s, (const uint16_t *)operands, sink, iters, scale_log2);
    else if (level == 1)
        hipLaunchKernelGGL(mfma_ceiling_kernel<1>, grid, block, 0, s, (const uint16_t *)operands, sink, iters, scale_log2);
    else
        hipLaunchKernelGGL(mfma_ceiling_kernel<2>, grid, block, 0, s, (const uint16_t *)operands, sink, iters, scale_log2);
    return (int)hipGetLastError();
}

// flops of one launch: workgroups x 8 waves x iters x 16 MFMAs x (2 * 32 * 32 * 16)
extern "C" double dskv_calib_mfma_loop_flops(int workgroups, int iters)
{
    return (double)workgroups * dskv::kCalibWaves * iters * 16.0 * 2.0 * 32 * 32 * 16;
}
