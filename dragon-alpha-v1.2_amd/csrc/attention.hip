// Attention block in one launch on the FP32 matrix cores of gfx950:
//     Y[b, i, :] = sum_j softmax_j(scale * <Q[b, i, :], K[b, j, :]>) * V[b, j, :]
// which the reference computes as batchMatMulT2 -> sdiv -> softmax -> batchMatMul, with a
// transpose(1, 2) on every tensor around them (nn/unit/complex/block/ChannelMHA.java:66-83 of
// alpha-Dragon-v1.2/src/z/dragon).  Here the score matrix never reaches memory: a workgroup owns 128
// queries of one (image, head), walks over the keys 64 at a time and keeps a reference maximum, a
// running sum and the un-normalised output per query ("online softmax").  Row strides are
// arguments, so the [N, L, head, d] tensors of the layer are read and written where they lie and
// the four transposes disappear as well.
//
// Both products are computed transposed, S^T = K.Q^T and Y^T = V^T.P^T, with
// v_mfma_f32_32x32x2_f32.  In that instruction's result layout lane (c, h) holds column c, and a
// column is a query in both S^T and Y^T: the maximum, the sum and the rescaling factor of a query
// live in the lane that needs them (the two halves h of a wavefront exchange one value per step),
// and the probabilities P^T come out of the first product exactly in the register layout the
// second product wants for its B operand -- no trip through LDS between the two.
//
//   S^T = K.Q^T :  A = K tile from LDS, [key][d] in 16-byte chunks, chunk swizzled like every
//                  K-inner tile of the matrix products (one ds_read_b128 feeds 4 MFMA steps);
//                  B = Q, 4 consecutive d per lane and group, loaded once into registers.
//   Y^T = V^T.P^T: A = V tile from LDS, [key][d], lane r reads column r of the d-block (a
//                  ds_read_b32 over 32 consecutive floats); B = P^T in place.
//   MFMA step v of the second product consumes key 8*(v/4) + 4*h + v%4 from lane half h, which
//   is the row the first product's result register v holds.
//
// K and V tiles are fetched one step ahead into registers (buffer loads, rows beyond the key
// count and chunks beyond the head dimension read as zero) and stored to the other LDS buffer
// after the step's matrix work; one barrier per step.
//
// The vector instructions of the softmax are not hidden behind the matrix work (taking them out
// shortens the kernel by exactly their issue time), so there are as few as possible: the scale
// is folded into Q when it is loaded; and the reference maximum that the exponentials subtract
// is only raised -- which costs a rescaling of the 32 output registers -- when some query's
// scores exceed it by more than 2^8.  Any reference gives the same result after the final
// division by the sum; letting it lag keeps every term below 2^8 and skips the rescaling in
// almost every step.
#include "gemm_mfma_kernel.h"
#include "runtime_internal.h"
#include "../../include/dragon_hip_gemm.h"

namespace dragon {
namespace {

constexpr int AQ = 128;   // queries per workgroup: 32 per wavefront
constexpr int LAG = 8;    // the reference maximum may lag the true one by 2^LAG

struct AttnParams {
    const float* Q; const float* K; const float* V; float* Y;
    int head, nq, nk;            // heads per image, queries, keys
    int dk4, dv4;                // head dimension of Q / K and of V / Y, multiples of 4
    int qtiles;                  // workgroups per (image, head)
    long long q_n, q_h; int q_l; // element strides: image, head, row
    long long k_n, k_h; int k_l;
    long long v_n, v_h; int v_l;
    long long y_n, y_h; int y_l;
    float c;                     // scale * log2(e): the exponentials are base 2
    const float* M;              // optional factor on the probabilities, M[.., query, key]
    long long m_b; int m_l;      // its element strides: (image, head) slice (0: one mask for all), row
};

__device__ __forceinline__ float xhalf(float x) { return __shfl_xor(x, 32, 64); }

// DB = 32-wide blocks of the head dimension in a row of the K / V tiles in LDS: 1 (d <= 32), 2 (d <= 64),
// 4 (d <= 128) or 8 (d <= 256: one workgroup per compute unit, its query and output registers fill the
// register file); DC <= DB = the blocks that hold anything for this head dimension -- only those are
// multiplied and kept in registers (d = 192: 6 of 8, a quarter of the matrix work less);
// KB = 32-key blocks per step;
// MASK: the probabilities are multiplied by M[query, key] AFTER the softmax, as the block's mask unit does
// (ChannelMHA.java:75-76: P = softmax(...); P = mask.forward(P)): the sum that normalises them runs over the
// unmasked terms, the second product takes the masked ones.
template <int DB, int DC, int KB, bool MASK>
__global__ __launch_bounds__(NTHREADS, DB > 4 ? 1 : 2) void attention_f32_mfma(const AttnParams p) {
    static_assert(DC >= 1 && DC <= DB && 2 * DC > DB, "a narrower tile row would do");
    constexpr int AK = KB * 32;            // keys per step
    constexpr int DW = DB * 32;            // tile width in floats
    constexpr int CPR = DW / 4;            // 16-byte chunks per tile row
    constexpr int RPP = NTHREADS / CPR;    // tile rows staged per pass
    constexpr int PASSES = AK / RPP;       // = DB * KB
    constexpr int NG = DC * 4;             // groups of 8 d (4 MFMA steps each) that the head dimension reaches
    // DB = 8: the query and output registers leave no room for staging registers, so the K / V tiles go from
    // global memory straight into the other LDS buffer (a lane's 16 bytes land at the wave's base + 16 * lane:
    // the chunk swizzle of the K tile moves to the global side)
    constexpr bool DMA = DB > 4;
    static_assert(PASSES * RPP == AK, "the key tile divides over the workgroup");

    __shared__ __attribute__((aligned(16))) float Ks[2][AK * DW];
    __shared__ __attribute__((aligned(16))) float Vs[2][AK * DW];

    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int r = lane & 31, h = lane >> 5;

    const int lid = xcd_contiguous_id(blockIdx.x, gridDim.x);   // one XCD's L2 serves whole heads
    const int bh = lid / p.qtiles, qt = lid - bh * p.qtiles;
    const int n = bh / p.head, hd = bh - n * p.head;
    const float* Qb = p.Q + n * p.q_n + hd * p.q_h;
    const float* Kb = p.K + n * p.k_n + hd * p.k_h;
    const float* Vb = p.V + n * p.v_n + hd * p.v_h;
    float* Yb = p.Y + n * p.y_n + hd * p.y_h;

    // ---- this lane's query: row r of the wavefront's 32, d = 8g + 4h .. +3 per group ----
    const int q = qt * AQ + wave * 32 + r;
    v4f qf[NG];
#pragma unroll
    for (int g = 0; g < NG; g++) {
        const int d = 8 * g + 4 * h;
        qf[g] = buffer_load_f4(Qb, (q < p.nq && d < p.dk4) ? (q * p.q_l + d) * 4 : OOB_OFFSET);
        qf[g] *= p.c;                       // scores come out in units of log2: scale * log2(e) * <q, k>
    }

    // ---- staging of the K / V tiles ----
    const int s_chunk = t % CPR, s_row = t / CPR;
    v4f kreg[DMA ? 1 : PASSES], vreg[DMA ? 1 : PASSES];
    // A lane's byte offsets inside a key tile never change (a chunk beyond the head dimension is out of
    // range for good).  The tile's first key goes into the buffer descriptor's base and the bytes up
    // to the end of the last key into its size, so the hardware returns zeros for rows beyond the key
    // count: a step's fetch costs scalar instructions only, no per-lane address or test.
    int koff[PASSES], voff[PASSES];
#pragma unroll
    for (int s = 0; s < PASSES; s++) {
        const int row = s_row + s * RPP;
        const int kchunk = DMA ? (s_chunk ^ kin_swizzle<DW>(row)) : s_chunk;   // the chunk that belongs at this LDS slot
        koff[s] = (kchunk * 4 < p.dk4) ? (row * p.k_l + kchunk * 4) * 4 : OOB_OFFSET;
        voff[s] = (s_chunk * 4 < p.dv4) ? (row * p.v_l + s_chunk * 4) * 4 : OOB_OFFSET;
    }
    const unsigned lds_k = (unsigned)(unsigned long long)(__attribute__((address_space(3))) float*)&Ks[0][0];
    const unsigned lds_v = (unsigned)(unsigned long long)(__attribute__((address_space(3))) float*)&Vs[0][0];
    const unsigned lds_wave = __builtin_amdgcn_readfirstlane(wave) * 1024;
    // DMA: the tiles of the step that starts at key0, into LDS buffer `into`
    auto fetch_direct = [&](int key0, int into) {
        const int left = p.nk - key0;   // > 0
        const unsigned long long bk = (unsigned long long)(Kb + (size_t)key0 * p.k_l);
        const unsigned long long bv = (unsigned long long)(Vb + (size_t)key0 * p.v_l);
        const v4u rk = {(unsigned)bk, (unsigned)(bk >> 32) & 0xffffu, (unsigned)(left * p.k_l * 4), (unsigned)RSRC_FLAGS};
        const v4u rv = {(unsigned)bv, (unsigned)(bv >> 32) & 0xffffu, (unsigned)(left * p.v_l * 4), (unsigned)RSRC_FLAGS};
        const unsigned tile_bytes = into * (AK * DW * 4);
        static_for<PASSES>([&](auto sc) {
            constexpr int s = decltype(sc)::value;
            dma_f4_lean<s * NTHREADS * 16>(rk, lds_k + tile_bytes + lds_wave, koff[s]);
            dma_f4_lean<s * NTHREADS * 16>(rv, lds_v + tile_bytes + lds_wave, voff[s]);
        });
    };
    auto fetch = [&](int key0) {
        const int left = p.nk - key0;   // > 0
        const __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc(
            (void*)(Kb + (size_t)key0 * p.k_l), 0, left * p.k_l * 4, RSRC_FLAGS);
        const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc(
            (void*)(Vb + (size_t)key0 * p.v_l), 0, left * p.v_l * 4, RSRC_FLAGS);
#pragma unroll
        for (int s = 0; s < PASSES; s++) {
            kreg[s] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rk, koff[s], 0, 0));
            vreg[s] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rv, voff[s], 0, 0));
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int s = 0; s < PASSES; s++) {
            const int row = s_row + s * RPP;
            *(v4f*)(&Ks[buf][row * DW + 4 * (s_chunk ^ kin_swizzle<DW>(row))]) = kreg[s];
            *(v4f*)(&Vs[buf][row * DW + 4 * s_chunk]) = vreg[s];
        }
    };

    // ---- this lane's row of the mask: keys 32kb + 8g + 4h .. +3 of a step in one 16-byte load; zeros beyond
    // the row's end (the descriptor ends there) and for a query that does not exist ----
    const float* Mrow = MASK ? p.M + (size_t)bh * p.m_b + (size_t)(q < p.nq ? q : 0) * p.m_l : nullptr;
    v4f mreg[MASK ? KB * 4 : 1];
    auto fetch_mask = [&](int key0) {
        if constexpr (MASK) {
            const __amdgpu_buffer_rsrc_t rm = __builtin_amdgcn_make_buffer_rsrc(
                (void*)(Mrow + key0), 0, q < p.nq ? (p.m_l - key0) * 4 : 0, RSRC_FLAGS);   // to the end of the row
#pragma unroll
            for (int kb = 0; kb < KB; kb++)
#pragma unroll
                for (int g = 0; g < 4; g++)
                    mreg[kb * 4 + g] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rm, (32 * kb + 8 * g + 4 * h) * 4, 0, 0));
        }
    };

    v16f o[DC];
#pragma unroll
    for (int b = 0; b < DC; b++) o[b] = (v16f)(0.0f);
    float m = -__builtin_inff(), l = 0.0f;      // reference maximum (shared by the halves), this half's sum

    const int steps = (p.nk + AK - 1) / AK;
    if constexpr (DMA) {
        fetch_direct(0, 0);
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    } else {
        fetch(0);
        stage(0);
    }
    __syncthreads();
    int buf = 0;
    for (int it = 0; it < steps; it++) {
        const bool more = it + 1 < steps;
        if (more) {
            if constexpr (DMA) fetch_direct((it + 1) * AK, buf ^ 1);   // nobody reads that buffer during this step
            else fetch((it + 1) * AK);
        }
        fetch_mask(it * AK);      // used behind the first product and the exponentials
        __builtin_amdgcn_sched_barrier(0);

        // ---- S^T[key][query] for this step's keys, one 32-key block after the other ----
        v16f s[KB];
        const float* ks = Ks[buf];
#pragma unroll
        for (int kb = 0; kb < KB; kb++) {
            s[kb] = (v16f)(0.0f);
#pragma unroll
            for (int g = 0; g < NG; g++) {
                const v4f kf = *(const v4f*)(ks + (kb * 32 + r) * DW + 4 * ((2 * g + h) ^ kin_swizzle<DW>(r)));
                s[kb] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf.x, qf[g].x, s[kb], 0, 0, 0);
                s[kb] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf.y, qf[g].y, s[kb], 0, 0, 0);
                s[kb] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf.z, qf[g].z, s[kb], 0, 0, 0);
                s[kb] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf.w, qf[g].w, s[kb], 0, 0, 0);
            }
        }

        // ---- online softmax, per lane = per query; register v of block kb is key 32kb + 8*(v/4) + 4h + v%4 ----
        if (!more && (p.nk & (AK - 1))) {           // the last step of a ragged key count
            const int left = p.nk - it * AK;
#pragma unroll
            for (int kb = 0; kb < KB; kb++)
#pragma unroll
                for (int v = 0; v < 16; v++)
                    if (32 * kb + 8 * (v / 4) + 4 * h + (v % 4) >= left) s[kb][v] = -__builtin_inff();
        }
        float mt = s[0][0];
#pragma unroll
        for (int kb = 0; kb < KB; kb++)
#pragma unroll
            for (int v = (kb == 0); v < 16; v++) mt = fmaxf(mt, s[kb][v]);
        mt = fmaxf(mt, xhalf(mt));
        if (__builtin_amdgcn_ballot_w64(mt > m + (float)LAG) != 0) {   // same decision for the whole wavefront
            const float m_new = fmaxf(m, mt);
            const float alpha = __builtin_amdgcn_exp2f(m - m_new);     // 0 on the first step (m = -inf)
            m = m_new;
            l *= alpha;
#pragma unroll
            for (int b = 0; b < DC; b++)
#pragma unroll
                for (int v = 0; v < 16; v++) o[b][v] *= alpha;
        }
        float sum = 0.0f;
#pragma unroll
        for (int kb = 0; kb < KB; kb++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                s[kb][v] = __builtin_amdgcn_exp2f(s[kb][v] - m);
                sum += s[kb][v];
            }
        l += sum;
        if constexpr (MASK) {
#pragma unroll
            for (int kb = 0; kb < KB; kb++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    s[kb][4 * g + 0] *= mreg[kb * 4 + g].x;
                    s[kb][4 * g + 1] *= mreg[kb * 4 + g].y;
                    s[kb][4 * g + 2] *= mreg[kb * 4 + g].z;
                    s[kb][4 * g + 3] *= mreg[kb * 4 + g].w;
                }
            if (!more && (p.nk & (AK - 1))) {       // whatever the mask's row holds beyond the last key does not count
                const int left = p.nk - it * AK;
#pragma unroll
                for (int kb = 0; kb < KB; kb++)
#pragma unroll
                    for (int v = 0; v < 16; v++)
                        if (32 * kb + 8 * (v / 4) + 4 * h + (v % 4) >= left) s[kb][v] = 0.0f;
            }
        }

        // ---- Y^T[d][query] += V^T[d][key] * P^T[key][query] ----
        const float* vs = Vs[buf];
#pragma unroll
        for (int kb = 0; kb < KB; kb++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int key = 32 * kb + 8 * (v / 4) + 4 * h + (v % 4);
#pragma unroll
                for (int b = 0; b < DC; b++)
                    o[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(vs[key * DW + b * 32 + r], s[kb][v], o[b], 0, 0, 0);
            }

        if constexpr (DMA) __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));   // this wave's part of the next tiles has landed
        else if (more) stage(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }

    // ---- normalise and store: register v of block b is d = 32b + 8*(v/4) + 4h + v%4 ----
    l += xhalf(l);
    const float inv = 1.0f / l;
    if (q < p.nq) {
        float* yrow = Yb + (size_t)q * p.y_l;
#pragma unroll
        for (int b = 0; b < DC; b++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int d = 32 * b + 8 * g + 4 * h;
                if (d < p.dv4) {
                    v4f y = {o[b][4 * g] * inv, o[b][4 * g + 1] * inv, o[b][4 * g + 2] * inv, o[b][4 * g + 3] * inv};
                    *(v4f*)(yrow + d) = y;
                }
            }
    }
}

inline bool aligned16(int64_t a) { return (a & 15) == 0; }

}  // namespace
}  // namespace dragon

using namespace dragon;

extern "C" {

static int attention_launch(const int64_t* streams, int32_t length, int64_t dQ, int64_t dK, int64_t dV, int64_t dMask,
                            int64_t dY, int32_t N, int32_t head, int32_t QL, int32_t VL, int32_t dK4, int32_t dV4,
                            int32_t head_inner, float scale, int32_t mask_pitch, int32_t mask_per_head) {
    if (streams == nullptr || length < 1 || length > 10) return hipErrorInvalidValue;
    if (dQ == 0 || dK == 0 || dV == 0 || dY == 0 || !aligned16(dQ) || !aligned16(dK) || !aligned16(dV) ||
        !aligned16(dY))
        return hipErrorInvalidValue;
    if (N <= 0 || head <= 0 || QL <= 0 || VL <= 0 || dK4 <= 0 || dV4 <= 0 || (dK4 & 3) || (dV4 & 3) || dK4 > 256 ||
        dV4 > 256 || !(scale - scale == 0.0f))   // NaN and the infinities fail the last test
        return hipErrorInvalidValue;
    if (dMask != 0 && (!aligned16(dMask) || mask_pitch < VL || (mask_pitch & 3) || (long long)mask_pitch * 4 >= 0x7ffffff0LL))
        return hipErrorInvalidValue;
    // offsets inside one (image, head) slice travel as 32-bit byte offsets
    const long long rowK = head_inner ? (long long)head * dK4 : dK4, rowV = head_inner ? (long long)head * dV4 : dV4;
    const long long maxL = QL > VL ? QL : VL, maxRow = rowK > rowV ? rowK : rowV;
    if ((maxL + AQ) * maxRow * 4 >= 0x7ffffff0LL || (long long)N * head > 0x7fffffffLL / ((QL + AQ - 1) / AQ))
        return hipErrorInvalidValue;
    AttnParams p;
    p.Q = (const float*)(intptr_t)dQ; p.K = (const float*)(intptr_t)dK; p.V = (const float*)(intptr_t)dV;
    p.Y = (float*)(intptr_t)dY;
    p.M = (const float*)(intptr_t)dMask;
    p.m_l = mask_pitch;
    p.m_b = mask_per_head ? (long long)QL * mask_pitch : 0;
    p.head = head; p.nq = QL; p.nk = VL; p.dk4 = dK4; p.dv4 = dV4;
    p.qtiles = (QL + AQ - 1) / AQ;
    if (head_inner) {   // [N, L, head, d]: a row of a head lies head*d apart from the next
        p.q_l = p.k_l = (int)rowK; p.v_l = p.y_l = (int)rowV;
        p.q_h = p.k_h = dK4; p.v_h = p.y_h = dV4;
        p.q_n = (long long)QL * rowK; p.k_n = (long long)VL * rowK;
        p.v_n = (long long)VL * rowV; p.y_n = (long long)QL * rowV;
    } else {            // [N, head, L, d]
        p.q_l = p.k_l = dK4; p.v_l = p.y_l = dV4;
        p.q_h = (long long)QL * dK4; p.k_h = (long long)VL * dK4;
        p.v_h = (long long)VL * dV4; p.y_h = (long long)QL * dV4;
        p.q_n = p.q_h * head; p.k_n = p.k_h * head; p.v_n = p.v_h * head; p.y_n = p.y_h * head;
    }
    dragon::split_ledger_touch(p.Y, (size_t)N * (size_t)p.y_n * 4);
    p.c = scale * 1.44269504088896340736f;
    hipStream_t s = (hipStream_t)(intptr_t)streams[0];
    const dim3 grid((unsigned)((long long)N * head * p.qtiles)), block(NTHREADS);
    const int dmax = dK4 > dV4 ? dK4 : dV4;
    const int dc = (dmax + 31) / 32;   // 32-wide blocks of the head dimension that hold anything
    const bool masked = dMask != 0;
#define ATTN_CASE(DB_, DC_, KB_)                                                                          \
    case DC_:                                                                                             \
        if (masked) hipLaunchKernelGGL((attention_f32_mfma<DB_, DC_, KB_, true>), grid, block, 0, s, p);  \
        else hipLaunchKernelGGL((attention_f32_mfma<DB_, DC_, KB_, false>), grid, block, 0, s, p);        \
        break;
    switch (dc) {
        ATTN_CASE(1, 1, 2)
        ATTN_CASE(2, 2, 2)
        ATTN_CASE(4, 3, 1)
        ATTN_CASE(4, 4, 1)
        ATTN_CASE(8, 5, 1)
        ATTN_CASE(8, 6, 1)
        ATTN_CASE(8, 7, 1)
        ATTN_CASE(8, 8, 1)
        default: return hipErrorInvalidValue;
    }
#undef ATTN_CASE
    return hipGetLastError();
}

int dragon_Cuda_attention_forward(const int64_t* streams, int32_t length, int64_t dQ, int64_t dK, int64_t dV,
                                  int64_t dY, int32_t N, int32_t head, int32_t QL, int32_t VL, int32_t dK4,
                                  int32_t dV4, int32_t head_inner, float scale) {
    return attention_launch(streams, length, dQ, dK, dV, 0, dY, N, head, QL, VL, dK4, dV4, head_inner, scale, 0, 0);
}

int dragon_Cuda_attention_forward_masked(const int64_t* streams, int32_t length, int64_t dQ, int64_t dK, int64_t dV,
                                         int64_t dMask, int64_t dY, int32_t N, int32_t head, int32_t QL, int32_t VL,
                                         int32_t dK4, int32_t dV4, int32_t head_inner, float scale,
                                         int32_t mask_pitch, int32_t mask_per_head) {
    if (dMask == 0) return hipErrorInvalidValue;
    return attention_launch(streams, length, dQ, dK, dV, dMask, dY, N, head, QL, VL, dK4, dV4, head_inner, scale,
                            mask_pitch, mask_per_head);
}

}  // extern "C"
