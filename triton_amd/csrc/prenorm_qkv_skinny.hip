// Fused RMSNorm + Q/K/V projection for a handful of tokens (decode: at most 32), where the GEMM is a stream of the
// weight matrices through HBM and nothing else matters: 100 MB of W for 16 tokens at the Llama3-8B widths.
//
// Same arithmetic and MFMA mapping as the larger tilings (C^T = W^T X^T, 32x32x16 fp16 MFMAs, tokens padded to one
// 32-wide block).  A workgroup owns a 64-column panel of one projection -- full 128-byte lines of every W row -- and
// its four waves split the contraction range between them; each wave streams its quarter of the panel through a
// private ring of six LDS stages filled by direct global->LDS loads, so there is not a single barrier in the main
// loop: a wave only ever reads what it requested itself and orders itself with s_waitcnt vmcnt(N), N = the loads
// issued behind the stage it needs (five stages = 30 KB per wave, 120 KB per CU in flight -- what it takes to keep
// HBM busy from a CU).  X (and gamma) take the same route, so every load in the loop is one of a fixed number of
// LDS-DMA requests per stage and the count is exact.  The four partial accumulators and the four partial sums of
// squares are added through LDS at the end.
#include "prenorm_qkv.h"

namespace trn {

[[maybe_unused]] constexpr int SN = 64, SK = 32, SS = 6;      // panel columns, contraction rows per stage, stages per wave

__global__ __launch_bounds__(256, 1) void prenorm_qkv_skinny_kernel(const GemmArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)   // buffer descriptors and LDS-load builtins exist in the device pass only
    // One array per stage (each holds the four waves' private parts): the compiler orders LDS reads after
    // outstanding global->LDS loads that may alias them, and only distinct variables are provably disjoint.
#define TRN_STAGE(i_)                                                               \
    __shared__ __attribute__((aligned(1024))) half_t Ws##i_[4 * SK * SN];           \
    __shared__ __attribute__((aligned(1024))) half_t Xs##i_[4 * 32 * SK];           \
    __shared__ __attribute__((aligned(256))) half_t Gs##i_[4 * 128];
    TRN_STAGE(0) TRN_STAGE(1) TRN_STAGE(2) TRN_STAGE(3) TRN_STAGE(4) TRN_STAGE(5)
#undef TRN_STAGE
    __shared__ float ss_part[4][32];

    const int tid = threadIdx.x, lane = tid & 63, c = lane & 31, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int panel = blockIdx.x;
    const int pi = panel >= a.p[2].tile0 ? 2 : (panel >= a.p[1].tile0 ? 1 : 0);
    const ProjOut P = a.p[pi];
    const int n0 = (panel - P.tile0) * SN;
    const int nst = (a.K + SK - 1) / SK;             // stages in all; this wave takes nsw of them from s0 on
    const int nsw = (nst + 3) / 4, s0 = wave * nsw;
    constexpr int kOut = 0x7ffffff0;                 // a byte offset past every buffer: the load returns zeros

    // ---- W: 32 rows x 128 bytes per stage, chunk c of row r stored at c ^ swz<64>(r).  A wave-wide load covers 8
    // rows; load i covers stage rows 8*i + lane/8, and the swizzle depends on the row's bits 1..3, i.e. on i % 2.
    const __amdgpu_buffer_rsrc_t wrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)P.w, 0, (int)(((int64_t)(a.K - 1) * P.ldw + P.n) * 2), 0x00020000);
    int w_vo[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int r = 8 * i + (lane >> 3);
        w_vo[i] = (int)((lane >> 3) * P.ldw * 2) + (n0 + 8 * ((lane & 7) ^ swz<64>(r))) * 2;
    }
    const int w_row8 = (int)(8 * P.ldw * 2), w_stage = (int)(SK * P.ldw * 2);
    // ---- X: 32 token rows x 64 bytes per stage, chunk c of row t stored at c ^ ((t/4) % 4).  A wave-wide load
    // covers 16 rows; tokens past the end read as zeros.
    const __amdgpu_buffer_rsrc_t xrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)a.x, 0, (int)(((int64_t)(a.T - 1) * a.ldx + a.K) * 2), 0x00020000);
    const int x_chunk = (lane & 3) ^ ((lane >> 4) & 3);
    int x_vo[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int t = 16 * j + (lane >> 2);
        x_vo[j] = t < a.T ? (int)(t * a.ldx * 2) + x_chunk * 16 : kOut;
    }
    // ---- gamma: 4 bytes per lane = 128 values from the stage's first column on (32 are used)
    const bool use_g = a.gamma != nullptr && a.norm;
    const __amdgpu_buffer_rsrc_t grs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(use_g ? a.gamma : a.x), 0, use_g ? a.K * 2 : 0, 0x00020000);
    // All loads of stage s (absolute index) into ring slot arrays W_, X_, G_: 4 + 2 (+ 1) LDS-DMA requests.
#define TRN_FETCH(s_, W_, X_, G_)                                                                                \
    do {                                                                                                         \
        const int st_ = (s_);                                                                                    \
        _Pragma("unroll") for (int i_ = 0; i_ < 4; ++i_)                                                         \
            __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                            \
                wrs, (__attribute__((address_space(3))) void*)(&W_[wave * SK * SN + i_ * 8 * SN]), 16,           \
                w_vo[i_ & 1], st_ * w_stage + i_ * w_row8, 0, 0);                                                \
        /* columns past hidden hold the next row's data: read zeros instead */                                   \
        const bool drop_ = st_ * SK + 8 * x_chunk >= a.K;                                                        \
        _Pragma("unroll") for (int j_ = 0; j_ < 2; ++j_)                                                         \
            __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                            \
                xrs, (__attribute__((address_space(3))) void*)(&X_[wave * 32 * SK + j_ * 16 * SK]), 16,          \
                drop_ ? kOut : x_vo[j_], st_ * SK * 2, 0, 0);                                                    \
        if (use_g)                                                                                               \
            __builtin_amdgcn_raw_ptr_buffer_load_lds(                                                            \
                grs, (__attribute__((address_space(3))) void*)(&G_[wave * 128]), 4, lane * 4, st_ * SK * 2, 0, 0); \
    } while (0)

    // ---- LDS read offsets (halfs) within this wave's part of a stage
    int xoff[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) xoff[ks] = wave * 32 * SK + c * SK + (((2 * ks + h) ^ ((c >> 2) & 3)) << 3);
    int woff_lo[2], woff_hi[2];     // W^T A-operand via the transposing read: rows 8h + (lane%16)/4 [+4] of a 16-row step
    {
        const int rl = 8 * h + ((lane & 15) >> 2), rh = rl + 4;
        const int lc = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1), sub = (lane & 1) * 4;
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            woff_lo[nb] = wave * SK * SN + rl * SN + (((nb * 4 + lc) ^ swz<64>(rl)) << 3) + sub;
            woff_hi[nb] = wave * SK * SN + rh * SN + (((nb * 4 + lc) ^ swz<64>(rh)) << 3) + sub;
        }
    }

    float16_t acc[2];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[nb][r] = 0.f;
    float ss = 0.f;

    // One stage: wait for it, read its operands, hand the slot back to the loader at once, then the four MFMAs.
    // Requests are issued unconditionally -- stages past this wave's range (or past hidden) read zeros and add
    // nothing -- so that exactly (SS-1) stages of 6 (7 with gamma) requests sit behind the one being waited for.
    auto stage = [&](int s, half_t* Wc, half_t* Xc, half_t* Gc) __attribute__((always_inline)) {
        if (use_g) __builtin_amdgcn_s_waitcnt(0x8f73);       // vmcnt(35)
        else __builtin_amdgcn_s_waitcnt(0x4f7e);             // vmcnt(30)
        half8_t xb[2], wa[2][2], g[2];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            xb[ks] = *reinterpret_cast<const half8_t*>(&Xc[xoff[ks]]);
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                const half4_t lo = lds_read_tr16(&Wc[ks * 16 * SN + woff_lo[nb]]);
                const half4_t hi = lds_read_tr16(&Wc[ks * 16 * SN + woff_hi[nb]]);
                wa[ks][nb] = half8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            }
            if (use_g) g[ks] = *reinterpret_cast<const half8_t*>(&Gc[wave * 128 + ks * 16 + 8 * h]);
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);                  // lgkmcnt(0): the reads have returned, the slot is free
        __builtin_amdgcn_sched_barrier(0);
        // (a stage of another wave's range or past hidden: harmless zeros / duplicates are never requested --
        // the range test is on the absolute stage index)
        TRN_FETCH(s + SS < s0 + nsw ? s + SS : nst, Wc, Xc, Gc);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            half8_t xv = xb[ks];
            if (a.norm) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const half2_t p = {xv[2 * e], xv[2 * e + 1]};
                    ss = __builtin_amdgcn_fdot2(p, p, ss, false);
                }
                if (use_g) xv = xv * g[ks];
            }
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) acc[nb] = mfma32(wa[ks][nb], xv, acc[nb]);
        }
    };
#define TRN_PRIME(i_) TRN_FETCH(s0 + i_ < s0 + nsw ? s0 + i_ : nst, Ws##i_, Xs##i_, Gs##i_)
    TRN_PRIME(0); TRN_PRIME(1); TRN_PRIME(2); TRN_PRIME(3); TRN_PRIME(4); TRN_PRIME(5);
#undef TRN_PRIME
    for (int s = s0; s < s0 + nsw; s += SS) {
        stage(s, Ws0, Xs0, Gs0);
        stage(s + 1, Ws1, Xs1, Gs1);
        stage(s + 2, Ws2, Xs2, Gs2);
        stage(s + 3, Ws3, Xs3, Gs3);
        stage(s + 4, Ws4, Xs4, Gs4);
        stage(s + 5, Ws5, Xs5, Gs5);
    }
#undef TRN_FETCH

    // ---- add the four waves' partial results through LDS (the rings are idle once every request has landed)
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();
    float* red01 = reinterpret_cast<float*>(Ws0);            // [2 waves][32 registers][64 lanes] floats = 16 KB
    float* red23 = reinterpret_cast<float*>(Ws1);
    {
        float* mine = (wave < 2 ? red01 : red23) + (wave & 1) * 32 * 64;
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int r = 0; r < 16; ++r) mine[(nb * 16 + r) * 64 + lane] = acc[nb][r];
        const float s = half_sum(ss);                        // both halves of a token's columns
        if (h == 0) ss_part[wave][c] = s;
    }
    __syncthreads();
    // wave w finishes accumulator registers 8w .. 8w+7: column block (8w)/16, rows 8*(r/4) + 4h + r%4 of it, token c
    const float rstd = a.norm ? 1.0f / __builtin_sqrtf((ss_part[0][c] + ss_part[1][c] + ss_part[2][c] + ss_part[3][c]) / (float)a.K + a.eps)
                              : 1.0f;
    const int nb = wave >> 1;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        const int r0 = (wave & 1) * 8 + q * 4;               // four consecutive registers = four consecutive columns
        const int n = n0 + nb * 32 + 8 * (r0 / 4) + 4 * h;
        const int64_t o_off = (int64_t)(n / a.head_dim) * P.stride_h + (int64_t)c * P.stride_s + (n % a.head_dim);
        const bool live = c < a.T && n < P.n;
        half4_t ad = {(half_t)0.f, (half_t)0.f, (half_t)0.f, (half_t)0.f};
        if (live && P.addend) ad = *reinterpret_cast<const half4_t*>(P.addend + o_off);
        half4_t ov;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int idx = ((nb * 16 + r0 + e) * 64 + lane);
            const float v = red01[idx] + red01[32 * 64 + idx] + red23[idx] + red23[32 * 64 + idx];
            ov[e] = (half_t)((float)(half_t)(v * rstd) + (float)ad[e]);     // the product rounded to fp16 first, as a separate GEMM would leave it
        }
        if (live) *reinterpret_cast<half4_t*>(P.out + o_off) = ov;
    }
#endif
}

int launch_prenorm_qkv_skinny(GemmArgs a, hipStream_t stream) {
    int t0 = 0;
    for (int i = 0; i < 3; ++i) { a.p[i].tile0 = t0; t0 += (a.p[i].n + SN - 1) / SN; }
    a.n_panels = t0;
    hipLaunchKernelGGL(prenorm_qkv_skinny_kernel, dim3((unsigned)a.n_panels), dim3(256), 0, stream, a);
    return hipGetLastError() == hipSuccess ? TRN_OK : TRN_E_LAUNCH;
}

}  // namespace trn
