// FP8 (e4m3 x e4m3) scaled GEMM for gfx950:  out[M,N] = bf16((A[M,K] . B[N,K]^T in fp32) * inv_a * inv_b)
// Replaces torch._scaled_mm as called at nanochat/fp8.py:143-153 (row-major A, K-contiguous B, fp32
// accumulation, bf16 output).  B may be several weight matrices stacked along N, each with its own
// tensorwise inv-scale (the reference's c_q/c_k/c_v are three Float8Linear modules).
//
// Both kernels use v_mfma_f32_16x16x128_f8f6f4 (the full-rate fp8 MFMA of CDNA4): a lane supplies 32
// consecutive K bytes of row (lane & 15) from K-block (lane >> 4).  Operands are issued as (B, A) so a
// lane ends up holding four consecutive output columns of one output row, which packs into one 8-byte
// bf16 store.
//
//   gemm_tile_kernel    M large (prefill, isolated Float8Linear): BMxBNx128 tiles, 4 waves in 2x2,
//                       double-buffered swizzled LDS, global loads of step k+1 overlap the MFMAs of step k.
//   gemm_skinny_kernel  M <= 128 (decode): weight-bandwidth bound.  A workgroup owns 64 output columns,
//                       each wave 16 of them over the whole K; weight rows stream global -> registers,
//                       the small activation panel is shared through LDS.
#include "nc_common.h"
#include "nc_kernels.h"

#define MFMA_F8(acc, b, a) __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4((b), (a), (acc), 0, 0, 0, 0, 0, 0)

struct EpilogueArgs {
    const float* inv_a;
    const float* inv_b;
    NcGemmSegs segs;
    void* out;
    int out_kind;
    float softcap;
    int ldc;
};

__device__ __forceinline__ float seg_scale(const EpilogueArgs& e, int col) {
    int s = 0;
#pragma unroll
    for (int i = 0; i < 3; i++)
        if (i + 1 < e.segs.nseg && col >= e.segs.end[i]) s = i + 1;
    return e.inv_b[s];
}

// four consecutive columns n..n+3 of output row m
__device__ __forceinline__ void store4(const EpilogueArgs& e, float inv_a, v4f acc, int m, int n, int M, int N) {
    if (m >= M || n >= N) return;
    const float inv_b = seg_scale(e, n);
    float v[4];
#pragma unroll
    for (int r = 0; r < 4; r++) v[r] = (acc[r] * inv_a) * inv_b;
    if (e.out_kind == 0) {
        bf16_t* o = (bf16_t*)e.out + (size_t)m * e.ldc + n;
        if (n + 3 < N) {
            uint2 p = make_uint2(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]));
            *(uint2*)o = p;
        } else {
            for (int r = 0; r < 4 && n + r < N; r++) o[r] = f32_to_bf16(v[r]);
        }
    } else {
        float* o = (float*)e.out + (size_t)m * e.ldc + n;
        for (int r = 0; r < 4 && n + r < N; r++) o[r] = e.softcap * tanhf(rbf(v[r]) / e.softcap);
    }
}

// ------------------------------------------------------------------------------------------------
// Tile kernel.  LDS rows are 128 bytes (one K step); 16-byte chunk c of row r lives at chunk slot
// c ^ ((r >> 1) & 7), which makes both the row-major fills and the per-lane fragment reads conflict free.
template <int BM, int BN>
__global__ __launch_bounds__(256) void gemm_tile_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                        EpilogueArgs ep, int M, int N, int K, int tiles_m, int tiles_n) {
    constexpr int WTM = BM / 32, WTN = BN / 32;          // 16x16 tiles per wave along M and N
    constexpr int A_CH = BM * 8 / 256, B_CH = BN * 8 / 256;
    extern __shared__ __align__(16) uint8_t lds[];
    auto tile_a = [&](int buf) -> uint8_t* { return lds + buf * (BM + BN) * 128; };
    auto tile_b = [&](int buf) -> uint8_t* { return lds + buf * (BM + BN) * 128 + BM * 128; };

    // Workgroups are handed to the 8 XCDs round robin; give each XCD a contiguous run of tiles (N fastest)
    // so the A row panels and the B panel it touches stay in that XCD's L2.
    const int ntiles = tiles_m * tiles_n;
    int pid = blockIdx.x;
    {
        const int per = ntiles / 8, rem = ntiles % 8;
        const int xcd = pid % 8, local = pid / 8;
        pid = xcd * per + (xcd < rem ? xcd : rem) + local;
    }
    const int m0 = (pid / tiles_n) * BM, n0 = (pid % tiles_n) * BN;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int frow = lane & 15, kb = lane >> 4;

    v4f acc[WTM][WTN];
#pragma unroll
    for (int i = 0; i < WTM; i++)
#pragma unroll
        for (int j = 0; j < WTN; j++) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

    uint4 ra[A_CH], rb[B_CH];
    auto load_regs = [&](int kt) {
#pragma unroll
        for (int c = 0; c < A_CH; c++) {
            const int id = tid + c * 256, row = id >> 3, ch = id & 7;
            const int gr = m0 + row, gk = kt * 128 + ch * 16;
            ra[c] = (gr < M && gk < K) ? *(const uint4*)(A + (size_t)gr * K + gk) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int c = 0; c < B_CH; c++) {
            const int id = tid + c * 256, row = id >> 3, ch = id & 7;
            const int gr = n0 + row, gk = kt * 128 + ch * 16;
            rb[c] = (gr < N && gk < K) ? *(const uint4*)(B + (size_t)gr * K + gk) : make_uint4(0, 0, 0, 0);
        }
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int c = 0; c < A_CH; c++) {
            const int id = tid + c * 256, row = id >> 3, ch = id & 7;
            *(uint4*)(tile_a(buf) + row * 128 + ((ch ^ ((row >> 1) & 7)) << 4)) = ra[c];
        }
#pragma unroll
        for (int c = 0; c < B_CH; c++) {
            const int id = tid + c * 256, row = id >> 3, ch = id & 7;
            *(uint4*)(tile_b(buf) + row * 128 + ((ch ^ ((row >> 1) & 7)) << 4)) = rb[c];
        }
    };
    auto read_frag = [&](const uint8_t* base, int row) -> v8i {
        const int sw = (row >> 1) & 7;
        const uint4 lo = *(const uint4*)(base + row * 128 + (((2 * kb) ^ sw) << 4));
        const uint4 hi = *(const uint4*)(base + row * 128 + (((2 * kb + 1) ^ sw) << 4));
        v8i f;
        f[0] = lo.x, f[1] = lo.y, f[2] = lo.z, f[3] = lo.w, f[4] = hi.x, f[5] = hi.y, f[6] = hi.z, f[7] = hi.w;
        return f;
    };

    const int ksteps = (K + 127) / 128;
    load_regs(0);
    store_lds(0);
    __syncthreads();
    for (int kt = 0; kt < ksteps; kt++) {
        const int buf = kt & 1;
        if (kt + 1 < ksteps) load_regs(kt + 1);
        v8i af[WTM];
#pragma unroll
        for (int i = 0; i < WTM; i++) af[i] = read_frag(tile_a(buf), wm * (BM / 2) + i * 16 + frow);
#pragma unroll
        for (int j = 0; j < WTN; j++) {
            const v8i bf = read_frag(tile_b(buf), wn * (BN / 2) + j * 16 + frow);
#pragma unroll
            for (int i = 0; i < WTM; i++) acc[i][j] = MFMA_F8(acc[i][j], bf, af[i]);
        }
        if (kt + 1 < ksteps) store_lds(buf ^ 1);
        __syncthreads();
    }

    const float inv_a = *ep.inv_a;
#pragma unroll
    for (int i = 0; i < WTM; i++)
#pragma unroll
        for (int j = 0; j < WTN; j++) {
            const int m = m0 + wm * (BM / 2) + i * 16 + frow;
            const int n = n0 + wn * (BN / 2) + j * 16 + 4 * kb;
            store4(ep, inv_a, acc[i][j], m, n, M, N);
        }
}

// ------------------------------------------------------------------------------------------------
// Skinny kernel: M <= 16*MB rows.  K is walked in super-steps of 512 bytes (four MFMA K-steps).
// LDS holds the activation panel of one super-step, 512-byte rows, chunk c (0..31) of row r at slot
// c ^ (r & 15).
template <int MB>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                          EpilogueArgs ep, int M, int N, int K) {
    constexpr int ROWS = MB * 16;
    constexpr int A_CH = ROWS * 32 / 256;   // 16-byte chunks per thread per super-step
    __shared__ __align__(16) uint8_t lds[2][ROWS * 512];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int frow = lane & 15, kb = lane >> 4;
    const int n0 = blockIdx.x * 64 + wave * 16;
    const int brow = n0 + frow;
    const bool brow_ok = brow < N;
    const uint8_t* bptr = B + (size_t)(brow_ok ? brow : 0) * K + kb * 32;

    v4f acc[MB];
#pragma unroll
    for (int i = 0; i < MB; i++) acc[i] = v4f{0.f, 0.f, 0.f, 0.f};

    uint4 ra[A_CH];
    uint4 rb[2][4][2];
    auto load_a = [&](int ks) {
#pragma unroll
        for (int c = 0; c < A_CH; c++) {
            const int id = tid + c * 256, row = id >> 5, ch = id & 31;
            const int gk = ks * 512 + ch * 16;
            ra[c] = (row < M && gk < K) ? *(const uint4*)(A + (size_t)row * K + gk) : make_uint4(0, 0, 0, 0);
        }
    };
    auto store_a = [&](int buf) {
#pragma unroll
        for (int c = 0; c < A_CH; c++) {
            const int id = tid + c * 256, row = id >> 5, ch = id & 31;
            *(uint4*)(&lds[buf][row * 512 + ((ch ^ (row & 15)) << 4)]) = ra[c];
        }
    };
    auto load_b = [&](int ks, int slot) {
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            const int gk = ks * 512 + kk * 128 + kb * 32;
#pragma unroll
            for (int h = 0; h < 2; h++)
                rb[slot][kk][h] = (brow_ok && gk + h * 16 < K) ? *(const uint4*)(bptr + ks * 512 + kk * 128 + h * 16)
                                                              : make_uint4(0, 0, 0, 0);
        }
    };

    const int nsteps = (K + 511) / 512;
    load_a(0);
    load_b(0, 0);
    store_a(0);
    __syncthreads();
#pragma unroll 1
    for (int ks = 0; ks < nsteps; ks += 2) {
        // two super-steps per trip so the register slots of rb are compile-time constants
#pragma unroll
        for (int half = 0; half < 2; half++) {
            const int s = ks + half;
            if (s < nsteps) {
                const bool more = s + 1 < nsteps;
                if (more) {
                    load_a(s + 1);
                    load_b(s + 1, half ^ 1);
                }
#pragma unroll
                for (int kk = 0; kk < 4; kk++) {
                    v8i bf;
                    const uint4 lo = rb[half][kk][0], hi = rb[half][kk][1];
                    bf[0] = lo.x, bf[1] = lo.y, bf[2] = lo.z, bf[3] = lo.w, bf[4] = hi.x, bf[5] = hi.y, bf[6] = hi.z, bf[7] = hi.w;
#pragma unroll
                    for (int i = 0; i < MB; i++) {
                        const int row = i * 16 + frow;
                        const int c0 = kk * 8 + 2 * kb;
                        const uint4 alo = *(const uint4*)(&lds[half][row * 512 + ((c0 ^ (row & 15)) << 4)]);
                        const uint4 ahi = *(const uint4*)(&lds[half][row * 512 + (((c0 + 1) ^ (row & 15)) << 4)]);
                        v8i af;
                        af[0] = alo.x, af[1] = alo.y, af[2] = alo.z, af[3] = alo.w, af[4] = ahi.x, af[5] = ahi.y, af[6] = ahi.z, af[7] = ahi.w;
                        acc[i] = MFMA_F8(acc[i], bf, af);
                    }
                }
                if (more) store_a(half ^ 1);
                __syncthreads();
            }
        }
    }

    const float inv_a = *ep.inv_a;
#pragma unroll
    for (int i = 0; i < MB; i++) store4(ep, inv_a, acc[i], i * 16 + frow, n0 + 4 * kb, M, N);
}

// ------------------------------------------------------------------------------------------------
template <int BM, int BN>
static int launch_tile(const uint8_t* a, const uint8_t* b, const EpilogueArgs& ep, int M, int N, int K, hipStream_t s) {
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const size_t lds_bytes = 2 * (size_t)(BM + BN) * 128;
    static bool configured = false;   // per instantiation; the attribute is per function, not per device state
    hipError_t e = hipFuncSetAttribute((const void*)gemm_tile_kernel<BM, BN>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e != hipSuccess) NC_FAIL(-2, "fp8_gemm: cannot reserve %zu bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
    (void)configured;
    hipLaunchKernelGGL((gemm_tile_kernel<BM, BN>), dim3(tiles_m * tiles_n), dim3(256), lds_bytes, s, a, b, ep, M, N, K, tiles_m, tiles_n);
    return 0;
}

int nc_launch_gemm(const uint8_t* a, const uint8_t* b, const float* inv_a, const float* inv_b, NcGemmSegs segs,
                   void* out, int out_kind, float softcap, int M, int N, int K, int ldc, int force_kernel, hipStream_t s) {
    NC_CHECK_ARG(a && b && inv_a && inv_b && out, "fp8_gemm: null pointer");
    NC_CHECK_ARG(M >= 0 && N > 0 && K > 0, "fp8_gemm: bad shape M=%d N=%d K=%d", M, N, K);
    NC_CHECK_ARG(K % 16 == 0, "fp8_gemm: K=%d must be a multiple of 16", K);
    NC_CHECK_ARG(ldc >= N, "fp8_gemm: ldc=%d < N=%d", ldc, N);
    NC_CHECK_ARG(((uintptr_t)a & 15) == 0 && ((uintptr_t)b & 15) == 0, "fp8_gemm: operands must be 16-byte aligned");
    NC_CHECK_ARG(out_kind == 0 || out_kind == 1, "fp8_gemm: out_kind must be 0 (bf16) or 1 (softcapped fp32)");
    NC_CHECK_ARG(segs.nseg >= 1 && segs.nseg <= 4, "fp8_gemm: 1..4 column segments supported, got %d", segs.nseg);
    for (int i = 0; i < segs.nseg; i++) {
        NC_CHECK_ARG(segs.end[i] % 4 == 0 || segs.end[i] == N, "fp8_gemm: segment end %d must be a multiple of 4", segs.end[i]);
        NC_CHECK_ARG(i == 0 || segs.end[i] > segs.end[i - 1], "fp8_gemm: segment ends must increase");
    }
    NC_CHECK_ARG(segs.end[segs.nseg - 1] == N, "fp8_gemm: last segment must end at N");
    if (out_kind == 0)
        NC_CHECK_ARG(((uintptr_t)out & 7) == 0 && ldc % 4 == 0, "fp8_gemm: bf16 output needs 8-byte alignment and ldc %% 4 == 0");
    if (M == 0) return 0;
    EpilogueArgs ep{inv_a, inv_b, segs, out, out_kind, softcap, ldc};
    NcProfScope prof(1, 2.0 * M * N * K, s);

    // force_kernel: 0 auto, 1 skinny, 2 tile 256x256, 3 tile 256x128, 4 tile 128x128
    int which = force_kernel;
    if (which == 0) {
        if (M <= 128) which = 1;
        else {
            const long t256 = (long)((M + 255) / 256) * ((N + 255) / 256);
            which = (t256 >= 512) ? 2 : (M >= 2048 ? 3 : 4);
        }
    }
    int rc = 0;
    if (which == 1) {
        NC_CHECK_ARG(M <= 128, "fp8_gemm: skinny kernel needs M <= 128, got %d", M);
        const int grid = (N + 63) / 64;
        if (M <= 16) hipLaunchKernelGGL(gemm_skinny_kernel<1>, dim3(grid), dim3(256), 0, s, a, b, ep, M, N, K);
        else if (M <= 32) hipLaunchKernelGGL(gemm_skinny_kernel<2>, dim3(grid), dim3(256), 0, s, a, b, ep, M, N, K);
        else if (M <= 64) hipLaunchKernelGGL(gemm_skinny_kernel<4>, dim3(grid), dim3(256), 0, s, a, b, ep, M, N, K);
        else hipLaunchKernelGGL(gemm_skinny_kernel<8>, dim3(grid), dim3(256), 0, s, a, b, ep, M, N, K);
    } else if (which == 2) rc = launch_tile<256, 256>(a, b, ep, M, N, K, s);
    else if (which == 3) rc = launch_tile<256, 128>(a, b, ep, M, N, K, s);
    else if (which == 4) rc = launch_tile<128, 128>(a, b, ep, M, N, K, s);
    else NC_FAIL(-1, "fp8_gemm: unknown kernel selector %d", force_kernel);
    if (rc) return rc;
    NC_CHECK_LAUNCH("fp8_gemm");
    return 0;
}
