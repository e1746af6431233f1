// FP8 (e4m3 x e4m3) scaled GEMM for gfx950:  out[M,N] = bf16((A[M,K] . B[N,K]^T in fp32) * inv_a * inv_b)
// Replaces torch._scaled_mm as called at nanochat/fp8.py:143-153 (row-major A, K-contiguous B, fp32
// accumulation, bf16 output).  B may be several weight matrices stacked along N, each with its own
// tensorwise inv-scale (the reference's c_q/c_k/c_v are three Float8Linear modules).
//
// The kernels use v_mfma_f32_16x16x128_f8f6f4 (the full-rate fp8 MFMA of CDNA4): a lane supplies 32
// consecutive K bytes of row (lane & 15) from K-block (lane >> 4).  Operands are issued as (B, A) so a
// lane ends up holding four consecutive output columns of one output row, which packs into one 8-byte
// bf16 store.
//
//   gemm_bl_kernel      M large (prefill, isolated Float8Linear): BMxBNx128 tiles, double-buffered swizzled LDS fed
//                       through two register stages of buffer loads (for the 128x128 tile the fills and loads are
//                       placed between the MFMA groups by hand), bf16 epilogue staged through LDS.
//   gemm_dl_kernel      256x256x128 tiles whose operands go from global memory straight into LDS (no staging registers,
//   gemm_dlp_kernel     no LDS fill instructions); the second is the persistent form for shapes of several rounds of tiles.
//   gemm_tile_kernel    the same tiling with plain global loads (64-bit addressing) for operands past 2 GiB.
//   M <= 128 (decode) is weight-bandwidth bound and handled by gemm_decode_kernel in nc_gemm_decode.hip.
#include <type_traits>
#include "nc_common.h"
#include "nc_kernels.h"

// 16-byte chunk c of LDS row r (128-byte rows) is kept at chunk slot c ^ NC_SWZ(r) by the buffer-load kernels.  Measured on
// gfx950: with this mapping a fragment read (16 rows per 16 lanes, ds_read_b128) runs at the rate of a lane-linear read
// (~215 B/clk/CU); XOR with (r & 7) alone, or with (r >> 1) & 7, runs at 60% of that.
#define NC_SWZ(row) (((row) & 7) ^ (((row) >> 3) & 1))
#define MFMA_F8(acc, b, a) __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4((b), (a), (acc), 0, 0, 0, 0, 0, 0)

struct EpilogueArgs {
    const float* inv_a;
    const float* inv_b;
    NcGemmSegs segs;
    void* out;
    int out_kind;            // 0 bf16, 1 fp32 softcap, 2 bf16 relu(v)^2 with the amax of the result published to out_amax
    float softcap;
    int ldc;
    uint32_t* out_amax;
};

// relu(bf16(v))^2, to be rounded to bf16 by the caller's pack: the two eager ops of nanochat/gpt.py:139 on a bf16 tensor
__device__ __forceinline__ float relu2_of(float v) {
    const float h = relu_keep_nan(rbf(v));
    return h * h;
}
// largest of eight non-negative bf16 values in a 16-byte vector, the first `count` of them
__device__ __forceinline__ float max_bf16x8(const uint4& v, int count) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t m = 0;
#pragma unroll
    for (int r = 0; r < 8; r++) {
        const uint32_t b = (w[r >> 1] >> ((r & 1) * 16)) & 0xffffu;
        if (r < count) m = b > m ? b : m;             // non-negative bf16: integer order is value order
    }
    return __uint_as_float(m << 16);
}

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

// Tile order.  Workgroups are dealt to the 8 XCDs round robin (workgroup id % 8) and each XCD has its own 4 MB L2,
// so (1) every XCD gets a contiguous run of the tile sequence, and (2) the sequence walks the tile grid in bands of
// GROUP_M tile rows, column by column inside a band: the ~64 tiles an XCD works on at one time then cover about
// GROUP_M rows x 8 columns and share GROUP_M A panels and 8 B panels (a few MB) instead of streaming all of B
// past one A panel.
#define NC_GROUP_M 8
__device__ __forceinline__ void tile_coords(int wg, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int ntiles = tiles_m * tiles_n;
    const int per = ntiles / 8, rem = ntiles % 8;
    const int xcd = wg % 8, local = wg / 8;
    const int seq = xcd * per + (xcd < rem ? xcd : rem) + local;
    const int band_tiles = NC_GROUP_M * tiles_n;
    const int band = seq / band_tiles, in_band = seq % band_tiles;
    const int rows_here = min(NC_GROUP_M, tiles_m - band * NC_GROUP_M);
    tm = band * NC_GROUP_M + in_band % rows_here;
    tn = in_band / rows_here;
}

// ------------------------------------------------------------------------------------------------
// Tile kernel.  LDS rows are 128 bytes (one K step); 16-byte chunk c of row r lives at chunk slot
// c ^ (r & 7), which makes both the row-major fills and the per-lane fragment reads conflict free.
template <int BM, int BN>
__global__ __launch_bounds__(256) void gemm_tile_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                        EpilogueArgs ep, int M, int N, int K, int tiles_m, int tiles_n) {
    constexpr int WTM = BM / 32, WTN = BN / 32;          // 16x16 tiles per wave along M and N
    constexpr int A_CH = BM * 8 / 256, B_CH = BN * 8 / 256;
    extern __shared__ __align__(16) uint8_t lds[];
    auto tile_a = [&](int buf) -> uint8_t* { return lds + buf * (BM + BN) * 128; };
    auto tile_b = [&](int buf) -> uint8_t* { return lds + buf * (BM + BN) * 128 + BM * 128; };

    int tm, tn;
    tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;

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
            *(uint4*)(tile_a(buf) + row * 128 + ((ch ^ (row & 7)) << 4)) = ra[c];
        }
#pragma unroll
        for (int c = 0; c < B_CH; c++) {
            const int id = tid + c * 256, row = id >> 3, ch = id & 7;
            *(uint4*)(tile_b(buf) + row * 128 + ((ch ^ (row & 7)) << 4)) = rb[c];
        }
    };
    auto read_frag = [&](const uint8_t* base, int row) -> v8i {
        const int sw = row & 7;
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

// Epilogue of the buffer-load kernels: scale, convert and store one workgroup tile.
template <int BM, int BN, int WGM, int WGN, int OUT_KIND>
__device__ __forceinline__ void bl_epilogue(v4f (&acc)[BM / WGM / 16][BN / WGN / 16], uint8_t* lds, const EpilogueArgs& ep, float inv_a,
                                            const float (&sc)[4], int m0, int n0, int M, int N) {
    constexpr int WTM = BM / WGM / 16, WTN = BN / WGN / 16;
    constexpr int STAGE = (BM + BN) * 128;
    const int lane = threadIdx.x & 63, wave = threadIdx.x / 64;
    const int wm = wave / WGN, wn = wave % WGN;
    const int frow = lane & 15, kb = lane >> 4;
    if (OUT_KIND != 1) {
        // bf16 output goes through LDS so that every store instruction writes whole 128-byte lines: each wave parks its
        // (BM/WGM) x (BN/WGN) block in its own LDS region (16-byte chunk c of row r at chunk c ^ (r & 7)), then reads it
        // back with one row segment per group of LPR lanes and stores 16 bytes per lane.
        constexpr int WROWS = BM / WGM, WCOLS = BN / WGN, ROWB = WCOLS * 2, LPR = ROWB / 16, RPI = 64 / LPR;
        static_assert(LPR % 8 == 0 && LPR <= 64 && WGM * WGN * WROWS * ROWB <= 2 * STAGE, "epilogue staging");
        constexpr bool relu2 = OUT_KIND == 2;
        float am = 0.f;
        __syncthreads();                                       // every wave is done with the operand tiles
        uint8_t* reg = lds + wave * WROWS * ROWB;
#pragma unroll
        for (int j = 0; j < WTN; j++) {
            const int n = n0 + wn * WCOLS + j * 16 + 4 * kb;
            float inv_b = sc[0];
#pragma unroll
            for (int i = 0; i < 3; i++)
                if (i + 1 < ep.segs.nseg && n >= ep.segs.end[i]) inv_b = sc[i + 1];
            const int chunk = 2 * j + (kb >> 1);
#pragma unroll
            for (int i = 0; i < WTM; i++) {
                const int row = i * 16 + frow;
                const v4f a4 = acc[i][j];
                float o4[4];
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    o4[r] = (a4[r] * inv_a) * inv_b;
                    if (relu2) o4[r] = relu2_of(o4[r]);
                }
                const uint2 pk = make_uint2(pack_bf16_hw(o4[0], o4[1]), pack_bf16_hw(o4[2], o4[3]));
                *(uint2*)(reg + row * ROWB + ((chunk ^ (row & 7)) << 4) + (kb & 1) * 8) = pk;
            }
        }
        // the region is private to the wave: its own LDS writes only have to land before its reads
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_s_waitcnt(0xc07f);                    // lgkmcnt(0)
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const bool vec16 = (ep.ldc % 8 == 0) && (((uintptr_t)ep.out & 15) == 0);
        const int lrow_e = lane / LPR, c = lane % LPR;
        const int n = n0 + wn * WCOLS + c * 8;
#pragma unroll
        for (int it = 0; it < WROWS / RPI; it++) {
            const int row = it * RPI + lrow_e;
            const int m = m0 + wm * WROWS + row;
            const uint4 v = *(const uint4*)(reg + row * ROWB + ((c ^ (row & 7)) << 4));
            if (m >= M || n >= N) continue;
            if (relu2) am = amax_join(am, max_bf16x8(v, N - n));
            bf16_t* o = (bf16_t*)ep.out + (size_t)m * ep.ldc + n;
            if (n + 8 <= N) {
                if (vec16) __builtin_nontemporal_store(v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w}, (v4i*)o);
                else {
                    *(uint2*)o = make_uint2(v.x, v.y);
                    *(uint2*)(o + 4) = make_uint2(v.z, v.w);
                }
            } else {
                const uint32_t w[4] = {v.x, v.y, v.z, v.w};
                for (int r = 0; r < 8 && n + r < N; r++) o[r] = (bf16_t)(w[r >> 1] >> ((r & 1) * 16));
            }
        }
        if (relu2) {
            // one publication per workgroup: the waves meet once more and the first thread joins their maxima
            __shared__ float wave_am[WGM * WGN];
            am = wave_amax(am);
            if (lane == 0) wave_am[wave] = am;
            __syncthreads();
            if (threadIdx.x == 0) {
                float t = wave_am[0];
#pragma unroll
                for (int w = 1; w < WGM * WGN; w++) t = amax_join(t, wave_am[w]);
                amax_publish(ep.out_amax, t);
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < WTN; j++) {
            const int n = n0 + wn * (BN / WGN) + j * 16 + 4 * kb;
            float inv_b = sc[0];
#pragma unroll
            for (int i = 0; i < 3; i++)
                if (i + 1 < ep.segs.nseg && n >= ep.segs.end[i]) inv_b = sc[i + 1];
#pragma unroll
            for (int i = 0; i < WTM; i++) {
                const int m = m0 + wm * (BM / WGM) + i * 16 + frow;
                if (m >= M || n >= N) continue;
                float* o = (float*)ep.out + (size_t)m * ep.ldc + n;
                for (int r = 0; r < 4 && n + r < N; r++)
                    o[r] = ep.softcap * tanhf(rbf((acc[i][j][r] * inv_a) * inv_b) / ep.softcap);
            }
        }
    }
    // no barrier and no wait here: the kernel ends, and a wave may retire with its stores still on their way, which frees the
    // CU for the next workgroup while the output drains
}

// ------------------------------------------------------------------------------------------------
// Buffer-load tile kernel: the same tiling, LDS layout and MFMA mapping as gemm_tile_kernel, with a main
// loop free of branches.  Global reads go through buffer descriptors, whose hardware range check returns
// zeros for rows past M / N and for the K tail, so no load sits under a lane mask and the loads of K-steps
// k+2 and k+3 stay in flight (two register stages) while step k is computed; the waits the compiler places
// then count outstanding loads instead of draining them.  Waves form a WGM x WGN grid over the BM x BN tile.
#define NC_BUF_OOB 0x80000000u
// Accumulate in place: tying the result to the accumulator operand keeps every 16x16 tile in the same four
// accumulation registers for the whole K loop (the builtin lets the register allocator pick a different result
// tuple, which it repairs with dozens of register copies per K-step once the loop is unrolled).
// A_FMT is the format of the activation-side operand (the instruction's second source, `blgp`): 0 = e4m3, 1 = e5m2, the
// gradient format of the backward GEMMs (nanochat/fp8.py:165).  The weight-side operand is always e4m3.
template <int A_FMT = 0>
__device__ __forceinline__ void mfma_f8_acc(v4f& acc, const v8i& b, const v8i& a) {
    if (A_FMT == 0) asm("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(acc) : "v"(b), "v"(a));
    else asm("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0 blgp:1" : "+a"(acc) : "v"(b), "v"(a));
}
// Same, pinned in program order against every memory operation: used where the LDS fills and global loads of the
// next steps are placed between groups of MFMAs by hand, so that the LDS, load and matrix pipes work at the same time.
template <int A_FMT = 0>
__device__ __forceinline__ void mfma_f8_acc_ordered(v4f& acc, const v8i& b, const v8i& a) {
    if (A_FMT == 0) asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(acc) : "v"(b), "v"(a) : "memory");
    else asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0 blgp:1" : "+a"(acc) : "v"(b), "v"(a) : "memory");
}
template <int BM, int BN, int WGM, int WGN, int OUT_KIND, bool INTERLEAVE = false, int A_FMT = 0>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm_bl_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                                 EpilogueArgs ep, int M, int N, int K, int tiles_m, int tiles_n) {
    constexpr int NT = 64 * WGM * WGN;
    constexpr int WTM = BM / WGM / 16, WTN = BN / WGN / 16;     // 16x16 tiles per wave along M and N
    constexpr int A_CH = BM * 8 / NT, B_CH = BN * 8 / NT;       // 16-byte pieces per thread and K-step
    constexpr int PASS_ROWS = NT / 8;                           // tile rows covered by one piece of every thread
    constexpr int STAGE = (BM + BN) * 128;
    static_assert(PASS_ROWS % 16 == 0 && BM % (16 * WGM) == 0 && BN % (16 * WGN) == 0, "tile shape");
    extern __shared__ __align__(16) uint8_t lds[];

    int tm, tn;
    tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid / 64;
    const int wm = wave / WGN, wn = wave % WGN;
    const int frow = lane & 15, kb = lane >> 4;

    const __amdgpu_buffer_rsrc_t desc_a = __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, M * K, 0x00020000);
    const __amdgpu_buffer_rsrc_t desc_b = __builtin_amdgcn_make_buffer_rsrc((void*)B, 0, N * K, 0x00020000);

    // this thread's pieces: chunk `ch` of rows lrow, lrow + PASS_ROWS, ...
    const int lrow = tid >> 3, ch = tid & 7;
    uint32_t avo[A_CH], bvo[B_CH];
#pragma unroll
    for (int c = 0; c < A_CH; c++) {
        const int r = m0 + lrow + c * PASS_ROWS;
        avo[c] = r < M ? (uint32_t)r * (uint32_t)K + ch * 16 : NC_BUF_OOB;
    }
#pragma unroll
    for (int c = 0; c < B_CH; c++) {
        const int r = n0 + lrow + c * PASS_ROWS;
        bvo[c] = r < N ? (uint32_t)r * (uint32_t)K + ch * 16 : NC_BUF_OOB;
    }
    const int lw = lrow * 128 + ((ch ^ NC_SWZ(lrow)) << 4);                 // LDS fill offset of piece 0 (PASS_ROWS keeps the swizzle)
    const int sw = NC_SWZ(frow);
    const int rd_lo = frow * 128 + (((2 * kb) ^ sw) << 4), rd_hi = frow * 128 + (((2 * kb + 1) ^ sw) << 4);
    const int a_rd = wm * (BM / WGM) * 128, b_rd = BM * 128 + wn * (BN / WGN) * 128;

    const int ksteps = (K + 127) / 128, kfull = K / 128;
    const bool ch_in_tail = ch * 16 >= K % 128;                            // only looked at for the partial last step

    v4f acc[WTM][WTN];
#pragma unroll
    for (int i = 0; i < WTM; i++)
#pragma unroll
        for (int j = 0; j < WTN; j++) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

    v4i ra[2][A_CH], rb[2][B_CH];
#define BL_LOAD(SLOT, T)                                                                                  \
    do {                                                                                                  \
        const int t__ = (T);                                                                              \
        const bool cut__ = t__ >= ksteps || (t__ == kfull && ch_in_tail);                                 \
        _Pragma("unroll") for (int c = 0; c < A_CH; c++)                                                  \
            ra[SLOT][c] = __builtin_amdgcn_raw_buffer_load_b128(desc_a, cut__ ? NC_BUF_OOB : avo[c], t__ * 128, 0); \
        _Pragma("unroll") for (int c = 0; c < B_CH; c++)                                                  \
            rb[SLOT][c] = __builtin_amdgcn_raw_buffer_load_b128(desc_b, cut__ ? NC_BUF_OOB : bvo[c], t__ * 128, 0); \
    } while (0)
#define BL_FILL(SLOT, BUF)                                                                                \
    do {                                                                                                  \
        uint8_t* st__ = lds + (BUF) * STAGE + lw;                                                         \
        _Pragma("unroll") for (int c = 0; c < A_CH; c++) *(v4i*)(st__ + c * PASS_ROWS * 128) = ra[SLOT][c]; \
        _Pragma("unroll") for (int c = 0; c < B_CH; c++) *(v4i*)(st__ + BM * 128 + c * PASS_ROWS * 128) = rb[SLOT][c]; \
    } while (0)
    auto frag = [&](const uint8_t* base) -> v8i {
        const v4i lo = *(const v4i*)(base + rd_lo);
        const v4i hi = *(const v4i*)(base + rd_hi);
        return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };
    auto compute = [&](int buf) {
        const uint8_t* st = lds + buf * STAGE;
        v8i af[WTM];
#pragma unroll
        for (int i = 0; i < WTM; i++) af[i] = frag(st + a_rd + i * 2048);
#pragma unroll
        for (int j = 0; j < WTN; j++) {
            const v8i bf = frag(st + b_rd + j * 2048);
#pragma unroll
            for (int i = 0; i < WTM; i++) mfma_f8_acc<A_FMT>(acc[i][j], bf, af[i]);
        }
    };
    // Step kt computes from LDS buffer kt & 1, then moves tile kt+1 (register slot (kt+1) & 1, loaded two
    // steps ago) into the other buffer and refills that slot with tile kt+3.
#define BL_STEP(KT, BUF)                 \
    do {                                 \
        compute(BUF);                    \
        BL_FILL((BUF) ^ 1, (BUF) ^ 1);   \
        BL_LOAD((BUF) ^ 1, (KT) + 3);    \
        __syncthreads();                 \
        __builtin_amdgcn_sched_barrier(0); \
    } while (0)
    // Interleaved step: the fill of the other LDS buffer and the reload of that register slot are cut into WTN
    // portions, one after each group of WTM MFMAs; B fragments are fetched one group ahead.
    constexpr int PIECES = A_CH + B_CH, PPG = (PIECES + WTN - 1) / WTN;
#define BL_STEP_I(KT, BUF)                                                                                     \
    do {                                                                                                       \
        const uint8_t* st__ = lds + (BUF) * STAGE;                                                             \
        uint8_t* fl__ = lds + ((BUF) ^ 1) * STAGE + lw;                                                        \
        const int t__ = (KT) + 3;                                                                              \
        const bool cut__ = t__ >= ksteps || (t__ == kfull && ch_in_tail);                                      \
        v8i af__[WTM], bf__[2];                                                                                \
        _Pragma("unroll") for (int i = 0; i < WTM; i++) af__[i] = frag(st__ + a_rd + i * 2048);                \
        bf__[0] = frag(st__ + b_rd);                                                                           \
        _Pragma("unroll") for (int j = 0; j < WTN; j++) {                                                      \
            if (j + 1 < WTN) bf__[(j + 1) & 1] = frag(st__ + b_rd + (j + 1) * 2048);                           \
            _Pragma("unroll") for (int q = 0; q < PPG; q++) {                                                  \
                const int p = j * PPG + q;                                                                     \
                const int pa = p < A_CH ? p : 0, pb = (p >= A_CH && p < PIECES) ? p - A_CH : 0;   /* in-range when not taken */ \
                if (p < A_CH) {                                                                                \
                    *(v4i*)(fl__ + pa * PASS_ROWS * 128) = ra[(BUF) ^ 1][pa];                                  \
                    ra[(BUF) ^ 1][pa] = __builtin_amdgcn_raw_buffer_load_b128(desc_a, cut__ ? NC_BUF_OOB : avo[pa], t__ * 128, 0); \
                } else if (p < PIECES) {                                                                       \
                    *(v4i*)(fl__ + BM * 128 + pb * PASS_ROWS * 128) = rb[(BUF) ^ 1][pb];                       \
                    rb[(BUF) ^ 1][pb] = __builtin_amdgcn_raw_buffer_load_b128(desc_b, cut__ ? NC_BUF_OOB : bvo[pb], t__ * 128, 0); \
                }                                                                                              \
            }                                                                                                  \
            _Pragma("unroll") for (int i = 0; i < WTM; i++) mfma_f8_acc_ordered<A_FMT>(acc[i][j], bf__[j & 1], af__[i]); \
        }                                                                                                      \
        __syncthreads();                                                                                       \
    } while (0)

    int kt = 0;
    {
        BL_LOAD(0, 0);
        BL_LOAD(1, 1);
        BL_FILL(0, 0);
        BL_LOAD(0, 2);
        __syncthreads();
        if (INTERLEAVE) {
            for (; kt + 1 < ksteps; kt += 2) {
                BL_STEP_I(kt, 0);
                BL_STEP_I(kt + 1, 1);
            }
        } else {
            for (; kt + 1 < ksteps; kt += 2) {
                BL_STEP(kt, 0);
                BL_STEP(kt + 1, 1);
            }
        }
        if (kt < ksteps) compute(0);
    }
#undef BL_STEP_I
#undef BL_LOAD
#undef BL_FILL
#undef BL_STEP

    // the last MFMAs must have left the pipeline before the accumulators are read (16 passes at most)
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
    for (int i = 0; i < WTM; i++)
#pragma unroll
        for (int j = 0; j < WTN; j++) asm volatile("" : "+a"(acc[i][j]));

    // epilogue: the (at most four) per-segment weight scales are fetched once
    const float inv_a = *ep.inv_a;
    float sc[4];
#pragma unroll
    for (int i = 0; i < 4; i++) sc[i] = ep.inv_b[i < ep.segs.nseg ? i : 0];
    bl_epilogue<BM, BN, WGM, WGN, OUT_KIND>(acc, lds, ep, inv_a, sc, m0, n0, M, N);
}


// Per-process caches of what never changes while the process lives: the number of CUs of a device, and which kernels have had their
// dynamic LDS limit raised on which device (hipFuncSetAttribute costs microseconds per call, a launch-bound caller notices).
#include <atomic>
namespace {
constexpr int NC_GEMM_MAX_DEVICES = 64;
int current_device() {
    int dev = 0;
    return hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < NC_GEMM_MAX_DEVICES ? dev : 0;
}
int cu_count() {
    static std::atomic<int> cached[NC_GEMM_MAX_DEVICES];
    const int dev = current_device();
    int cus = cached[dev].load(std::memory_order_relaxed);
    if (cus == 0) {
        cus = 256;
        (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
        cached[dev].store(cus, std::memory_order_relaxed);
    }
    return cus;
}
// slot: one per kernel family that asks for dynamic LDS (the attribute is set for the instantiation actually launched, so the
// cache is keyed by the function pointer as well)
hipError_t reserve_lds(const void* fn, int bytes) {
    struct Entry {
        std::atomic<const void*> fn;
        std::atomic<int> bytes;
    };
    static Entry done[NC_GEMM_MAX_DEVICES][32];
    const int dev = current_device();
    for (auto& e : done[dev]) {
        const void* f = e.fn.load(std::memory_order_acquire);
        if (f == fn && e.bytes.load(std::memory_order_relaxed) >= bytes) return hipSuccess;
        if (f == nullptr || f == fn) {
            const hipError_t rc = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
            if (rc == hipSuccess) {
                e.bytes.store(bytes, std::memory_order_relaxed);
                e.fn.store(fn, std::memory_order_release);
            }
            return rc;
        }
    }
    return hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);      // table full: just set it
}
}  // namespace

int nc_cu_count() { return cu_count(); }

template <int BM, int BN, int WGM, int WGN, bool INTERLEAVE, int A_FMT, int OUT_KIND>
static int launch_bl_as(const uint8_t* a, const uint8_t* b, const EpilogueArgs& ep, int M, int N, int K, hipStream_t s) {
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const size_t lds_bytes = 2 * (size_t)(BM + BN) * 128;
    const void* fn = (const void*)gemm_bl_kernel<BM, BN, WGM, WGN, OUT_KIND, INTERLEAVE, A_FMT>;
    hipError_t e = reserve_lds(fn, (int)lds_bytes);
    if (e != hipSuccess) NC_FAIL(-2, "fp8_gemm: cannot reserve %zu bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
    hipLaunchKernelGGL((gemm_bl_kernel<BM, BN, WGM, WGN, OUT_KIND, INTERLEAVE, A_FMT>), dim3(tiles_m * tiles_n), dim3(64 * WGM * WGN), lds_bytes, s, a, b,
                       ep, M, N, K, tiles_m, tiles_n);
    return 0;
}
template <int BM, int BN, int WGM, int WGN, bool INTERLEAVE = false, int A_FMT = 0>
static int launch_bl(const uint8_t* a, const uint8_t* b, const EpilogueArgs& ep, int M, int N, int K, hipStream_t s) {
    NC_CHECK_ARG((long)M * K < (1L << 31) && (long)N * K < (1L << 31), "fp8_gemm: buffer-load kernels need M*K and N*K below 2^31");
    if (ep.out_kind == 0) return launch_bl_as<BM, BN, WGM, WGN, INTERLEAVE, A_FMT, 0>(a, b, ep, M, N, K, s);
    NC_CHECK_ARG(A_FMT == 0, "fp8_gemm: an e5m2 operand goes with plain bf16 output");
    if (ep.out_kind == 1) return launch_bl_as<BM, BN, WGM, WGN, INTERLEAVE, 0, 1>(a, b, ep, M, N, K, s);
    return launch_bl_as<BM, BN, WGM, WGN, INTERLEAVE, 0, 2>(a, b, ep, M, N, K, s);
}


// ------------------------------------------------------------------------------------------------
// Direct-to-LDS kernels: 256x256x128 tiles, 8 waves (4 x 2, 64x128 outputs each), one workgroup per CU.  The operand
// tiles never pass through registers: every wave issues eight 1 KB `buffer_load_dwordx4 ... lds` per K-step, each of
// which lands 8 rows x 128 bytes in consecutive LDS; the swizzle of the LDS layout (chunk c of row r at slot
// c ^ NC_SWZ(r)) is applied on the global side, lane (sub, slot) fetching chunk slot ^ NC_SWZ(row) of its row, so each
// group of 8 lanes still reads one whole 128-byte line.  That removes the ds_write phase (a 64 KB stage costs ~860
// cycles at the 76 B/clk LDS write rate, next to 2048 cycles of MFMA) and the staging registers.  K must be a multiple
// of 128 (a K tail would need zero fill inside rows, which the range check of the descriptor cannot give); bf16 output.
typedef __attribute__((address_space(3))) void* lds_ptr_t;

struct DlGeom {
    int lane, wave, wm, wn, frow, kb;
    int sub, gch;          // this lane's row inside an 8-row block and the global chunk that belongs in its LDS slot
    int rd_lo, rd_hi;      // fragment read offsets inside a 16-row block
};
__device__ __forceinline__ DlGeom dl_geom() {
    DlGeom g;
    g.lane = threadIdx.x & 63, g.wave = threadIdx.x / 64;
    g.wm = g.wave / 2, g.wn = g.wave % 2;
    g.frow = g.lane & 15, g.kb = g.lane >> 4;
    g.sub = g.lane >> 3, g.gch = (g.lane & 7) ^ g.sub ^ (g.wave & 1);
    const int sw = NC_SWZ(g.frow);
    g.rd_lo = g.frow * 128 + (((2 * g.kb) ^ sw) << 4), g.rd_hi = g.frow * 128 + (((2 * g.kb + 1) ^ sw) << 4);
    return g;
}
__device__ __forceinline__ v8i dl_frag(const uint8_t* base, const DlGeom& g) {
    const v4i lo = *(const v4i*)(base + g.rd_lo);
    const v4i hi = *(const v4i*)(base + g.rd_hi);
    return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}
// FIRST starts the accumulation from zero (C operand 0) instead of reading the accumulators.
template <int A_FMT = 0>
__device__ __forceinline__ void mfma_f8_first_ordered(v4f& acc, const v8i& b, const v8i& a) {
    if (A_FMT == 0) asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, 0" : "=a"(acc) : "v"(b), "v"(a) : "memory");
    else asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, 0 blgp:1" : "=a"(acc) : "v"(b), "v"(a) : "memory");
}
// One K-step of a wave: 64 rows x (128 or, for a half-width tile, 64) columns from the stage at `st`.
// `behind_first_reads` runs once the step's first fragment reads are on their way: the place to issue the operand loads of a later
// step, so that they do not stand between the barrier and the reads the first MFMA waits for.
struct DlNothing {
    __device__ void operator()() const {}
};
template <bool HALF, bool FIRST = false, int A_FMT = 0, typename F = DlNothing>
__device__ __forceinline__ void dl_compute(v4f (&acc)[4][8], const uint8_t* st, const DlGeom& g, F&& behind_first_reads = F()) {
    constexpr int WTN = HALF ? 4 : 8;
    const uint8_t* a = st + g.wm * 64 * 128;
    const uint8_t* b = st + 256 * 128 + g.wn * (HALF ? 64 : 128) * 128;
    v8i af[4], bf[2];
    bf[0] = dl_frag(b, g);
#pragma unroll
    for (int i = 0; i < 4; i++) af[i] = dl_frag(a + i * 2048, g);
    behind_first_reads();
#pragma unroll
    for (int j = 0; j < WTN; j++) {
        if (j + 1 < WTN) bf[(j + 1) & 1] = dl_frag(b + (j + 1) * 2048, g);    // one group ahead of its use
#pragma unroll
        for (int i = 0; i < 4; i++) {
            if (FIRST) mfma_f8_first_ordered<A_FMT>(acc[i][j], bf[j & 1], af[i]);
            else mfma_f8_acc_ordered<A_FMT>(acc[i][j], bf[j & 1], af[i]);
        }
    }
}

// The barrier that ends a K-step of the direct-to-LDS kernels.  The operand loads write LDS behind the compiler's back,
// so the wait for them is explicit: every vector memory operation of this wave has completed (the loads of the next step, and
// the stores of the previous tile's epilogue that were issued behind them), then the workgroup meets.  (Left to the compiler, the
// barrier after the first K-step of a tile came out as vmcnt(6), which on the first tile does not cover all of the step's loads.
// Letting the 16 stores of the previous tile stay in flight across this barrier, vmcnt(16), was measured 1 % slower.)
__device__ __forceinline__ void dl_step_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0x0F70);     // vmcnt(0), other counters untouched
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// One tile per workgroup, launched tile by tile (any M, N).
template <int A_FMT, bool RELU2>
__global__ __launch_bounds__(512) void gemm_dl_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, EpilogueArgs ep, int M,
                                                      int N, int K, int tiles_m, int tiles_n) {
    constexpr int STAGE = 512 * 128;
    extern __shared__ __align__(16) uint8_t lds[];
    int tm, tn;
    tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
    const int m0 = tm * 256, n0 = tn * 256;
    const DlGeom g = dl_geom();
    const int wave_s = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const __amdgpu_buffer_rsrc_t desc_a = __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, M * K, 0x00020000);
    const __amdgpu_buffer_rsrc_t desc_b = __builtin_amdgcn_make_buffer_rsrc((void*)B, 0, N * K, 0x00020000);

    // piece i of this wave is the 1 KB block (wave + 8 i) of the stage: tile rows 8 wave + 64 i + sub, A for i < 4, B after
    uint32_t vo[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int ra = m0 + 8 * g.wave + 64 * i + g.sub, rb = n0 + 8 * g.wave + 64 * i + g.sub;
        vo[i] = ra < M ? (uint32_t)ra * (uint32_t)K + g.gch * 16 : NC_BUF_OOB;
        vo[4 + i] = rb < N ? (uint32_t)rb * (uint32_t)K + g.gch * 16 : NC_BUF_OOB;
    }
    const int ksteps = K / 128;

    v4f acc[4][8];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 8; j++) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

    auto fetch = [&](int t, int buf) {
        if (t < ksteps) {
            uint8_t* st = lds + buf * STAGE + wave_s * 1024;      // uniform: the LDS address of a load goes through M0
#pragma unroll
            for (int i = 0; i < 8; i++)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(i < 4 ? desc_a : desc_b, (lds_ptr_t)(st + i * 8192), 16, vo[i], t * 128, 0, 0);
        }
    };
    // step kt computes from buffer kt & 1 while the loads of step kt + 1 land in the other one; the barrier at its end
    // says both that those loads are complete for every wave and that nobody reads buffer kt & 1 any more
    fetch(0, 0);
    dl_step_barrier();
    int kt = 0;
    for (; kt + 1 < ksteps; kt += 2) {
        dl_compute<false, false, A_FMT>(acc, lds, g, [&] { fetch(kt + 1, 1); });
        dl_step_barrier();
        dl_compute<false, false, A_FMT>(acc, lds + STAGE, g, [&] { fetch(kt + 2, 0); });
        dl_step_barrier();
    }
    if (kt < ksteps) dl_compute<false, false, A_FMT>(acc, lds, g);

    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 8; j++) asm volatile("" : "+a"(acc[i][j]));
    const float inv_a = *ep.inv_a;
    float sc[4];
#pragma unroll
    for (int i = 0; i < 4; i++) sc[i] = ep.inv_b[i < ep.segs.nseg ? i : 0];
    bl_epilogue<256, 256, 4, 2, RELU2 ? 2 : 0>(acc, lds, ep, inv_a, sc, m0, n0, M, N);
}

// ------------------------------------------------------------------------------------------------
// The same tile-by-tile kernel with a narrower tile: 256 rows x 32 NJ columns (NJ = 4 .. 7 blocks of 16 columns per wave).  A launch of
// one round -- a prompt of one to two thousand rows -- lasts as long as one tile, whatever the number of CUs that got one: 1792 x 4992
// is 140 tiles of 256 x 256 on 256 CUs, but 224 tiles of 256 x 160, each 5/8 of the matrix work.  The launch picks NJ (dl_pick_nj).
// A wave's B pieces beyond the tile's 32 NJ rows are not loaded (the test is uniform per wave), the stage is 256 + 32 NJ rows.
template <int NJ, int A_FMT = 0, typename F = DlNothing>
__device__ __forceinline__ void dln_compute(v4f (&acc)[4][NJ], const uint8_t* st, const DlGeom& g, F&& behind_first_reads = F()) {
    const uint8_t* a = st + g.wm * 64 * 128;
    const uint8_t* b = st + 256 * 128 + g.wn * (16 * NJ) * 128;
    v8i af[4], bf[2];
    bf[0] = dl_frag(b, g);
#pragma unroll
    for (int i = 0; i < 4; i++) af[i] = dl_frag(a + i * 2048, g);
    behind_first_reads();
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        if (j + 1 < NJ) bf[(j + 1) & 1] = dl_frag(b + (j + 1) * 2048, g);    // one group ahead of its use
#pragma unroll
        for (int i = 0; i < 4; i++) mfma_f8_acc_ordered<A_FMT>(acc[i][j], bf[j & 1], af[i]);
    }
}

// Epilogue for a wave block of 64 x 16 NJ outputs, bf16 (RELU2: relu(v)^2 and its maximum): the block is parked in the wave's own
// LDS region (rows of 32 NJ + 16 bytes) and leaves as a linear sequence of 16-byte pieces, so a store instruction writes runs of
// 32 NJ contiguous bytes per row.
template <int NJ, bool RELU2>
__device__ __forceinline__ void dln_epilogue(v4f (&acc)[4][NJ], uint8_t* lds, const EpilogueArgs& ep, float inv_a, const float (&sc)[4],
                                             const DlGeom& g, int m0, int n0, int M, int N) {
    constexpr int WCOLS = 16 * NJ, ROWB = WCOLS * 2, PITCH = ROWB + 16, LPR = ROWB / 16, PIECES = 64 * LPR;
    static_assert(8 * 64 * PITCH <= 2 * (256 + 32 * NJ) * 128, "epilogue staging");
    float am = 0.f;
    __syncthreads();                                       // every wave is done with the operand tiles
    uint8_t* reg = lds + g.wave * 64 * PITCH;
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const int n = n0 + g.wn * WCOLS + j * 16 + 4 * g.kb;
        float inv_b = sc[0];
#pragma unroll
        for (int i = 0; i < 3; i++)
            if (i + 1 < ep.segs.nseg && n >= ep.segs.end[i]) inv_b = sc[i + 1];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int row = i * 16 + g.frow;
            const v4f a4 = acc[i][j];
            float o4[4];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                o4[r] = (a4[r] * inv_a) * inv_b;
                if (RELU2) o4[r] = relu2_of(o4[r]);
            }
            *(uint2*)(reg + row * PITCH + j * 32 + g.kb * 8) = make_uint2(pack_bf16_hw(o4[0], o4[1]), pack_bf16_hw(o4[2], o4[3]));
        }
    }
    // the region is private to the wave: its own LDS writes only have to land before its reads
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_s_waitcnt(0xc07f);                    // lgkmcnt(0)
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const bool vec16 = (ep.ldc % 8 == 0) && (((uintptr_t)ep.out & 15) == 0);
#pragma unroll
    for (int it = 0; it < PIECES / 64; it++) {
        const int id = it * 64 + g.lane, row = id / LPR, c = id % LPR;
        const int m = m0 + g.wm * 64 + row, n = n0 + g.wn * WCOLS + c * 8;
        const uint4 v = *(const uint4*)(reg + row * PITCH + c * 16);
        if (m >= M || n >= N) continue;
        if (RELU2) am = amax_join(am, max_bf16x8(v, N - n));
        bf16_t* o = (bf16_t*)ep.out + (size_t)m * ep.ldc + n;
        if (n + 8 <= N) {
            if (vec16) __builtin_nontemporal_store(v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w}, (v4i*)o);
            else {
                *(uint2*)o = make_uint2(v.x, v.y);
                *(uint2*)(o + 4) = make_uint2(v.z, v.w);
            }
        } else {
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
            for (int r = 0; r < 8 && n + r < N; r++) o[r] = (bf16_t)(w[r >> 1] >> ((r & 1) * 16));
        }
    }
    if (RELU2) {
        __shared__ float wave_am[8];
        am = wave_amax(am);
        if (g.lane == 0) wave_am[g.wave] = am;
        __syncthreads();
        if (threadIdx.x == 0) {
            float t = wave_am[0];
#pragma unroll
            for (int w = 1; w < 8; w++) t = amax_join(t, wave_am[w]);
            amax_publish(ep.out_amax, t);
        }
    }
}

// the operand loads of one K-step: `st` is the wave's first 1 KB piece of the stage (uniform: the LDS address of a load goes through M0)
template <int NJ>
__device__ __forceinline__ void dln_fetch(const uint8_t* A, int a_bytes, const uint8_t* B, int b_bytes, uint8_t* st, const uint32_t* vo_a,
                                          const uint32_t* vo_b, int wave_s, int k_off) {
    const __amdgpu_buffer_rsrc_t desc_a = __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, a_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t desc_b = __builtin_amdgcn_make_buffer_rsrc((void*)B, 0, b_bytes, 0x00020000);
#pragma unroll
    for (int i = 0; i < 4; i++) __builtin_amdgcn_raw_ptr_buffer_load_lds(desc_a, (lds_ptr_t)(st + i * 8192), 16, vo_a[i], k_off, 0, 0);
#pragma unroll
    for (int i = 0; i < (4 * NJ + 7) / 8; i++)
        if (wave_s + 8 * i < 4 * NJ)                      // uniform per wave
            __builtin_amdgcn_raw_ptr_buffer_load_lds(desc_b, (lds_ptr_t)(st + 256 * 128 + i * 8192), 16, vo_b[i], k_off, 0, 0);
}

template <int NJ, bool RELU2, int A_FMT = 0>
__global__ __launch_bounds__(512) void gemm_dln_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, EpilogueArgs ep, int M,
                                                       int N, int K, int tiles_m, int tiles_n) {
    constexpr int BN = 32 * NJ, STAGE = (256 + BN) * 128, B_PIECES = BN / 8, B_ROUNDS = (B_PIECES + 7) / 8;
    extern __shared__ __align__(16) uint8_t lds[];
    int tm, tn;
    tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
    const int m0 = tm * 256, n0 = tn * BN;
    const DlGeom g = dl_geom();
    const int wave_s = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

    // piece i of this wave is the 1 KB block (wave + 8 i) of its operand's part of the stage: tile rows 8 wave + 64 i + sub
    uint32_t vo_a[4], vo_b[B_ROUNDS];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int ra = m0 + 8 * g.wave + 64 * i + g.sub;
        vo_a[i] = ra < M ? (uint32_t)ra * (uint32_t)K + g.gch * 16 : NC_BUF_OOB;
    }
#pragma unroll
    for (int i = 0; i < B_ROUNDS; i++) {
        const int rb = n0 + 8 * g.wave + 64 * i + g.sub;
        vo_b[i] = rb < N ? (uint32_t)rb * (uint32_t)K + g.gch * 16 : NC_BUF_OOB;
    }
    const int ksteps = K / 128;

    v4f acc[4][NJ];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < NJ; j++) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

    auto fetch = [&](int t, int buf) {
        if (t < ksteps) dln_fetch<NJ>(A, M * K, B, N * K, lds + buf * STAGE + wave_s * 1024, vo_a, vo_b, wave_s, t * 128);
    };
    fetch(0, 0);
    dl_step_barrier();
    int kt = 0;
    for (; kt + 1 < ksteps; kt += 2) {
        dln_compute<NJ, A_FMT>(acc, lds, g, [&] { fetch(kt + 1, 1); });
        dl_step_barrier();
        dln_compute<NJ, A_FMT>(acc, lds + STAGE, g, [&] { fetch(kt + 2, 0); });
        dl_step_barrier();
    }
    if (kt < ksteps) dln_compute<NJ, A_FMT>(acc, lds, g);

    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < NJ; j++) asm volatile("" : "+a"(acc[i][j]));
    const float inv_a = *ep.inv_a;
    float sc[4];
#pragma unroll
    for (int i = 0; i < 4; i++) sc[i] = ep.inv_b[i < ep.segs.nseg ? i : 0];
    dln_epilogue<NJ, RELU2>(acc, lds, ep, inv_a, sc, g, m0, n0, M, N);
}

// the operand loads of one K-step of gemm_dr_kernel: `st` is the wave's first 1 KB piece of the stage, its pieces lie 4 KB apart
template <int A_P>
__device__ __forceinline__ void dr_fetch(const uint8_t* A, int a_bytes, const uint8_t* B, int b_bytes, uint8_t* st, int b_part, const uint32_t* vo_a,
                                         const uint32_t* vo_b, int k_off) {
    const __amdgpu_buffer_rsrc_t desc_a = __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, a_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t desc_b = __builtin_amdgcn_make_buffer_rsrc((void*)B, 0, b_bytes, 0x00020000);
#pragma unroll
    for (int i = 0; i < A_P; i++) __builtin_amdgcn_raw_ptr_buffer_load_lds(desc_a, (lds_ptr_t)(st + i * 4096), 16, vo_a[i], k_off, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; i++) __builtin_amdgcn_raw_ptr_buffer_load_lds(desc_b, (lds_ptr_t)(st + b_part + i * 4096), 16, vo_b[i], k_off, 0, 0);
}

// ------------------------------------------------------------------------------------------------
// Direct-to-LDS tiles for a narrow weight under a prompt: BM x 128 outputs (BM = 64, 96, 128), four waves (2 x 2, BM/2 x 64 each), and a
// ring of FOUR operand stages.  Where the 256-row tiles would leave most CUs without one (1792 x 1664: 49 or 91 tiles), the launch is
// one round of small tiles, one workgroup of one wave per SIMD on each CU: nothing hides the latency of a K-step's operands then but
// the depth of the prefetch.  The register-staged tiles have two K-steps in flight and pay a ds_write phase per step; here the operands
// of three steps ahead are on their way into LDS while one is multiplied, and a step costs its MFMAs or the L2's bandwidth, whichever
// is longer.  Past the end of K the loads are issued all the same (the first step's operands again, into stages nobody reads), so that
// the count the barrier waits for is the same in every step.
template <int BM, int OUT_KIND>
__global__ __launch_bounds__(256) void gemm_dr_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, EpilogueArgs ep, int M,
                                                      int N, int K, int tiles_m, int tiles_n) {
    constexpr int WTM = BM / 32, STAGE = (BM + 128) * 128, A_P = BM / 32, LOADS = A_P + 4;
    // s_waitcnt vmcnt(2 * LOADS), other counters untouched: the loads of the two youngest steps may still be in flight
    constexpr int WAIT2 = 0x0F70 | ((2 * LOADS) & 15) | (((2 * LOADS) >> 4) << 14);
    extern __shared__ __align__(16) uint8_t lds[];
    int tm, tn;
    tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * 128;
    DlGeom g = dl_geom();
    g.wm = g.wave >> 1, g.wn = g.wave & 1;
    const int wave_s = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // piece i of this wave is the 1 KB block (wave + 4 i) of its operand's part of the stage: tile rows 8 wave + 32 i + sub
    uint32_t vo_a[A_P], vo_b[4];
#pragma unroll
    for (int i = 0; i < A_P; i++) {
        const int ra = m0 + 8 * g.wave + 32 * i + g.sub;
        vo_a[i] = ra < M ? (uint32_t)ra * (uint32_t)K + g.gch * 16 : NC_BUF_OOB;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int rb = n0 + 8 * g.wave + 32 * i + g.sub;
        vo_b[i] = rb < N ? (uint32_t)rb * (uint32_t)K + g.gch * 16 : NC_BUF_OOB;
    }
    const int ksteps = K / 128;

    v4f acc[WTM][4];
#pragma unroll
    for (int i = 0; i < WTM; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

    auto fetch = [&](int t) {
        dr_fetch<A_P>(A, M * K, B, N * K, lds + (t & 3) * STAGE + wave_s * 1024, BM * 128, vo_a, vo_b, t < ksteps ? t * 128 : 0);
    };
    auto compute = [&](int t) {
        const uint8_t* st = lds + (t & 3) * STAGE;
        const uint8_t* a = st + g.wm * (BM / 2) * 128;
        const uint8_t* b = st + BM * 128 + g.wn * 64 * 128;
        v8i af[WTM], bf[2];
        bf[0] = dl_frag(b, g);
#pragma unroll
        for (int i = 0; i < WTM; i++) af[i] = dl_frag(a + i * 2048, g);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (j + 1 < 4) bf[(j + 1) & 1] = dl_frag(b + (j + 1) * 2048, g);
#pragma unroll
            for (int i = 0; i < WTM; i++) mfma_f8_acc_ordered<0>(acc[i][j], bf[j & 1], af[i]);
        }
    };
    fetch(0);
    fetch(1);
    fetch(2);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(WAIT2);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    for (int kt = 0; kt < ksteps; kt++) {
        fetch(kt + 3);                       // into the stage that was read in step kt - 1: everyone is past the barrier that ended it
        compute(kt);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(WAIT2);   // the operands of step kt + 1 have landed (this wave's share; the barrier says everybody's)
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    }
    // the loads past the end of K are still landing in the stages: they must be done before the epilogue reuses the memory
    dl_step_barrier();

    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
    for (int i = 0; i < WTM; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) asm volatile("" : "+a"(acc[i][j]));
    const float inv_a = *ep.inv_a;
    float sc[4];
#pragma unroll
    for (int i = 0; i < 4; i++) sc[i] = ep.inv_b[i < ep.segs.nseg ? i : 0];
    bl_epilogue<BM, 128, 2, 2, OUT_KIND>(acc, lds, ep, inv_a, sc, m0, n0, M, N);
}

// Epilogue of the persistent kernel: the wave's 64 x (128 | 64) block leaves 16 rows at a time through a 4 KB LDS region of
// its own (past the two operand stages, so the loads of the next tile keep landing meanwhile), every store instruction
// writing whole 128-byte lines.
template <bool HALF, bool RELU2>
__device__ __forceinline__ void dlp_epilogue(v4f (&acc)[4][8], uint8_t* reg, const EpilogueArgs& ep, float inv_a, const float (&sc)[4],
                                             const DlGeom& g, int m0, int n0, int M, int N) {
    constexpr int WTN = HALF ? 4 : 8, WCOLS = WTN * 16, ROWB = WCOLS * 2, LPR = ROWB / 16, RPI = 64 / LPR;
    const bool vec16 = (ep.ldc % 8 == 0) && (((uintptr_t)ep.out & 15) == 0);
    const uint32_t reg_off = (uint32_t)(uintptr_t)(lds_ptr_t)reg;       // the region's byte offset in LDS
    constexpr bool relu2 = RELU2;
    float am = 0.f;
    const int lrow_e = g.lane / LPR, c = g.lane % LPR;
    const int n_st = n0 + g.wn * WCOLS + c * 8;
    float inv_b[WTN];
#pragma unroll
    for (int j = 0; j < WTN; j++) {
        const int n = n0 + g.wn * WCOLS + j * 16 + 4 * g.kb;
        inv_b[j] = sc[0];
#pragma unroll
        for (int i = 0; i < 3; i++)
            if (i + 1 < ep.segs.nseg && n >= ep.segs.end[i]) inv_b[j] = sc[i + 1];
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
        for (int j = 0; j < WTN; j++) {
            const int chunk = 2 * j + (g.kb >> 1);
            const v4f a4 = acc[i][j];
            float o4[4];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                o4[r] = (a4[r] * inv_a) * inv_b[j];
                if (relu2) o4[r] = relu2_of(o4[r]);
            }
            const v2i pk = {(int)pack_bf16_hw(o4[0], o4[1]), (int)pack_bf16_hw(o4[2], o4[3])};
            // written and read back with explicit instructions: an LDS access the compiler generates here waits for the next
            // tile's operand loads (vmcnt(0)), because it cannot tell this region from the stages they are landing in
            asm volatile("ds_write_b64 %0, %1" ::"v"(reg_off + g.frow * ROWB + ((chunk ^ (g.frow & 7)) << 4) + (g.kb & 1) * 8), "v"(pk) : "memory");
        }
        // the region is private to the wave: its own LDS writes only have to land before its reads
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_s_waitcnt(0xc07f);                    // lgkmcnt(0)
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        v4i rd[16 / RPI];
#pragma unroll
        for (int it = 0; it < 16 / RPI; it++) {
            const int row = it * RPI + lrow_e;
            asm volatile("ds_read_b128 %0, %1" : "=v"(rd[it]) : "v"(reg_off + row * ROWB + ((c ^ (row & 7)) << 4)) : "memory");
        }
        if (16 / RPI == 4) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(rd[0]), "+v"(rd[1]), "+v"(rd[2 % (16 / RPI)]), "+v"(rd[3 % (16 / RPI)])::"memory");
        else asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(rd[0]), "+v"(rd[1])::"memory");
#pragma unroll
        for (int it = 0; it < 16 / RPI; it++) {
            const int row = it * RPI + lrow_e;
            const int m = m0 + g.wm * 64 + i * 16 + row;
            const uint4 v = make_uint4((uint32_t)rd[it][0], (uint32_t)rd[it][1], (uint32_t)rd[it][2], (uint32_t)rd[it][3]);
            if (m >= M || n_st >= N) continue;
            if (relu2) am = amax_join(am, max_bf16x8(v, N - n_st));
            bf16_t* o = (bf16_t*)ep.out + (size_t)m * ep.ldc + n_st;
            if (n_st + 8 <= N) {
                if (vec16) __builtin_nontemporal_store(v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w}, (v4i*)o);
                else {
                    *(uint2*)o = make_uint2(v.x, v.y);
                    *(uint2*)(o + 4) = make_uint2(v.z, v.w);
                }
            } else {
                const uint32_t w[4] = {v.x, v.y, v.z, v.w};
                for (int r = 0; r < 8 && n_st + r < N; r++) o[r] = (bf16_t)(w[r >> 1] >> ((r & 1) * 16));
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");   // the reads are done before the next 16 rows overwrite the region
    }
    if (relu2) {
        am = wave_amax(am);
        if (g.lane == 0) amax_publish(ep.out_amax, am);
    }
}

// Persistent form: 8 x 32 workgroups, each walking its own list of tiles as one uninterrupted stream of K-steps (the
// first loads of the next tile are in flight while the current one is finished and stored).  XCD x (workgroup id % 8)
// owns `rows_per_xcd` consecutive tile rows; its 32 workgroups form rows_per_xcd x (32 / rows_per_xcd) slots, slot
// (r, c) owning tile row r and the c-th share of the N range counted in 128-column units.  A share is cut into full
// 256-column tiles plus, when its unit count is odd, one half-width tile at its end, so no workgroup rounds its work up
// to whole 256x256 tiles.
template <int A_FMT, bool RELU2>
__global__ __launch_bounds__(512) void gemm_dlp_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, EpilogueArgs ep,
                                                       int M, int N, int K, int rows_per_xcd, int nu) {
    constexpr int STAGE = 512 * 128;
    extern __shared__ __align__(16) uint8_t lds[];
    const DlGeom g = dl_geom();
    const int wave_s = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int xcd = blockIdx.x % 8, slot = blockIdx.x / 8;
    const int cols = 32 / rows_per_xcd;
    const int sc_c = slot % cols, sc_r = slot / cols;
    const int m0 = (xcd * rows_per_xcd + sc_r) * 256;
    const int ub = nu * sc_c / cols, ue = nu * (sc_c + 1) / cols;
    const int count = ue - ub, nitems = (count + 1) / 2;
    const bool has_half = count & 1;
    if (nitems == 0) return;
    // A share with an odd unit count has one half-width tile: at its end in the even slots, at its start in the odd ones, so that the
    // workgroups do not all reach their epilogues -- 128 KB of stores each -- at the same moments (M = 8192, N = 4992: 63 -> 61 us,
    // N = 6656: 82.5 -> 80 us, alternating in one process)
    const bool half_first = has_half && (slot & 1);
    auto item = [&](int q, int& n0, bool& half) {
        half = has_half && q == (half_first ? 0 : nitems - 1);
        n0 = (ub + 2 * q - ((half_first && q > 0) ? 1 : 0)) * 128;
    };

    const __amdgpu_buffer_rsrc_t desc_a = __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, M * K, 0x00020000);
    const __amdgpu_buffer_rsrc_t desc_b = __builtin_amdgcn_make_buffer_rsrc((void*)B, 0, N * K, 0x00020000);
    const int ksteps = K / 128;
    uint32_t vo_a[4], vo_b[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int ra = m0 + 8 * g.wave + 64 * i + g.sub;
        vo_a[i] = ra < M ? (uint32_t)ra * (uint32_t)K + g.gch * 16 : NC_BUF_OOB;
    }
    // the fetch cursor runs ahead of the compute cursor, across tile boundaries
    int fq = 0, fkt = 0, fbuf = 0;
    bool f_half = false;
    auto set_fetch_item = [&](int q) {
        int n0;
        item(q, n0, f_half);
        // The lane's row and chunk are worked out again here from the lane id rather than kept in registers across the K loop:
        // the kernel has none to spare (kept live, the row offset was spilled, and its reload put a vmcnt(0) into the stream
        // of operand loads once per tile).  The asm keeps the compiler from hoisting the computation back out.
        int lane_id;
        asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane_id));
        const int sub = lane_id >> 3, gch = (lane_id & 7) ^ sub ^ (wave_s & 1);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int rb = n0 + 8 * wave_s + 64 * i + sub;
            vo_b[i] = rb < N ? (uint32_t)rb * (uint32_t)K + gch * 16 : NC_BUF_OOB;
        }
    };
    auto fetch_next = [&]() {
        if (fq >= nitems) return;
        uint8_t* st = lds + fbuf * STAGE + wave_s * 1024;      // uniform: the LDS address of a load goes through M0
#pragma unroll
        for (int i = 0; i < 4; i++) __builtin_amdgcn_raw_ptr_buffer_load_lds(desc_a, (lds_ptr_t)(st + i * 8192), 16, vo_a[i], fkt * 128, 0, 0);
#pragma unroll
        for (int i = 0; i < 2; i++) __builtin_amdgcn_raw_ptr_buffer_load_lds(desc_b, (lds_ptr_t)(st + (4 + i) * 8192), 16, vo_b[i], fkt * 128, 0, 0);
        if (!f_half) {
#pragma unroll
            for (int i = 2; i < 4; i++) __builtin_amdgcn_raw_ptr_buffer_load_lds(desc_b, (lds_ptr_t)(st + (4 + i) * 8192), 16, vo_b[i], fkt * 128, 0, 0);
        }
        fbuf ^= 1;
        if (++fkt == ksteps) {
            fkt = 0;
            if (++fq < nitems) set_fetch_item(fq);
        }
    };

    // the scales live in scalar registers across the K loops (as vector registers they were spilled, and the reloads in the
    // epilogue waited for the operand loads issued just before it)
    auto uniform = [](float v) { return __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(v))); };
    const float inv_a = uniform(*ep.inv_a);
    float sc[4];
#pragma unroll
    for (int i = 0; i < 4; i++) sc[i] = uniform(ep.inv_b[i < ep.segs.nseg ? i : 0]);
    uint8_t* epi = lds + 2 * STAGE + wave_s * 4096;

    // Invariant at the top of every K-step: its own operands have landed (the barrier before it) and the loads of the step
    // after it are already in flight.  After the barrier that ends a step, its buffer is free and takes the loads of
    // the step after next; at the end of a tile those are the next tile's, and they travel while the tile is stored.
    set_fetch_item(0);
    fetch_next();
    dl_step_barrier();
    fetch_next();
    int buf = 0;
    auto tile = [&](int n0, auto half_tag) {
        constexpr bool HALF = decltype(half_tag)::value;
        v4f acc[4][8];
        dl_compute<HALF, true, A_FMT>(acc, lds + buf * STAGE, g);
        dl_step_barrier();
        buf ^= 1;
        for (int kt = 1; kt < ksteps; kt++) {
            // the loads into the buffer that the barrier has just freed go out behind this step's first fragment reads
            dl_compute<HALF, false, A_FMT>(acc, lds + buf * STAGE, g, fetch_next);
            dl_step_barrier();
            buf ^= 1;
        }
        fetch_next();
        // the last MFMAs must have left the pipeline before the accumulators are read
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < (HALF ? 4 : 8); j++) asm volatile("" : "+a"(acc[i][j]));
        int m0_here = m0;
        asm volatile("" : "+s"(m0_here));          // keeps the store addresses of all tiles from being precomputed (and spilled)
        // the epilogue's lane geometry is worked out afresh (see set_fetch_item): values kept for it across the K loop were
        // spilled, and their reloads at this point waited for the next tile's operand loads that had just been issued
        int lane_e;
        asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane_e));
        DlGeom ge;
        ge.lane = lane_e, ge.wave = wave_s, ge.wm = wave_s / 2, ge.wn = wave_s % 2, ge.frow = lane_e & 15, ge.kb = lane_e >> 4;
        ge.sub = ge.gch = ge.rd_lo = ge.rd_hi = 0;
        dlp_epilogue<HALF, RELU2>(acc, epi, ep, inv_a, sc, ge, m0_here, n0, M, N);
    };
    for (int q = 0; q < nitems; q++) {
        int n0;
        bool half;
        item(q, n0, half);
        if (half) tile(n0, std::true_type{});
        else tile(n0, std::false_type{});
    }
}

static bool dlp_eligible(int M, int /*N*/, int K) {
    const int tiles_m = (M + 255) / 256;
    if (K % 128 != 0 || tiles_m % 8 != 0) return false;
    const int rx = tiles_m / 8;
    return rx >= 1 && rx <= 32 && (rx & (rx - 1)) == 0;
}

template <int A_FMT, bool RELU2>
static int launch_dl_as(const uint8_t* a, const uint8_t* b, const EpilogueArgs& ep, int M, int N, int K, bool persistent, hipStream_t s) {
    const int tiles_m = (M + 255) / 256, tiles_n = (N + 255) / 256;
    const size_t lds_bytes = 2 * 512 * 128 + (persistent ? 8 * 4096 : 0);
    const void* fn = persistent ? (const void*)gemm_dlp_kernel<A_FMT, RELU2> : (const void*)gemm_dl_kernel<A_FMT, RELU2>;
    hipError_t e = reserve_lds(fn, (int)lds_bytes);
    if (e != hipSuccess) NC_FAIL(-2, "fp8_gemm: cannot reserve %zu bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
    if (persistent)
        hipLaunchKernelGGL((gemm_dlp_kernel<A_FMT, RELU2>), dim3(256), dim3(512), lds_bytes, s, a, b, ep, M, N, K, tiles_m / 8, (N + 127) / 128);
    else
        hipLaunchKernelGGL((gemm_dl_kernel<A_FMT, RELU2>), dim3(tiles_m * tiles_n), dim3(512), lds_bytes, s, a, b, ep, M, N, K, tiles_m, tiles_n);
    return 0;
}

// Blocks of 16 columns per wave (tile width 32 NJ, NJ = 4 .. 8) for a launch of 256-row tiles that is not persistent.  Measured at
// K = 1664 a round of tiles lasts about 6 + NJ units (the A side of a K-step, the launch and the epilogue cost the same at any width:
// 16.6 / 18.5 / 19.7 / 22.0 / 23.4 us for NJ = 4 .. 8 with 80 tiles) and up to a fifth longer when every CU has a tile (28.1 us with 240
// tiles of 256 x 256).  The full width is kept unless a narrower tile is at least 8 % cheaper by that count:
// 1792 x 4992: 140 tiles of 256 x 256, 24.1 us -> 224 of 256 x 160, 20.6 us; 1792 x 6656: 182 tiles, 25.4 -> 245 of 256 x 192, 22.2 us.
static double dl_cost(int nj, int M, int N, int cus, long* tiles_out) {
    const long tiles = (long)((M + 255) / 256) * ((N + 32 * nj - 1) / (32 * nj));
    if (tiles_out) *tiles_out = tiles;
    double cost = 0.0;
    for (long left = tiles; left > 0; left -= cus) cost += (6.0 + nj) * (1.0 + 0.2 * (double)(left < cus ? left : cus) / cus);
    return cost;
}
static int dl_pick_nj(int M, int N) {
    const int cus = cu_count();
    int best = 8;
    const double full = dl_cost(8, M, N, cus, nullptr);
    double best_cost = 0.92 * full;
    for (int nj = 7; nj >= 4; nj--) {
        const double c = dl_cost(nj, M, N, cus, nullptr);
        if (c < best_cost) best = nj, best_cost = c;
    }
    return best;
}
// whether some narrower tile gives the launch one round with at least 150 of 256 CUs busy (then the 256-row tiles beat the 128 x 128
// ones although the 256 x 256 tiles would leave most CUs idle: 1024 x 4992 x 1664 16.6 us against 18.4)
static bool dl_narrow_fills(int M, int N) {
    const int cus = cu_count();
    for (int nj = 4; nj <= 7; nj++) {
        long tiles;
        (void)dl_cost(nj, M, N, cus, &tiles);
        if (tiles <= cus && 256 * tiles >= 150L * cus) return true;
    }
    return false;
}
template <int NJ, bool RELU2, int A_FMT>
static int launch_dln_as(const uint8_t* a, const uint8_t* b, const EpilogueArgs& ep, int M, int N, int K, hipStream_t s) {
    const int tiles_m = (M + 255) / 256, tiles_n = (N + 32 * NJ - 1) / (32 * NJ);
    const size_t lds_bytes = 2 * (256 + 32 * NJ) * 128;
    const void* fn = (const void*)gemm_dln_kernel<NJ, RELU2, A_FMT>;
    hipError_t e = reserve_lds(fn, (int)lds_bytes);
    if (e != hipSuccess) NC_FAIL(-2, "fp8_gemm: cannot reserve %zu bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
    hipLaunchKernelGGL((gemm_dln_kernel<NJ, RELU2, A_FMT>), dim3(tiles_m * tiles_n), dim3(512), lds_bytes, s, a, b, ep, M, N, K, tiles_m, tiles_n);
    return 0;
}
template <int NJ>
static int launch_dln_nj(int a_fmt, const uint8_t* a, const uint8_t* b, const EpilogueArgs& ep, int M, int N, int K, hipStream_t s) {
    if (a_fmt == 1) return launch_dln_as<NJ, false, 1>(a, b, ep, M, N, K, s);
    return ep.out_kind == 2 ? launch_dln_as<NJ, true, 0>(a, b, ep, M, N, K, s) : launch_dln_as<NJ, false, 0>(a, b, ep, M, N, K, s);
}
// bf16 or (e4m3 first operand only) relu^2 output, K a multiple of 128
static int launch_dln(int nj, int a_fmt, const uint8_t* a, const uint8_t* b, const EpilogueArgs& ep, int M, int N, int K, hipStream_t s) {
    NC_CHECK_ARG((long)M * K < (1L << 31) && (long)N * K < (1L << 31), "fp8_gemm: buffer-load kernels need M*K and N*K below 2^31");
    NC_CHECK_ARG(K % 128 == 0, "fp8_gemm: the direct-to-LDS kernels need K %% 128 == 0, got %d", K);
    NC_CHECK_ARG(ep.out_kind != 1, "fp8_gemm: the direct-to-LDS kernels write bf16 only");
    NC_CHECK_ARG(a_fmt == 0 || ep.out_kind == 0, "fp8_gemm: the relu^2 epilogue goes with an e4m3 first operand");
    switch (nj) {
        case 4: return launch_dln_nj<4>(a_fmt, a, b, ep, M, N, K, s);
        case 5: return launch_dln_nj<5>(a_fmt, a, b, ep, M, N, K, s);
        case 6: return launch_dln_nj<6>(a_fmt, a, b, ep, M, N, K, s);
        case 7: return launch_dln_nj<7>(a_fmt, a, b, ep, M, N, K, s);
    }
    NC_FAIL(-1, "fp8_gemm: tile widths of 128, 160, 192 and 224 columns only, not %d", 32 * nj);
}

template <int BM, int OUT_KIND>
static int launch_dr_as(const uint8_t* a, const uint8_t* b, const EpilogueArgs& ep, int M, int N, int K, hipStream_t s) {
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + 127) / 128;
    const size_t lds_bytes = 4 * (size_t)(BM + 128) * 128;
    const void* fn = (const void*)gemm_dr_kernel<BM, OUT_KIND>;
    hipError_t e = reserve_lds(fn, (int)lds_bytes);
    if (e != hipSuccess) NC_FAIL(-2, "fp8_gemm: cannot reserve %zu bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
    hipLaunchKernelGGL((gemm_dr_kernel<BM, OUT_KIND>), dim3(tiles_m * tiles_n), dim3(256), lds_bytes, s, a, b, ep, M, N, K, tiles_m, tiles_n);
    return 0;
}
// e4m3 operands, bf16 or relu^2 output, K a multiple of 128
template <int BM>
static int launch_dr(const uint8_t* a, const uint8_t* b, const EpilogueArgs& ep, int M, int N, int K, hipStream_t s) {
    NC_CHECK_ARG((long)M * K < (1L << 31) && (long)N * K < (1L << 31), "fp8_gemm: buffer-load kernels need M*K and N*K below 2^31");
    NC_CHECK_ARG(K % 128 == 0, "fp8_gemm: the direct-to-LDS kernels need K %% 128 == 0, got %d", K);
    NC_CHECK_ARG(ep.out_kind != 1, "fp8_gemm: the direct-to-LDS kernels write bf16 only");
    return ep.out_kind == 2 ? launch_dr_as<BM, 2>(a, b, ep, M, N, K, s) : launch_dr_as<BM, 0>(a, b, ep, M, N, K, s);
}

// the relu^2 epilogue is a variant of its own so that the plain kernels keep their register budget
template <int A_FMT>
static int launch_dl(const uint8_t* a, const uint8_t* b, const EpilogueArgs& ep, int M, int N, int K, bool persistent, hipStream_t s) {
    NC_CHECK_ARG((long)M * K < (1L << 31) && (long)N * K < (1L << 31), "fp8_gemm: buffer-load kernels need M*K and N*K below 2^31");
    NC_CHECK_ARG(K % 128 == 0, "fp8_gemm: the direct-to-LDS kernels need K %% 128 == 0, got %d", K);
    NC_CHECK_ARG(ep.out_kind != 1, "fp8_gemm: the direct-to-LDS kernels write bf16 only");
    if (persistent)
        NC_CHECK_ARG(dlp_eligible(M, N, K), "fp8_gemm: the persistent kernel needs M/256 (rounded up) to be 8, 16, ... 256 tile rows, got M=%d", M);
    if (A_FMT == 0 && ep.out_kind == 2) return launch_dl_as<0, true>(a, b, ep, M, N, K, persistent, s);
    NC_CHECK_ARG(ep.out_kind == 0, "fp8_gemm: the relu^2 epilogue goes with an e4m3 first operand");
    return launch_dl_as<A_FMT, false>(a, b, ep, M, N, K, persistent, s);
}

// ------------------------------------------------------------------------------------------------
template <int BM, int BN>
static int launch_tile(const uint8_t* a, const uint8_t* b, const EpilogueArgs& ep, int M, int N, int K, hipStream_t s) {
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const size_t lds_bytes = 2 * (size_t)(BM + BN) * 128;
    hipError_t e = reserve_lds((const void*)gemm_tile_kernel<BM, BN>, (int)lds_bytes);
    if (e != hipSuccess) NC_FAIL(-2, "fp8_gemm: cannot reserve %zu bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
    hipLaunchKernelGGL((gemm_tile_kernel<BM, BN>), dim3(tiles_m * tiles_n), dim3(256), lds_bytes, s, a, b, ep, M, N, K, tiles_m, tiles_n);
    return 0;
}

int nc_launch_gemm(const uint8_t* a, const uint8_t* b, const float* inv_a, const float* inv_b, NcGemmSegs segs,
                   void* out, int out_kind, float softcap, int M, int N, int K, int ldc, int force_kernel, void* workspace,
                   size_t workspace_bytes, hipStream_t s, int a_fmt, uint32_t* out_amax) {
    NC_CHECK_ARG(a && b && inv_a && inv_b && out, "fp8_gemm: null pointer");
    NC_CHECK_ARG(M >= 0 && N > 0 && K > 0, "fp8_gemm: bad shape M=%d N=%d K=%d", M, N, K);
    NC_CHECK_ARG(K % 16 == 0, "fp8_gemm: K=%d must be a multiple of 16", K);
    NC_CHECK_ARG(ldc >= N, "fp8_gemm: ldc=%d < N=%d", ldc, N);
    NC_CHECK_ARG(((uintptr_t)a & 15) == 0 && ((uintptr_t)b & 15) == 0, "fp8_gemm: operands must be 16-byte aligned");
    NC_CHECK_ARG(out_kind >= 0 && out_kind <= 2, "fp8_gemm: out_kind must be 0 (bf16), 1 (softcapped fp32) or 2 (bf16 relu^2 + amax)");
    NC_CHECK_ARG(out_kind != 2 || (out_amax && M > 128 && (long)M * K < (1L << 31) && (long)N * K < (1L << 31) && (force_kernel == 0 || force_kernel >= 5)),
                 "fp8_gemm: the relu^2 epilogue needs an amax word, M > 128, operands below 2 GiB and a buffer-load kernel");
    NC_CHECK_ARG(segs.nseg >= 1 && segs.nseg <= 4, "fp8_gemm: 1..4 column segments supported, got %d", segs.nseg);
    for (int i = 0; i < segs.nseg; i++) {
        NC_CHECK_ARG(segs.end[i] % 4 == 0 || segs.end[i] == N, "fp8_gemm: segment end %d must be a multiple of 4", segs.end[i]);
        NC_CHECK_ARG(i == 0 || segs.end[i] > segs.end[i - 1], "fp8_gemm: segment ends must increase");
    }
    NC_CHECK_ARG(segs.end[segs.nseg - 1] == N, "fp8_gemm: last segment must end at N");
    if (out_kind != 1)
        NC_CHECK_ARG(((uintptr_t)out & 7) == 0 && ldc % 4 == 0, "fp8_gemm: bf16 output needs 8-byte alignment and ldc %% 4 == 0");
    NC_CHECK_ARG(a_fmt == 0 || a_fmt == 1, "fp8_gemm: the format of a must be 0 (e4m3fn) or 1 (e5m2)");
    if (M == 0) return 0;
    EpilogueArgs ep{inv_a, inv_b, segs, out, out_kind, softcap, ldc, out_amax};
    if (a_fmt == 1) {
        // gradient operand (the backward GEMMs): bf16 output through the 128x128 buffer-load tile or the 256x256 direct-to-LDS tiles
        NC_CHECK_ARG(out_kind == 0, "fp8_gemm: an e5m2 operand goes with bf16 output");
        NC_CHECK_ARG((long)M * K < (1L << 31) && (long)N * K < (1L << 31), "fp8_gemm: e5m2 operands need M*K and N*K below 2^31");
        int which = force_kernel;
        if (which == 0) {
            const int cus = cu_count();
            const long t256 = (long)((M + 255) / 256) * ((N + 255) / 256);
            which = (K % 128 == 0 && (8 * t256 >= 5 * cus || dl_narrow_fills(M, N))) ? ((t256 >= 2 * cus && dlp_eligible(M, N, K)) ? 9 : 8) : 5;
            if (which == 8) {
                const int nj = dl_pick_nj(M, N);
                if (nj < 8) which = 8 + nj;               // 12 .. 15: the narrower 256-row tiles
            }
        }
        NC_CHECK_ARG(which == 5 || which == 8 || which == 9 || (which >= 12 && which <= 15),
                     "fp8_gemm: kernels 5, 8, 9 and 12..15 take an e5m2 operand, not %d", force_kernel);
        NcProfScope prof(1, 2.0 * M * N * K, s, ((int64_t)N << 32) | (uint32_t)K);
        int rc = which == 5 ? launch_bl<128, 128, 2, 2, true, 1>(a, b, ep, M, N, K, s)
                            : (which >= 12 ? launch_dln(which - 8, 1, a, b, ep, M, N, K, s) : launch_dl<1>(a, b, ep, M, N, K, which == 9, s));
        if (rc) return rc;
        NC_CHECK_LAUNCH("fp8_gemm");
        return 0;
    }

    // force_kernel: 0 auto, 1 small-M, 4 plain-load tile 128x128, 5/6/7 buffer-load tiles 128x128 / 256x128 / 256x256,
    // 8 direct-to-LDS 256x256 tile by tile, 9 the same persistent, 10 / 11 buffer-load tiles 64x128 / 96x128,
    // 12 .. 15 direct-to-LDS tiles of 256 x 128 / 160 / 192 / 224 tile by tile, 16 / 17 / 18 direct-to-LDS tiles of 64 / 96 / 128 x 128
    // with four stages
    int which = force_kernel;
    if (which == 0) {
        if (M <= 128) which = 1;
        else if ((long)M * K >= (1L << 31) || (long)N * K >= (1L << 31)) which = 4;   // past the 32-bit buffer offsets
        else {
            const int cus = cu_count();
            const long t256 = (long)((M + 255) / 256) * ((N + 255) / 256);
            const long rounds = (t256 + cus - 1) / cus;
            const long t128 = (long)((M + 127) / 128) * ((N + 127) / 128);
            if (out_kind != 1 && K % 128 == 0 && (8 * t256 >= 5 * cus || t128 > 2 * cus || dl_narrow_fills(M, N))) {
                // 256x256 tiles fed straight into LDS whenever they occupy at least 5/8 of the CUs, or the 128x128 tiles, four times
                // as many, would not fit the chip in one round of two workgroups per CU (below that the small tiles fill the chip
                // better: 18 us against 22 for 1280 x 4992 x 1664, but 25 against 22.4 for 1792 rows); from two rounds of tiles on,
                // the persistent form, which neither rounds the last round up nor pays a prologue per tile
                which = (t256 >= 2 * cus && dlp_eligible(M, N, K)) ? 9 : 8;
                if (which == 8) {
                    const int nj = dl_pick_nj(M, N);
                    if (nj < 8) which = 8 + nj;           // 12 .. 15
                }
            } else {
                // 256x256 tiles move half the bytes per flop through L2 and LDS but run one workgroup per CU: take them
                // when their count fills whole rounds of the CUs well, else the 128x128 tiles (two workgroups per CU)
                which = (M >= 1024 && N >= 512 && 10 * t256 >= 8 * rounds * cus && rounds <= 2) ? 7 : 5;
                // a prompt of a few hundred to two thousand rows against a narrow weight leaves CUs without a 128x128 tile, and each
                // tile's K loop is one dependent step after the other: lower tiles put a workgroup on more CUs with less MFMA work per
                // step, as long as they still fit one round of one workgroup per CU (512..1024 rows x 1664 columns with 64-row tiles:
                // 8 us against 10.7 at K = 1664, 21 against 31 at K = 6656; 1792 rows with 96-row tiles: 10.0 / 11.5 and 27.9 / 30.5)
                if (which == 5 && out_kind != 2) {
                    const long tn = (N + 127) / 128;
                    if ((long)((M + 63) / 64) * tn <= cus) which = 10;
                    else if ((long)((M + 95) / 96) * tn <= cus) which = 11;
                    // the same tiles fed straight into a ring of four LDS stages where K allows it: three K-steps of operands on their
                    // way instead of two and no ds_write phase (1792 x 1664 x 6656: 27.5 -> 25.6 us, 1024 rows: 21.9 -> 20.8 us; what is
                    // left is the L2's bandwidth: 28 KB per K-step and CU for tiles this small)
                    if (which >= 10 && K % 128 == 0 && out_kind == 0) which += 6;
                }
            }
        }
    }
    int rc = 0;
    if (which != 1) NC_CHECK_ARG(which >= 4 && which <= 18, "fp8_gemm: unknown kernel selector %d", force_kernel);
    NcProfScope prof(which == 1 ? -1 : 1, 2.0 * M * N * K, s, ((int64_t)N << 32) | (uint32_t)K);
    if (which == 1) {
        NC_CHECK_ARG(M <= 128, "fp8_gemm: the small-M kernel needs M <= 128, got %d", M);
        // split-K when the caller brought room for the partial sums, finished by a second small kernel
        int ks = nc_gemm_decode_splits(N, K);
        if (ks > 1 && (!workspace || workspace_bytes < (size_t)ks * M * N * sizeof(float))) ks = 1;
        int used = 1;
        rc = nc_launch_gemm_decode(a, 0, nullptr, inv_a, b, inv_b, segs, out, out_kind, softcap, nullptr, M, N, K, ldc, (float*)workspace,
                                   workspace_bytes, ks, &used, s);
        if (rc) return rc;
        if (used > 1)
            return nc_launch_finish_partials((const float*)workspace, used, nullptr, inv_a, inv_b, segs, out, out_kind, softcap, nullptr, M,
                                             N, ldc, s);
        return 0;
    } else if (which == 4) rc = launch_tile<128, 128>(a, b, ep, M, N, K, s);
    else if (which == 5) rc = launch_bl<128, 128, 2, 2, true>(a, b, ep, M, N, K, s);
    else if (which == 6) rc = launch_bl<256, 128, 4, 2, false>(a, b, ep, M, N, K, s);
    else if (which == 7) rc = launch_bl<256, 256, 4, 2, false>(a, b, ep, M, N, K, s);
    else if (which == 8) rc = launch_dl<0>(a, b, ep, M, N, K, false, s);
    else if (which == 9) rc = launch_dl<0>(a, b, ep, M, N, K, true, s);
    else if (which == 10) rc = launch_bl<64, 128, 2, 2, true>(a, b, ep, M, N, K, s);
    else if (which == 11) rc = launch_bl<96, 128, 2, 2, true>(a, b, ep, M, N, K, s);
    else if (which == 16) rc = launch_dr<64>(a, b, ep, M, N, K, s);
    else if (which == 17) rc = launch_dr<96>(a, b, ep, M, N, K, s);
    else if (which == 18) rc = launch_dr<128>(a, b, ep, M, N, K, s);
    else if (which >= 12) rc = launch_dln(which - 8, 0, a, b, ep, M, N, K, s);
    else NC_FAIL(-1, "fp8_gemm: unknown kernel selector %d", force_kernel);
    if (rc) return rc;
    NC_CHECK_LAUNCH("fp8_gemm");
    return 0;
}
