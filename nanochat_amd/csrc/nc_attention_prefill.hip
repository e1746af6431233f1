// Attention of many query positions per row over the KV cache (prefill): the T > 1 case of
// flash_attn_with_kvcache (nanochat/flash_attention.py:139-185) and of flash_attn_func (:115-136), causal with an
// optional left window, GQA by kv head = q head / (H / Hkv), head_dim 128, bf16 in, fp32 softmax, bf16 out.
// The new keys and values are already in the cache (qkv_rope_append); a query at cache position p sees keys
// [max(0, p - window), p].
//
// Flash-attention forward on the bf16 matrix cores, written "transposed" so that nothing has to move between lanes:
//   S^T = K . Q^T   (v_mfma_f32_32x32x16_bf16, A = K rows from LDS, B = the wave's 32 queries held in registers):
//                   a lane ends up with 16 scores of ONE query (column lane % 32), so the running max / sum of the
//                   online softmax are per-lane scalars plus one exchange with lane ^ 32;
//   O^T = V^T . P^T (same instruction, A = V^T, B = P^T): the B operand is exactly the S^T accumulator registers converted to
//                   bf16 (the key order inside a 16-key chunk is the accumulator's row order, and V^T is read in that order),
//                   and the output columns are again the lane's own query, so the softmax rescale is a per-lane multiply.
// Keys and values go through LDS in blocks of 32, both as [key][d] (K rows padded to 272 B, V rows to 320 B); the V^T operand
// comes out of LDS through the transposing read (ds_read_b64_tr_b16), so nothing is shuffled while staging.  The loads of the
// next block are in flight while the current one is multiplied.
#include "nc_common.h"
#include "nc_kernels.h"

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef short v4s __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4s* lds_v4s_t;
typedef __attribute__((address_space(3))) uint8_t* lds_u8_t;

#define PF_KPITCH 272          // bytes per K row in LDS (256 + 16)
#define PF_VPITCH 320          // bytes per V row in LDS (256 + 64: four consecutive keys start 16 banks apart)
#define PF_KBYTES (32 * PF_KPITCH)
#define PF_VBYTES (32 * PF_VPITCH)
#define PF_MASKED (-1.0e30f)   // raw score of a key that the query does not see
#define PF_LAZY 6.0f           // log2 units the running maximum may lag behind before the accumulators are rescaled
#define PF_M_FLOOR (-1.0e20f)  // running maximum (scaled units) before any visible key: far above PF_MASKED * scale, far below any score

__device__ __forceinline__ v8bf as_v8bf(uint4 v) { return __builtin_bit_cast(v8bf, v); }

// GS = query heads of one kv head that share a workgroup (1, 2 or 4), KS = waves that share one block of 32 queries and split
// its keys between them (1 or 2), GS * KS <= 4.  Wave w serves head (w % GS) of the group, key share (w / GS) % KS and the
// (w / (GS * KS))-th block of 32 queries, so a workgroup covers 128 / (GS * KS) queries of GS heads and the keys and values it
// stages are used by all of its waves.  Keys go through LDS 64 at a time (two sub-blocks of 32, each laid out and multiplied as
// described above): one pair of barriers and one round of loads in flight per 64 keys.  With KS = 1 a wave works through both
// sub-blocks, with KS = 2 through one of them, and the two partial softmax states of a query block are merged through LDS at the end:
// that doubles the number of workgroups when a launch has too few of them to fill the chip (a single long prompt).
// A wave skips a sub-block that none of its queries can see (past the causal diagonal, or wholly before the window of its first
// query), and a sub-block that all of its queries see in full takes the path without the mask arithmetic.  The running maximum only
// triggers a rescale of the 64 output accumulators when it moved for some lane of the wave.  Tiles are handed out from the end of the
// sequence, longest key ranges first.
// Which (tile, head) unit the workgroup with a given linear index takes, when the launch says so (one row, every key visible, a
// grid of at most 512 workgroups): see pf_balance_units.
struct PfUnitMap {
    int on;
    uint16_t unit[512];
};
template <int GS, int KS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void attn_prefill_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache,
                                                           const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ cache_seqlens,
                                                           int window_left, int seqlens_include_new, bf16_t* __restrict__ out,
                                                           uint32_t* __restrict__ amax_ws, int T, int H, int Hkv, int Tmax, PfUnitMap map) {
    constexpr int QT = 128 / (GS * KS);                        // queries per workgroup
    __shared__ __align__(16) uint8_t lds[2 * PF_KBYTES + 2 * PF_VBYTES];
    __shared__ float red[4];
    uint8_t* const lds_k = lds;
    uint8_t* const lds_v = lds + 2 * PF_KBYTES;
    const lds_u8_t lds_v3 = (lds_u8_t)lds + 2 * PF_KBYTES;     // the same place as an LDS address, for the transposing reads
    const int G = H / Hkv, parts = G / GS;                     // workgroups per kv head along the head axis
    // Workgroups go to the eight XCDs in turn by their linear index, and each XCD has an L2 of its own: the (tile, head) pairs of a
    // row are numbered so that one XCD gets a contiguous run of them, i.e. all tiles of a few heads, and the keys and values of a head
    // are then read into one L2 instead of all eight.  Within a head the tiles come from the end of the sequence, longest first.
    const int b = blockIdx.z;
    int qb0, hy;
    {
        const int nx = gridDim.x, total = nx * (int)gridDim.y, lid = (int)blockIdx.x + nx * (int)blockIdx.y;
        const int xcd = lid & 7, slot = lid >> 3;
        const int unit = map.on ? (int)map.unit[lid] : xcd * (total >> 3) + min(xcd, total & 7) + slot;
        hy = unit / nx;
        qb0 = (nx - 1 - unit % nx) * QT;
    }
    const int hk = hy / parts;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = hk * G + (hy % parts) * GS + wave % GS;
    const int ks = (wave / GS) % KS;                           // which of the KS key shares this wave takes
    const int qw0 = qb0 + (wave / (GS * KS)) * 32;             // first query of this wave
    const int col = lane & 31, hl = lane >> 5;

    int pos0 = cache_seqlens[b];
    if (seqlens_include_new) pos0 -= T;
    // this lane's query
    const int t = qw0 + col;
    const bool q_ok = t < T;
    const int qpos = pos0 + (q_ok ? t : T - 1);
    const int q_lo = window_left < 0 ? 0 : max(0, qpos - window_left);

    // key range of the workgroup
    const int t_last = min(qb0 + QT - 1, T - 1);
    int k_hi = pos0 + t_last;
    if (k_hi > Tmax - 1) k_hi = Tmax - 1;
    int k_lo = window_left < 0 ? 0 : pos0 + qb0 - window_left;
    if (k_lo < 0) k_lo = 0;
    const int kb_first = k_lo & ~63;

    // what the wave as a whole can see: keys [w_lo, w_hi]; what every one of its queries sees in full: keys [f_lo, f_hi]
    const int qpos_first = pos0 + min(qw0, T - 1), qpos_last = pos0 + min(qw0 + 31, T - 1);
    const int w_hi = qpos_last;
    const int w_lo = window_left < 0 ? 0 : max(0, qpos_first - window_left);
    const int f_hi = min(qpos_first, k_hi);
    const int f_lo = window_left < 0 ? 0 : max(0, qpos_last - window_left);

    // Q fragments: B operand of K.Q^T, lane = (query col, d half hl): Q[query][16c + 8hl .. +7]
    v8bf qf[8];
    {
        const bf16_t* qrow = q + (((size_t)b * T + (q_ok ? t : T - 1)) * H + h) * 128;
#pragma unroll
        for (int c = 0; c < 8; c++) qf[c] = as_v8bf(*(const uint4*)(qrow + 16 * c + 8 * hl));
    }

    v16f o[4];
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[dt][r] = 0.f;
    float m_run = PF_M_FLOOR, l_run = 0.f;
    const float sc = 1.4426950408889634f * 0.08838834764831845f;     // log2(e) / sqrt(128)

    // staging: thread = (16-byte chunk ch of a key, key pair kp): keys 2kp, 2kp+1 of each 32-key sub-block
    const int ch = tid & 15, kp = tid >> 4;
    // Keys and values come through buffer descriptors that end behind key k_hi of this row: a load past the workgroup's range returns
    // zeros without a branch or a select, and the eight loads of a stage are eight instructions (plus one add each for the stage's
    // offset; the range check looks at the vector offset only, so the stage cannot go into the scalar offset).
    const uint32_t key_bytes = (uint32_t)Hkv * 256;
    const uint32_t row_bytes = (uint32_t)(k_hi + 1) * key_bytes;
    const __amdgpu_buffer_rsrc_t desc_k = __builtin_amdgcn_make_buffer_rsrc((void*)(k_cache + (size_t)b * Tmax * Hkv * 128), 0, row_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t desc_v = __builtin_amdgcn_make_buffer_rsrc((void*)(v_cache + (size_t)b * Tmax * Hkv * 128), 0, row_bytes, 0x00020000);
    const uint32_t lane_off = (uint32_t)(2 * kp) * key_bytes + (uint32_t)hk * 256 + (uint32_t)ch * 16;
    typedef int pf_v4i __attribute__((ext_vector_type(4)));
    uint4 rk[2][2], rv[2][2];
    // the 64 keys from kb on: sub-block sb, key 2 kp + i of it
    auto fetch = [&](int kb) {
        const uint32_t base = lane_off + (uint32_t)kb * key_bytes;
#pragma unroll
        for (int sb = 0; sb < 2; sb++)
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const uint32_t off = base + (uint32_t)(32 * sb + i) * key_bytes;
                const pf_v4i kv = __builtin_amdgcn_raw_buffer_load_b128(desc_k, off, 0, 0);
                const pf_v4i vv = __builtin_amdgcn_raw_buffer_load_b128(desc_v, off, 0, 0);
                rk[sb][i] = make_uint4((uint32_t)kv[0], (uint32_t)kv[1], (uint32_t)kv[2], (uint32_t)kv[3]);
                rv[sb][i] = make_uint4((uint32_t)vv[0], (uint32_t)vv[1], (uint32_t)vv[2], (uint32_t)vv[3]);
            }
    };
    auto stage = [&]() {
#pragma unroll
        for (int sb = 0; sb < 2; sb++)
#pragma unroll
            for (int i = 0; i < 2; i++) {
                *(uint4*)(lds_k + sb * PF_KBYTES + (2 * kp + i) * PF_KPITCH + ch * 16) = rk[sb][i];
                *(uint4*)(lds_v + sb * PF_VBYTES + (2 * kp + i) * PF_VPITCH + ch * 16) = rv[sb][i];
            }
    };
    // Transposed read of V (ds_read_b64_tr_b16): in every group of 16 lanes, lane r points at four consecutive d of key r / 4
    // (d offset 4 (r % 4)), and lane i receives element d = i of the 16 the group covers, for those four keys.  The groups are
    // (d half of the 32-row block, key half hl), which makes the result the A operand of the second product as laid out below.
    const uint32_t vtr_off = (uint32_t)(4 * hl + ((lane & 15) >> 2)) * PF_VPITCH + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
    // one sub-block of 32 keys starting at kb, staged in slot sb; MASKED = some (query, key) pair of it is not visible
    auto sub_block = [&](int kb, int sb, bool masked) {
        // ---- S^T = K . Q^T : rows = keys kb + 8*(r/4) + 4*hl + r%4, column = this lane's query
        v16f s;
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = 0.f;
        const uint8_t* kt = lds_k + sb * PF_KBYTES;
#pragma unroll
        for (int c = 0; c < 8; c++) {
            const v8bf kf = as_v8bf(*(const uint4*)(kt + col * PF_KPITCH + (16 * c + 8 * hl) * 2));
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[c], s, 0, 0, 0);
        }
        // ---- mask, online softmax (per lane = per query; the other half of the keys sits in lane ^ 32)
        if (masked) {                      // wave-uniform
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int key = kb + 8 * (r >> 2) + 4 * hl + (r & 3);
                const bool vis = key <= qpos && key >= q_lo && key <= k_hi;
                s[r] = vis ? s[r] : PF_MASKED;
            }
        }
        float mx = s[0];
#pragma unroll
        for (int r = 1; r < 16; r++) mx = fmaxf(mx, s[r]);
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        // (a sub-block with nothing visible for this lane leaves the maximum where it was: PF_MASKED * sc lies below the floor,
        // and its weights come out as exp2(-huge) = 0)
        // The reference point of the exponentials only follows the maximum when it has moved by more than PF_LAZY (in log2 units)
        // for some lane of the wave: until then the weights may exceed 1 (by at most 2^PF_LAZY, nothing for fp32 sums or bf16
        // weights), the quotient sum(p v) / sum(p) is the same, and the 64 accumulators are spared the multiply.
        const float m_new = fmaxf(m_run, mx * sc);
        if (__builtin_amdgcn_ballot_w64(m_new > m_run + PF_LAZY) != 0) {      // wave-uniform
            const float corr = __builtin_amdgcn_exp2f(m_run - m_new);
            l_run *= corr;
#pragma unroll
            for (int dt = 0; dt < 4; dt++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[dt][r] *= corr;
            m_run = m_new;
        }
        float psum = 0.f;
        v8bf pf[2];
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const float p = __builtin_amdgcn_exp2f(fmaf(s[r], sc, -m_run));
            psum += p;
            pf[r >> 3][r & 7] = (__bf16)p;
        }
        l_run += psum;
        // ---- O^T += V^T . P^T : chunk c2 of 16 keys uses accumulator rows 8*c2 .. 8*c2+7, i.e. keys
        //      kb + 16*c2 + 4*hl + {0..3} and kb + 16*c2 + 8 + 4*hl + {0..3}; V^T is read in the same order
#pragma unroll
        for (int c2 = 0; c2 < 2; c2++)
#pragma unroll
            for (int dt = 0; dt < 4; dt++) {
                const lds_u8_t vblk = lds_v3 + sb * PF_VBYTES + vtr_off + 16 * c2 * PF_VPITCH + 32 * dt * 2;
                const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t)vblk);
                const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t)(vblk + 8 * PF_VPITCH));
                const v8bf vf = __builtin_bit_cast(v8bf, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[c2], o[dt], 0, 0, 0);
            }
    };
    // (wave-uniform tests: a skipped sub-block holds no key that any query of this wave sees)
    auto visit = [&](int kb, int sb) {
        if (kb <= w_hi && kb + 31 >= w_lo) sub_block(kb, sb, !(kb >= f_lo && kb + 31 <= f_hi));
    };

    if (kb_first <= k_hi) fetch(kb_first);
    for (int kb = kb_first; kb <= k_hi; kb += 64) {
        __syncthreads();                    // everyone is done with the previous block's tiles
        stage();
        __syncthreads();
        if (kb + 64 <= k_hi) fetch(kb + 64);
        if (KS == 1) {
#pragma unroll 1
            for (int sb = 0; sb < 2; sb++) visit(kb + 32 * sb, sb);
        } else {
            visit(kb + 32 * ks, ks);
        }
    }

    if (KS == 2) {
        // the wave with the odd sub-blocks hands its state to its partner through the tile memory: [value][lane] floats,
        // values 0..63 the accumulators, 64 the maximum, 65 the sum
        __syncthreads();
        float* xch = (float*)lds + (wave / (2 * GS) * GS + wave % GS) * (66 * 64);
        if (ks == 1) {
#pragma unroll
            for (int dt = 0; dt < 4; dt++)
#pragma unroll
                for (int r = 0; r < 16; r++) xch[(16 * dt + r) * 64 + lane] = o[dt][r];
            xch[64 * 64 + lane] = m_run;
            xch[65 * 64 + lane] = l_run;
        }
        __syncthreads();
        if (ks == 0) {
            const float m2 = xch[64 * 64 + lane], l2 = xch[65 * 64 + lane];
            const float m_new = fmaxf(m_run, m2);
            const float wa = __builtin_amdgcn_exp2f(m_run - m_new), wb = __builtin_amdgcn_exp2f(m2 - m_new);
            l_run = l_run * wa + l2 * wb;
#pragma unroll
            for (int dt = 0; dt < 4; dt++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[dt][r] = o[dt][r] * wa + xch[(16 * dt + r) * 64 + lane] * wb;
        }
    }

    // ---- finish: total weight of the query = both lane halves
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    const float inv_l = l_tot > 0.f ? 1.0f / l_tot : 0.f;
    float am = 0.f;
    if (q_ok && ks == 0) {
        bf16_t* orow = out + (((size_t)b * T + t) * H + h) * 128;
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
#pragma unroll
            for (int g4 = 0; g4 < 4; g4++) {
                const int d = 32 * dt + 8 * g4 + 4 * hl;
                const uint2 pk = make_uint2(pack_bf16(o[dt][4 * g4] * inv_l, o[dt][4 * g4 + 1] * inv_l),
                                            pack_bf16(o[dt][4 * g4 + 2] * inv_l, o[dt][4 * g4 + 3] * inv_l));
                *(uint2*)(orow + d) = pk;
                am = amax_fold(amax_fold(amax_fold(amax_fold(am, bf16_lo(pk.x)), bf16_hi(pk.x)), bf16_lo(pk.y)), bf16_hi(pk.y));
            }
    }
    if (amax_ws) {
        am = wave_amax(am);
        __syncthreads();
        if (lane == 0) red[wave] = am;
        __syncthreads();
        if (tid == 0) amax_publish(amax_ws, amax_join(amax_join(red[0], red[1]), amax_join(red[2], red[3])));
    }
}

// ------------------------------------------------------------------------------------------------
// The shared part of a decode step whose rows all start with the same tokens (Engine.generate prefills one prompt at batch 1 and
// replicates its cache to every row, nanochat/engine.py:198-214): positions [0, shared_len) of every row of the cache hold the same
// keys and values, so the new token of every row attends to ONE copy of them.  The rows play the part that the query positions
// play in the kernel above: a workgroup takes up to 128 / (GS * KS) rows x GS query heads of one kv head and a chunk of the shared
// keys, read from row 0 of the cache, once for all of its rows, and multiplies on the matrix cores (the per-row streaming kernel
// would pull the same bytes through every CU once per row: 64 rows x 1792 keys x 13 heads x 512 B = 763 MB per layer instead of
// 12 MB).  All rows sit at the same position (cache_seqlens[0], the Engine's loop), every query sees the same keys
// [max(0, p - window), shared_len), and nothing is masked inside that range.  The result is not normalised: per (row, head, chunk)
// the running maximum (log2 units), the sum of weights and the weighted value sums, which the per-row kernel merges with what it
// finds in the row's own tail of the cache (attn_partial_kernel, `extra`).
#define SP_PART_STRIDE 132     // floats per partial: m, l, pad, pad, acc[128] (the layout of the per-row kernel's split partials)
template <int GS, int KS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void attn_shared_prefix_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ cache_seqlens,
    int shared_len, int window_left, int seqlens_include_new, float* __restrict__ partials, int nparts, int chunk_keys, int nqtiles, int rows,
    int H, int Hkv, int Tmax) {
    constexpr int QT = 128 / (GS * KS);                        // rows per workgroup
    __shared__ __align__(16) uint8_t lds[2 * PF_KBYTES + 2 * PF_VBYTES];
    uint8_t* const lds_k = lds;
    uint8_t* const lds_v = lds + 2 * PF_KBYTES;
    const lds_u8_t lds_v3 = (lds_u8_t)lds + 2 * PF_KBYTES;
    const int G = H / Hkv, parts = G / GS;
    const int qb0 = ((int)blockIdx.x % nqtiles) * QT, chunk = (int)blockIdx.x / nqtiles, hy = blockIdx.y;
    const int hk = hy / parts;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = hk * G + (hy % parts) * GS + wave % GS;
    const int ks = (wave / GS) % KS;
    const int qw0 = qb0 + (wave / (GS * KS)) * 32;             // first row of this wave
    const int col = lane & 31, hl = lane >> 5;
    const int t = qw0 + col;                                   // this lane's row of the batch
    const bool q_ok = t < rows;

    // keys of this chunk that the step sees: [k_lo, k_hi], the same for every row
    const int pos = cache_seqlens[0] - (seqlens_include_new ? 1 : 0);
    int k_lo = window_left < 0 ? 0 : max(0, pos - window_left);
    k_lo = max(k_lo, chunk * chunk_keys);
    const int k_hi = min(min(shared_len, pos), (chunk + 1) * chunk_keys) - 1;
    float* part = partials + (((size_t)(q_ok ? t : 0) * H + h) * nparts + chunk) * SP_PART_STRIDE;
    if (k_lo > k_hi) {
        // nothing of this chunk is visible: a partial of weight zero
        if (q_ok && ks == 0) {
            if (hl == 0) part[0] = PF_M_FLOOR, part[1] = 0.f;
#pragma unroll
            for (int i = 0; i < 16; i++) *(float4*)(part + 4 + 64 * hl + 4 * i) = make_float4(0.f, 0.f, 0.f, 0.f);
        }
        return;
    }
    const int kb_first = k_lo & ~63;

    v8bf qf[8];
    {
        const bf16_t* qrow = q + ((size_t)(q_ok ? t : rows - 1) * H + h) * 128;
#pragma unroll
        for (int c = 0; c < 8; c++) qf[c] = as_v8bf(*(const uint4*)(qrow + 16 * c + 8 * hl));
    }
    v16f o[4];
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[dt][r] = 0.f;
    float m_run = PF_M_FLOOR, l_run = 0.f;
    const float sc = 1.4426950408889634f * 0.08838834764831845f;     // log2(e) / sqrt(128)

    const int ch = tid & 15, kp = tid >> 4;
    const uint32_t key_stride = (uint32_t)Hkv * 128;
    const bf16_t* kbase = k_cache + (size_t)hk * 128 + ch * 8;        // row 0 of the cache
    const bf16_t* vbase = v_cache + (size_t)hk * 128 + ch * 8;
    uint4 rk[2][2], rv[2][2];
    auto fetch_one = [&](int kb, int j) {
        const int sb = j >> 2, i = (j >> 1) & 1;
        const int key = kb + 32 * sb + 2 * kp + i;
        const bool ok = key <= k_hi;
        const uint32_t off = (uint32_t)key * key_stride;
        if (j & 1) rv[sb][i] = ok ? *(const uint4*)(vbase + off) : make_uint4(0, 0, 0, 0);
        else rk[sb][i] = ok ? *(const uint4*)(kbase + off) : make_uint4(0, 0, 0, 0);
    };
    auto fetch = [&](int kb) {
#pragma unroll
        for (int j = 0; j < 8; j++) fetch_one(kb, j);
    };
    auto stage = [&]() {
#pragma unroll
        for (int sb = 0; sb < 2; sb++)
#pragma unroll
            for (int i = 0; i < 2; i++) {
                *(uint4*)(lds_k + sb * PF_KBYTES + (2 * kp + i) * PF_KPITCH + ch * 16) = rk[sb][i];
                *(uint4*)(lds_v + sb * PF_VBYTES + (2 * kp + i) * PF_VPITCH + ch * 16) = rv[sb][i];
            }
    };
    const uint32_t vtr_off = (uint32_t)(4 * hl + ((lane & 15) >> 2)) * PF_VPITCH + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
    auto sub_block = [&](int kb, int sb, bool masked) {
        v16f s;
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = 0.f;
        const uint8_t* kt = lds_k + sb * PF_KBYTES;
#pragma unroll
        for (int c = 0; c < 8; c++) {
            const v8bf kf = as_v8bf(*(const uint4*)(kt + col * PF_KPITCH + (16 * c + 8 * hl) * 2));
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[c], s, 0, 0, 0);
        }
        if (masked) {                      // wave-uniform: the chunk's first or last sub-block
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int key = kb + 8 * (r >> 2) + 4 * hl + (r & 3);
                s[r] = (key >= k_lo && key <= k_hi) ? s[r] : PF_MASKED;
            }
        }
        float mx = s[0];
#pragma unroll
        for (int r = 1; r < 16; r++) mx = fmaxf(mx, s[r]);
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m_run, mx * sc);
        if (__builtin_amdgcn_ballot_w64(m_new > m_run + PF_LAZY) != 0) {      // wave-uniform
            const float corr = __builtin_amdgcn_exp2f(m_run - m_new);
            l_run *= corr;
#pragma unroll
            for (int dt = 0; dt < 4; dt++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[dt][r] *= corr;
            m_run = m_new;
        }
        float psum = 0.f;
        v8bf pf[2];
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const float p = __builtin_amdgcn_exp2f(fmaf(s[r], sc, -m_run));
            psum += p;
            pf[r >> 3][r & 7] = (__bf16)p;
        }
        l_run += psum;
#pragma unroll
        for (int c2 = 0; c2 < 2; c2++)
#pragma unroll
            for (int dt = 0; dt < 4; dt++) {
                const lds_u8_t vblk = lds_v3 + sb * PF_VBYTES + vtr_off + 16 * c2 * PF_VPITCH + 32 * dt * 2;
                const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t)vblk);
                const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t)(vblk + 8 * PF_VPITCH));
                const v8bf vf = __builtin_bit_cast(v8bf, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[c2], o[dt], 0, 0, 0);
            }
    };
    auto visit = [&](int kb, int sb) {
        if (kb <= k_hi && kb + 31 >= k_lo) sub_block(kb, sb, !(kb >= k_lo && kb + 31 <= k_hi));
    };

    fetch(kb_first);
    for (int kb = kb_first; kb <= k_hi; kb += 64) {
        __syncthreads();
        stage();
        __syncthreads();
        if (kb + 64 <= k_hi) fetch(kb + 64);
        if (KS == 1) {
#pragma unroll 1
            for (int sb = 0; sb < 2; sb++) visit(kb + 32 * sb, sb);
        } else {
            visit(kb + 32 * ks, ks);
        }
    }
    if (KS == 2) {
        __syncthreads();
        float* xch = (float*)lds + (wave / (2 * GS) * GS + wave % GS) * (66 * 64);
        if (ks == 1) {
#pragma unroll
            for (int dt = 0; dt < 4; dt++)
#pragma unroll
                for (int r = 0; r < 16; r++) xch[(16 * dt + r) * 64 + lane] = o[dt][r];
            xch[64 * 64 + lane] = m_run;
            xch[65 * 64 + lane] = l_run;
        }
        __syncthreads();
        if (ks == 0) {
            const float m2 = xch[64 * 64 + lane], l2 = xch[65 * 64 + lane];
            const float m_new = fmaxf(m_run, m2);
            const float wa = __builtin_amdgcn_exp2f(m_run - m_new), wb = __builtin_amdgcn_exp2f(m2 - m_new);
            l_run = l_run * wa + l2 * wb;
            m_run = m_new;
#pragma unroll
            for (int dt = 0; dt < 4; dt++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[dt][r] = o[dt][r] * wa + xch[(16 * dt + r) * 64 + lane] * wb;
        }
    }
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    if (q_ok && ks == 0) {
        if (hl == 0) part[0] = m_run, part[1] = l_tot;
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
#pragma unroll
            for (int g4 = 0; g4 < 4; g4++)
                *(float4*)(part + 4 + 32 * dt + 8 * g4 + 4 * hl) = make_float4(o[dt][4 * g4], o[dt][4 * g4 + 1], o[dt][4 * g4 + 2], o[dt][4 * g4 + 3]);
    }
}

// keys per chunk and chunks of the shared part: chunks of at least 128 keys (two staging rounds), as many as give the launch about one
// workgroup per CU
void nc_attn_shared_plan(int rows, int H, int Hkv, int shared_len, int* chunk_keys_out, int* nchunks_out) {
    const int G = H / Hkv;
    const int GS = G % 4 == 0 ? 4 : (G % 2 == 0 ? 2 : 1), KS = GS <= 2 ? 2 : 1, QT = 128 / (GS * KS);
    const long per_chunk = (long)((rows + QT - 1) / QT) * Hkv * (G / GS);
    int want = (int)((nc_cu_count() + per_chunk - 1) / per_chunk);
    if (want < 1) want = 1;
    int ck = (shared_len + want - 1) / want;
    ck = (ck + 63) & ~63;
    if (ck < 128) ck = 128;
    *chunk_keys_out = ck;
    *nchunks_out = (shared_len + ck - 1) / ck;
}
size_t nc_attn_shared_partial_bytes(int rows, int H, int Hkv, int shared_len) {
    int ck, nc;
    nc_attn_shared_plan(rows, H, Hkv, shared_len, &ck, &nc);
    return (size_t)rows * H * nc * SP_PART_STRIDE * sizeof(float);
}

int nc_launch_attention_shared_prefix(const bf16_t* q, const bf16_t* k_cache, const bf16_t* v_cache, const int32_t* cache_seqlens, int shared_len,
                                      int window_left, int seqlens_include_new, float* partials, size_t partial_bytes, int rows, int H, int Hkv,
                                      int Tmax, int* nchunks_out, hipStream_t s) {
    NC_CHECK_ARG(q && k_cache && v_cache && cache_seqlens && partials, "shared_prefix_attention: null pointer");
    NC_CHECK_ARG(rows > 0 && H > 0 && Hkv > 0 && H % Hkv == 0 && shared_len > 0 && shared_len <= Tmax, "shared_prefix_attention: bad shape");
    NC_CHECK_ARG((long long)Tmax * Hkv * 128 < (1LL << 31), "shared_prefix_attention: one row of the cache must stay below 2^31 elements");
    NC_CHECK_ARG((((uintptr_t)q | (uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)partials) & 15) == 0,
                 "shared_prefix_attention: pointers must be 16-byte aligned");
    int ck, nchunks;
    nc_attn_shared_plan(rows, H, Hkv, shared_len, &ck, &nchunks);
    NC_CHECK_ARG(partial_bytes >= (size_t)rows * H * nchunks * SP_PART_STRIDE * sizeof(float), "shared_prefix_attention: %zu bytes of partial sums needed",
                 (size_t)rows * H * nchunks * SP_PART_STRIDE * sizeof(float));
    const int G = H / Hkv;
    const int GS = G % 4 == 0 ? 4 : (G % 2 == 0 ? 2 : 1), KS = GS <= 2 ? 2 : 1, QT = 128 / (GS * KS);
    const int nqtiles = (rows + QT - 1) / QT;
    const dim3 grid(nqtiles * nchunks, Hkv * (G / GS));
    NC_CHECK_ARG(grid.y <= 65535, "shared_prefix_attention: too many heads in one launch");
    NcProfScope prof(0, 0.0, s);
#define SP_LAUNCH(GG, KK)                                                                                                          \
    hipLaunchKernelGGL((attn_shared_prefix_kernel<GG, KK>), grid, dim3(256), 0, s, q, k_cache, v_cache, cache_seqlens, shared_len,  \
                       window_left, seqlens_include_new, partials, nchunks, ck, nqtiles, rows, H, Hkv, Tmax)
    if (GS == 4) SP_LAUNCH(4, 1);
    else if (GS == 2) SP_LAUNCH(2, 2);
    else SP_LAUNCH(1, 2);
#undef SP_LAUNCH
    NC_CHECK_LAUNCH("shared_prefix_attention");
    if (nchunks_out) *nchunks_out = nchunks;
    return 0;
}

// A causal launch over one long row has tiles of very different lengths (tile t of a head reads t + 1 blocks of keys) and more workgroups
// than CUs, but fewer than two per CU: some CUs get two workgroups that then run at half speed each, and with the plain order (each XCD:
// a run of units, longest first) the second workgroup of a CU lands beside one of the longest.  Here each XCD's units are dealt so that
// the longest stay alone and the rest are paired long with short: with C CUs per XCD and P = units - C pairs, the workgroups dispatched
// P .. C-1 (alone on their CU, if the dispatcher deals the second round in the order of the first) take the longest units, 0 .. P-1 the
// next longest and C + k the (k+1)-th shortest.  Only the order changes, every unit is still computed by exactly one workgroup.
// d26, 1792 tokens, full-context layers (28 tiles x 13 heads = 364 workgroups): 40 -> 33.3 us, which is the longest tile alone on its CU.
static void pf_balance_units(PfUnitMap& map, int nx, int ny, int cus) {
    const int total = nx * ny, C = cus / 8;
    map.on = 0;
    if (total > 512 || C <= 0) return;
    for (int xcd = 0; xcd < 8; xcd++) {
        const int per = (total >> 3) + (xcd < (total & 7) ? 1 : 0), base = xcd * (total >> 3) + (xcd < (total & 7) ? xcd : (total & 7));
        if (per <= C || per > 2 * C) return;
        // units of this XCD in descending length: a unit's length grows with its tile index nx - 1 - unit % nx
        int order[128];
        if (per > 128) return;
        for (int i = 0; i < per; i++) order[i] = base + i;
        for (int i = 1; i < per; i++) {              // insertion sort, stable: longest first
            const int u = order[i], key = nx - 1 - u % nx;
            int j = i - 1;
            while (j >= 0 && (nx - 1 - order[j] % nx) < key) order[j + 1] = order[j], j--;
            order[j + 1] = u;
        }
        const int P = per - C, S = C - P;
        for (int slot = 0; slot < per; slot++) {
            const int rank = slot < P ? S + slot : (slot < C ? slot - P : per - 1 - (slot - C));
            map.unit[xcd + 8 * slot] = (uint16_t)order[rank];
        }
    }
    map.on = 1;
}

int nc_launch_attention_prefill(const bf16_t* q, const bf16_t* k_cache, const bf16_t* v_cache, const int32_t* cache_seqlens,
                                int window_left, bf16_t* out, int B, int T, int H, int Hkv, int Tmax, int seqlens_include_new,
                                uint32_t* amax_ws, hipStream_t s) {
    NC_CHECK_ARG(q && k_cache && v_cache && cache_seqlens && out, "prefill_attention: null pointer");
    NC_CHECK_ARG(B > 0 && T > 0 && H > 0 && Hkv > 0 && Tmax > 0 && H % Hkv == 0, "prefill_attention: bad shape");
    NC_CHECK_ARG(B <= 65535 && H <= 65535, "prefill_attention: more than 65535 rows or heads in one launch");
    NC_CHECK_ARG((long long)Tmax * Hkv * 128 < (1LL << 31), "prefill_attention: one row of the cache must stay below 2^31 elements");
    NC_CHECK_ARG((((uintptr_t)q | (uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)out) & 15) == 0,
                 "prefill_attention: pointers must be 16-byte aligned");
    NcProfScope prof(0, 0.0, s);
    const int G = H / Hkv;
    const int GS = G % 4 == 0 ? 4 : (G % 2 == 0 ? 2 : 1);       // query heads of a kv head per workgroup
    // two waves per query block, each with half of the keys, when whole-key-range workgroups would not give every CU two of them
    const long long wgs1 = (long long)B * Hkv * (G / GS) * ((T + 128 / GS - 1) / (128 / GS));
    const int KS = (GS <= 2 && wgs1 < 2LL * nc_cu_count()) ? 2 : 1;
    const int QT = 128 / (GS * KS);
    const dim3 grid((T + QT - 1) / QT, Hkv * (G / GS), B);
    NC_CHECK_ARG(grid.y <= 65535, "prefill_attention: too many heads in one launch");
    PfUnitMap map;                         // passed by value
    map.on = 0;
    // one row whose queries see every key before them (a window of at least the cache length is none): the long prompt of a prefill
    if (B == 1 && (window_left < 0 || window_left >= Tmax)) pf_balance_units(map, (int)grid.x, (int)grid.y, nc_cu_count());
#define PF_LAUNCH(GG, KK)                                                                                                              \
    hipLaunchKernelGGL((attn_prefill_kernel<GG, KK>), grid, dim3(256), 0, s, q, k_cache, v_cache, cache_seqlens, window_left,          \
                       seqlens_include_new, out, amax_ws, T, H, Hkv, Tmax, map)
    if (GS == 4) PF_LAUNCH(4, 1);
    else if (GS == 2 && KS == 2) PF_LAUNCH(2, 2);
    else if (GS == 2) PF_LAUNCH(2, 1);
    else if (KS == 2) PF_LAUNCH(1, 2);
    else PF_LAUNCH(1, 1);
#undef PF_LAUNCH
    NC_CHECK_LAUNCH("prefill_attention");
    return 0;
}
