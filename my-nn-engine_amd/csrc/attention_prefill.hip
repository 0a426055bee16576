// Causal / full prefill attention on the matrix cores (flash-attention form), replacing the
// reference's attention_tc (attention.cuh:45-314: mma.m16n8k16, S and P round-tripping through
// shared memory, 16 lanes doing the softmax serially).
//
// One workgroup = 4 waves = 128 query rows of one (batch, query head); each wave owns 32 rows.  Two workgroups
// per CU (two waves per SIMD, up to 256 registers a lane: at three the kernel spilled into scratch inside the
// key loop).  Workgroups are dispatched longest first: grid y = query block, last block (most keys) first.
// Per 64-key tile (staged once in LDS for the four waves, K row-major, V transposed; two 32-key S^T tiles):
//   S^T = K . Q^T      v_mfma_f32_32x32x16: A = K rows from LDS, B = Q kept in registers
//   softmax            each lane owns ONE query column and 16 of the 32 keys of each S^T tile, so the
//                      row max / sum are in-lane plus a single exchange with lane ^ 32
//   O^T += V^T . P^T   the D-layout of S^T is already the B-operand layout of P^T (keys are
//                      contracted in the permuted order 4g+0..3, 8+4g+0..3), so P never leaves
//                      registers; A = V^T read from LDS with two 8-byte reads
// The rescale factor of the online softmax is a per-lane scalar because O^T keeps the same query
// column per lane; the rescale is skipped when no lane of the wave moved its maximum (most tiles after the
// first few).  Key tiles past a wave's last causal position are skipped.
// rope_q: the queries are read un-rotated from the projection's output and rotated in registers (the RoPE launch
// then only has the keys and values left to do).
// A thread stages CH neighbouring keys of the same 8 dims, so V^T goes to LDS CH keys at a time (4- or 8-byte
// writes of values gathered with v_perm) instead of one 2-byte write per value.
#include <type_traits>

#include "attention.h"
#include "mfma.h"

namespace mynn {

constexpr int kPfThreads = 256, kPfRows = 128, kPfKeys = 64;

// PAGED: K/V rows are found through a page table (AttnParams::page_table) of at most 64 pages per sequence, each a
// power of two >= 64 rows: a 64-key tile lies in one page, and the sequence's table row sits in one register (lane i =
// page i) from which a tile picks its entry with v_readlane.
template <typename T, int D, bool PAGED>
__global__ __launch_bounds__(kPfThreads, 2) void attn_prefill_kernel(AttnParams p) {
    constexpr int LDK = D + 8;          // K tile row stride (elements): conflict-free 16-byte reads
    constexpr int LDV = kPfKeys + 4;    // V^T tile row stride
    constexpr int KS = D / 16;          // k-steps of the S^T product
    constexpr int DT = D / 32;          // 32-row tiles of O^T
    constexpr int CH = (kPfKeys * D / 8) / kPfThreads;  // 16-byte chunks per thread and tile (2 or 4): neighbouring keys
    constexpr int NPF = D == 64 ? 2 : 1;                // tiles in flight in registers ahead of the one in LDS
    static_assert(CH == 2 || CH == 4, "a thread stages 2 or 4 neighbouring keys");
    __shared__ __align__(16) uint16_t Ks[2][kPfKeys * LDK];
    __shared__ __align__(16) uint16_t Vt[2][D * LDV];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, g = lane >> 5;
    const int bh = blockIdx.x, b = bh / p.Hq, h = bh % p.Hq;
    const int G = p.Hq / p.Hkv, hkv = h / G;
    const int Sq = p.Sq;
    const int active = p.d_active ? *p.d_active : p.active;
    const int qoff = p.d_active ? active - Sq : p.q_pos_offset;
    const int kv_bound = min(active, p.cache_len);

    const int q_blk = ((int)gridDim.y - 1 - (int)blockIdx.y) * kPfRows;  // the blocks with the most keys are dispatched first
    const int qrow = q_blk + wave * 32 + col;           // this lane's query row
    const int qrow_c = min(qrow, Sq - 1);
    // keys this lane's query may see, and the furthest any row of the wave / workgroup may see
    const int my_bound = p.is_causal ? min(kv_bound, qoff + qrow_c + 1) : kv_bound;
    const int wave_last = min(q_blk + wave * 32 + 31, Sq - 1);
    const int wave_bound = p.is_causal ? min(kv_bound, qoff + wave_last + 1) : kv_bound;
    const int blk_last = min(q_blk + kPfRows - 1, Sq - 1);
    const int blk_bound = p.is_causal ? min(kv_bound, qoff + blk_last + 1) : kv_bound;
    const int ntiles = (blk_bound + kPfKeys - 1) / kPfKeys;

    const T *Kg = (const T *)p.k + (PAGED ? 0 : (size_t)(b * p.Hkv + hkv) * p.cache_len * D);
    const T *Vg = (const T *)p.v + (PAGED ? 0 : (size_t)(b * p.Hkv + hkv) * p.cache_len * D);
    const int psh = p.page_shift, pmask = (1 << psh) - 1;
    int pg_reg = 0;
    if constexpr (PAGED) {
        if (lane < p.pages_per_seq) pg_reg = p.page_table[(size_t)b * p.pages_per_seq + lane];
    }
    // a tile travels global -> registers (NPF iterations ahead of) -> LDS (one iteration ahead of) the MFMAs.
    // Thread t stages the keys CH * (t / (D/8)) + 0 .. CH-1 of a tile, dims 8 * (t % (D/8)) .. +7.
    // Rows past the end are clamped to the last visible key: whatever they hold is masked out.
    const int key0 = (tid / (D / 8)) * CH, dd = (tid % (D / 8)) * 8;
    U4 rk[NPF][CH], rv[NPF][CH];
    auto load_tile = [&](int t, U4 *k_, U4 *v_) {
        size_t po = 0;  // PAGED: first row of the tile's page, in rows of one head of the pool
        if constexpr (PAGED) {
            const int pg = __builtin_amdgcn_readlane(pg_reg, __builtin_amdgcn_readfirstlane((t * kPfKeys) >> psh));
            po = ((size_t)pg * p.Hkv + hkv) << psh;
        }
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int key = min(t * kPfKeys + key0 + c, blk_bound - 1);
            const size_t row = PAGED ? po + (size_t)(key & pmask) : (size_t)key;
            k_[c] = *(const U4 *)(Kg + row * D + dd);
            v_[c] = *(const U4 *)(Vg + row * D + dd);
        }
    };
    auto store_tile = [&](int buf, const U4 *k_, const U4 *v_) {
#pragma unroll
        for (int c = 0; c < CH; c++) *(U4 *)&Ks[buf][(key0 + c) * LDK + dd] = k_[c];
        // V^T[d][key0 .. key0 + CH - 1] for the 8 dims: dword i of a chunk holds dims 2i (low half) and 2i + 1
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint32_t w[CH];
#pragma unroll
            for (int c = 0; c < CH; c++) w[c] = i == 0 ? v_[c].x : i == 1 ? v_[c].y : i == 2 ? v_[c].z : v_[c].w;
            uint16_t *lo = &Vt[buf][(dd + 2 * i) * LDV + key0], *hi = &Vt[buf][(dd + 2 * i + 1) * LDV + key0];
            if constexpr (CH == 2) {
                *(uint32_t *)lo = __builtin_amdgcn_perm(w[1], w[0], 0x05040100u);
                *(uint32_t *)hi = __builtin_amdgcn_perm(w[1], w[0], 0x07060302u);
            } else {
                *(uint2 *)lo = uint2{__builtin_amdgcn_perm(w[1], w[0], 0x05040100u), __builtin_amdgcn_perm(w[3], w[2], 0x05040100u)};
                *(uint2 *)hi = uint2{__builtin_amdgcn_perm(w[1], w[0], 0x07060302u), __builtin_amdgcn_perm(w[3], w[2], 0x07060302u)};
            }
        }
    };

    // the first tile's loads are on their way before the queries (and their RoPE table rows) are asked for
    if (ntiles > 0) load_tile(0, rk[0], rv[0]);
    // Q^T fragments: B operand, lane (query col, g): d = 16*ks + 8*g .. +7
    const T *Q = (const T *)p.q + (size_t)b * p.q_bs + (size_t)h * p.q_hs + (size_t)qrow_c * p.q_rs;
    U4 qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qf[ks] = *(const U4 *)(Q + 16 * ks + 8 * g);
    if (p.rope_q) {
        // the query rows arrive un-rotated (straight from the projection): RoPE by the row's position, the arithmetic of
        // rope.cuh:18-46 -- lo' = lo*cos[j] - hi*sin[j], hi' = hi*cos[j + D/2] + lo*sin[j + D/2], separate products, one
        // rounding.  Dims d and d + D/2 sit in fragments ks and ks + KS/2 of the same lane.
        const size_t tab = (size_t)p.d_pos[qrow_c] * D;
        const T *cs = (const T *)p.cos_t + tab, *sn = (const T *)p.sin_t + tab;
#pragma unroll
        for (int ks = 0; ks < KS / 2; ks++) {
            const int d0 = 16 * ks + 8 * g;
            float xl[8], xh[8], cl[8], ch[8], sl[8], sh[8], ol[8], oh[8];
            widen8<T>(qf[ks], xl);
            widen8<T>(qf[ks + KS / 2], xh);
            widen8<T>(*(const U4 *)(cs + d0), cl);
            widen8<T>(*(const U4 *)(cs + d0 + D / 2), ch);
            widen8<T>(*(const U4 *)(sn + d0), sl);
            widen8<T>(*(const U4 *)(sn + d0 + D / 2), sh);
#pragma unroll
            for (int i = 0; i < 8; i++) {
                ol[i] = xl[i] * cl[i] - xh[i] * sl[i];
                oh[i] = xh[i] * ch[i] + xl[i] * sh[i];
            }
            qf[ks] = U4{pack2<T>(ol[0], ol[1]), pack2<T>(ol[2], ol[3]), pack2<T>(ol[4], ol[5]), pack2<T>(ol[6], ol[7])};
            qf[ks + KS / 2] = U4{pack2<T>(oh[0], oh[1]), pack2<T>(oh[2], oh[3]), pack2<T>(oh[4], oh[5]), pack2<T>(oh[6], oh[7])};
        }
    }


    f16x_t o[DT];
#pragma unroll
    for (int t = 0; t < DT; t++)
#pragma unroll
        for (int e = 0; e < 16; e++) o[t][e] = 0.f;
    // running max in units of log2: scores are turned into exponents of two with one FMA each,
    // p = 2^(s * scale * log2(e) - m); the softmax scale is positive, so the max may be taken on raw scores
    float m = -INFINITY, l = 0.f;
    const float scale2 = p.scale * 1.4426950408889634f;
    // keys every query row of this wave may see: tiles that end at or below it need no masking
    const int wave_first = min(q_blk + wave * 32, Sq - 1);
    const int wave_all = p.is_causal ? min(kv_bound, qoff + wave_first + 1) : kv_bound;

    // one tile of 64 keys = two S^T tiles (rows = keys, cols = queries), one softmax update, 4 k-steps of P.V
    auto tile = [&](int buf, int k0, auto masked) {
        constexpr bool MASKED = decltype(masked)::value;
        f16x_t s[2];
#pragma unroll
        for (int hf = 0; hf < 2; hf++)
#pragma unroll
            for (int e = 0; e < 16; e++) s[hf][e] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ks++)
#pragma unroll
            for (int hf = 0; hf < 2; hf++) {
                const U4 a = *(const U4 *)&Ks[buf][(32 * hf + col) * LDK + 16 * ks + 8 * g];
                s[hf] = Mfma<T>::run(a, qf[ks], s[hf]);
            }
        // ---- online softmax for this lane's query over its 32 keys (+ partner lane's 32)
        float mloc = -INFINITY;
#pragma unroll
        for (int hf = 0; hf < 2; hf++)
#pragma unroll
            for (int e = 0; e < 16; e++) {
                if (MASKED) {
                    const int key = k0 + 32 * hf + 8 * (e >> 2) + 4 * g + (e & 3);
                    if (key >= my_bound) s[hf][e] = -INFINITY;
                }
                mloc = fmaxf(mloc, s[hf][e]);
            }
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));  // (the row swap instruction measured slower here)
        const float mn = fmaxf(m, mloc * scale2);
        float corr = 1.f;
        if (MASKED && mn == -INFINITY) {
#pragma unroll
            for (int hf = 0; hf < 2; hf++)
#pragma unroll
                for (int e = 0; e < 16; e++) s[hf][e] = 0.f;
        } else {
            corr = __builtin_amdgcn_exp2f(m - mn);
            float ls = 0.f;
#pragma unroll
            for (int hf = 0; hf < 2; hf++)
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    s[hf][e] = __builtin_amdgcn_exp2f(fmaf(s[hf][e], scale2, -mn));
                    ls += s[hf][e];
                }
            l = fmaf(l, corr, ls);
            m = mn;
        }
        // (a factor of exactly 1 in every lane leaves O^T as it is: the multiplications are skipped)
        if (__builtin_amdgcn_ballot_w64(corr != 1.f) != 0) {
#pragma unroll
            for (int t2 = 0; t2 < DT; t2++)
#pragma unroll
                for (int e = 0; e < 16; e++) o[t2][e] *= corr;
        }
        // ---- O^T += V^T . P^T, keys contracted in the order the D-layout delivers them
#pragma unroll
        for (int st = 0; st < 4; st++) {
            const f16x_t &ph = s[st >> 1];
            const int e0 = 8 * (st & 1);
            const U4 pf = U4{pack2<T>(ph[e0 + 0], ph[e0 + 1]), pack2<T>(ph[e0 + 2], ph[e0 + 3]),
                             pack2<T>(ph[e0 + 4], ph[e0 + 5]), pack2<T>(ph[e0 + 6], ph[e0 + 7])};
#pragma unroll
            for (int t2 = 0; t2 < DT; t2++) {
                const uint16_t *vr = &Vt[buf][(32 * t2 + col) * LDV + 16 * st + 4 * g];
                const uint2 lo = *(const uint2 *)vr, hi = *(const uint2 *)(vr + 8);
                o[t2] = Mfma<T>::run(U4{lo.x, lo.y, hi.x, hi.y}, pf, o[t2]);
            }
        }
    };
    auto compute = [&](int t) {
        const int k0 = t * kPfKeys;
        if (k0 + kPfKeys <= wave_all) tile(t & 1, k0, std::false_type{});
        else if (k0 < wave_bound) tile(t & 1, k0, std::true_type{});
    };

    // tile 0 goes straight to LDS; tiles 1 .. NPF wait in registers (slot j holds tile 1 + j, then 1 + j + NPF, ..)
    if (ntiles > 0) {
        store_tile(0, rk[0], rv[0]);
#pragma unroll
        for (int j = 0; j < NPF; j++) load_tile(min(1 + j, ntiles - 1), rk[j], rv[j]);
    }
    __syncthreads();
    int t = 0;
    // groups of NPF iterations that all still issue a load (unconditional, so the waits on older loads can be counted)
    for (; t + 2 * NPF < ntiles; t += NPF) {
#pragma unroll
        for (int j = 0; j < NPF; j++) {
            store_tile((t + j + 1) & 1, rk[j], rv[j]);  // tile t + j + 1, loaded NPF iterations ago; its buffer was released by the last barrier
            load_tile(t + j + 1 + NPF, rk[j], rv[j]);   // (< ntiles by the loop bound)
            compute(t + j);
            __syncthreads();
        }
    }
    // the rest: every tile still missing from LDS is in registers already or on its way
    for (; t < ntiles; t += NPF) {
#pragma unroll
        for (int j = 0; j < NPF; j++) {
            if (t + j < ntiles) {
                if (t + j + 1 < ntiles) store_tile((t + j + 1) & 1, rk[j], rv[j]);
                if (t + j + 1 + NPF < ntiles) load_tile(t + j + 1 + NPF, rk[j], rv[j]);
                compute(t + j);
                __syncthreads();
            }
        }
    }

    // ---- out[query, d] = O^T[d, query] / l
    l += __shfl_xor(l, 32, 64);
    if (qrow < Sq) {
        T *out = (T *)p.out + (size_t)b * p.o_bs + (size_t)h * p.o_hs + (size_t)qrow * p.o_rs;
        const float inv = 1.0f / l;
#pragma unroll
        for (int t2 = 0; t2 < DT; t2++)
#pragma unroll
            for (int e4 = 0; e4 < 4; e4++) {
                const int d = 32 * t2 + 8 * e4 + 4 * g;
                uint2 w;
                w.x = pack2<T>(o[t2][4 * e4 + 0] * inv, o[t2][4 * e4 + 1] * inv);
                w.y = pack2<T>(o[t2][4 * e4 + 2] * inv, o[t2][4 * e4 + 3] * inv);
                *(uint2 *)(out + d) = w;
            }
    }
}

bool attention_prefill_supported(const AttnParams &p, int D, int dtype, int kv_int8) {
    if (kv_int8 || (dtype != MYNN_F16 && dtype != MYNN_BF16)) return false;
    if (D != 64 && D != 128) return false;
    if (p.Sq < 16) return false;  // a handful of rows: the per-row kernel wastes less
    if (!(p.scale > 0.f)) return false;  // the running max is taken on unscaled scores
    // 16-byte loads of Q rows and 8-byte stores of out rows
    if ((p.q_rs % 8) || (p.q_hs % 8) || (p.q_bs % 8) || (p.o_rs % 4) || (p.o_hs % 4) || (p.o_bs % 4)) return false;
    if (((uintptr_t)p.q & 15) || ((uintptr_t)p.out & 7) || ((uintptr_t)p.k & 15) || ((uintptr_t)p.v & 15)) return false;
    return true;
}

int attention_prefill_launch(const AttnParams &p, int D, int dtype, hipStream_t s) {
    MYNN_REQUIRE((p.Sq + kPfRows - 1) / kPfRows <= 65535, MYNN_ERR_UNSUPPORTED, "attention: Sq = %d exceeds the grid", p.Sq);
    if (p.page_table) {
        const int P = 1 << p.page_shift;
        MYNN_REQUIRE(P >= kPfKeys && p.pages_per_seq <= 64 && p.cache_len == p.pages_per_seq << p.page_shift, MYNN_ERR_UNSUPPORTED,
                     "paged prefill attention: %d pages of %d rows per sequence (at most 64 pages of 2^n >= %d rows)",
                     p.pages_per_seq, P, kPfKeys);
    }
    dim3 grid(p.B * p.Hq, (p.Sq + kPfRows - 1) / kPfRows);
    return dispatch_dtype16(dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        if (p.page_table) {
            if (D == 64) MYNN_LAUNCH((attn_prefill_kernel<T, 64, true>), grid, dim3(kPfThreads), 0, s, p);
            else MYNN_LAUNCH((attn_prefill_kernel<T, 128, true>), grid, dim3(kPfThreads), 0, s, p);
        } else {
            if (D == 64) MYNN_LAUNCH((attn_prefill_kernel<T, 64, false>), grid, dim3(kPfThreads), 0, s, p);
            else MYNN_LAUNCH((attn_prefill_kernel<T, 128, false>), grid, dim3(kPfThreads), 0, s, p);
        }
        return launch_status("attn_prefill_kernel");
    });
}

}  // namespace mynn
