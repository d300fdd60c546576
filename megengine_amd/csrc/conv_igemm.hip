// Dense int8 ConvBias as an implicit GEMM on the gfx950 matrix cores.
//
//   D[oc][pixel] = sum_k  F[oc][k] * X[pixel][k]        k = (channel block, fh, fw, channel-in-block)
//
// computed with v_mfma_i32_32x32x32_i8 (A = filter rows, B = pixels, int32 accumulate) and
// requantised in registers by the fused epilogue (epilogue.h).  Activations and filters in the
// reference's NCHW4 / NCHW32 layouts already hold the 16 consecutive k-bytes an MFMA lane needs
// (NCHW32: one 16-byte run; NCHW4: four 4-byte runs), so the im2col matrix is never materialised:
// each stage gathers a BN x BK activation tile and a BM x BK filter tile straight into LDS.
//
// Schedule: persistent workgroups.  Each workgroup walks a list of output tiles and, inside a
// tile, the k-stages; the two loops are flattened into one iteration space so that the global
// loads of the next TWO iterations (registers R0/R1) are always in flight -- across tile
// boundaries too, i.e. under the epilogue of the previous tile.  LDS is double buffered.
//
// Data layout in LDS (per buffer and operand): [row][BK bytes], BK = KCH * 32, 16-byte slot s of
// row r stored at slot s ^ swz(r).  A k-unit table {byte offset, fh, fw} for every 32-byte (NCHW32)
// or 4-byte (NCHW4) k-unit is built once per workgroup, so the loaders do no divisions.
//
// Accumulator layout of the 32x32 MFMA (lane l, register v): pixel = l % 32,
// oc = 8*(v/4) + 4*(l/32) + v%4.  NCHW4 output stores one dword (4 channels) per register quad;
// NCHW32 output first exchanges quads between lanes l and l+32 (v_permlane32_swap) so that each
// lane owns 16 consecutive channels of one pixel and stores 16 bytes.
#include <string.h>

#include <atomic>

#include "igemm_shared.h"

namespace mi355 {
namespace {

// PW = pointwise fast path: 1x1 filter, no padding.  Its loaders need no
// bounds tests and no k-unit table: every address is a per-row base plus a wave-uniform term.
template <int PIN, int POUT, int BM, int BN, int WM, int WN, int KCH, bool PW>
struct IgemmKernel {
    static constexpr int WTM = BM / WM, WTN = BN / WN;
    static constexpr int MT = WTM / 32, NT = WTN / 32;
    static constexpr int S = KCH * 2;              // 16-byte slots per LDS row
    static constexpr int ROWB = KCH * 32;          // bytes per LDS row
    static constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB;
    static constexpr int UA = BM * S / IG_THREADS;  // 16-byte units per thread per stage
    static constexpr int UB = BN * S / IG_THREADS;
    // Activation unit j: row pass j % RB (rows (t/2) + 128 * pass), k-chunk csel + CSB * (j / RB): lanes run along
    // pixels, which are contiguous in memory for one channel block.
    // Filter unit j: slot t % S of row t / S + RPA * j: lanes run along k, so that every filter row contributes one
    // whole contiguous BK-byte run (full cache lines) per load instruction.
    static constexpr int RB = BN >= 128 ? BN / 128 : 1;
    static constexpr int CSB = BN >= 128 ? 1 : 128 / BN;
    static constexpr int RPA = IG_THREADS / S;  // filter rows per loader pass
    static constexpr int BIAS_BYTES = 2 * BM * 4;          // bias of the current / next tile's channels
    static constexpr int STAGE_BYTES = 2 * (A_BYTES + B_BYTES) + BIAS_BYTES;
    static_assert(WM * WN * 64 == IG_THREADS, "4 waves");
    static_assert(UA >= 1 && UB >= 1, "tile too small for 256 loader threads");
    static_assert(MT >= 1 && NT >= 1, "wave tile");

    struct Regs {
        v4i a[UA];
        v4i b[UB];
    };
    // loader-side state: which (tile, stage) the next issue() fetches, and the rows of that tile
    struct Loader {
        int tile, stage, kc0;   // position in this workgroup's sequence; kc0 = stage * KCH
        int a_base[UA];         // filter row byte offset (+ lane slot), SENT for rows past OC
        int b_base[RB];         // pixel byte offset (+ lane half); PW: SENT for rows past M
        int ih0[RB], iw0[RB];   // table path: top-left input coordinate (ih0 = -0x8000 for rows past M)
    };

    __device__ static __forceinline__ int rowA(int t, int j) { return t / S + RPA * j; }
    __device__ static __forceinline__ int rowB(int t, int j) { return BN >= 128 ? (t >> 1) + 128 * (j % RB) : (t >> 1) % BN; }
    // wave-uniform first chunk of this thread's units (non-zero only for tiles with fewer than 128 rows)
    __device__ static __forceinline__ int cselB(int t) { return BN >= 128 ? 0 : __builtin_amdgcn_readfirstlane((t >> 1) / BN); }

    __device__ static __forceinline__ void tile_coords(const IgemmArgs& a, int tile, int& oc0, int& pix0) {
        const int tn = tile / a.tiles_m, tm = tile - tn * a.tiles_m;
        oc0 = tm * BM;
        pix0 = tn * BN;
    }

    __device__ static __forceinline__ void loader_enter_tile(const IgemmArgs& a, Loader& L, int tile, int t) {
        int oc0, pix0;
        tile_coords(a, tile, oc0, pix0);
#pragma unroll
        for (int r = 0; r < UA; ++r) {
            const int oc = oc0 + rowA(t, r);
            L.a_base[r] = oc < a.OC ? oc * a.kbytes + (t % S) * 16 : SENT;
        }
#pragma unroll
        for (int r = 0; r < RB; ++r) {
            const int m = pix0 + rowB(t, r);
            const bool ok = m < a.M;
            const uint32_t mm = ok ? m : 0;
            const uint32_t n = fdiv(mm, a.div_ohw), rem = mm - n * a.OHW;
            const uint32_t oh = fdiv(rem, a.div_ow), ow = rem - oh * a.OW;
            const int ih0 = (int)oh * a.sh - a.ph, iw0 = (int)ow * a.sw - a.pw;
            const int lane_part = PIN == 32 ? (t & 1) * 16 : (PW ? (t & 1) * 4 * a.src_scb : 0);
            const int base = (int)n * a.src_sn + (ih0 * a.IW + iw0) * PIN + lane_part;
            L.b_base[r] = (PW && !ok) ? SENT : base;
            L.ih0[r] = ok ? ih0 : -0x8000;  // makes every tap fail the bounds test
            L.iw0[r] = iw0;
        }
    }

    __device__ static __forceinline__ void loader_kill(Loader& L) {
        // past the end of this workgroup's work: every further load is out of range (returns 0, moves no
        // data), which keeps issue/stash unconditional in the steady-state loop
#pragma unroll
        for (int r = 0; r < UA; ++r) L.a_base[r] = SENT;
#pragma unroll
        for (int r = 0; r < RB; ++r) {
            L.b_base[r] = SENT;
            L.ih0[r] = -0x8000;
        }
        L.kc0 = 0;
    }

    // Global loads of one stage into registers.  Straight-line code: every offset is fully bounds-checked
    // by the buffer descriptor, invalid rows/taps use the SENT offset and return zeros.
    __device__ static __forceinline__ void issue(const IgemmArgs& a, const Loader& L, const KEntry* tab,
                                                 const __amdgpu_buffer_rsrc_t& rs_src,
                                                 const __amdgpu_buffer_rsrc_t& rs_flt, Regs& R, int t) {
        const int cb = cselB(t);
        // bytes past the end of a filter row (last stage of a K that is not a multiple of BK) belong to the next
        // row or are out of range (zeros): either way they meet zero activations
#pragma unroll
        for (int j = 0; j < UA; ++j)
            R.a[j] = __builtin_amdgcn_raw_buffer_load_b128(rs_flt, L.a_base[j] + L.kc0 * 32, 0, 0);
#pragma unroll
        for (int j = 0; j < UB; ++j) {
            const int r = j % RB;
            const int kc = L.kc0 + cb + CSB * (j / RB);  // wave-uniform
            if (PW) {
                // channel blocks past the last one (K not a whole number of stages) read as zeros
                if (PIN == 32) {
                    R.b[j] = __builtin_amdgcn_raw_buffer_load_b128(rs_src, kc < a.KC ? L.b_base[r] + kc * a.src_scb : SENT, 0, 0);
                } else {
                    const int lim = (a.kbytes >> 2) - (t & 1) * 4;  // this lane's half starts 4 blocks further on
                    v4i x;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int cbi = kc * 8 + i;
                        x[i] = __builtin_amdgcn_raw_buffer_load_b32(rs_src, cbi < lim ? L.b_base[r] + cbi * a.src_scb : SENT, 0, 0);
                    }
                    R.b[j] = x;
                }
            } else if (PIN == 32) {
                const KEntry k = tab[kc];
                const int k_off = __builtin_amdgcn_readfirstlane(k.off), k_fhfw = __builtin_amdgcn_readfirstlane(k.fhfw);
                const int ih = L.ih0[r] + (k_fhfw & 0xffff), iw = L.iw0[r] + (k_fhfw >> 16);
                const bool ok = (unsigned)ih < (unsigned)a.IH && (unsigned)iw < (unsigned)a.IW;
                R.b[j] = __builtin_amdgcn_raw_buffer_load_b128(rs_src, ok ? L.b_base[r] + k_off : SENT, 0, 0);
            } else {
                const int e0 = kc * 8 + (t & 1) * 4;
                v4i x;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const KEntry k = tab[e0 + i];
                    const int ih = L.ih0[r] + (k.fhfw & 0xffff), iw = L.iw0[r] + (k.fhfw >> 16);
                    const bool ok = (unsigned)ih < (unsigned)a.IH && (unsigned)iw < (unsigned)a.IW;
                    x[i] = __builtin_amdgcn_raw_buffer_load_b32(rs_src, ok ? L.b_base[r] + k.off : SENT, 0, 0);
                }
                R.b[j] = x;
            }
        }
    }

    __device__ static __forceinline__ void stash(int8_t* sA, int8_t* sB, const Regs& R, int t) {
        const int cb = cselB(t);
#pragma unroll
        for (int j = 0; j < UA; ++j) {
            const int row = rowA(t, j);
            const int slot = (t % S) ^ swz<S>(row);
            *reinterpret_cast<v4i*>(sA + row * ROWB + slot * 16) = R.a[j];
        }
#pragma unroll
        for (int j = 0; j < UB; ++j) {
            const int row = rowB(t, j), chunk = cb + CSB * (j / RB);
            const int slot = (chunk * 2 + (t & 1)) ^ swz<S>(row);
            *reinterpret_cast<v4i*>(sB + row * ROWB + slot * 16) = R.b[j];
        }
    }

    // accumulators start from the bias of their output channel (held in LDS per tile)
    __device__ static __forceinline__ void init_acc(v16i (&acc)[MT][NT], const int* sBias, int wm, int lh) {
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            v16i init;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const v4i b = *reinterpret_cast<const v4i*>(sBias + wm * WTM + i * 32 + 8 * q + 4 * lh);
                init[4 * q + 0] = b[0]; init[4 * q + 1] = b[1]; init[4 * q + 2] = b[2]; init[4 * q + 3] = b[3];
            }
#pragma unroll
            for (int j = 0; j < NT; ++j) acc[i][j] = init;
        }
    }

    __device__ static __forceinline__ int fetch_bias(const IgemmArgs& a, int oc0, int t) {
        const int oc = oc0 + t;
        return (a.has_bias && t < BM && oc < a.OC) ? a.bias[oc] : 0;
    }

    __device__ static __forceinline__ void run(const IgemmArgs& a) {
        extern __shared__ __attribute__((aligned(16))) int8_t lds[];
        int8_t* sA = lds;                  // 2 buffers of A_BYTES
        int8_t* sB = lds + 2 * A_BYTES;    // 2 buffers of B_BYTES
        int* sBias = reinterpret_cast<int*>(lds + 2 * (A_BYTES + B_BYTES));  // 2 x BM
        KEntry* tab = reinterpret_cast<KEntry*>(lds + STAGE_BYTES);

        const int t = threadIdx.x;
        const int lane = t & 63, wave = t >> 6;
        const int l32 = lane & 31, lh = lane >> 5;
        const int wm = wave / WN, wn = wave % WN;

        // ---- this workgroup's tile sequence: first, first + step, ... (< last).
        // Workgroups are dealt round-robin to the 8 XCDs; when the grid is a multiple of 8 every XCD
        // owns a contiguous range of tiles (neighbouring tiles share activations and halos in that
        // XCD's L2) and its workgroups stride through the range.
        int first, step, last;
        {
            const int G = gridDim.x, b = blockIdx.x;
            if ((G & 7) == 0) {
                const int x = b & 7, j = b >> 3, gx = G >> 3;
                const int per = a.tiles >> 3, rem = a.tiles & 7;
                const int t0 = x * per + (x < rem ? x : rem);
                last = t0 + per + (x < rem ? 1 : 0);
                first = t0 + j;
                step = gx;
            } else {
                first = b; step = G; last = a.tiles;
            }
        }
        const int my_tiles = first < last ? (last - first + step - 1) / step : 0;
        const int total = my_tiles * a.nstages;

        // ---- k-unit table (not needed by the pointwise path)
        if (!PW) {
            constexpr int UPC = PIN == 32 ? 1 : 8;  // units per 32-byte chunk
            const int cap = a.nstages * KCH * UPC;
            for (int e = t; e < cap; e += IG_THREADS) {
                KEntry k;
                if (e < a.entries) {
                    const uint32_t cb = fdiv(e, a.div_t), tap = e - cb * a.T;
                    const uint32_t fh = fdiv(tap, a.div_fw), fw = tap - fh * a.FW;
                    k.off = (int)cb * a.src_scb + ((int)fh * a.IW + (int)fw) * PIN;
                    k.fhfw = (int)(fh | (fw << 16));
                } else {
                    k.off = 0;
                    k.fhfw = 0x4000;
                }
                tab[e] = k;
            }
        }
        if (total == 0) return;

        const __amdgpu_buffer_rsrc_t rs_src = make_rsrc(a.src, a.src_bytes);
        const __amdgpu_buffer_rsrc_t rs_flt = make_rsrc(a.flt, a.flt_bytes);

        Loader L;
        L.tile = first;
        L.stage = 0;
        L.kc0 = 0;
        loader_enter_tile(a, L, first, t);
        int issued = 0;  // iterations whose loads have been issued
        auto advance = [&]() __attribute__((always_inline)) {
            ++issued;
            L.kc0 += KCH;
            if (++L.stage == a.nstages) {
                L.stage = 0;
                L.kc0 = 0;
                L.tile += step;
                if (issued < total) loader_enter_tile(a, L, L.tile, t);
            }
            if (issued >= total) loader_kill(L);
        };

        Regs R0, R1;
        __syncthreads();  // table ready
        issue(a, L, tab, rs_src, rs_flt, R0, t);
        advance();
        issue(a, L, tab, rs_src, rs_flt, R1, t);
        advance();

        // consumer-side state
        int c_tile = first, c_stage = 0, c_oc0, c_pix0;
        tile_coords(a, c_tile, c_oc0, c_pix0);
        int c_par = 0;          // which half of sBias the current tile uses
        int bias_next = 0;      // prefetched bias word of the next tile (threads < BM)
        if (t < BM) sBias[t] = fetch_bias(a, c_oc0, t);
        v16i acc[MT][NT];
        // a wave with a single 32x32 tile alternates two accumulators so that consecutive MFMAs are independent
        constexpr bool DUAL = MT * NT == 1;
        v16i alt;

        stash(sA, sB, R0, t);
        __syncthreads();

        auto phase = [&](int it, int buf, Regs& Rfree, Regs& Rnext) __attribute__((always_inline)) {
            // Rfree was stashed into LDS in the previous phase; Rnext holds iteration it + 1
            if (c_stage == 0) {
                init_acc(acc, sBias + c_par * BM, wm, lh);
                if (DUAL) alt = v16i{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            }
            const bool last_stage = it < total && c_stage + 1 == a.nstages;
            int n_oc0 = c_oc0, n_pix0 = c_pix0;
            if (last_stage && it + 1 < total) {
                tile_coords(a, c_tile + step, n_oc0, n_pix0);
                if (a.tiles_m > 1) bias_next = fetch_bias(a, n_oc0, t);  // lands during the MFMAs + epilogue
            }
            // ---- one straight-line block: loads of iteration it + 2, MFMAs of iteration it with their
            // LDS fragment reads running one k-chunk ahead, then iteration it + 1 goes to the other buffer
            issue(a, L, tab, rs_src, rs_flt, Rfree, t);
            const int8_t* pA = sA + buf * A_BYTES;
            const int8_t* pB = sB + buf * B_BYTES;
            // Fragment reads run ahead of the MFMAs: the whole stage when it fits in registers, else one
            // k-chunk ahead.  The LDS writes of iteration it + 1 are issued before the MFMAs so that their
            // latency hides under the matrix pipeline.
            constexpr int FD = KCH * (MT + NT) <= 12 ? KCH : 2;
            v4i fa[FD][MT], fb[FD][NT];
            auto frags = [&](int c, v4i (&xa)[MT], v4i (&xb)[NT]) __attribute__((always_inline)) {
#pragma unroll
                for (int i = 0; i < MT; ++i) {
                    const int row = wm * WTM + i * 32 + l32;
                    const int slot = (c * 2 + lh) ^ swz<S>(row);
                    xa[i] = *reinterpret_cast<const v4i*>(pA + row * ROWB + slot * 16);
                }
#pragma unroll
                for (int j = 0; j < NT; ++j) {
                    const int row = wn * WTN + j * 32 + l32;
                    const int slot = (c * 2 + lh) ^ swz<S>(row);
                    xb[j] = *reinterpret_cast<const v4i*>(pB + row * ROWB + slot * 16);
                }
            };
            auto mfmas = [&](int c, const v4i (&xa)[MT], const v4i (&xb)[NT]) __attribute__((always_inline)) {
#pragma unroll
                for (int i = 0; i < MT; ++i)
#pragma unroll
                    for (int j = 0; j < NT; ++j) {
                        if (DUAL && (c & 1))
                            alt = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa[i], xb[j], alt, 0, 0, 0);
                        else
                            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa[i], xb[j], acc[i][j], 0, 0, 0);
                    }
            };
            if (FD == KCH) {
#pragma unroll
                for (int c = 0; c < KCH; ++c) frags(c, fa[c], fb[c]);
                __builtin_amdgcn_sched_barrier(0);
                stash(sA + (buf ^ 1) * A_BYTES, sB + (buf ^ 1) * B_BYTES, Rnext, t);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int c = 0; c < KCH; ++c) mfmas(c, fa[c], fb[c]);
            } else {
                frags(0, fa[0], fb[0]);
                stash(sA + (buf ^ 1) * A_BYTES, sB + (buf ^ 1) * B_BYTES, Rnext, t);
#pragma unroll
                for (int c = 0; c < KCH; ++c) {
                    if (c + 1 < KCH) frags(c + 1, fa[(c + 1) & 1], fb[(c + 1) & 1]);
                    mfmas(c, fa[c & 1], fb[c & 1]);
                }
            }
            // ---- bookkeeping
            if (last_stage) {
                if (DUAL) acc[0][0] += alt;
                if (POUT == 1)
                    igemm_epilogue_planar<MT, NT>(a, acc, c_oc0 + wm * WTM, c_pix0 + wn * WTN, l32, lh);
                else
                    igemm_run_epilogue<POUT, MT, NT>(a, acc, c_oc0 + wm * WTM, c_pix0 + wn * WTN, l32, lh);
                c_stage = 0;
                c_tile += step;
                if (a.tiles_m > 1) {
                    c_par ^= 1;
                    if (t < BM) sBias[c_par * BM + t] = bias_next;
                }
                c_oc0 = n_oc0;
                c_pix0 = n_pix0;
            } else {
                ++c_stage;
            }
            advance();
            __syncthreads();
        };

        for (int it = 0; it < total; it += 2) {
            phase(it, 0, R0, R1);
            if (it + 1 >= total) break;  // leaving the loop here keeps the loads inside both phases unconditional
            phase(it + 1, 1, R1, R0);
        }
    }

};

template <int PIN, int POUT, int BM, int BN, int WM, int WN, int KCH, int MINW, bool PW>
__global__ __launch_bounds__(IG_THREADS, MINW) void igemm_kernel(IgemmArgs a) {
    IgemmKernel<PIN, POUT, BM, BN, WM, WN, KCH, PW>::run(a);
}

struct TileCfg {
    const char* name;
    int bm, bn, kch;
};
// index = tile_cfg of mi355_algo
const TileCfg kCfgs[] = {
        {"128x128x64", 128, 128, 2},
        {"64x256x64", 64, 256, 2},
        {"256x128x64", 256, 128, 2},
        {"64x64x128", 64, 64, 4},
        {"32x256x128", 32, 256, 4},
        {"128x128x128", 128, 128, 4},
        {"64x128x128", 64, 128, 4},
        {"128x64x128", 128, 64, 4},
};
constexpr int kNumCfgs = sizeof(kCfgs) / sizeof(kCfgs[0]);

template <int PIN, int POUT, int BM, int BN, int WM, int WN, int KCH, int MINW, bool PW>
int launch_pw(hipStream_t st, IgemmArgs& a, int cu_count) {
    using K = IgemmKernel<PIN, POUT, BM, BN, WM, WN, KCH, PW>;
    a.tiles_m = (a.OC + BM - 1) / BM;
    a.tiles_n = (a.M + BN - 1) / BN;
    const int64_t tiles = (int64_t)a.tiles_m * a.tiles_n;
    if (tiles <= 0 || tiles > 0x3fffffff) return (int)hipErrorInvalidValue;
    a.tiles = (int)tiles;
    a.nstages = (a.KC + KCH - 1) / KCH;
    const int tab_entries = PW ? 0 : a.nstages * KCH * (PIN == 32 ? 1 : 8);
    const int lds = K::STAGE_BYTES + tab_entries * 8;
    auto kern = igemm_kernel<PIN, POUT, BM, BN, WM, WN, KCH, MINW, PW>;
    // per-instantiation caches; atomics, because operators on different streams may launch from several threads
    static std::atomic<int> max_lds_set{0};
    if (lds > max_lds_set.load(std::memory_order_relaxed)) {
        const int want = K::STAGE_BYTES + IG_MAX_ENTRIES * 8;
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, want);
        if (e != hipSuccess) return (int)e;
        max_lds_set.store(want, std::memory_order_relaxed);
    }
    // persistent grid: as many workgroups as fit on the device at once
    static std::atomic<uint64_t> occ_cache{0};  // LDS bytes of the last query << 32 | its result
    const uint64_t cached = occ_cache.load(std::memory_order_relaxed);
    int occ = (int)(uint32_t)cached;
    if ((cached >> 32) != (uint64_t)lds || occ < 1) {
        hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, reinterpret_cast<const void*>(kern),
                                                                    IG_THREADS, (size_t)lds);
        if (e != hipSuccess || occ < 1) {
            (void)hipGetLastError();
            occ = 1;
        }
        occ_cache.store(((uint64_t)lds << 32) | (uint32_t)occ, std::memory_order_relaxed);
    }
    if (cu_count <= 0) cu_count = 256;
    int64_t grid = (int64_t)occ * cu_count;
    // a multiple of 8 (one contiguous slab of the tile space per XCD).  When every tile has a workgroup of its own the
    // count is rounded UP -- a few workgroups find no tile and leave -- because rounding down would hand some workgroups
    // a second tile and double the launch's duration; otherwise down, inside what the device holds at once.
    if (grid > tiles) grid = tiles;
    if (grid >= 8) grid = grid == tiles ? (grid + 7) & ~(int64_t)7 : grid & ~(int64_t)7;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(IG_THREADS), lds, st, a);
    return (int)hipGetLastError();
}

template <int PIN, int POUT, int BM, int BN, int WM, int WN, int KCH, int MINW>
int launch_one(hipStream_t st, IgemmArgs& a, int cu_count) {
    // pointwise fast path: 1x1, no padding (any K: the loaders zero the channel blocks past the last one)
    const bool pw = a.T == 1 && a.ph == 0 && a.pw == 0;
    if (pw) return launch_pw<PIN, POUT, BM, BN, WM, WN, KCH, MINW, true>(st, a, cu_count);
    return launch_pw<PIN, POUT, BM, BN, WM, WN, KCH, MINW, false>(st, a, cu_count);
}

template <int PIN, int POUT>
int launch_fmt(hipStream_t st, IgemmArgs& a, int cfg, int cu) {
    switch (cfg) {
        case 0: return launch_one<PIN, POUT, 128, 128, 2, 2, 2, 2>(st, a, cu);
        case 1: return launch_one<PIN, POUT, 64, 256, 1, 4, 2, 2>(st, a, cu);
        case 2: return launch_one<PIN, POUT, 256, 128, 2, 2, 2, 1>(st, a, cu);
        case 3: return launch_one<PIN, POUT, 64, 64, 2, 2, 4, 3>(st, a, cu);
        case 4: return launch_one<PIN, POUT, 32, 256, 1, 4, 4, 2>(st, a, cu);
        case 5: return launch_one<PIN, POUT, 128, 128, 2, 2, 4, 2>(st, a, cu);
        case 6: return launch_one<PIN, POUT, 64, 128, 2, 2, 4, 3>(st, a, cu);
        case 7: return launch_one<PIN, POUT, 128, 64, 2, 2, 4, 2>(st, a, cu);
        default: return (int)hipErrorInvalidValue;
    }
}

}  // namespace

// tile_cfg numbering: register-staged tiles, LDS-direct tiles, second-generation tiles, patch-staged tiles, weight-resident
// tiles, the 32-packed streaming kernel
int igemm_num_cfgs() { return kNumCfgs + igemm_dma_num_cfgs() + igemm2_num_cfgs() + igemm3_num_cfgs() + igemm4_num_cfgs() + 1; }
int igemm_first_v2_cfg() { return kNumCfgs + igemm_dma_num_cfgs(); }
// planar destination (NCHW4_NCHW): two of the register-staged tiles
static int launch_planar(hipStream_t st, IgemmArgs& a, int cfg, int cu) {
    switch (cfg) {
        case 0: return launch_one<4, 1, 128, 128, 2, 2, 2, 2>(st, a, cu);
        case 3: return launch_one<4, 1, 64, 64, 2, 2, 4, 3>(st, a, cu);
        default: return (int)hipErrorInvalidConfiguration;
    }
}

static int igemm_first_v3_cfg() { return igemm_first_v2_cfg() + igemm2_num_cfgs(); }
static int igemm_first_v4_cfg() { return igemm_first_v3_cfg() + igemm3_num_cfgs(); }
static int igemm_pw32s_cfg() { return igemm_first_v4_cfg() + igemm4_num_cfgs(); }
const char* igemm_cfg_name(int cfg) {
    if (cfg >= 0 && cfg < kNumCfgs) return kCfgs[cfg].name;
    if (cfg < igemm_first_v2_cfg()) return igemm_dma_cfg_name(cfg - kNumCfgs);
    if (cfg < igemm_first_v3_cfg()) return igemm2_cfg_name(cfg - igemm_first_v2_cfg());
    if (cfg < igemm_first_v4_cfg()) return igemm3_cfg_name(cfg - igemm_first_v3_cfg());
    if (cfg < igemm_pw32s_cfg()) return igemm4_cfg_name(cfg - igemm_first_v4_cfg());
    return "pw32_stream";
}

static bool igemm_needs_general(const ConvProblem& p) {
    return p.d.dst_dtype != MI355_DT_QS8 || p.d.bias_mode == MI355_BIAS_FULL || !p.epi.fast;
}

// NCHW4 group convolution with whole channel blocks of 4 per group on both sides (the reference's NCHW4 group filter
// (G, OCpg, ICpg/4, FH, FW, 4), dnn/src/common/convolution.cpp:392-407): every group is a dense NCHW4 convolution on
// batch-strided views of src, dst and z, with its own contiguous piece of filter and bias -- one launch of the dense
// tiles per group, the way the reference's CUDA backend runs group convolutions over a dense algorithm
// (dnn/src/cuda/conv_bias/group_conv.cpp:10-44,76-104).
constexpr uint32_t kMaxGroupLaunches = 1024;
static bool igemm_group_by_launch(const ConvProblem& p) {
    const mi355_conv_desc& d = p.d;
    if (!(d.group > 1 && d.group <= kMaxGroupLaunches && !p.dw4 && p.icpg % 4 == 0)) return false;
    if (d.format == MI355_FMT_NCHW4) return p.ocpg % 4 == 0 && !igemm_needs_general(p);
    // planar destination: a group's output channels are a contiguous run of planes of every image (any ocpg); a
    // full-shape bias is indexed by the whole tensor's channel count, which a group's view does not have
    // (every group's piece of the filter starts 16-byte aligned)
    return d.format == MI355_FMT_NCHW4_NCHW && d.dst_dtype != MI355_DT_QS32 && d.bias_mode != MI355_BIAS_FULL &&
           ((uint64_t)p.ocpg * p.icpg * d.fh * d.fw) % 16 == 0;
}
static ConvProblem igemm_group_view(const ConvProblem& p) {
    ConvProblem q = p;
    q.d.group = 1;
    q.d.sparse = MI355_SPARSE_DENSE;
    q.d.ic = p.icpg;
    q.d.oc = p.ocpg;
    return q;  // batch strides stay those of the whole tensors
}

bool igemm_usable(const ConvProblem& p) {
    const mi355_conv_desc& d = p.d;
    if (p.dw4) return false;
    // group convolution: 32-packed tensors whose groups are whole channel blocks (second-generation tiles only), or
    // NCHW4 with whole blocks of 4 on both sides, one dense launch per group (igemm_group_view)
    if (d.group != 1 && !(p.pin == 32 && p.icpg % 32 == 0 && p.ocpg % 32 == 0) && !igemm_group_by_launch(p)) return false;
    // planar destination (NCHW4_NCHW: QuantizedS8 or Float32 dst, any bias shape, any scales): dense, on two of the
    // register-staged tiles, whose planar epilogue covers all of it
    const bool planar = d.format == MI355_FMT_NCHW4_NCHW;
    if (planar && ((d.group != 1 && !igemm_group_by_launch(p)) || d.dst_dtype == MI355_DT_QS32)) return false;
    if (d.format != MI355_FMT_NCHW4 && d.format != MI355_FMT_NCHW32 && d.format != MI355_FMT_NCHW4_NCHW32 &&
        d.format != MI355_FMT_NCHW32_NCHW4 && !planar)
        return false;
    if (d.mode != MI355_MODE_CROSS_CORRELATION || d.dilate_h != 1 || d.dilate_w != 1) return false;
    // QuantizedS32 dst (without a residual), full-shape bias and scales outside the fast forms' envelope run the
    // second-generation tiles with their general epilogue: 32-packed inputs only
    if (igemm_needs_general(p) && !planar) {
        if (p.pin != 32) return false;
        if (d.dst_dtype == MI355_DT_F32) return false;
    }
    if (d.fh > 255 || d.fw > 255 || d.pad_h > 0xfff || d.pad_w > 0xfff || d.ih > 0x3000 || d.iw > 0x3000) return false;
    // 32-bit byte offsets and buffer descriptors
    const int64_t lim = (int64_t)1 << 31;
    const int64_t src_b = (int64_t)(d.n - 1) * p.src_sn + (int64_t)d.ic * d.ih * d.iw;
    const int64_t dst_b = (int64_t)(d.n - 1) * p.dst_sn + (int64_t)d.oc * p.oh * p.ow;
    const int64_t z_b = d.has_z ? (int64_t)(d.n - 1) * p.z_sn + (int64_t)d.oc * p.oh * p.ow : 0;
    const int64_t flt_b = (int64_t)d.oc * p.icpg * d.fh * d.fw;
    if (src_b >= lim || dst_b >= lim || z_b >= lim || flt_b >= lim) return false;
    if ((int64_t)d.n * p.oh * p.ow >= lim) return false;
    const int64_t entries = p.pin == 32 ? (int64_t)(p.icpg / 32) * d.fh * d.fw : (int64_t)(p.icpg / 4) * d.fh * d.fw;
    // table capacity incl. the padding entries of the last stage (<= 8 chunks of 8 units)
    if (entries + 64 > IG_MAX_ENTRIES) return false;
    return true;
}

static int pick_cfg_by_shape(const ConvProblem& p, int cu_count, bool will_preprocess) {
    const mi355_conv_desc& d = p.d;
    if (p.pout == 1) {
        // planar destination: 128 x 128 tiles once they fill the device, else 64 x 64
        const int64_t t128 = (int64_t)((d.oc + 127) / 128) * (((int64_t)d.n * p.oh * p.ow + 127) / 128);
        return d.oc > 64 && t128 >= (cu_count > 0 ? cu_count : 256) ? 0 : 3;
    }
    if (p.pin == 32 && p.pout == 32 && d.group == 1 && !igemm_needs_general(p) && d.fh == 3 && d.fw == 3 &&
        d.stride_h == 1 && d.stride_w == 1 && d.pad_h == 1 && d.pad_w == 1 && (d.ic == 32 || d.ic == 64)) {
        // 3x3 over 32 or 64 channels with five and more 64 x 128 tiles for each of the two workgroups of a CU: the
        // weight-resident tile, whose workgroups load the filter once (64 -> 64 at 56 x 56, batch 128: 24.4 against 26.7 us
        // on the second-generation tile; at batch 64, three tiles per workgroup, its longer prologue loses: 15.7 against 14.8)
        const int64_t t = (int64_t)((d.oc + 63) / 64) * d.n * ((p.oh * p.ow + 127) / 128);
        const int v4 = igemm_first_v4_cfg();
        if (t >= 10 * (int64_t)(cu_count > 0 ? cu_count : 256) && igemm_resolve_cfg(p, v4) == v4) return v4;
    }
    if (p.pin == 32 && p.pout == 32 && d.group == 1 && !igemm_needs_general(p) && d.fh == 1 && d.fw == 1 && d.pad_h == 0 &&
        d.pad_w == 0 && d.ic <= 64 && d.oc <= 64) {
        // pointwise over at most 64 channels on both sides (the first 1x1 of a network's first bottleneck): nothing to
        // tile -- the streaming kernel, filter rows in registers (64 -> 64 at 56 x 56, batch 64: 7.3 against 8.0 us alone,
        // -3 us inside the ResNet-50 stack)
        const int s = igemm_pw32s_cfg();
        if (igemm_resolve_cfg(p, s) == s) return s;
    }
    if (p.pin == 32 && p.pout == 32 && d.group == 1 && !igemm_needs_general(p) && d.fh == 1 && d.fw == 1 && d.pad_h == 0 &&
        d.pad_w == 0 && d.has_z && d.ic <= 128) {
        // pointwise with a residual over at most 128 channels (the expanding 1x1 of a bottleneck block): bound by the
        // vector instructions of the requantisation, which the residual table form halves -- the streaming kernel where
        // the host has a proof for these scales (64 -> 256 at 56 x 56, batch 64: 20.5 against 23.4 us on the tiled kernel;
        // 128 -> 512 at 28 x 28: 14.6 against 16.1)
        // Over at most 64 channels the streaming kernel wins without a table too (64 -> 256 at 56 x 56 with the
        // multi-step form, inside the ResNet-50 stack: -4 us per step against the tiled kernel, alternating bench runs).
        float c;
        const float* tab;
        const int s = igemm_pw32s_cfg();
        if ((d.ic <= 64 || epi_residual_table(p.epi, &c, &tab)) && igemm_resolve_cfg(p, s) == s) return s;
    }
    if (will_preprocess && p.pin == 32 && p.pout == 32 && d.group == 1 && !igemm_needs_general(p)) {
        // The caller re-tiles the filter for the chosen algorithm (weight pre-processing): the second-generation tiles
        // then copy whole kilobytes for both operands.  Every tile was forced on every ResNet-50 shape in turn and timed
        // as whole-stack replays of one captured graph, against the unchanged stack in the same process.
        enum { V128x128x64r4 = 0, V128x128x128r3 = 2, V64x128x128r3 = 3, V64x128x64r4 = 4, V64x64x128r3 = 7, V64x64x128r4 = 8, V128x256x64w8 = 10, V256x256x64w8 = 11 };
        enum { V3_128x128x256r3 = 6 };
        const int v2 = igemm_first_v2_cfg();
        const int cu = cu_count > 0 ? cu_count : 256;
        const int64_t M = (int64_t)d.n * p.oh * p.ow;
        const int64_t t128 = ((d.oc + 127) / 128) * ((M + 127) / 128);
        const int kb = (int)(p.icpg * d.fh * d.fw);
        const bool pw = d.fh == 1 && d.fw == 1 && d.pad_h == 0 && d.pad_w == 0;
        // Large convolutions (six and more 128 x 128 tiles per CU, long reductions), with or without a residual: the
        // 8-wave tiles of 256 rows or columns, which read a residual in the epilogue instead of staging it in LDS
        // (1.8 / 2.2 / 2.1 Pop/s against 1.5 / 1.9 / 1.9 on the first-generation tiles for 3x3 256->256 at 64x64, 3x3
        // stride 2 512->1024 at 32x32 and 5x5 128->128 at 80x80, batch 128, residual + H_SWISH).
        if (t128 >= 6 * (int64_t)cu && kb >= 1024 && d.oc > 64) return v2 + (d.oc >= 256 ? V256x256x64w8 : V128x256x64w8);
        if (!d.has_z) {
            // the layers without a residual; the others stay on the first-generation tiles below, where the residual
            // costs no LDS
            if (d.oc <= 64) return v2 + V64x128x64r4;
            if (t128 >= cu) return v2 + V128x128x64r4;
            // a handful of tiles (small batches): the smallest tile puts the most CUs to work (3x3 256->256 at 14x14,
            // batch 1 and 8: 7.4 / 7.6 us against 8.9 / 9.1 on 64 x 128 tiles)
            const int64_t t64 = (int64_t)((d.oc + 63) / 64) * ((M + 127) / 128);
            if (2 * t64 < cu) return v2 + V64x64x128r3;
            const bool s1 = d.stride_h == 1 && d.stride_w == 1;
            // 3x3 over 256 channels at stride 1 with one 128 x 128 tile for most CUs: the patch-staged tile, whose stage of
            // eight k-chunks halves both the bytes through the CU's copy path and the stage boundaries (-1.4 us per
            // launch against the tile below on 256 -> 256 at 14 x 14, batch 64; falls back when the patch does not fit)
            if (d.fh == 3 && d.fw == 3 && s1 && kb >= 2304 && kb < 4608 && 2 * t128 >= cu) return igemm_first_v3_cfg() + V3_128x128x256r3;
            // long reductions with a 128 x 128 tile for more than half of the CUs: that tile, with half the operand bytes per
            // MAC of the 64 x 64 one (2048 -> 512 at 7 x 7, batch 128: 8.9 against 12.6 us; 3x3 512 -> 512: 17 against 24.6)
            if (kb >= 2048 && 2 * t128 > cu && (pw || s1 || kb >= 4608)) return v2 + V128x128x128r3;
            // pointwise: more pixels than channels per tile; with few tiles and a very long reduction the small tile with
            // the deepest ring
            if (pw) return v2 + (kb >= 2048 ? V64x64x128r4 : V64x128x128r3);
            if (kb >= 4608) return v2 + V64x64x128r4;
            if (s1) return v2 + V64x128x128r3;
            // few tiles, strided 3x3 over at most 256 channels: the first-generation tiles below
        }
    }
    const int64_t M = (int64_t)d.n * p.oh * p.ow;
    const int OC = d.oc;
    if (cu_count <= 0) cu_count = 256;
    // group convolution and the general epilogue: second-generation tiles only; a channel tile never spans two groups
    if (d.group != 1 || igemm_needs_general(p)) return igemm_first_v2_cfg() + (p.ocpg <= 64 ? 3 : 0);
    auto tiles = [&](int cfg) { return ((OC + kCfgs[cfg].bm - 1) / kCfgs[cfg].bm) * ((M + kCfgs[cfg].bn - 1) / kCfgs[cfg].bn); };
    const int kbytes = d.ic * d.fh * d.fw;
    if (p.pin == 4 && p.pout == 4 && d.fh == 1 && d.fw == 1 && d.pad_h == 0 && d.pad_w == 0) {
        // 4-packed pointwise layers (per-tile sweep of the MobileNetV2 1x1 layers): the LDS-direct tiles win wherever the
        // register-staged loop is latency-bound -- narrow outputs, and few tiles with a long reduction
        enum { D4_128x128x64 = kNumCfgs + 19, D4_64x64x128 = kNumCfgs + 20, D4_128x64x128 = kNumCfgs + 21, PW4_STREAM = kNumCfgs + 23 };
        // at most 64 channels in, many out (the expansions): the streaming kernel, which has no per-tile pipeline
        if (kbytes <= 64 && OC >= 64 && OC <= 1024) return PW4_STREAM;
        // one channel block out (the narrow projections): the same kernel, up to six k-steps
        if (OC <= 32 && kbytes <= 192) return PW4_STREAM;
        if (OC <= 32 && kbytes <= 256) return D4_128x128x64;
        if (OC > 32 && 2 * tiles(0) < 3 * cu_count) return kbytes >= 192 ? D4_64x64x128 : D4_128x64x128;
    }
    if (OC <= 32) {
        // 32 x 256 tiles waste no matrix rows, but need enough pixels to fill the chip (measured on the 4-packed
        // 1x1 projections of MobileNetV2)
        if (p.pin == 32 || tiles(4) >= 2 * cu_count) return 4;
        return tiles(0) >= cu_count ? 0 : 3;
    }
    if (p.pin == 32) {
        // 32-packed inputs: LDS-direct tiles (ids after the register-staged ones), chosen from a sweep of every
        // tile over the ResNet-50 / large-convolution shapes.  t128 = number of 128x128 tiles.
        enum {
            D128x128x64 = kNumCfgs + 0, D64x64x128 = kNumCfgs + 1, D128x128x128r2 = kNumCfgs + 7, D64x64x64r4 = kNumCfgs + 10,
            D128x64x128r2 = kNumCfgs + 11, D64x128x128r2 = kNumCfgs + 13, D128x128x64w8 = kNumCfgs + 14,
            D128x64x128w8 = kNumCfgs + 15, D256x128x64w8 = kNumCfgs + 16, D128x128x128r2w8 = kNumCfgs + 17,
            D64x64x128r2 = kNumCfgs + 6, D64x128x128w8 = kNumCfgs + 18, D64x64x128r4 = kNumCfgs + 12
        };
        if (OC <= 64) return kbytes <= 64 ? D128x128x64w8 : kbytes <= 256 ? D64x64x128r2 : D64x128x128r2;
        const int64_t t128 = tiles(0);
        // layers with a residual and a short reduction (the expanding 1x1 of a bottleneck block) are bound by their
        // epilogue: three 8-wave workgroups per CU at every size (whole-stack graph replays, each tile in turn)
        if (d.has_z && t128 >= cu_count && (kbytes <= 128 || (kbytes <= 512 && t128 < 2 * cu_count))) return D128x128x64w8;
        if (t128 >= 4 * cu_count)
            return kbytes >= 1024 ? (OC >= 256 ? D256x128x64w8 : D128x128x128r2) : (kbytes <= 128 ? D128x128x64w8 : D128x128x128r2w8);
        if (t128 >= 2 * cu_count) return D128x64x128r2;
        if (2 * t128 >= 3 * cu_count) return kbytes >= 512 ? D128x128x128r2w8 : D128x128x64;
        // few tiles, long reductions: the deeper ring hides the cold first touch of every weight byte; the longest
        // ones (3x3 over 256 channels) run best with more pixels than channels per tile
        if (kbytes >= 2304 && tiles(6) >= cu_count) return D64x128x128w8;
        if (tiles(7) >= cu_count) return D128x64x128w8;
        // fewer tiles than CUs: the longest reductions (3x3 over 512 channels) take the deepest ring, 2048-channel
        // pointwise layers the 8-wave tile with more pixels than channels
        if (kbytes >= 4608) return D64x64x128r4;
        return kbytes >= 2048 && 4 * tiles(6) >= 3 * cu_count ? D64x128x128w8 : D64x64x128;
    }
    if (OC <= 64) return tiles(1) >= cu_count ? 1 : 3;
    // 128x128 tiles as soon as they give every CU 1.5 tiles; the deeper k stage pays once the
    // reduction is long enough to amortise its larger prologue
    if (tiles(0) >= 2 * cu_count) return kbytes >= 512 ? 5 : 0;
    if (2 * tiles(0) >= 3 * cu_count) return kbytes >= 1024 ? 5 : 0;
    if (OC >= 256 && tiles(7) >= cu_count) return 7;
    if (tiles(6) >= cu_count) return 6;
    return 3;
}

size_t igemm_preprocessed_bytes(const ConvProblem& p, int cfg) {
    // the weight-resident tiles read the reference layout (once per workgroup: nothing to gain from re-tiling)
    if (p.pin != 32 || cfg < igemm_first_v2_cfg() || cfg >= igemm_first_v4_cfg()) return 0;
    return igemm2_preprocessed_bytes((int)p.d.oc, (int)(p.icpg * p.d.fh * p.d.fw));
}

int launch_igemm_preprocess(hipStream_t st, const ConvProblem& p, const int8_t* flt, int8_t* out) {
    return launch_igemm2_preprocess(st, flt, out, (int)p.d.oc, (int)(p.icpg * p.d.fh * p.d.fw));
}

// The chooser's tile, as the launch code will run it: what query() hands out names the kernel that executes.
int igemm_pick_cfg(const ConvProblem& p, int cu_count, bool will_preprocess) {
    if (igemm_group_by_launch(p)) return igemm_pick_cfg(igemm_group_view(p), cu_count, will_preprocess);
    const int c = pick_cfg_by_shape(p, cu_count, will_preprocess);
    const int r = igemm_resolve_cfg(p, c);
    return r >= 0 ? r : c;
}

// everything of IgemmArgs that follows from the problem alone (no tensor pointers, no tile)
static void igemm_fill_args(const ConvProblem& p, IgemmArgs& a) {
    const mi355_conv_desc& d = p.d;
    memset(&a, 0, sizeof(a));
    a.IH = d.ih; a.IW = d.iw; a.OH = p.oh; a.OW = p.ow; a.OHW = p.oh * p.ow;
    a.FH = d.fh; a.FW = d.fw; a.T = d.fh * d.fw;
    a.sh = d.stride_h; a.sw = d.stride_w; a.ph = d.pad_h; a.pw = d.pad_w;
    a.OC = d.oc;
    a.M = d.n * p.oh * p.ow;
    a.kbytes = p.icpg * d.fh * d.fw;
    a.KC = (a.kbytes + 31) / 32;
    a.entries = p.pin == 32 ? a.KC : (p.icpg / 4) * a.T;
    a.src_sn = (int)p.src_sn;
    a.src_scb = d.ih * d.iw * p.pin;
    a.dst_sn = (int)p.dst_sn;
    a.dst_scb = p.oh * p.ow * p.pout;
    a.z_sn = (int)p.z_sn;
    a.src_bytes = (uint32_t)((int64_t)(d.n - 1) * p.src_sn + (int64_t)d.ic * d.ih * d.iw);
    a.flt_bytes = (uint32_t)((int64_t)d.oc * a.kbytes);  // (groups x ocpg) rows of icpg * fh * fw bytes
    a.dst_bytes = (uint32_t)((int64_t)(d.n - 1) * p.dst_sn + (int64_t)d.oc * a.OHW);
    a.z_bytes = d.has_z ? (uint32_t)((int64_t)(d.n - 1) * p.z_sn + (int64_t)d.oc * a.OHW) : 0;
    a.has_bias = d.bias_mode == MI355_BIAS_BROADCAST_CHANNEL;
    a.div_ohw = make_fastdiv(a.OHW);
    a.div_ow = make_fastdiv(a.OW);
    a.div_t = make_fastdiv(a.T);
    a.div_fw = make_fastdiv(a.FW);
    a.epi = p.epi;
    a.flt_rstride = a.kbytes;
    a.flt_kstride = 32;
    a.NB = d.n;
    a.groups = d.group;
    a.ocpg = p.ocpg;
    a.src_sg = (p.icpg / p.pin) * a.src_scb;
    a.general = igemm_needs_general(p) && p.pout != 1 ? 1 : 0;
    a.dst_f32 = d.dst_dtype == MI355_DT_F32;
    if (a.dst_f32) a.has_bias = 0;  // a Float32 bias is added by the planar epilogue, not to the int32 accumulators
    a.dst_s32 = d.dst_dtype == MI355_DT_QS32;
    a.bias_full = d.bias_mode == MI355_BIAS_FULL;
    if (a.dst_s32) a.epi.s_b = a.epi.s_d;  // the sum lives in dst and is dequantised with the dtype of dst
}

static int staged_tile_of_shape(int bm, int bn, int kch) {
    int cfg = 0;
    for (int i = 0; i < kNumCfgs; ++i)
        if (kCfgs[i].bm == bm && kCfgs[i].bn == bn && kCfgs[i].kch == kch) cfg = i;
    return cfg;
}

int igemm_resolve_cfg(const ConvProblem& p, int cfg) {
    if (cfg < 0 || cfg >= igemm_num_cfgs()) return -1;
    if (igemm_group_by_launch(p)) return igemm_resolve_cfg(igemm_group_view(p), cfg);
    const mi355_conv_desc& d = p.d;
    IgemmArgs a;
    igemm_fill_args(p, a);
    if (a.M == 0 || a.OC == 0) return cfg;  // nothing is launched
    if (p.pout == 1) return cfg == 3 ? 3 : 0;  // planar destination: two register-staged tiles
    const int first_v2 = igemm_first_v2_cfg();
    // group convolutions and the general epilogue exist on the second-generation tiles only
    if ((d.group != 1 || a.general) && cfg < first_v2) cfg = first_v2 + (p.ocpg <= 64 ? 3 : 0);
    if (cfg == igemm_pw32s_cfg()) {
        // the 32-packed streaming kernel: pointwise over at most 128 channels; otherwise as above
        if (pw32s_usable(a, p.pin, p.pout)) return cfg;
        cfg = first_v2;
    }
    if (cfg >= igemm_first_v4_cfg()) {
        // the weight-resident tiles: 3x3 / stride 1 / pad 1 over 32 or 64 channels; otherwise as above
        if (igemm4_can_run(a, p.pin, p.pout, cfg - igemm_first_v4_cfg())) return cfg;
        cfg = first_v2;
    }
    if (cfg >= igemm_first_v3_cfg()) {
        // the patch-staged tiles: stride 1, a filter window, 32-packed, the fast epilogue; otherwise the second-generation
        // tile of 128 x 128 (resolved below like any other request for it)
        if (igemm3_can_run(a, p.pin, p.pout, cfg - igemm_first_v3_cfg())) return cfg;
        cfg = first_v2;
    }
    if (cfg >= first_v2) {
        if (p.pin == 32) {
            int v = cfg - first_v2;
            if (igemm2_can_run(a, p.pout, v)) return cfg;
            int bm, bn, kch;
            igemm2_cfg_shape(v, &bm, &bn, &kch);
            // the general epilogue exists on two tiles: the one with the asked tile's channel count, or the smaller one
            if (a.general) v = bm <= 64 ? 3 : 0;
            if (igemm2_can_run(a, p.pout, v)) return first_v2 + v;
            // ring + residual slots beyond the LDS of a CU: 128 x 128 x 64 with a ring of three always fits
            return first_v2 + 1;
        }
        // 4-packed inputs: the register-staged tile of the same shape
        int bm, bn, kch;
        igemm2_cfg_shape(cfg - first_v2, &bm, &bn, &kch);
        return staged_tile_of_shape(bm, bn, kch);
    }
    if (cfg >= kNumCfgs) {
        const int dcfg = cfg - kNumCfgs;
        const bool c4 = igemm_dma_cfg_is_pin4(dcfg);
        if (!c4 && p.pin == 32) return cfg;
        if (c4 && p.pin == 4 && p.pout == 4 && a.T == 1 && a.ph == 0 && a.pw == 0) {
            // the streaming kernel where it applies, else the 128 x 128 x 64 tile
            if (dcfg == igemm_dma_num_cfgs() - 1 && !pw4s_usable(a)) return kNumCfgs + igemm_dma_first_pin4_cfg();
            return cfg;
        }
        // no LDS-direct kernel for this packing / filter: the register-staged tile of the same shape
        int bm, bn, kch;
        igemm_dma_cfg_shape(dcfg, &bm, &bn, &kch);
        return staged_tile_of_shape(bm, bn, kch);
    }
    return cfg;
}

int launch_conv_igemm(hipStream_t st, const ConvProblem& p, int cfg, int cu_count, const int8_t* src,
                      const int8_t* flt, const int32_t* bias, const int8_t* z, int8_t* dst, bool flt_preprocessed) {
    if (igemm_group_by_launch(p)) {
        if (flt_preprocessed) return (int)hipErrorInvalidValue;
        const ConvProblem q = igemm_group_view(p);
        const mi355_conv_desc& d = p.d;
        const int64_t src_g = (int64_t)p.icpg * d.ih * d.iw, dst_g = (int64_t)p.ocpg * p.oh * p.ow;
        const int64_t flt_g = (int64_t)p.ocpg * p.icpg * d.fh * d.fw;
        const int64_t eb = d.dst_dtype == MI355_DT_F32 ? 4 : 1;  // bytes per element of dst and z (bias: 4 either way)
        for (uint32_t g = 0; g < d.group; ++g) {
            const int rc = launch_conv_igemm(st, q, cfg, cu_count, src + g * src_g, flt + g * flt_g,
                                             bias ? bias + (int64_t)g * p.ocpg : nullptr, z ? z + g * dst_g * eb : nullptr,
                                             dst + g * dst_g * eb, false);
            if (rc) return rc;
        }
        return 0;
    }
    IgemmArgs a;
    igemm_fill_args(p, a);
    a.src = src; a.flt = flt; a.bias = bias; a.z = z; a.dst = dst;
    if (a.M == 0 || a.OC == 0) return 0;
    cfg = igemm_resolve_cfg(p, cfg);
    if (cfg < 0) return (int)hipErrorInvalidValue;
    if (flt_preprocessed) {
        if (igemm_preprocessed_bytes(p, cfg) == 0) return (int)hipErrorInvalidValue;
        const int ocp = (a.OC + 31) / 32 * 32;
        a.flt_rstride = 32;
        a.flt_kstride = ocp * 32;
        a.flt_bytes = (uint32_t)igemm_preprocessed_bytes(p, cfg);
    }
    if (p.pout == 1) {
        if (p.d.bias_mode == MI355_BIAS_NONE) a.bias = nullptr;  // the planar epilogue tests the pointer
        return launch_planar(st, a, cfg, cu_count);
    }
    const int first_v2 = igemm_first_v2_cfg();
    a.ztab = nullptr;
    if (cfg == igemm_pw32s_cfg() && !a.general) {
        // the streaming kernel holds the residual table in LDS: it takes the table form where the host has proved it
        // for these scales.  (The first-generation LDS-direct kernel with the table behind its ring, tried on the
        // residual layers over 256 and 512 channels, changed the ResNet-50 step by +1 us: those are not bound by their
        // vector instructions.)
        float c;
        const float* tab;
        if (epi_residual_table(a.epi, &c, &tab)) {
            a.epi.zlin = 1;
            a.epi.lin_c = c;
            a.ztab = tab;
        }
    }
    if (cfg == igemm_pw32s_cfg()) return launch_pw32s(st, a, cu_count);
    if (cfg >= igemm_first_v4_cfg()) return launch_igemm4(st, a, p.pin, p.pout, cfg - igemm_first_v4_cfg(), cu_count);
    if (cfg >= igemm_first_v3_cfg()) return launch_igemm3(st, a, p.pin, p.pout, cfg - igemm_first_v3_cfg());
    if (cfg >= first_v2) return launch_igemm2(st, a, p.pout, cfg - first_v2, cu_count);
    if (cfg >= kNumCfgs) return launch_igemm_dma(st, a, p.pout, cfg - kNumCfgs, cu_count);
    if (p.pin == 32 && p.pout == 32) return launch_fmt<32, 32>(st, a, cfg, cu_count);
    if (p.pin == 4 && p.pout == 4) return launch_fmt<4, 4>(st, a, cfg, cu_count);
    if (p.pin == 4 && p.pout == 32) return launch_fmt<4, 32>(st, a, cfg, cu_count);
    return launch_fmt<32, 4>(st, a, cfg, cu_count);
}

}  // namespace mi355
