// Implicit-GEMM int8 ConvBias with LDS-direct operand staging (32-packed inputs: NCHW32, NCHW32_NCHW4; 4-packed
// inputs on the pointwise path, NCHW4 in and out: see PIN = 4 at DmaKernel).
//
// Same tiling, MFMA layout, LDS swizzle and fused epilogue as conv_igemm.hip; what differs is how a
// k-stage travels from global memory to LDS:
//
//   * buffer_load_dwordx4 ... lds: one wave instruction copies 64 x 16 bytes straight into LDS, lane l to
//     address M0 + 16 * l (out-of-range lanes write zeros).  No staging registers, no ds_write.  The LDS
//     side of a copy is therefore lane-linear -- 64 consecutive 16-byte slots, i.e. 64 / S whole rows of a
//     tile -- and the swizzle is applied on the GLOBAL side: the lane that owns physical slot p of row r
//     fetches logical slot p ^ swz(r).
//   * a ring of NS stage buffers in LDS.  Iteration i waits until ITS stage has landed (all but the
//     (NS - 2) * (UA + UB) youngest copies of this wave complete), passes the workgroup barrier, refills the
//     buffer that iteration i - 1 just finished reading with stage i + NS - 1, and multiplies.  The copies are
//     issued from inline assembly and waited for with explicit s_waitcnt vmcnt(n): vector-memory operations
//     complete in order, so any compiler-issued load or store in between can only make such a wait
//     stricter, never too weak; and because the compiler does not see the copies, it cannot serialise them.
//   * before the workgroup ends it waits for every copy (vmcnt(0)): a copy landing after the LDS allocation
//     has been handed to another workgroup would corrupt it.
//   * the stages of a tile split into a steady loop, whose refills stay inside the tile (no tile bookkeeping: with 16
//     waves on a CU the one scalar unit paces a loop that carries it), and the last NS stages, whose refills cross
//     into the workgroup's next tile.  The bias of the workgroup's channel tile sits in LDS, written once: tiles of
//     one workgroup are a multiple of the channel-tile count apart whenever that count is a power of two.
#include <atomic>

#include "igemm_shared.h"
#include "lds_copy.h"

namespace mi355 {
namespace {

// PIN = 4 (4-packed activations, pointwise only): a pixel's 4 channels are the only contiguous bytes, so the
// activation tile travels as 64 x 4-byte copies -- lane = pixel, one channel block per copy -- and sits in LDS as
// [block of 64 pixels][channel block][pixel] dwords; an MFMA B fragment (16 k-bytes of one pixel = 4 channel blocks)
// is read as four dwords 256 bytes apart.  Filters are laid out and copied exactly as for 32-packed inputs.
template <int POUT, int BM, int BN, int WM, int WN, int KCH, int NS, bool PW, int PIN = 32>
struct DmaKernel {
    static constexpr int NW = WM * WN;             // waves per workgroup (4 or 8)
    static constexpr int THREADS = NW * 64;
    static constexpr int WTM = BM / WM, WTN = BN / WN;
    static constexpr int MT = WTM / 32, NT = WTN / 32;
    static constexpr int S = KCH * 2;              // 16-byte slots per LDS row
    static constexpr int ROWB = KCH * 32;          // bytes per LDS row
    static constexpr int RPL = 64 / S;             // rows per wave copy (64 slots = 1 KiB)
    static constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB;
    static constexpr int STG = A_BYTES + B_BYTES;  // one stage
    static constexpr int UA = BM / (RPL * NW);     // copies per wave per stage
    static constexpr int UB32 = BN / (RPL * NW);
    static constexpr int NB64 = BN / 64;           // 4-packed: blocks of 64 pixels
    static constexpr int CB = KCH * 8;             // 4-packed: channel blocks per stage
    static constexpr int UB4 = NB64 * CB / NW;     // 4-packed: dword copies per wave per stage
    static constexpr int CPB = CB / NW;            // ... of which per pixel block
    static constexpr int UB = PIN == 4 ? UB4 : UB32;
    static constexpr int NOFF = PIN == 4 ? (NB64 > 0 ? NB64 : 1) : UB32;  // per-lane activation offsets kept by the loader
    static constexpr int U = UA + UB;
    static_assert(PIN == 32 || (PIN == 4 && PW && BN % 64 == 0 && CB % NW == 0), "4-packed inputs: pointwise tiles of whole 64-pixel blocks");
    // bias of the workgroup's channel tile; it arrives by whole-wave copies of 64 dwords (a 32-row tile leaves half of one unused)
    static constexpr int BIAS_BYTES = (BM < 64 ? 64 : BM) * 4;
    static constexpr int RING_BYTES = NS * STG + BIAS_BYTES;
    static_assert(NW == 4 || NW == 8, "4 or 8 waves");
    static_assert(UA >= 1 && UB >= 1 && BM % (RPL * NW) == 0 && (PIN == 4 || BN % (RPL * NW) == 0), "tile vs copy granularity");
    static_assert(NS >= 2 && (NS - 2) * U < 64, "ring depth");
    // swz() looks at row bits 0..3; rows of copy j of wave w are (NW j + w) * RPL + lane / S, so with RPL >= 8 those
    // bits never depend on j: a lane's logical slot is the same for all of its copies
    static_assert(RPL >= 8, "slot must not depend on the copy index");

    struct Loader {
        int tile, stage, kc0;
        int a_off[UA];            // filter: byte offset of (row, logical slot), SENT past OC
        int b_off[NOFF];          // activation: byte offset of the pixel (+ chunk / half for the pointwise path)
        int ih0[NOFF], iw0[NOFF]; // table path: top-left input coordinate (ih0 = -0x8000 past M)
    };

    __device__ static __forceinline__ void tile_coords(const IgemmArgs& a, int tile, int& oc0, int& pix0) {
        const int tn = (int)fdiv((uint32_t)tile, a.div_tiles_m), tm = tile - tn * a.tiles_m;
        oc0 = tm * BM;
        pix0 = tn * BN;
    }

    // lane's row inside copy j of wave w, and its logical slot (constant per lane)
    __device__ static __forceinline__ int row_of(int w, int lane, int j) { return (NW * j + w) * RPL + lane / S; }
    __device__ static __forceinline__ int slot_of(int w, int lane) { return (lane % S) ^ swz<S>(w * RPL + lane / S); }

    __device__ static __forceinline__ void loader_enter_tile(const IgemmArgs& a, Loader& L, int tile, int w, int lane) {
        int oc0, pix0;
        tile_coords(a, tile, oc0, pix0);
        const int s = slot_of(w, lane);
#pragma unroll
        for (int j = 0; j < UA; ++j) {
            const int oc = oc0 + row_of(w, lane, j);
            L.a_off[j] = oc < a.OC ? oc * a.kbytes + s * 16 : SENT;
        }
        if (PIN == 4) {
#pragma unroll
            for (int b = 0; b < NB64; ++b) {
                const int m = pix0 + b * 64 + lane;
                const bool ok = m < a.M;
                const uint32_t mm = ok ? m : 0;
                const uint32_t n = fdiv(mm, a.div_ohw), rem = mm - n * a.OHW;
                const uint32_t oh = fdiv(rem, a.div_ow), ow = rem - oh * a.OW;
                L.b_off[b] = ok ? (int)n * a.src_sn + ((int)oh * a.sh * a.IW + (int)ow * a.sw) * 4 : SENT;
            }
            return;
        }
#pragma unroll
        for (int j = 0; j < UB; ++j) {
            const int m = pix0 + row_of(w, lane, j);
            const bool ok = m < a.M;
            const uint32_t mm = ok ? m : 0;
            const uint32_t n = fdiv(mm, a.div_ohw), rem = mm - n * a.OHW;
            const uint32_t oh = fdiv(rem, a.div_ow), ow = rem - oh * a.OW;
            const int ih0 = (int)oh * a.sh - a.ph, iw0 = (int)ow * a.sw - a.pw;
            const int base = (int)n * a.src_sn + (ih0 * a.IW + iw0) * 32 + (s & 1) * 16;
            if (PW) {
                L.b_off[j] = ok ? base + (s >> 1) * a.src_scb : SENT;
            } else {
                L.b_off[j] = base;
                L.ih0[j] = ok ? ih0 : -0x8000;  // makes every tap fail the bounds test
                L.iw0[j] = iw0;
            }
        }
    }

    __device__ static __forceinline__ void loader_kill(Loader& L) {
#pragma unroll
        for (int j = 0; j < UA; ++j) L.a_off[j] = SENT;
#pragma unroll
        for (int j = 0; j < NOFF; ++j) {
            L.b_off[j] = SENT;
            L.ih0[j] = -0x8000;
        }
        L.kc0 = 0;
    }

    // copies of one stage into ring buffer `buf` (LDS byte address lds0 + buf * STG); always U copies per wave.
    // PF: the caller already holds this lane's table entry (*pk), read one iteration ahead
    template <bool PF = false>
    __device__ static __forceinline__ void issue(const IgemmArgs& a, const Loader& L, const KEntry* tab, const v4i& rs_src,
                                                 const v4i& rs_flt, uint32_t stage_addr, int w, int lane,
                                                 const KEntry* pk = nullptr) {
        const int a_k = L.kc0 * 32;
#pragma unroll
        for (int j = 0; j < UA; ++j) {
            // SENT plus a stage offset is still out of range
            lds_copy64x16(stage_addr + (uint32_t)((NW * j + w) * 1024), L.a_off[j] + a_k, rs_flt);
        }
        if (PIN == 4) {
            // copy j of wave w: pixel block j / CPB, channel block (j % CPB) * NW + w of this stage.  A channel block
            // past the last one (K not a whole number of stages) reads as zeros: SENT plus a pixel offset stays out
            // of range; SENT plus SENT (a row past M as well) wraps to offset 0, whose bytes only meet discarded rows
            const int icb = a.kbytes >> 2;
#pragma unroll
            for (int j = 0; j < UB4; ++j) {
                const int cbl = (j % CPB) * NW + w;
                const int cb = L.kc0 * 8 + cbl;
                const int k_off = cb < icb ? cb * a.src_scb : SENT;  // wave-uniform
                lds_copy64x4(stage_addr + (uint32_t)(A_BYTES + ((j / CPB) * CB + cbl) * 256), (int)((uint32_t)L.b_off[j / CPB] + (uint32_t)k_off), rs_src);
            }
        } else if (PW) {
            const int b_k = L.kc0 * a.src_scb;
#pragma unroll
            for (int j = 0; j < UB; ++j) {
                lds_copy64x16(stage_addr + (uint32_t)(A_BYTES + (NW * j + w) * 1024), L.b_off[j] + b_k, rs_src);
            }
        } else {
            const KEntry k = PF ? *pk : tab[L.kc0 + (slot_of(w, lane) >> 1)];  // this lane's k-chunk: channel block and tap
            const int fh = k.fhfw & 0xffff, fw = k.fhfw >> 16;
#pragma unroll
            for (int j = 0; j < UB; ++j) {
                const int ih = L.ih0[j] + fh, iw = L.iw0[j] + fw;
                const bool ok = (unsigned)ih < (unsigned)a.IH && (unsigned)iw < (unsigned)a.IW;
                lds_copy64x16(stage_addr + (uint32_t)(A_BYTES + (NW * j + w) * 1024), ok ? L.b_off[j] + k.off : SENT, rs_src);
            }
        }
    }

    __device__ static __forceinline__ void init_acc_lds(v16i (&acc)[MT][NT], const int* sBias, int wm, int lh) {
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

    // Per tile: a steady loop whose refills stay inside the tile -- the loader only steps along k, so the loop carries no
    // tile bookkeeping (with 16 waves on a CU its one scalar unit paces a loop that does) -- then the last NS stages, whose
    // refills cross into the next tile and which carry the residual prefetch and the next tile's coordinates.
    __device__ static __forceinline__ void run(const IgemmArgs& a) {
        extern __shared__ __attribute__((aligned(16))) int8_t lds[];
        KEntry* tab = reinterpret_cast<KEntry*>(lds + RING_BYTES);
        const uint32_t lds0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)lds);

        const int t = threadIdx.x;
        const int lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
        const int l32 = lane & 31, lh = lane >> 5;
        const int wm = wave / WN, wn = wave % WN;

        // this workgroup's tile sequence (XCD-contiguous ranges, see conv_igemm.hip)
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
        const int my_tiles = first < last ? (int)fdiv((uint32_t)(last - first + step - 1), a.div_step) : 0;
        const int total = my_tiles * a.nstages;

        // The bias of the workgroup's channel tile lives in LDS, copied there once: workgroups mostly stay on one channel
        // tile (their tile stride is a multiple of the number of channel tiles whenever that is a power of two), so the
        // copy is read at every tile start and almost never rewritten.
        int* sBias = reinterpret_cast<int*>(lds + NS * STG);
        int c_tile = first, c_oc0, c_pix0;
        tile_coords(a, c_tile, c_oc0, c_pix0);
        // An LDS-direct copy like the operands' (no register is the target of a load the compiler does not know about),
        // requested before the prologue's copies: its cold miss overlaps theirs, and it is older than all of them.
        // Without a bias the buffer has no bytes: every lane writes 0, and so do channels past the last one.
        const v4i rs_bias = uniform_rsrc(a.bias, a.has_bias ? (uint32_t)a.OC * 4u : 0u);
        const bool bias_wave = wave * 64 < BM;  // wave-uniform
        if (total != 0 && bias_wave) lds_copy64x4(lds0 + (uint32_t)(NS * STG + wave * 256), (c_oc0 + t) * 4, rs_bias);

        if (!PW) {
            const int cap = a.nstages * KCH;
            for (int e = t; e < cap; e += THREADS) {
                KEntry k;
                if (e < a.entries) {
                    const uint32_t cb = fdiv(e, a.div_t), tap = e - cb * a.T;
                    const uint32_t fh = fdiv(tap, a.div_fw), fw = tap - fh * a.FW;
                    k.off = (int)cb * a.src_scb + ((int)fh * a.IW + (int)fw) * 32;
                    k.fhfw = (int)(fh | (fw << 16));
                } else {
                    k.off = 0;
                    k.fhfw = 0x4000;
                }
                tab[e] = k;
            }
        }
        if (total == 0) return;

        const v4i rs_src = uniform_rsrc(a.src, a.src_bytes);
        const v4i rs_flt = uniform_rsrc(a.flt, a.flt_bytes);

        Loader L;
        L.tile = first;
        L.stage = 0;
        L.kc0 = 0;
        loader_enter_tile(a, L, first, wave, lane);
        int issued = 0;
        auto advance = [&]() __attribute__((always_inline)) {
            ++issued;
            L.kc0 += KCH;
            if (++L.stage == a.nstages) {
                L.stage = 0;
                L.kc0 = 0;
                L.tile += step;
                if (issued < total) loader_enter_tile(a, L, L.tile, wave, lane);
            }
            if (issued >= total) loader_kill(L);
        };

        if (!PW) __syncthreads();  // table ready

        // prologue: stages 0 .. NS - 2 go to buffers 0 .. NS - 2
#pragma unroll
        for (int s = 0; s < NS - 1; ++s) {
            issue(a, L, tab, rs_src, rs_flt, lds0 + (uint32_t)(s * STG), wave, lane);
            advance();
        }
        v16i acc[MT][NT];
        // the bias copy is older than every copy of the prologue (the counter holds at most 63: with more copies than
        // that in the prologue the oldest operations, this one first, have completed by the time the last copy was accepted)
        wait_vmcnt<((NS - 1) * U < 63 ? (NS - 1) * U : 63)>();
        __syncthreads();
        init_acc_lds(acc, sBias, wm, lh);
        int rd_off = 0;                                     // byte offset of the stage being multiplied
        uint32_t wr_addr = lds0 + (uint32_t)((NS - 1) * STG);  // LDS address of the stage buffer refilled next

        constexpr bool DUAL = MT * NT == 1;
        v16i alt;

        // stage `rd` times the accumulators, then both ring positions step
        auto multiply = [&]() __attribute__((always_inline)) {
            const int8_t* pA = lds + rd_off;
            const int8_t* pB = pA + A_BYTES;
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
                    if (PIN == 4) {
                        const int* q = reinterpret_cast<const int*>(pB) + ((row >> 6) * CB + c * 8 + lh * 4) * 64 + (row & 63);
                        xb[j][0] = q[0]; xb[j][1] = q[64]; xb[j][2] = q[128]; xb[j][3] = q[192];
                    } else {
                        const int slot = (c * 2 + lh) ^ swz<S>(row);
                        xb[j] = *reinterpret_cast<const v4i*>(pB + row * ROWB + slot * 16);
                    }
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
#pragma unroll
                for (int c = 0; c < KCH; ++c) mfmas(c, fa[c], fb[c]);
            } else {
                frags(0, fa[0], fb[0]);
#pragma unroll
                for (int c = 0; c < KCH; ++c) {
                    if (c + 1 < KCH) frags(c + 1, fa[(c + 1) & 1], fb[(c + 1) & 1]);
                    mfmas(c, fa[c & 1], fb[c & 1]);
                }
            }
            rd_off = rd_off + STG == NS * STG ? 0 : rd_off + STG;
            wr_addr = wr_addr + STG == lds0 + NS * STG ? lds0 : wr_addr + STG;
        };

        // Stages of one tile split into a steady part, whose refills stay inside the tile (the loader only steps
        // along k: no tile bookkeeping in that loop), and the last NS stages, whose refills cross into the next tile.
        const int steady = a.nstages > NS ? a.nstages - NS : 0;
        for (int ti = 0; ti < my_tiles; ++ti) {
            if (DUAL) alt = v16i{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            KEntry nk;  // the table entry of the next refill, read while the current stage multiplies
            if (!PW && steady > 0) nk = tab[L.kc0 + (slot_of(wave, lane) >> 1)];
            for (int s = 0; s < steady; ++s) {
                // this wave's copies of the stage have landed once at most the NS - 2 younger stages are in flight
                wait_vmcnt<(NS - 2) * U>();
                __syncthreads();  // ... of every wave; and every wave is done reading the buffer refilled next
                issue<!PW>(a, L, tab, rs_src, rs_flt, wr_addr, wave, lane, &nk);
                ++issued;
                ++L.stage;
                L.kc0 += KCH;
                if (!PW) nk = tab[L.kc0 + (slot_of(wave, lane) >> 1)];
                multiply();
            }
            ZRegs<MT, NT> zr;
            int n_oc0 = c_oc0, n_pix0 = c_pix0;
            for (int s = steady; s < a.nstages; ++s) {
                wait_vmcnt<(NS - 2) * U>();
                __syncthreads();
                // the residual of a tile is requested at the start of its last stage -- before this iteration's
                // copies, so that waiting for it in the epilogue does not also wait for them
                const bool last_stage = s + 1 == a.nstages;
                if (last_stage && a.epi.has_z)
                    igemm_load_z<POUT, MT, NT>(a, zr, c_oc0 + wm * WTM, c_pix0 + wn * WTN, l32, lh);
                issue(a, L, tab, rs_src, rs_flt, wr_addr, wave, lane);
                advance();
                if (last_stage && ti + 1 < my_tiles) {
                    tile_coords(a, c_tile + step, n_oc0, n_pix0);
                }
                multiply();
            }
            if (DUAL) acc[0][0] += alt;
            igemm_run_epilogue<POUT, MT, NT, true>(a, acc, c_oc0 + wm * WTM, c_pix0 + wn * WTN, l32, lh, &zr);
            c_tile += step;
            if (ti + 1 < my_tiles) {
                if (n_oc0 != c_oc0) {
                    // rare: another channel tile.  Everyone is done with the old copy before it is replaced, and
                    // sees the new one before it is read (a workgroup-uniform branch: barriers are safe here)
                    __syncthreads();
                    if (t < BM) sBias[t] = fetch_bias(a, n_oc0, t);
                    __syncthreads();
                }
                init_acc_lds(acc, sBias, wm, lh);
            }
            c_oc0 = n_oc0;
            c_pix0 = n_pix0;
        }
        // the trailing (out-of-range, zero-filling) copies must land before this workgroup's LDS is released
        wait_vmcnt<0>();
    }
};

template <int POUT, int BM, int BN, int WM, int WN, int KCH, int NS, int MINW, bool PW, int PIN = 32>
__global__ __launch_bounds__(WM * WN * 64, MINW) void igemm_dma_kernel(IgemmArgs a) {
    DmaKernel<POUT, BM, BN, WM, WN, KCH, NS, PW, PIN>::run(a);
}

struct DmaCfg {
    const char* name;
    int bm, bn, kch;
};
// tile_cfg of mi355_algo = number of register-staged tiles + index here
const DmaCfg kDma[] = {
        {"dma128x128x64", 128, 128, 2},
        {"dma64x64x128", 64, 64, 4},
        {"dma128x64x128", 128, 64, 4},
        {"dma64x128x128", 64, 128, 4},
        {"dma128x128x128", 128, 128, 4},
        {"dma64x256x64", 64, 256, 2},
        {"dma64x64x128r2", 64, 64, 4},
        {"dma128x128x128r2", 128, 128, 4},
        {"dma256x128x64", 256, 128, 2},
        {"dma128x128x64r4", 128, 128, 2},
        {"dma64x64x64r4", 64, 64, 2},
        {"dma128x64x128r2", 128, 64, 4},
        {"dma64x64x128r4", 64, 64, 4},
        {"dma64x128x128r2", 64, 128, 4},
        {"dma128x128x64w8", 128, 128, 2},
        {"dma128x64x128w8", 128, 64, 4},
        {"dma256x128x64w8", 256, 128, 2},
        {"dma128x128x128r2w8", 128, 128, 4},
        {"dma64x128x128w8", 64, 128, 4},
        // 4-packed pointwise (NCHW4 in and out); other problems run the register-staged tile of the same shape
        {"dma4_128x128x64", 128, 128, 2},
        {"dma4_64x64x128", 64, 64, 4},
        {"dma4_128x64x128", 128, 64, 4},
        {"dma4_32x256x128", 32, 256, 4},
        // no tile at all: the streaming kernel of conv_pw4.hip where it applies, else dma4_128x128x64
        {"pw4_stream", 128, 128, 2},
};
constexpr int kFirstDma4 = 19;
constexpr int kNumDma = sizeof(kDma) / sizeof(kDma[0]);

template <int POUT, int BM, int BN, int WM, int WN, int KCH, int NS, int MINW, bool PW, int PIN = 32>
int launch_pw(hipStream_t st, IgemmArgs& a, int cu_count) {
    using K = DmaKernel<POUT, BM, BN, WM, WN, KCH, NS, PW, PIN>;
    a.tiles_m = (a.OC + BM - 1) / BM;
    a.div_tiles_m = make_fastdiv((uint32_t)a.tiles_m);
    a.tiles_n = (a.M + BN - 1) / BN;
    const int64_t tiles = (int64_t)a.tiles_m * a.tiles_n;
    if (tiles <= 0 || tiles > 0x3fffffff) return (int)hipErrorInvalidValue;
    a.tiles = (int)tiles;
    a.nstages = (a.KC + KCH - 1) / KCH;
    const int tab_entries = PW ? 0 : a.nstages * KCH;
    const int lds = K::RING_BYTES + tab_entries * 8;
    auto kern = igemm_dma_kernel<POUT, BM, BN, WM, WN, KCH, NS, MINW, PW, PIN>;
    // per-instantiation caches; atomics, because operators on different streams may launch from several threads
    static std::atomic<int> max_lds_set{0};
    if (lds > max_lds_set.load(std::memory_order_relaxed)) {
        const int want = K::RING_BYTES + IG_MAX_ENTRIES * 8;
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, want);
        if (e != hipSuccess) return (int)e;
        max_lds_set.store(want, std::memory_order_relaxed);
    }
    static std::atomic<uint64_t> occ_cache{0};  // LDS bytes of the last query << 32 | its result
    const uint64_t cached = occ_cache.load(std::memory_order_relaxed);
    int occ = (int)(uint32_t)cached;
    if ((cached >> 32) != (uint64_t)lds || occ < 1) {
        hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, reinterpret_cast<const void*>(kern),
                                                                    K::THREADS, (size_t)lds);
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
    a.div_step = make_fastdiv((uint32_t)((grid & 7) == 0 ? grid >> 3 : grid));  // the kernel's tile stride
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(K::THREADS), lds, st, a);
    return (int)hipGetLastError();
}

template <int POUT, int BM, int BN, int WM, int WN, int KCH, int NS, int MINW>
int launch_one(hipStream_t st, IgemmArgs& a, int cu) {
    const bool pw = a.T == 1 && a.ph == 0 && a.pw == 0 && a.kbytes % (32 * KCH) == 0;
    return pw ? launch_pw<POUT, BM, BN, WM, WN, KCH, NS, MINW, true>(st, a, cu)
              : launch_pw<POUT, BM, BN, WM, WN, KCH, NS, MINW, false>(st, a, cu);
}

template <int POUT>
int launch_fmt(hipStream_t st, IgemmArgs& a, int cfg, int cu) {
    switch (cfg) {
        case 0: return launch_one<POUT, 128, 128, 2, 2, 2, 3, 2>(st, a, cu);
        case 1: return launch_one<POUT, 64, 64, 2, 2, 4, 3, 3>(st, a, cu);
        case 2: return launch_one<POUT, 128, 64, 2, 2, 4, 3, 2>(st, a, cu);
        case 3: return launch_one<POUT, 64, 128, 2, 2, 4, 3, 2>(st, a, cu);
        case 4: return launch_one<POUT, 128, 128, 2, 2, 4, 3, 2>(st, a, cu);
        case 5: return launch_one<POUT, 64, 256, 1, 4, 2, 3, 2>(st, a, cu);
        case 6: return launch_one<POUT, 64, 64, 2, 2, 4, 2, 3>(st, a, cu);
        case 7: return launch_one<POUT, 128, 128, 2, 2, 4, 2, 2>(st, a, cu);
        case 8: return launch_one<POUT, 256, 128, 2, 2, 2, 3, 1>(st, a, cu);
        case 9: return launch_one<POUT, 128, 128, 2, 2, 2, 4, 2>(st, a, cu);
        case 10: return launch_one<POUT, 64, 64, 2, 2, 2, 4, 3>(st, a, cu);
        case 11: return launch_one<POUT, 128, 64, 2, 2, 4, 2, 2>(st, a, cu);
        case 12: return launch_one<POUT, 64, 64, 2, 2, 4, 4, 3>(st, a, cu);
        case 13: return launch_one<POUT, 64, 128, 2, 2, 4, 2, 2>(st, a, cu);
        case 14: return launch_one<POUT, 128, 128, 2, 4, 2, 3, 6>(st, a, cu);  // 80 VGPRs: three 8-wave workgroups per CU
        case 15: return launch_one<POUT, 128, 64, 4, 2, 4, 3, 2>(st, a, cu);
        case 16: return launch_one<POUT, 256, 128, 4, 2, 2, 3, 4>(st, a, cu);
        case 17: return launch_one<POUT, 128, 128, 2, 4, 4, 2, 2>(st, a, cu);
        case 18: return launch_one<POUT, 64, 128, 2, 4, 4, 3, 2>(st, a, cu);
        case 19: return launch_pw<4, 128, 128, 2, 2, 2, 3, 2, true, 4>(st, a, cu);
        case 20: return launch_pw<4, 64, 64, 2, 2, 4, 4, 3, true, 4>(st, a, cu);
        case 21: return launch_pw<4, 128, 64, 2, 2, 4, 3, 2, true, 4>(st, a, cu);
        case 22: return launch_pw<4, 32, 256, 1, 4, 4, 3, 2, true, 4>(st, a, cu);
        case 23: return pw4s_usable(a) ? launch_pw4s(st, a, cu) : launch_pw<4, 128, 128, 2, 2, 2, 3, 2, true, 4>(st, a, cu);
        default: return (int)hipErrorInvalidValue;
    }
}

}  // namespace

int igemm_dma_num_cfgs() { return kNumDma; }
const char* igemm_dma_cfg_name(int cfg) { return cfg >= 0 && cfg < kNumDma ? kDma[cfg].name : "?"; }
void igemm_dma_cfg_shape(int cfg, int* bm, int* bn, int* kch) {
    *bm = kDma[cfg].bm; *bn = kDma[cfg].bn; *kch = kDma[cfg].kch;
}

bool igemm_dma_cfg_is_pin4(int cfg) { return cfg >= kFirstDma4; }
int igemm_dma_first_pin4_cfg() { return kFirstDma4; }

int launch_igemm_dma(hipStream_t st, IgemmArgs& a, int pout, int cfg, int cu_count) {
    return pout == 32 ? launch_fmt<32>(st, a, cfg, cu_count) : launch_fmt<4>(st, a, cfg, cu_count);
}

}  // namespace mi355
