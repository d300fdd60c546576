// Implicit-GEMM int8 ConvBias for 32-packed inputs with filters larger than 1x1 at stride 1 (NCHW32, dense): the
// activations of a tile are staged in LDS ONCE per channel block, as the patch of input pixels that the tile's outputs
// touch, and every filter tap reads its MFMA fragments from that patch.  The implicit-GEMM kernels of conv_igemm2.hip
// copy the im2col matrix instead: FH x FW times the same bytes through the CU's 64 bytes-per-clock path from L2.
// Measured: the activation copies this kernel saves are worth 2-3 % on 3x3 256 -> 256 at 64 x 64, batch 128 (1.93 against
// 1.87 Pop/s on the best second-generation tile) and nothing or less on the other large shapes and on every ResNet-50
// layer, where the second-generation tiles' L2 hits are cheap and this kernel's per-tile patch prologue is not.  The
// tiles are therefore selectable by id and profiled by fast-run, but not chosen by the heuristic.
//
//   D[oc][pixel] = sum over (channel block, tap) of F[oc][block, tap, 32] . X[pixel + tap][block, 32]
//
// The filter side is the second-generation kernel's: a ring of NS stage buffers of KCH k-chunks (one chunk = 32 bytes
// = one tap of one channel block), filled by LDS-direct copies, chunk-major [chunk][block of 32 rows][1 KiB].
//
// The patch.  Number the rows of the zero-padded batch R = n (IH + 2 ph) + (ih + ph): an image followed by the next,
// each with its own padding rows.  At stride 1 the output pixel (n, oh, ow) reads, for tap (fh, fw), padded row
// R(n, oh) + fh and padded column ow + fw.  A tile of BN consecutive output pixels therefore touches a contiguous range
// of padded rows, and with the patch stored as those rows, PW = IW + 2 pw pixels each, the LDS address of a fragment is
//     base(lane's pixel) + (fh PW + fw) 16        -- a per-lane constant plus a term that is uniform over the wave.
// A pixel's 32 channels are kept as two planes of 16 bytes (plane 0: channels 0-15 of every patch pixel, then plane
// 1): the 16 lanes of a quarter wave read 16 consecutive pixels of one plane, 256 contiguous bytes, no bank conflict
// (two lanes collide where a quarter wave spans the end of an image row).  Padding pixels are out-of-range lanes of
// the copies, which write zeros.  NP patches are resident: the one being multiplied, the next one arriving (its copies
// are dealt out over the stages of the current channel block, PCS per wave and stage so that the count of copies in
// flight stays a compile-time constant for the explicit vmcnt waits), and the slots being recycled.
//
// One workgroup runs one tile (the launch has one workgroup per tile: the hardware's dispatcher staggers them).
#include <atomic>
#include <type_traits>
#include <utility>

#include "igemm_shared.h"
#include "lds_copy.h"

namespace mi355 {
namespace {

template <int BM, int BN, int WM, int WN, int KCH, int NS, int NP, int PCS>
struct Igemm3 {
    static constexpr int NW = WM * WN;
    static constexpr int THREADS = NW * 64;
    static constexpr int WTM = BM / WM, WTN = BN / WN;
    static constexpr int MT = WTM / 32, NT = WTN / 32;
    static constexpr int NBA = BM / 32;
    static constexpr int STG = KCH * NBA * 1024;   // filter bytes of one stage
    static constexpr int UA = KCH * NBA / NW;      // filter copies per wave per stage
    static constexpr int RA = NBA >= NW ? NBA / NW : 1;
    static constexpr int U = UA + PCS;             // copies per wave per stage at most: filter copies and patch-copy slots
    static constexpr int PCW_MAX = 4;              // patch copies per wave and patch, at most
    static constexpr int BIAS_OFF = NS * STG, PATCH_OFF = BIAS_OFF + BM * 4;
    static_assert(NW == 4 || NW == 8, "4 or 8 waves");
    static_assert(MT >= 1 && NT >= 1 && WTM % 32 == 0 && WTN % 32 == 0, "wave tile");
    static_assert((KCH * NBA) % NW == 0 && (NBA >= NW ? NBA % NW == 0 : NW % NBA == 0), "filter copies divide over the waves");
    static_assert(KCH % 2 == 0, "fragment double buffer: the first chunk of a stage uses register set 0");
    static_assert(NS >= 3 && (NS - 1) * U + PCW_MAX < 64, "ring depth vs the 6-bit vmcnt");

    __device__ static __forceinline__ int copy_chunk(int j, int w) { return NBA >= NW ? j / RA : j * (NW / NBA) + w / NBA; }
    __device__ static __forceinline__ int copy_bi(int j) { return NBA >= NW ? j % RA : 0; }
    __device__ static __forceinline__ int row_block(int bi, int w) { return NBA >= NW ? bi * NW + w : w % NBA; }

    template <int N>
    __host__ __device__ static constexpr int step_of(int j) { return N >= KCH ? j / (N / KCH) : j * (KCH / N); }
    template <int N>
    __host__ __device__ static constexpr int nth_in_step(int j) {
        int n = 0;
        for (int q = 0; q < j; ++q) n += step_of<N>(q) == step_of<N>(j) ? 1 : 0;
        return n;
    }
    template <int N>
    __host__ __device__ static constexpr int copies_in_step(int c) {
        int n = 0;
        for (int j = 0; j < N; ++j) n += step_of<N>(j) == c ? 1 : 0;
        return n;
    }
    static_assert(UA >= KCH ? UA % KCH == 0 : KCH % UA == 0, "filter copies vs chunk steps");
    static_assert(PCS >= 1 && PCS <= KCH && KCH % PCS == 0, "patch copies vs chunk steps");
    static constexpr int CA_LAST = copies_in_step<UA>(KCH - 1);
    // Patch copies are issued before the filter copies of their chunk step, and no patch-copy slot lies behind the last step
    // that has a filter copy: every patch copy issued with a stage is older than that stage's last filter copy.
    static_assert(copies_in_step<PCS>(KCH - 1) == 0 && step_of<PCS>(PCS - 1) <= step_of<UA>(UA - 1), "patch slots vs filter copies");
    static_assert(NS <= 4, "the waits look two issued stages back");

    // s_waitcnt vmcnt(B + extra) for a wave-uniform extra in 0 .. MAXE (the count is an immediate of the instruction)
    template <int B, int MAXE>
    __device__ static __forceinline__ void wait_vmcnt_plus(int extra) {
        if constexpr (MAXE == 0) {
            wait_vmcnt<B>();
        } else {
            if (extra >= MAXE)
                wait_vmcnt<B + MAXE>();
            else
                wait_vmcnt_plus<B, MAXE - 1>(extra);
        }
    }

    // M0 = wave-uniform LDS address, offset = per-lane base + wave-uniform term (the add sits between the write of M0 and
    // the copy, which needs one wait state after it)
    __device__ static __forceinline__ void copy_at(uint32_t lds_addr, int koff, int base, const v4i& rsrc) {
        int tmp;
        asm volatile(
            "s_mov_b32 m0, %1\n\t"
            "v_add_u32 %0, %2, %3\n\t"
            "buffer_load_dwordx4 %0, %4, 0 offen lds"
            : "=&v"(tmp)
            : "s"(lds_addr), "s"(koff), "v"(base), "s"(rsrc)
            : "memory", "m0");
    }

    template <class F, int... C>
    __device__ static __forceinline__ void for_each(F&& f, std::integer_sequence<int, C...>) {
        (f(std::integral_constant<int, C>{}), ...);
    }

    __device__ static __forceinline__ void run(const IgemmArgs& a) {
        // every kernel argument the path to the first copy reads, requested in one batch of scalar loads (left alone the
        // compiler fetches them where they are first used: several dependent round trips to the argument segment)
        asm volatile("" ::"s"(a.src), "s"(a.flt), "s"(a.bias), "s"(a.src_bytes), "s"(a.flt_bytes), "s"(a.M), "s"(a.OC),
                     "s"(a.tiles), "s"(a.tiles_m), "s"(a.nstages), "s"(a.KC), "s"(a.T), "s"(a.FW), "s"(a.src_sn), "s"(a.src_scb),
                     "s"(a.flt_rstride), "s"(a.flt_kstride), "s"(a.OHW), "s"(a.OW), "s"(a.IW), "s"(a.IH), "s"(a.ph), "s"(a.pw),
                     "s"(a.has_bias), "s"(a.NB), "s"(a.p_w), "s"(a.p_himg), "s"(a.pxp), "s"(a.pcw), "s"(a.cbs));
        asm volatile("" ::"s"(a.div_ohw.m), "s"(a.div_ohw.s1), "s"(a.div_ohw.s2), "s"(a.div_ow.m), "s"(a.div_ow.s1),
                     "s"(a.div_ow.s2), "s"(a.div_tiles_m.m), "s"(a.div_tiles_m.s1), "s"(a.div_tiles_m.s2), "s"(a.div_t.m),
                     "s"(a.div_t.s1), "s"(a.div_t.s2), "s"(a.div_fw.m), "s"(a.div_fw.s1), "s"(a.div_fw.s2), "s"(a.div_pw.m),
                     "s"(a.div_pw.s1), "s"(a.div_pw.s2), "s"(a.div_phimg.m), "s"(a.div_phimg.s1), "s"(a.div_phimg.s2));
        extern __shared__ __attribute__((aligned(16))) int8_t lds[];
        const uint32_t lds0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)lds);
        const int t = threadIdx.x;
        const int lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
        const int l32 = lane & 31, lh = lane >> 5;
        const int wm = wave / WN, wn = wave % WN;

        // workgroup b runs on XCD b % 8 (round-robin dispatch); each XCD takes one contiguous slab of the tile space
        int tile;
        {
            const int b = blockIdx.x, x = b & 7, j = b >> 3;
            const int per = a.tiles >> 3, rem = a.tiles & 7;
            if (j >= per + (x < rem ? 1 : 0)) return;  // workgroup-uniform: the grid is rounded up to a multiple of 8
            tile = x * per + (x < rem ? x : rem) + j;
        }
        const int tn = (int)fdiv((uint32_t)tile, a.div_tiles_m), tm = tile - tn * a.tiles_m;
        const int oc0 = tm * BM, pix0 = tn * BN;
        const int nst = a.nstages, T = a.T, KC = a.KC, PW = a.p_w, PHI = a.p_himg;
        const int patch_bytes = a.pxp * 32;

        // bias of the channel tile: an LDS-direct copy, older than every other copy
        const v4i rs_bias = uniform_rsrc(a.bias, a.has_bias ? (uint32_t)a.OC * 4u : 0u);
        if (wave * 64 < BM) lds_copy64x4(lds0 + (uint32_t)(BIAS_OFF + wave * 256), (oc0 + t) * 4, rs_bias);
        const v4i rs_src = uniform_rsrc(a.src, a.src_bytes);
        const v4i rs_flt = uniform_rsrc(a.flt, a.flt_bytes);

        // first padded row of the tile
        const uint32_t n0 = fdiv((uint32_t)pix0, a.div_ohw), rem0 = (uint32_t)pix0 - n0 * a.OHW;
        const int R0 = (int)n0 * PHI + (int)fdiv(rem0, a.div_ow);

        // chunk -> LDS offset of (its channel block's patch slot, its tap); two stages of padding entries
        int* tab = reinterpret_cast<int*>(lds + PATCH_OFF + NP * patch_bytes);
        for (int e = t; e < (nst + 2) * KCH; e += THREADS) {
            const int kc = e < KC ? e : 0;
            const uint32_t cb = fdiv((uint32_t)kc, a.div_t), tap = kc - cb * T;
            const uint32_t fh = fdiv(tap, a.div_fw), fw = tap - fh * a.FW;
            tab[e] = PATCH_OFF + (int)(cb % NP) * patch_bytes + ((int)fh * PW + (int)fw) * 16;
        }

        // patch copies of this wave: copy id = k NW + wave covers 64 patch pixels of one 16-byte plane
        const int cpp = a.pxp >> 6;  // copies per plane
        const int npct = 2 * cpp;    // ... per patch; a.pcw = copies per wave = ceil(npct / NW) <= PCW_MAX
        // (four scalars, not an array: a selection among array elements by the run-time copy index would be folded into an
        // indexed load from scratch memory, and a scratch load in the loop waits for every copy in flight)
        auto patch_offset = [&](int k) __attribute__((always_inline)) -> int {
            const int id = k * NW + wave;
            const int plane = id >= cpp ? 1 : 0;
            const int u = (id - plane * cpp) * 64 + lane;  // patch pixel
            const uint32_t prow = fdiv((uint32_t)u, a.div_pw);
            const int pcol = u - (int)prow * PW;
            const uint32_t R = (uint32_t)R0 + prow;
            const uint32_t n = fdiv(R, a.div_phimg);
            const int ih = (int)(R - n * (uint32_t)PHI) - a.ph, iw = pcol - a.pw;
            const bool ok = id < npct && (int)n < a.NB && (unsigned)ih < (unsigned)a.IH && (unsigned)iw < (unsigned)a.IW;
            return ok ? (int)n * a.src_sn + (ih * a.IW + iw) * 32 + plane * 16 : SENT;
        };
        static_assert(PCW_MAX == 4, "four patch-copy offsets per lane");
        // (only the copies this launch has: the count is uniform over the launch)
        const int poff0 = patch_offset(0), poff1 = a.pcw > 1 ? patch_offset(1) : SENT, poff2 = a.pcw > 2 ? patch_offset(2) : SENT,
                  poff3 = a.pcw > 3 ? patch_offset(3) : SENT;

        // filter copies: byte offset of (row, half) of this lane, chunk added per copy
        const int rib = 16 * (lane >> 5) + (lane & 15), half = (lane >> 4) & 1;
        int va[UA];
        {
            int a_base[RA];
#pragma unroll
            for (int bi = 0; bi < RA; ++bi) {
                const int oc = oc0 + row_block(bi, wave) * 32 + rib;
                a_base[bi] = oc < a.OC ? oc * a.flt_rstride + half * 16 : SENT;
            }
#pragma unroll
            for (int j = 0; j < UA; ++j) va[j] = (int)((uint32_t)a_base[copy_bi(j)] + (uint32_t)(copy_chunk(j, wave) * a.flt_kstride));
        }

        // fragment side: LDS offset of this lane's pixel (plane lh) inside a patch, per pixel block
        int vB[NT];
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const int m = pix0 + (wn * NT + j) * 32 + l32;
            const uint32_t mm = m < a.M ? m : pix0;
            const uint32_t n = fdiv(mm, a.div_ohw), rem = mm - n * a.OHW;
            const uint32_t oh = fdiv(rem, a.div_ow), ow = rem - oh * a.OW;
            vB[j] = ((((int)n * PHI + (int)oh) - R0) * PW + (int)ow) * 16 + lh * (a.pxp * 16);
        }

        // ---- loader state: the stage it issues next, and the patch it is fetching
        int l_kc0 = 0, l_kA = 0;                 // first chunk of the stage, kc0 * flt_kstride
        const int dA = KCH * a.flt_kstride;
        int p_cb = 1, p_slot = 0;                // channel block being fetched, copies of it issued by this wave
        uint32_t p_dst = lds0 + (uint32_t)(PATCH_OFF + (1 % NP) * patch_bytes);
        int p_src = a.src_scb;
        const int pcw = a.pcw, cbs = a.cbs;
        const uint32_t wave_k = (uint32_t)(wave * 1024);

        int pc_cur = 0, pc_prev = 0;  // patch copies this wave issued with the stage being issued / with the one before
        auto patch_copy = [&]() __attribute__((always_inline)) {
            // The next copy of the patch being fetched, if this wave has one left (wave-uniform).  The explicit waits count
            // the copies that may stay in flight exactly: the filter copies of the stages behind the awaited one, a
            // compile-time number, plus the patch copies issued with those stages, counted here.  (A wait that ignored the
            // patch copies would wait for copies issued a moment ago; a copy with every lane out of range in each empty
            // slot, to make the number constant, costs more than the real copies.)
            if (p_slot < pcw && p_cb < cbs && p_slot * NW + wave < npct) {
#ifdef V3_ABLATE_CONTIG
                const int off = lane * 16 + p_slot * 1024;
#else
                const int off = p_slot == 0 ? poff0 : p_slot == 1 ? poff1 : p_slot == 2 ? poff2 : poff3;
#endif
                copy_at(p_dst + (uint32_t)(p_slot * NW * 1024) + wave_k, p_src, off, rs_src);
                ++pc_cur;
            }
            ++p_slot;
        };
        auto patch_switch = [&]() __attribute__((always_inline)) {
            // the stage about to be issued touches the channel block whose patch was being fetched: that patch is complete
            // (it had at least floor(T / KCH) stages of PCS copies per wave), the next one starts
            if (l_kc0 + KCH > p_cb * T) {
                ++p_cb;
                p_slot = 0;
                p_src += a.src_scb;
                p_dst += (uint32_t)patch_bytes;
                if (p_dst == lds0 + (uint32_t)(PATCH_OFF + NP * patch_bytes)) p_dst = lds0 + (uint32_t)PATCH_OFF;
            }
        };
        auto filter_copy = [&](auto jj, uint32_t stage_addr) __attribute__((always_inline)) {
            constexpr int j = decltype(jj)::value;
            // chunks past the end of the reduction read zeros (in the reference layout the bytes there are the next row's)
            const int koff = l_kc0 + copy_chunk(j, wave) < KC ? l_kA : SENT;
            copy_at(stage_addr + (uint32_t)(j * NW * 1024) + wave_k, koff, va[j], rs_flt);
        };
        auto loader_advance = [&]() __attribute__((always_inline)) {
            l_kc0 += KCH;
            l_kA += dA;
            pc_prev = pc_cur;
            pc_cur = 0;
        };

        __syncthreads();  // table ready

        // prologue: the first patch whole, then stages 0 .. NS - 2
        {
            const int pk[PCW_MAX] = {poff0, poff1, poff2, poff3};
#pragma unroll
            for (int k = 0; k < PCW_MAX; ++k) {
                const int id = k * NW + wave;
                if (k < pcw && id < npct) copy_at(lds0 + (uint32_t)(PATCH_OFF + id * 1024), 0, pk[k], rs_src);
            }
        }
#pragma unroll
        for (int s = 0; s < NS - 1; ++s) {
            patch_switch();
#pragma unroll
            for (int i = 0; i < PCS; ++i) patch_copy();
            for_each([&](auto jj) __attribute__((always_inline)) { filter_copy(jj, lds0 + (uint32_t)(s * STG)); },
                     std::make_integer_sequence<int, UA>{});
            loader_advance();
        }
        wait_vmcnt<(NS - 2) * UA>();  // stage 0, the first patch, the bias (and, stricter than needed, the patch copies behind them)
        __syncthreads();

        const int fragpos = ((l32 >> 4) * 2 + lh) * 256 + (l32 & 15) * 16;
        const int8_t* fragA = lds + fragpos + wm * MT * 1024;
        int rd_off = 0, wr_off = (NS - 1) * STG;
        int bc[KCH], bn[KCH];  // patch offsets of the chunks of the stage being multiplied / of the next one
#pragma unroll
        for (int c = 0; c < KCH; ++c) {
            bc[c] = tab[c];
            bn[c] = tab[KCH + c];
        }
        int c_stage = 0;

        v4i fa[2][MT], fb[2][NT];
        v16i acc[MT][NT];
        {
            const int* sBias = reinterpret_cast<const int*>(lds + BIAS_OFF);
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
#pragma unroll
        for (int i = 0; i < MT; ++i) fa[0][i] = *reinterpret_cast<const v4i*>(fragA + i * 1024);
#pragma unroll
        for (int j = 0; j < NT; ++j) fb[0][j] = *reinterpret_cast<const v4i*>(lds + vB[j] + bc[0]);

        // One chunk step: the MFMAs of chunk c run while the fragments of chunk c + 1 are read (from the next stage's buffer
        // on the last step, behind the stage boundary: wait, barrier) and while this step's share of the copies of the
        // stage NS - 1 ahead is issued; the pieces are dealt out between the MFMAs.
        auto chunk_step = [&](auto cc) __attribute__((always_inline)) {
            constexpr int c = decltype(cc)::value;
            constexpr bool LAST = c + 1 == KCH;
            if (LAST) {
                wait_lgkmcnt0();
                wait_vmcnt_plus<(NS - 2) * UA - CA_LAST, (NS - 2) * PCS>(pc_cur + (NS >= 4 ? pc_prev : 0));
                __syncthreads();
            }
            constexpr int CA = copies_in_step<UA>(c), CP = copies_in_step<PCS>(c);
            constexpr int PC = MT + NT;
            constexpr int P = PC + (c == 0 ? 1 : 0) + CA + CP + (LAST ? 1 : 0);
            constexpr int M = MT * NT;
            constexpr int PER = (P + M - 1) / M;
            constexpr int cn = LAST ? 0 : c + 1;
            const int rd_nxt = rd_off + STG == NS * STG ? 0 : rd_off + STG;
            const int rd_frag = LAST ? rd_nxt : rd_off;
            const int bo = LAST ? bn[0] : bc[cn];
            auto piece = [&](auto kk) __attribute__((always_inline)) {
                constexpr int k = decltype(kk)::value;
                constexpr int K0 = PC + (c == 0 ? 1 : 0);
                if constexpr (k < MT) {
                    fa[cn & 1][k] = *reinterpret_cast<const v4i*>(fragA + rd_frag + (cn * NBA + k) * 1024);
                } else if constexpr (k < PC) {
                    fb[cn & 1][k - MT] = *reinterpret_cast<const v4i*>(lds + vB[k - MT] + bo);
                } else if constexpr (c == 0 && k == PC) {
                    patch_switch();  // before the first copy of the stage
                } else if constexpr (k < K0 + CP) {
                    patch_copy();
                } else if constexpr (k < K0 + CP + CA) {
                    for_each([&](auto jj) __attribute__((always_inline)) {
                        constexpr int j = decltype(jj)::value;
                        if constexpr (step_of<UA>(j) == c && nth_in_step<UA>(j) == k - K0 - CP) filter_copy(jj, lds0 + (uint32_t)wr_off);
                    }, std::make_integer_sequence<int, UA>{});
                } else if constexpr (LAST && k == K0 + CA + CP) {
                    loader_advance();
                    wr_off = rd_off;
                    rd_off = rd_nxt;
                    ++c_stage;
#pragma unroll
                    for (int q = 0; q < KCH; ++q) {
                        bc[q] = bn[q];
                        bn[q] = tab[(c_stage + 1) * KCH + q];
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            };
            auto slot = [&](auto mm) __attribute__((always_inline)) {
                constexpr int m = decltype(mm)::value;
                constexpr int i = m / NT, j = m % NT;
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[c & 1][i], fb[c & 1][j], acc[i][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                for_each([&](auto qq) __attribute__((always_inline)) { piece(std::integral_constant<int, m * PER + decltype(qq)::value>{}); },
                         std::make_integer_sequence<int, PER>{});
            };
            __builtin_amdgcn_sched_barrier(0);
            for_each(slot, std::make_integer_sequence<int, M>{});
        };

        for (int s = 0; s < nst; ++s)
            for_each([&](auto cc) __attribute__((always_inline)) { chunk_step(cc); }, std::make_integer_sequence<int, KCH>{});

        igemm_run_epilogue<32, MT, NT, false>(a, acc, oc0 + wm * WTM, pix0 + wn * WTN, l32, lh, nullptr, a.OC);
        // the trailing (out-of-range, zero-filling) copies must land before this workgroup's LDS is released
        wait_vmcnt<0>();
    }
};

template <int BM, int BN, int WM, int WN, int KCH, int NS, int NP, int PCS, int MINW>
__global__ __launch_bounds__(WM * WN * 64, MINW) void igemm3_kernel(IgemmArgs a) {
    Igemm3<BM, BN, WM, WN, KCH, NS, NP, PCS>::run(a);
}

constexpr int kLdsPerCu = 160 * 1024;

struct Cfg3 {
    const char* name;
    int bm, bn, kch;
};
const Cfg3 kCfg3[] = {
        {"v3_128x128x64r4", 128, 128, 2},
        {"v3_64x128x64r4", 64, 128, 2},
        {"v3_128x256x64r4w8", 128, 256, 2},
        {"v3_256x256x64r3w8", 256, 256, 2},
        {"v3_128x128x128r3", 128, 128, 4},
        {"v3_64x128x256r3", 64, 128, 8},
        {"v3_128x128x256r3", 128, 128, 8},
        {"v3_64x64x256r3", 64, 64, 8},
};
constexpr int kNumCfg3 = sizeof(kCfg3) / sizeof(kCfg3[0]);

// -1: this tile cannot run the problem (patch or ring beyond the LDS of a CU, too many patch copies per wave)
template <int BM, int BN, int WM, int WN, int KCH, int NS, int NP, int PCS, int MINW>
int launch_k(hipStream_t st, IgemmArgs& a) {
    using K = Igemm3<BM, BN, WM, WN, KCH, NS, NP, PCS>;
    a.tiles_m = (a.OC + BM - 1) / BM;
    a.div_tiles_m = make_fastdiv((uint32_t)a.tiles_m);
    a.tiles_n = (a.M + BN - 1) / BN;
    const int64_t tiles = (int64_t)a.tiles_m * a.tiles_n;
    if (tiles <= 0 || tiles > 0x0fffffff) return -1;
    a.tiles = (int)tiles;
    a.nstages = (a.KC + KCH - 1) / KCH;
    // padded geometry: rows of PW pixels, PHI rows per image; the rows that BN consecutive output pixels can span
    a.p_w = a.IW + 2 * a.pw;
    a.p_himg = a.IH + 2 * a.ph;
    // (the tile starts repeat with period OHW / gcd(BN, OHW): walk one period, or take the bound for long ones)
    int64_t span = 0;
    {
        int g = BN, r = a.OHW;
        while (r) { const int q = g % r; g = r; r = q; }
        const int period = a.OHW / g;
        if (period <= 4096) {
            for (int i = 0; i < period && i < a.tiles_n; ++i) {
                const int64_t p0 = (int64_t)i * BN, p1 = p0 + BN - 1 < a.M - 1 ? p0 + BN - 1 : a.M - 1;
                const int64_t r0 = p0 / a.OHW * a.p_himg + p0 % a.OHW / a.OW, r1 = p1 / a.OHW * a.p_himg + p1 % a.OHW / a.OW;
                if (r1 - r0 + a.FH > span) span = r1 - r0 + a.FH;
            }
        } else {
            span = (BN - 1) / a.OW + 2 + (int64_t)((BN - 1) / a.OHW + 1) * (a.FH - 1) + (a.FH - 1);
        }
    }
    const int64_t px = span * a.p_w;
    if (px > 65536) return -1;
    a.pxp = (int)((px + 63) / 64 * 64);
    a.pcw = (2 * (a.pxp / 64) + K::NW - 1) / K::NW;
    a.cbs = a.KC / a.T;
    if (a.pcw > K::PCW_MAX) return -1;
    // a patch is fetched during the stages of the channel block before it, at least floor(T / KCH) of them
    if (PCS * (a.T / KCH) < a.pcw) return -1;
    // ... into the slot whose patch was last read NP - 1 channel blocks earlier, by a stage the ring has left behind
    if (NS * KCH >= (NP - 2) * a.T + 2) return -1;
    a.div_pw = make_fastdiv((uint32_t)a.p_w);
    a.div_phimg = make_fastdiv((uint32_t)a.p_himg);
    const int lds = K::PATCH_OFF + NP * a.pxp * 32 + (a.nstages + 2) * KCH * 4;
    if (lds > kLdsPerCu) return -1;
    if (a.dry_run) return 0;
    auto kern = igemm3_kernel<BM, BN, WM, WN, KCH, NS, NP, PCS, MINW>;
    static std::atomic<int> max_lds_set{0};
    if (lds > max_lds_set.load(std::memory_order_relaxed)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsPerCu);
        if (e != hipSuccess) return (int)e;
        max_lds_set.store(kLdsPerCu, std::memory_order_relaxed);
    }
    const int64_t grid = (tiles + 7) / 8 * 8;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(K::THREADS), lds, st, a);
    return (int)hipGetLastError();
}

int launch_cfg(hipStream_t st, IgemmArgs& a, int cfg) {
    // 3x3 filters: a channel block is 9 chunks, the ring of four stages of two chunks stays inside it (NP = 3); 5x5: 25
    // chunks per channel block
    switch (cfg) {
        case 0: return launch_k<128, 128, 2, 2, 2, 4, 3, 1, 2>(st, a);
        case 1: return launch_k<64, 128, 2, 2, 2, 4, 3, 1, 2>(st, a);
        case 2: return launch_k<128, 256, 2, 4, 2, 4, 3, 1, 4>(st, a);
        case 3: return launch_k<256, 256, 4, 2, 2, 3, 3, 1, 2>(st, a);
        case 4: return launch_k<128, 128, 2, 2, 4, 3, 4, 2, 2>(st, a);
        case 5: return launch_k<64, 128, 2, 2, 8, 3, 5, 2, 2>(st, a);
        case 6: return launch_k<128, 128, 2, 2, 8, 3, 5, 2, 2>(st, a);
        case 7: return launch_k<64, 64, 2, 2, 8, 3, 5, 2, 2>(st, a);
        default: return -1;
    }
}

bool shape_ok(const IgemmArgs& a, int pin, int pout) {
    // 32-packed on both sides, dense, stride 1, a real filter window, the fast epilogue
    return pin == 32 && pout == 32 && a.groups == 1 && !a.general && a.sh == 1 && a.sw == 1 && a.T > 1 && a.T <= 49 &&
           a.OH == a.IH + 2 * a.ph - a.FH + 1 && a.OW == a.IW + 2 * a.pw - a.FW + 1;
}

}  // namespace

int igemm3_num_cfgs() { return kNumCfg3; }
const char* igemm3_cfg_name(int cfg) { return cfg >= 0 && cfg < kNumCfg3 ? kCfg3[cfg].name : "?"; }

bool igemm3_can_run(const IgemmArgs& a, int pin, int pout, int cfg) {
    if (!shape_ok(a, pin, pout)) return false;
    IgemmArgs t = a;
    t.dry_run = 1;
    return launch_cfg(nullptr, t, cfg) == 0;
}

int launch_igemm3(hipStream_t st, IgemmArgs& a, int pin, int pout, int cfg) {
    if (!shape_ok(a, pin, pout)) return (int)hipErrorInvalidConfiguration;
    const int rc = launch_cfg(st, a, cfg);
    return rc < 0 ? (int)hipErrorInvalidConfiguration : rc;
}

}  // namespace mi355
