// Implicit-GEMM int8 ConvBias for 32-packed inputs (NCHW32, NCHW32_NCHW4; dense and group), second generation:
// a software-pipelined k-loop whose matrix instructions never wait for an LDS read of their own chunk.
//
//   D[oc][pixel] = sum_k F[oc][k] * X[pixel][k]      v_mfma_i32_32x32x32_i8, A = 32 filter rows, B = 32 pixels
//
// What differs from conv_igemm_dma.hip (same epilogue, same persistent XCD-contiguous schedule):
//
//   * LDS layout of a stage: [k-chunk of 32 bytes][block of 32 rows][1 KiB].  One LDS-direct wave copy
//     (buffer_load_dwordx4 ... lds, 64 lanes x 16 bytes, lane l lands at M0 + 16 l) fills exactly one block: the
//     32-byte k-chunk of 32 consecutive rows.  For activations those 32 x 32 bytes are ONE contiguous kilobyte of
//     global memory (consecutive pixels of one channel block), so every copy moves whole cache lines; with the
//     row-major stage of the first-generation kernel a copy touched 32-byte granules of four channel blocks.
//     Inside a block the lane that lands at 16-byte position p fetches row 16 (p / 32) + p % 16, half (p / 16) % 2:
//     an MFMA fragment read (lane = row l % 32, half l / 32) then finds the 16 lanes of every quarter wave on 16
//     distinct positions mod 16, which is what ds_read_b128 needs to run without bank conflicts on gfx950; no XOR
//     swizzle, and the k-chunk of a copy is wave-uniform, so filter taps and bounds are computed once per copy.
//   * the k-loop is software pipelined over chunks: the fragments of chunk c + 1 are read while the MFMAs of chunk c
//     run, across stage boundaries too.  The one barrier per stage sits before the LAST chunk's MFMAs of a stage: by then
//     every fragment of the stage is in registers, so the stage buffer is refilled at once (a ring of NS buffers
//     keeps NS - 1 stages in flight plus the one being read) and the first fragments of the next stage are requested
//     before those MFMAs issue.
//   * the filter is addressed as  row * flt_rstride + chunk * flt_kstride: the reference layout as it is, or the
//     pre-processed layout [k-chunk][channel][32] whose copies are contiguous kilobytes as well.
//   * group convolution: a channel tile lies inside one group; the group moves the activation base.
//   * the residual travels through LDS as well: each wave copies the residual of its NEXT tile's outputs into one of two
//     LDS slots while the current tile is multiplied (LDS-direct copies again: no register is the target of a load
//     the compiler does not know about), and the epilogue reads it back lane for lane.
#include <atomic>
#include <type_traits>
#include <utility>

#include "igemm_shared.h"
#include "lds_copy.h"

namespace mi355 {
namespace {

// KS > 1: the waves of a workgroup also split the reduction.  KS groups of WM x WN waves each multiply the whole output
// tile over their own chunks of every stage (CPS = KCH / KS chunk steps per stage instead of KCH: a serial chain KS
// times shorter, and with wave tiles of 64 x 64 four MFMAs per four fragment reads), the int32 partial sums meet in LDS
// -- in the ring, which is idle by then -- and every wave requantises and stores its share of the blocks.  Integer
// addition is exact in any order, nothing leaves the workgroup, the workspace stays 0.  Such a workgroup runs ONE tile
// (the launch gives every tile its own): these are the tiles for long reductions over few tiles.
template <int POUT, int BM, int BN, int WM, int WN, int KCH, int NS, bool PW, int KS = 1>
struct Igemm2 {
    static constexpr int WMN = WM * WN;      // waves of one reduction group
    static constexpr int NW = WMN * KS;      // waves per workgroup
    static constexpr int CPS = KCH / KS;     // chunk steps per stage of one wave
    static constexpr int THREADS = NW * 64;
    static constexpr int WTM = BM / WM, WTN = BN / WN;
    static constexpr int MT = WTM / 32, NT = WTN / 32;
    static constexpr int NBA = BM / 32, NBB = BN / 32;  // 1 KiB blocks per k-chunk
    static constexpr int A_BYTES = KCH * NBA * 1024, B_BYTES = KCH * NBB * 1024;
    static constexpr int STG = A_BYTES + B_BYTES;
    static constexpr int UA = KCH * NBA / NW, UB = KCH * NBB / NW;  // copies per wave per stage
    static constexpr int U = UA + UB;
    static constexpr int RA = NBA >= NW ? NBA / NW : 1;  // row blocks a wave copies
    static constexpr int RB = NBB >= NW ? NBB / NW : 1;
    static constexpr int BIAS_BYTES = BM * 4;
    static constexpr int RING_BYTES = NS * STG + BIAS_BYTES;
    // The 8-wave tiles of 256 x 128 outputs and more read the residual in the epilogue, straight from global memory:
    // an LDS slot for it (BM * BN bytes) would cost them a workgroup per CU, and a tile of theirs runs long enough to
    // hide the fetch of one block behind the requantisation of the previous one.
    static constexpr bool ZD = BM * BN >= 256 * 128 || KS > 1;  // (the split tiles keep their LDS for the ring)
    // partial sums of the blocks a wave does not finish itself: (KS - 1) / KS of its MT x NT blocks of 4 KiB
    static constexpr int OB = MT * NT / KS;  // blocks a wave finishes
    static constexpr int RED_BYTES = KS > 1 ? NW * OB * (KS - 1) * 4096 : 0;
    static_assert(KCH % KS == 0 && CPS % 2 == 0, "chunk steps per wave and stage: even (fragment double buffer)");
    static_assert(KS == 1 || ((MT * NT) % KS == 0 && RED_BYTES <= NS * STG), "partial sums fit the idle ring");
    static_assert(NW == 4 || NW == 8, "4 or 8 waves");
    static_assert(MT >= 1 && NT >= 1 && WTM % 32 == 0 && WTN % 32 == 0, "wave tile");
    static_assert((KCH * NBA) % NW == 0 && (KCH * NBB) % NW == 0, "copies divide over the waves");
    static_assert(NBA >= NW ? NBA % NW == 0 : NW % NBA == 0, "filter blocks vs waves");
    static_assert(NBB >= NW ? NBB % NW == 0 : NW % NBB == 0, "pixel blocks vs waves");

    static_assert(NS >= 3 && (NS - 1) * U < 64, "ring depth (one buffer read, one refilled, the rest in flight) vs the 6-bit vmcnt");

    // copy j of wave w is block j * NW + w of the stage in [chunk][row block] order
    template <int NB, int R>
    __device__ static __forceinline__ int copy_chunk(int j, int w) {
        return NB >= NW ? j / R : j * (NW / NB) + w / NB;
    }
    template <int NB, int R>
    __device__ static __forceinline__ int copy_bi(int j) {
        return NB >= NW ? j % R : 0;
    }
    template <int NB>
    __device__ static __forceinline__ int row_block(int bi, int w) {
        return NB >= NW ? bi * NW + w : w % NB;
    }

    struct Loader {
        int ti, stage, kc0;        // position: tile index in this workgroup's sequence, stage, first chunk of the stage
        int kA, kB;                // kc0 * flt_kstride, kc0 * src_scb
        int va[UA];                // filter copy j: byte offset of (row, half, chunk of the copy), SENT past the last channel
        int vb[PW ? UB : 1];       // pointwise activation copy j: the same for (pixel, half, chunk); SENT past M
        int b_base[RB];            // table path: byte offset of the pixel (+ half)
        int ih0[RB], iw0[RB];      // table path: top-left input coordinate (ih0 = -0x8000 past M)
    };

    struct Tile {
        int oc0, oc_end, pix0, src_goff;
    };

    __device__ static __forceinline__ Tile tile_coords(const IgemmArgs& a, int tile) {
        Tile c;
        const int tn = (int)fdiv((uint32_t)tile, a.div_tiles_m), tmg = tile - tn * a.tiles_m;
        const int g = (int)fdiv((uint32_t)tmg, a.div_tiles_m_pg), tm = tmg - g * a.tiles_m_pg;
        c.oc0 = g * a.ocpg + tm * BM;
        c.oc_end = (g + 1) * a.ocpg;
        c.pix0 = tn * BN;
        c.src_goff = g * a.src_sg;
        return c;
    }

    __device__ static __forceinline__ void loader_enter_tile(const IgemmArgs& a, Loader& L, const Tile& c, int w, int lane) {
        const int rib = 16 * (lane >> 5) + (lane & 15);  // row inside a block
        const int half = (lane >> 4) & 1;
        int a_base[RA];
#pragma unroll
        for (int bi = 0; bi < RA; ++bi) {
            const int oc = c.oc0 + row_block<NBA>(bi, w) * 32 + rib;
            a_base[bi] = oc < c.oc_end ? oc * a.flt_rstride + half * 16 : SENT;
        }
        // SENT plus a chunk offset stays out of range
#pragma unroll
        for (int j = 0; j < UA; ++j)
            L.va[j] = (int)((uint32_t)a_base[copy_bi<NBA, RA>(j)] + (uint32_t)(copy_chunk<NBA, RA>(j, w) * a.flt_kstride));
        int p_base[RB];
#pragma unroll
        for (int bi = 0; bi < RB; ++bi) {
            const int m = c.pix0 + row_block<NBB>(bi, w) * 32 + rib;
            const bool ok = m < a.M;
            const uint32_t mm = ok ? m : 0;
            const uint32_t n = fdiv(mm, a.div_ohw), rem = mm - n * a.OHW;
            const uint32_t oh = fdiv(rem, a.div_ow), ow = rem - oh * a.OW;
            const int ih0 = (int)oh * a.sh - a.ph, iw0 = (int)ow * a.sw - a.pw;
            const int base = (int)n * a.src_sn + c.src_goff + (ih0 * a.IW + iw0) * 32 + half * 16;
            if (PW) {
                p_base[bi] = ok ? base : SENT;
            } else {
                L.b_base[bi] = base;
                L.ih0[bi] = ok ? ih0 : -0x8000;  // makes every tap fail the bounds test
                L.iw0[bi] = iw0;
            }
        }
        if (PW) {
#pragma unroll
            for (int j = 0; j < UB; ++j)
                L.vb[j] = (int)((uint32_t)p_base[copy_bi<NBB, RB>(j)] + (uint32_t)(copy_chunk<NBB, RB>(j, w) * a.src_scb));
        }
    }

    __device__ static __forceinline__ void loader_kill(Loader& L) {
#pragma unroll
        for (int j = 0; j < UA; ++j) L.va[j] = SENT;
        if (PW) {
#pragma unroll
            for (int j = 0; j < UB; ++j) L.vb[j] = SENT;
        }
#pragma unroll
        for (int bi = 0; bi < RB; ++bi) {
            L.b_base[bi] = SENT;
            L.ih0[bi] = -0x8000;
        }
        L.kc0 = 0;
        L.kA = 0;
        L.kB = 0;
    }

    // table entries of the stage the loader fetches next: one per activation copy of this wave (wave-uniform index)
    __device__ static __forceinline__ void load_entries(const Loader& L, const KEntry* tab, KEntry (&nk)[UB], int w) {
        if (PW) return;
#pragma unroll
        for (int j = 0; j < UB; ++j) nk[j] = tab[L.kc0 + copy_chunk<NBB, RB>(j, w)];
    }

    // One copy whose global offset is a per-lane base plus a wave-uniform term: M0 = wave_addr + IMM, offset = base + koff.
    // The vector add sits between the write of M0 and the copy, which needs one wait state after it.
    template <int IMM>
    __device__ static __forceinline__ void copy_at(uint32_t wave_addr, int koff, int base, const v4i& rsrc) {
        int tmp;
        asm volatile(
            "s_add_u32 m0, %1, %2\n\t"
            "v_add_u32 %0, %3, %4\n\t"
            "buffer_load_dwordx4 %0, %5, 0 offen lds"
            : "=&v"(tmp)
            : "s"(wave_addr), "n"(IMM), "s"(koff), "v"(base), "s"(rsrc)
            : "memory", "m0", "scc");
    }
    // ... whose offset is already complete
    template <int IMM>
    __device__ static __forceinline__ void copy_to(uint32_t wave_addr, int voff, const v4i& rsrc) {
        asm volatile(
            "s_add_u32 m0, %0, %1\n\t"
            "s_nop 0\n\t"
            "buffer_load_dwordx4 %2, %3, 0 offen lds"
            :
            : "s"(wave_addr), "n"(IMM), "v"(voff), "s"(rsrc)
            : "memory", "m0", "scc");
    }

    // The copies of a stage are spread over the KCH chunk steps of the stage during which they are issued (a burst of
    // U copies fills the address path's queue and blocks the wave's in-order issue -- its MFMAs too -- until it drains).
    // Copy j of wave w is block j * NW + w of the stage, at LDS address wave_addr + j * NW KiB.
    template <int N>
    __device__ static constexpr int step_of(int j) {  // chunk step in which copy j of N is issued
        return N >= CPS ? j / (N / CPS) : j * (CPS / N);
    }
    template <int N>
    __device__ static constexpr int nth_in_step(int j) {  // position of copy j among the copies of its step
        int n = 0;
        for (int q = 0; q < j; ++q) n += step_of<N>(q) == step_of<N>(j) ? 1 : 0;
        return n;
    }
    template <int N>
    __device__ static constexpr int copies_in_step(int c) {
        int n = 0;
        for (int j = 0; j < N; ++j) n += step_of<N>(j) == c ? 1 : 0;
        return n;
    }
    static_assert(UA >= CPS ? UA % CPS == 0 : CPS % UA == 0, "filter copies vs chunk steps");
    static_assert(UB >= CPS ? UB % CPS == 0 : CPS % UB == 0, "activation copies vs chunk steps");
    static constexpr int CS_LAST = copies_in_step<UA>(CPS - 1) + copies_in_step<UB>(CPS - 1);

    // KT: the reduction is not a whole number of stages, chunks past its end read zeros (the activations' zeros meet
    // whatever the filter copy returns there).
    template <bool KT, int C>
    __device__ static __forceinline__ void issue_step(const IgemmArgs& a, const Loader& L, const KEntry (&nk)[UB], const v4i& rs_src,
                                                      const v4i& rs_flt, uint32_t wave_addr, int w) {
        issue_a<C>(L, rs_flt, wave_addr, std::make_integer_sequence<int, UA>{});
        issue_b<KT, C>(a, L, nk, rs_src, wave_addr, w, std::make_integer_sequence<int, UB>{});
    }
    template <bool KT>
    __device__ static __forceinline__ void issue_all(const IgemmArgs& a, const Loader& L, const KEntry (&nk)[UB], const v4i& rs_src,
                                                     const v4i& rs_flt, uint32_t wave_addr, int w) {
        issue_all_steps<KT>(a, L, nk, rs_src, rs_flt, wave_addr, w, std::make_integer_sequence<int, CPS>{});
    }
    template <bool KT, int... C>
    __device__ static __forceinline__ void issue_all_steps(const IgemmArgs& a, const Loader& L, const KEntry (&nk)[UB],
                                                           const v4i& rs_src, const v4i& rs_flt, uint32_t wave_addr, int w,
                                                           std::integer_sequence<int, C...>) {
        (issue_step<KT, C>(a, L, nk, rs_src, rs_flt, wave_addr, w), ...);
    }
    template <int C, int... J>
    __device__ static __forceinline__ void issue_a(const Loader& L, const v4i& rs_flt, uint32_t wave_addr,
                                                   std::integer_sequence<int, J...>) {
        ((step_of<UA>(J) == C ? copy_at<J * NW * 1024>(wave_addr, L.kA, L.va[J], rs_flt) : (void)0), ...);
    }
    template <bool KT, int C, int... J>
    __device__ static __forceinline__ void issue_b(const IgemmArgs& a, const Loader& L, const KEntry (&nk)[UB], const v4i& rs_src,
                                                   uint32_t wave_addr, int w, std::integer_sequence<int, J...>) {
        ((step_of<UB>(J) == C ? issue_b1<KT, J>(a, L, nk, rs_src, wave_addr, w) : (void)0), ...);
    }
    // the K-th copy of chunk step C
    template <int C, int K, int... J>
    __device__ static __forceinline__ void issue_a1(const Loader& L, const v4i& rs_flt, uint32_t wave_addr,
                                                    std::integer_sequence<int, J...>) {
        ((step_of<UA>(J) == C && nth_in_step<UA>(J) == K ? copy_at<J * NW * 1024>(wave_addr, L.kA, L.va[J], rs_flt) : (void)0), ...);
    }
    template <bool KT, int C, int K, int... J>
    __device__ static __forceinline__ void issue_bk(const IgemmArgs& a, const Loader& L, const KEntry (&nk)[UB], const v4i& rs_src,
                                                    uint32_t wave_addr, int w, std::integer_sequence<int, J...>) {
        ((step_of<UB>(J) == C && nth_in_step<UB>(J) == K ? issue_b1<KT, J>(a, L, nk, rs_src, wave_addr, w) : (void)0), ...);
    }
    template <bool KT, int J>
    __device__ static __forceinline__ void issue_b1(const IgemmArgs& a, const Loader& L, const KEntry (&nk)[UB], const v4i& rs_src,
                                                    uint32_t wave_addr, int w) {
        constexpr int IMM = A_BYTES + J * NW * 1024;
        if (PW) {
            // SENT plus a pixel offset stays out of range; SENT plus SENT (a row past M as well) wraps to offset 0,
            // whose bytes only meet discarded rows
            int koff = L.kB;
            if (KT) koff = L.kc0 + copy_chunk<NBB, RB>(J, w) < a.KC ? koff : SENT;
            copy_at<IMM>(wave_addr, koff, L.vb[J], rs_src);
        } else {
            const int bi = copy_bi<NBB, RB>(J);
            const KEntry k = nk[J];
            const int fh = k.fhfw & 0xffff, fw = k.fhfw >> 16;
            const int ih = L.ih0[bi] + fh, iw = L.iw0[bi] + fw;
            const bool ok = (unsigned)ih < (unsigned)a.IH && (unsigned)iw < (unsigned)a.IW;
            copy_to<IMM>(wave_addr, ok ? L.b_base[bi] + k.off : SENT, rs_src);
        }
    }

    // kg: the wave's reduction group; the bias enters the sum once, through group 0
    __device__ static __forceinline__ void init_acc_lds(v16i (&acc)[MT][NT], const int* sBias, int wm, int lh, int kg = 0) {
        if (KS > 1 && kg != 0) {  // wave-uniform
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int j = 0; j < NT; ++j) acc[i][j] = v16i{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            return;
        }
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

    static constexpr int ZWAVE = MT * NT * 1024;  // residual bytes of one wave tile
    static constexpr int ZSLOT = NW * ZWAVE;      // ... of a workgroup tile (= BM * BN)

    // Copies the residual of the wave tile at (oc_w, pix_w) into LDS at zaddr, in the order the epilogue consumes it:
    // POUT = 32: block (i, j) is 1 KiB, lane l holds the 16 consecutive channels of its pixel; POUT = 4: four copies of
    // 256 bytes per block, lane l holds one dword (4 channels) in each.
    __device__ static __forceinline__ void issue_z(const IgemmArgs& a, const v4i& rs_z, uint32_t zaddr, int oc_w, int pix_w,
                                                   int l32, int lh) {
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const int m = pix_w + j * 32 + l32;
            const bool pok = m < a.M;
            const uint32_t mm = pok ? m : 0;
            const uint32_t n = fdiv(mm, a.div_ohw), rem = mm - n * a.OHW;
            const int z_pix = (int)n * a.z_sn + (int)rem * POUT;
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                const int ocb = oc_w + i * 32;
                const uint32_t dst = zaddr + (uint32_t)((i * NT + j) * 1024);
                if (POUT == 32) {
                    const int blk_off = (ocb >> 5) * a.dst_scb + lh * 16;
                    lds_copy64x16(dst, (pok && ocb < a.OC) ? z_pix + blk_off : SENT, rs_z);
                } else {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int oc4 = ocb + 8 * q + 4 * lh;
                        const int off = (oc4 >> 2) * a.dst_scb;
                        lds_copy64x4(dst + (uint32_t)(q * 256), (pok && oc4 < a.OC) ? z_pix + off : SENT, rs_z);
                    }
                }
            }
        }
    }
    // number of copy instructions of issue_z
    static constexpr int NZ = MT * NT * (POUT == 32 ? 1 : 4);

    __device__ static __forceinline__ void read_z(ZRegs<MT, NT>& zr, const int8_t* zslot, int lane) {
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                const int8_t* blk = zslot + (i * NT + j) * 1024;
                if (POUT == 32) {
                    zr.v[i][j] = *reinterpret_cast<const v4i*>(blk + lane * 16);
                } else {
#pragma unroll
                    for (int q = 0; q < 4; ++q) zr.v[i][j][q] = *reinterpret_cast<const int*>(blk + q * 256 + lane * 4);
                }
            }
    }

    template <class F, int... C>
    __device__ static __forceinline__ void for_each_chunk(F&& f, std::integer_sequence<int, C...>) {
        (f(std::integral_constant<int, C>{}), ...);
    }

    // KT: the reduction is not a whole number of stages.  GEN: the general epilogue (its own instantiations: the fast
    // epilogue's kernels carry none of its registers)
    template <bool KT, bool GEN>
    __device__ static __forceinline__ void run(const IgemmArgs& a) {
        // Every kernel argument that the path to the first copy reads is requested here, in one batch of scalar loads:
        // left to itself the compiler fetches them where they are first used, behind branches, which made four
        // dependent round trips to the argument segment (~500 clocks each) out of the first 2000 clocks of a workgroup.
        asm volatile("" ::"s"(a.src), "s"(a.flt), "s"(a.bias), "s"(a.src_bytes), "s"(a.flt_bytes), "s"(a.M), "s"(a.OC),
                     "s"(a.tiles), "s"(a.tiles_m), "s"(a.tiles_m_pg), "s"(a.nstages), "s"(a.KC), "s"(a.src_sn), "s"(a.src_scb),
                     "s"(a.flt_rstride), "s"(a.flt_kstride), "s"(a.OHW), "s"(a.OW), "s"(a.IW), "s"(a.IH), "s"(a.sh), "s"(a.sw),
                     "s"(a.ph), "s"(a.pw), "s"(a.ocpg), "s"(a.src_sg), "s"(a.has_bias), "s"(a.zslots), "s"(a.entries));
        asm volatile("" ::"s"(a.div_ohw.m), "s"(a.div_ohw.s1), "s"(a.div_ohw.s2), "s"(a.div_ow.m), "s"(a.div_ow.s1),
                     "s"(a.div_ow.s2), "s"(a.div_tiles_m.m), "s"(a.div_tiles_m.s1), "s"(a.div_tiles_m.s2),
                     "s"(a.div_tiles_m_pg.m), "s"(a.div_tiles_m_pg.s1), "s"(a.div_tiles_m_pg.s2), "s"(a.div_step.m),
                     "s"(a.div_step.s1), "s"(a.div_step.s2), "s"(a.z), "s"(a.z_bytes), "s"(a.epi.has_z));
        if (!PW)  // the k-unit table
            asm volatile("" ::"s"(a.div_t.m), "s"(a.div_t.s1), "s"(a.div_t.s2), "s"(a.div_fw.m), "s"(a.div_fw.s1), "s"(a.div_fw.s2),
                         "s"(a.T), "s"(a.FW));
        extern __shared__ __attribute__((aligned(16))) int8_t lds[];
        int* sBias = reinterpret_cast<int*>(lds + NS * STG);
        // [ring][bias][residual slots, only for launches with a residual][k-unit table]
        const int zslots = ZD ? 0 : a.zslots;
        KEntry* tab = reinterpret_cast<KEntry*>(lds + RING_BYTES + zslots * ZSLOT);
        const uint32_t lds0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)lds);

        const int t = threadIdx.x;
        const int lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
        const int l32 = lane & 31, lh = lane >> 5;
        const int kg = KS > 1 ? wave / WMN : 0, wmn = KS > 1 ? wave - kg * WMN : wave;  // reduction group, wave inside it
        const int wm = wmn / WN, wn = wmn % WN;

        // this workgroup's tile sequence: workgroup b runs on XCD b % 8 (round-robin dispatch), and each XCD works on
        // one contiguous slab of the tile space, so that its L2 sees disjoint pixels and one set of filter rows
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
        if (my_tiles == 0) return;  // workgroup-uniform
        const int nst = a.nstages;

        int c_tile = first;
        Tile cur = tile_coords(a, c_tile);
        // The bias of the workgroup's channel tile goes straight into LDS (no register is the target of a load the
        // compiler does not know about); it is older than every copy of the prologue.  Without a bias the buffer has no
        // bytes: every lane writes 0.
        const v4i rs_bias = uniform_rsrc(a.bias, a.has_bias ? (uint32_t)a.OC * 4u : 0u);
        if (wave * 64 < BM) lds_copy64x4(lds0 + (uint32_t)(NS * STG + wave * 256), (cur.oc0 + t) * 4, rs_bias);
        const v4i rs_flt = uniform_rsrc(a.flt, a.flt_bytes);

        if (!PW) {
            const int cap = (nst + 1) * KCH;  // one stage of padding entries, read when the loader stands at the end of a tile
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

        const v4i rs_src = uniform_rsrc(a.src, a.src_bytes);
        const v4i rs_z = uniform_rsrc(a.z, a.epi.has_z ? a.z_bytes : 0u);
        const int dA = KCH * a.flt_kstride, dB = KCH * a.src_scb;  // k-offset steps of one stage

        Loader L;
        L.ti = 0;
        L.stage = 0;
        L.kc0 = 0;
        L.kA = 0;
        L.kB = 0;
        loader_enter_tile(a, L, cur, wave, lane);
        // after a stage was issued: the general step, which may move on to the workgroup's next tile or past its last
        auto advance = [&]() __attribute__((always_inline)) {
            L.kc0 += KCH;
            L.kA += dA;
            L.kB += dB;
            if (++L.stage == nst) {
                L.stage = 0;
                L.kc0 = 0;
                L.kA = 0;
                L.kB = 0;
                if (++L.ti < my_tiles)
                    loader_enter_tile(a, L, tile_coords(a, first + L.ti * step), wave, lane);
                else
                    loader_kill(L);
            }
        };

        if (!PW) __syncthreads();  // table ready

        // Residual slots: with two, a tile's residual is copied while the previous tile is multiplied (the first
        // tile's here: it is older than every copy of the prologue); with one, at the start of its own tile.
        const int8_t* zbuf = lds + RING_BYTES + wave * ZWAVE;
        const uint32_t zbuf_addr = lds0 + (uint32_t)(RING_BYTES + wave * ZWAVE);
        int zslot = 0;  // slot of the tile being multiplied
        if (zslots == 2) issue_z(a, rs_z, zbuf_addr, cur.oc0 + wm * WTM, cur.pix0 + wn * WTN, l32, lh);

        // prologue: stages 0 .. NS - 2 into buffers 0 .. NS - 2
        KEntry nk[UB];
        load_entries(L, tab, nk, wave);
        const uint32_t wave_lds = lds0 + (uint32_t)(wave * 1024);
#pragma unroll
        for (int s = 0; s < NS - 1; ++s) {
            issue_all<KT>(a, L, nk, rs_src, rs_flt, wave_lds + (uint32_t)(s * STG), wave);
            advance();
            load_entries(L, tab, nk, wave);
        }
        wait_vmcnt<(NS - 2) * U>();  // this wave's copies of stage 0, and the older bias and residual copies
        __syncthreads();             // ... and everyone's

        const int fragpos = ((l32 >> 4) * 2 + lh) * 256 + (l32 & 15) * 16;
        // (a reduction group reads its own CPS chunks of every stage)
        const int8_t* fragA = lds + fragpos + wm * MT * 1024 + kg * (CPS * NBA * 1024);
        const int8_t* fragB = lds + fragpos + A_BYTES + wn * NT * 1024 + kg * (CPS * NBB * 1024);
        int rd_off = 0;               // byte offset of the stage being multiplied
        int wr_off = (NS - 1) * STG;  // ... of the buffer refilled during this stage: the one read before it

        v4i fa[2][MT], fb[2][NT];
        auto frags = [&](int c, v4i (&xa)[MT], v4i (&xb)[NT]) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < MT; ++i) xa[i] = *reinterpret_cast<const v4i*>(fragA + rd_off + (c * NBA + i) * 1024);
#pragma unroll
            for (int j = 0; j < NT; ++j) xb[j] = *reinterpret_cast<const v4i*>(fragB + rd_off + (c * NBB + j) * 1024);
        };

        v16i acc[MT][NT];
        constexpr bool DUAL = MT * NT == 1;  // one accumulator block: alternate two, so consecutive MFMAs do not depend
        v16i alt;
        // One stage: chunk c's MFMAs run while chunk c + 1 is read and while the copies of chunk step c (of the stage
        // NS - 1 ahead, into the buffer that the previous stage was read from) are issued.  Before the last chunk's MFMAs
        // -- every fragment of the stage is then in registers -- the stage boundary: wait for the next stage, barrier
        // (which also frees this stage's buffer for the refill during the next stage), first fragments of the next
        // stage.  STEADY: the loader stays inside its tile, which takes three scalar additions; otherwise it may step
        // into the next tile or past the last one.
        auto chunk_step = [&](auto steady, auto cc) __attribute__((always_inline)) {
            constexpr bool STEADY = decltype(steady)::value;
            constexpr int c = decltype(cc)::value;
            constexpr bool LAST = c + 1 == CPS;
            if (LAST) {
                wait_lgkmcnt0();
                // copies younger than the next stage's: NS - 3 whole stages and the chunk steps of this stage so far
                wait_vmcnt<(NS - 2) * U - CS_LAST>();
                __syncthreads();  // the next stage has landed for everyone; everyone is done with this stage's buffer
            }
            // The step's other work, cut into pieces that are dealt out between its MFMAs: a wave issues in order, so
            // whatever follows an MFMA issues while the matrix pipe is busy with it (eight issue slots per MFMA), and
            // nothing but the next MFMA waits for the pipe.  Pieces: the reads of the next chunk's fragments, the step's
            // copies, the loader's bookkeeping (last step).
            constexpr int CA = copies_in_step<UA>(c), CB = copies_in_step<UB>(c);
            constexpr int PC = MT + NT;  // first copy piece: the reads come first, their data is needed soonest
            constexpr int P = PC + CA + CB + (LAST ? 1 : 0);
            constexpr int M = MT * NT;
            constexpr int PER = (P + M - 1) / M;
            constexpr int cn = LAST ? 0 : c + 1;  // the chunk whose fragments this step reads ...
            const int rd_nxt = rd_off + STG == NS * STG ? 0 : rd_off + STG;
            const int rd_frag = LAST ? rd_nxt : rd_off;  // ... from this stage's buffer or the next one's
            auto piece = [&](auto kk) __attribute__((always_inline)) {
                constexpr int k = decltype(kk)::value;
                if constexpr (k < MT) {
                    fa[cn & 1][k] = *reinterpret_cast<const v4i*>(fragA + rd_frag + (cn * NBA + k) * 1024);
                } else if constexpr (k < PC) {
                    constexpr int j = k - MT;
                    fb[cn & 1][j] = *reinterpret_cast<const v4i*>(fragB + rd_frag + (cn * NBB + j) * 1024);
                } else if constexpr (k < PC + CA) {
                    issue_a1<c, k - PC>(L, rs_flt, wave_lds + (uint32_t)wr_off, std::make_integer_sequence<int, UA>{});
                } else if constexpr (k < PC + CA + CB) {
                    issue_bk<KT, c, k - PC - CA>(a, L, nk, rs_src, wave_lds + (uint32_t)wr_off, wave, std::make_integer_sequence<int, UB>{});
                } else if constexpr (LAST && k == PC + CA + CB) {
                    if (STEADY) {
                        L.kc0 += KCH;
                        L.kA += dA;
                        L.kB += dB;
                    } else {
                        advance();
                    }
                    load_entries(L, tab, nk, wave);
                    wr_off = rd_off;
                    rd_off = rd_nxt;
                }
                __builtin_amdgcn_sched_barrier(0);
            };
            auto slot = [&](auto mm) __attribute__((always_inline)) {
                constexpr int m = decltype(mm)::value;
                constexpr int i = m / NT, j = m % NT;
                if (DUAL && (c & 1))
                    alt = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[c & 1][i], fb[c & 1][j], alt, 0, 0, 0);
                else
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[c & 1][i], fb[c & 1][j], acc[i][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                for_each_chunk([&](auto qq) __attribute__((always_inline)) { piece(std::integral_constant<int, m * PER + decltype(qq)::value>{}); },
                               std::make_integer_sequence<int, PER>{});
            };
            __builtin_amdgcn_sched_barrier(0);
            for_each_chunk(slot, std::make_integer_sequence<int, M>{});
        };
        auto stage = [&](auto steady) __attribute__((always_inline)) {
            for_each_chunk([&](auto cc) __attribute__((always_inline)) { chunk_step(steady, cc); },
                           std::make_integer_sequence<int, CPS>{});
        };

        frags(0, fa[0], fb[0]);
        init_acc_lds(acc, sBias, wm, lh, kg);

        // stages whose refill stays inside the tile: the loader runs NS - 1 stages ahead
        const int steady = nst > NS - 1 ? nst - (NS - 1) : 0;
        for (int ti = 0; ti < my_tiles; ++ti) {
            if (DUAL) alt = v16i{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            Tile nxt = cur;
            if (ti + 1 < my_tiles) nxt = tile_coords(a, c_tile + step);
            // residual copies: older than every stage copy of this tile (later waits are only stricter for them); the
            // slot they fill was read last by an earlier epilogue of this wave
            if (zslots == 2) {
                if (ti + 1 < my_tiles)
                    issue_z(a, rs_z, zbuf_addr + (uint32_t)((zslot ^ 1) * ZSLOT), nxt.oc0 + wm * WTM, nxt.pix0 + wn * WTN, l32, lh);
            } else if (zslots == 1) {
                issue_z(a, rs_z, zbuf_addr, cur.oc0 + wm * WTM, cur.pix0 + wn * WTN, l32, lh);
            }
            for (int s = 0; s < steady; ++s) stage(std::true_type{});
            if (steady > 0) {
                // the loader has issued the last stage of its tile
                L.stage = nst - 1;
                L.kc0 -= KCH;
                L.kA -= dA;
                L.kB -= dB;
                advance();
                load_entries(L, tab, nk, wave);
            }
            for (int s = steady; s < nst; ++s) stage(std::false_type{});
            if (DUAL) acc[0][0] += alt;
            if constexpr (KS > 1) {
                // The partial sums of the KS reduction groups meet in the ring: every copy has landed (the loader's trailing
                // copies are out-of-range zero fills, but they do write), everyone is done reading.  Block b of a wave tile
                // is finished by group b % KS: a wave parks its sums of the other blocks, lane-linear 16-byte stores, and
                // collects the other groups' sums of its own.
                wait_vmcnt<0>();
                __syncthreads();
                int8_t* red = lds + lane * 16;
                auto slot = [&](int owner, int ob, int src) __attribute__((always_inline)) {
                    return ((((owner * WMN + wmn) * OB + ob) * (KS - 1)) + (src < owner ? src : src - 1)) * 4096;
                };
#pragma unroll
                for (int b = 0; b < MT * NT; ++b) {
                    if (b % KS == kg) continue;  // wave-uniform
                    int8_t* p = red + slot(b % KS, b / KS, kg);
                    const v16i& c = acc[b / NT][b % NT];
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        *reinterpret_cast<v4i*>(p + q * 1024) = v4i{c[4 * q], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3]};
                }
                __syncthreads();
#pragma unroll
                for (int b = 0; b < MT * NT; ++b) {
                    if (b % KS != kg) continue;
                    v16i& c = acc[b / NT][b % NT];
                    for (int src = 0; src < KS; ++src) {
                        if (src == kg) continue;
                        const int8_t* p = red + slot(kg, b / KS, src);
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const v4i v = *reinterpret_cast<const v4i*>(p + q * 1024);
                            c[4 * q] += v[0]; c[4 * q + 1] += v[1]; c[4 * q + 2] += v[2]; c[4 * q + 3] += v[3];
                        }
                    }
                }
            }
            ZRegs<MT, NT> zr;
            if (zslots) {
                // A residual slot is complete once a stage boundary has waited with at least (NS - 2) U - CS_LAST younger
                // copies issued: boundary k after the request sees k U - CS_LAST of them.  Otherwise wait here: the U
                // copies of the last stage are younger.
                const int boundaries = zslots == 2 ? 2 * nst : nst;
                if (boundaries < NS - 2) wait_vmcnt<U>();
                read_z(zr, zbuf + zslot * ZSLOT, lane);
                if (zslots == 2) zslot ^= 1;
            }
            if constexpr (GEN)
                igemm_epilogue_general<POUT, MT, NT>(a, acc, cur.oc0 + wm * WTM, cur.pix0 + wn * WTN, l32, lh, cur.oc_end);
            else if constexpr (KS > 1)  // the blocks this wave finishes
                igemm_run_epilogue<POUT, MT, NT, false>(a, acc, cur.oc0 + wm * WTM, cur.pix0 + wn * WTN, l32, lh, nullptr, cur.oc_end, KS, kg);
            else if constexpr (ZD)
                igemm_run_epilogue<POUT, MT, NT, false>(a, acc, cur.oc0 + wm * WTM, cur.pix0 + wn * WTN, l32, lh, nullptr, cur.oc_end);
            else
                igemm_run_epilogue<POUT, MT, NT, true>(a, acc, cur.oc0 + wm * WTM, cur.pix0 + wn * WTN, l32, lh, &zr, cur.oc_end);
            c_tile += step;
            if (ti + 1 < my_tiles) {
                if (nxt.oc0 != cur.oc0) {
                    // another channel tile: everyone is done with the old bias copy before it is replaced and sees the
                    // new one before it is read (a workgroup-uniform branch)
                    __syncthreads();
                    if (t < BM) sBias[t] = fetch_bias(a, nxt.oc0, t);
                    __syncthreads();
                }
                init_acc_lds(acc, sBias, wm, lh, kg);
            }
            cur = nxt;
        }
        // the trailing (out-of-range, zero-filling) copies must land before this workgroup's LDS is released
        wait_vmcnt<0>();
    }
};

template <int POUT, int BM, int BN, int WM, int WN, int KCH, int NS, int MINW, bool PW, bool KT, bool GEN, int KS = 1>
__global__ __launch_bounds__(WM * WN * KS * 64, MINW) void igemm2_kernel(IgemmArgs a) {
    Igemm2<POUT, BM, BN, WM, WN, KCH, NS, PW, KS>::template run<KT, GEN>(a);
}

constexpr int kLdsPerCu = 160 * 1024;
constexpr int kNoFit = -1;  // not a hipError_t
constexpr int kNoGen = -2;  // this tile has no instantiation with the general epilogue

struct Cfg2 {
    const char* name;
    int bm, bn, kch;
};
const Cfg2 kCfg2[] = {
        {"v2_128x128x64r4", 128, 128, 2},
        {"v2_128x128x64r3", 128, 128, 2},
        {"v2_128x128x128r3", 128, 128, 4},
        {"v2_64x128x128r3", 64, 128, 4},
        {"v2_64x128x64r4", 64, 128, 2},
        {"v2_128x64x128r3", 128, 64, 4},
        {"v2_128x64x64r4", 128, 64, 2},
        {"v2_64x64x128r3", 64, 64, 4},
        {"v2_64x64x128r4", 64, 64, 4},
        {"v2_256x128x64r3w8", 256, 128, 2},
        {"v2_128x256x64r3w8", 128, 256, 2},
        {"v2_256x256x64r3w8", 256, 256, 2},
        {"v2_128x128x64r4w8", 128, 128, 2},
        {"v2_64x128x64r5", 64, 128, 2},
        {"v2_128x64x128r3k2", 128, 64, 4},
        {"v2_128x64x256r3k4w8", 128, 64, 8},
        {"v2_64x128x128r3k2", 64, 128, 4},
        {"v2_128x128x128r3k2w8", 128, 128, 4},
};
constexpr int kNumCfg2 = sizeof(kCfg2) / sizeof(kCfg2[0]);

template <int POUT, int BM, int BN, int WM, int WN, int KCH, int NS, int MINW, bool PW, bool KT, bool GEN, int KS = 1>
int launch_k(hipStream_t st, IgemmArgs& a, int cu_count) {
    using K = Igemm2<POUT, BM, BN, WM, WN, KCH, NS, PW, KS>;
    a.tiles_m_pg = (a.ocpg + BM - 1) / BM;
    a.tiles_m = a.tiles_m_pg * a.groups;
    a.div_tiles_m = make_fastdiv((uint32_t)a.tiles_m);
    a.div_tiles_m_pg = make_fastdiv((uint32_t)a.tiles_m_pg);
    a.tiles_n = (a.M + BN - 1) / BN;
    const int64_t tiles = (int64_t)a.tiles_m * a.tiles_n;
    if (tiles <= 0 || tiles > 0x3fffffff) return (int)hipErrorInvalidValue;
    a.tiles = (int)tiles;
    a.nstages = (a.KC + KCH - 1) / KCH;
    // one stage of padding entries: the loader reads the entries of the stage after the one it just issued
    const int tab_entries = PW ? 0 : (a.nstages + 1) * KCH;
    if (tab_entries > IG_MAX_ENTRIES) return (int)hipErrorInvalidValue;
    // Residual slots: short reductions copy a tile's residual one tile ahead (two slots); long ones have the whole
    // tile to hide it behind (one slot, and room for a second workgroup per CU)
    const int fixed = K::RING_BYTES + tab_entries * 8;
    a.zslots = 0;
    if (a.epi.has_z && !a.general && !K::ZD) {
        a.zslots = a.nstages <= 2 ? 2 : 1;
        if (fixed + a.zslots * K::ZSLOT > kLdsPerCu) a.zslots = 1;
    }
    const int lds = fixed + a.zslots * K::ZSLOT;
    if (lds > kLdsPerCu) return kNoFit;  // ring + residual slot of this tile do not fit
    if (a.dry_run) return 0;             // the question was only whether this tile can run the problem
    auto kern = igemm2_kernel<POUT, BM, BN, WM, WN, KCH, NS, MINW, PW, KT, GEN, KS>;
    // per-instantiation caches; atomics, because operators on different streams may launch from several threads
    static std::atomic<int> max_lds_set{0};
    if (lds > max_lds_set.load(std::memory_order_relaxed)) {
        int want = K::RING_BYTES + 2 * K::ZSLOT + IG_MAX_ENTRIES * 8;
        if (want > kLdsPerCu) want = kLdsPerCu;
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, want);
        if (e != hipSuccess) return (int)e;
        max_lds_set.store(want, std::memory_order_relaxed);
    }
    static std::atomic<uint64_t> occ_cache{0};  // LDS bytes of the last query << 32 | its result
    const uint64_t cached = occ_cache.load(std::memory_order_relaxed);
    int occ = (int)(uint32_t)cached;
    if ((cached >> 32) != (uint64_t)lds || occ < 1) {
        hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, reinterpret_cast<const void*>(kern), K::THREADS, (size_t)lds);
        if (e != hipSuccess || occ < 1) {
            (void)hipGetLastError();
            occ = 1;
        }
        occ_cache.store(((uint64_t)lds << 32) | (uint32_t)occ, std::memory_order_relaxed);
    }
    if (cu_count <= 0) cu_count = 256;
    int64_t grid = (int64_t)occ * cu_count;
    if (KS > 1) grid = tiles;  // a workgroup that splits the reduction runs one tile (its ring doubles as the meeting place)
    // a multiple of 8 (one contiguous slab of the tile space per XCD).  When every tile has a workgroup of its own the
    // count is rounded UP -- a few workgroups find no tile and leave -- because rounding down would hand some workgroups
    // a second tile and double the launch's duration; otherwise down, inside what the device holds at once.
    if (grid > tiles) grid = tiles;
    if (grid >= 8) grid = grid == tiles ? (grid + 7) & ~(int64_t)7 : grid & ~(int64_t)7;
    a.div_step = make_fastdiv((uint32_t)((grid & 7) == 0 ? grid >> 3 : grid));  // the kernel's tile stride
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(K::THREADS), lds, st, a);
    return (int)hipGetLastError();
}

template <int POUT, int BM, int BN, int WM, int WN, int KCH, int NS, int MINW, bool GEN, int KS = 1>
int launch_gen(hipStream_t st, IgemmArgs& a, int cu) {
    const bool pw = a.T == 1 && a.ph == 0 && a.pw == 0;
    const bool kt = a.KC % KCH != 0;
    if (pw)
        return kt ? launch_k<POUT, BM, BN, WM, WN, KCH, NS, MINW, true, true, GEN, KS>(st, a, cu)
                  : launch_k<POUT, BM, BN, WM, WN, KCH, NS, MINW, true, false, GEN, KS>(st, a, cu);
    // the k-unit table carries the end of the reduction (padding entries)
    return launch_k<POUT, BM, BN, WM, WN, KCH, NS, MINW, false, false, GEN, KS>(st, a, cu);
}

// a tile whose waves also split the reduction (fast epilogue only)
template <int POUT, int BM, int BN, int WM, int WN, int KCH, int NS, int MINW, int KS>
int launch_split(hipStream_t st, IgemmArgs& a, int cu) {
    if (a.general) return kNoGen;
    return launch_gen<POUT, BM, BN, WM, WN, KCH, NS, MINW, false, KS>(st, a, cu);
}

// GENOK: the tile is also instantiated with the general epilogue (two tiles are: every general problem runs on one of them)
template <int POUT, int BM, int BN, int WM, int WN, int KCH, int NS, int MINW, bool GENOK = false>
int launch_one(hipStream_t st, IgemmArgs& a, int cu) {
    if (a.general) {
        if constexpr (GENOK)
            return launch_gen<POUT, BM, BN, WM, WN, KCH, NS, MINW, true>(st, a, cu);
        else
            return kNoGen;
    }
    return launch_gen<POUT, BM, BN, WM, WN, KCH, NS, MINW, false>(st, a, cu);
}

template <int POUT>
int launch_fmt(hipStream_t st, IgemmArgs& a, int cfg, int cu) {
    switch (cfg) {
        case 0: return launch_one<POUT, 128, 128, 2, 2, 2, 4, 2, true>(st, a, cu);
        case 1: return launch_one<POUT, 128, 128, 2, 2, 2, 3, 2>(st, a, cu);
        case 2: return launch_one<POUT, 128, 128, 2, 2, 4, 3, 1>(st, a, cu);
        case 3: return launch_one<POUT, 64, 128, 2, 2, 4, 3, 2, true>(st, a, cu);
        case 4: return launch_one<POUT, 64, 128, 2, 2, 2, 4, 2>(st, a, cu);
        case 5: return launch_one<POUT, 128, 64, 2, 2, 4, 3, 2>(st, a, cu);
        case 6: return launch_one<POUT, 128, 64, 2, 2, 2, 4, 2>(st, a, cu);
        case 7: return launch_one<POUT, 64, 64, 2, 2, 4, 3, 3>(st, a, cu);
        case 8: return launch_one<POUT, 64, 64, 2, 2, 4, 4, 3>(st, a, cu);
        case 9: return launch_one<POUT, 256, 128, 4, 2, 2, 3, 4>(st, a, cu);
        case 10: return launch_one<POUT, 128, 256, 2, 4, 2, 3, 4>(st, a, cu);
        case 11: return launch_one<POUT, 256, 256, 4, 2, 2, 3, 2>(st, a, cu);
        case 12: return launch_one<POUT, 128, 128, 2, 4, 2, 4, 4>(st, a, cu);
        case 13: return launch_one<POUT, 64, 128, 2, 2, 2, 5, 2>(st, a, cu);
        // reduction split over the waves of the workgroup: wave tiles of 64 x 64
        case 14: return launch_split<POUT, 128, 64, 2, 1, 4, 3, 2, 2>(st, a, cu);
        case 15: return launch_split<POUT, 128, 64, 2, 1, 8, 3, 2, 4>(st, a, cu);
        case 16: return launch_split<POUT, 64, 128, 1, 2, 4, 3, 2, 2>(st, a, cu);
        case 17: return launch_split<POUT, 128, 128, 2, 2, 4, 3, 2, 2>(st, a, cu);
        default: return (int)hipErrorInvalidValue;
    }
}

}  // namespace

int igemm2_num_cfgs() { return kNumCfg2; }
const char* igemm2_cfg_name(int cfg) { return cfg >= 0 && cfg < kNumCfg2 ? kCfg2[cfg].name : "?"; }
void igemm2_cfg_shape(int cfg, int* bm, int* bn, int* kch) {
    *bm = kCfg2[cfg].bm; *bn = kCfg2[cfg].bn; *kch = kCfg2[cfg].kch;
}

namespace {
// [k-chunk][channel, padded to 32][32 bytes]: the 32-byte k-chunk of 32 consecutive filter rows is one contiguous
// kilobyte -- what one LDS-direct wave copy of the kernel above fetches.  One thread moves 16 bytes.
__global__ __launch_bounds__(256) void igemm2_preprocess_kernel(const int8_t* flt, int8_t* out, int oc, int ocp, int kbytes,
                                                                int64_t units) {
    const int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (u >= units) return;
    const int64_t kc = u / (ocp * 2);
    const int r = (int)(u - kc * (ocp * 2));
    const int row = r >> 1, half = r & 1;
    v4i v = {0, 0, 0, 0};
    if (row < oc) v = *reinterpret_cast<const v4i*>(flt + (int64_t)row * kbytes + kc * 32 + half * 16);
    *reinterpret_cast<v4i*>(out + u * 16) = v;
}
}  // namespace

size_t igemm2_preprocessed_bytes(int oc, int kbytes) {
    const int64_t ocp = (oc + 31) / 32 * 32, kc = (kbytes + 31) / 32;
    return (size_t)(kc * ocp * 32);
}

int launch_igemm2_preprocess(hipStream_t st, const int8_t* flt, int8_t* out, int oc, int kbytes) {
    const int ocp = (oc + 31) / 32 * 32, kc = (kbytes + 31) / 32;
    const int64_t units = (int64_t)kc * ocp * 2;
    if (units == 0) return 0;
    hipLaunchKernelGGL(igemm2_preprocess_kernel, dim3((unsigned)((units + 255) / 256)), dim3(256), 0, st, flt, out, oc, ocp,
                       kbytes, units);
    return (int)hipGetLastError();
}

// A tile that cannot run the problem (no instantiation with the general epilogue, or ring + residual slot beyond the
// LDS of a CU) is an error here: igemm_resolve_cfg (conv_igemm.hip) names the tile that runs before anything is launched.
int launch_igemm2(hipStream_t st, IgemmArgs& a, int pout, int cfg, int cu_count) {
    const int rc = pout == 32 ? launch_fmt<32>(st, a, cfg, cu_count) : launch_fmt<4>(st, a, cfg, cu_count);
    return rc == kNoFit || rc == kNoGen ? (int)hipErrorInvalidConfiguration : rc;
}

bool igemm2_can_run(const IgemmArgs& a, int pout, int cfg) {
    IgemmArgs t = a;
    t.dry_run = 1;
    return (pout == 32 ? launch_fmt<32>(nullptr, t, cfg, 256) : launch_fmt<4>(nullptr, t, cfg, 256)) == 0;
}

}  // namespace mi355
