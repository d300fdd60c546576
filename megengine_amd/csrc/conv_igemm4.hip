// Weight-resident kernel for 3x3 / stride 1 / pad 1 ConvBias over few input channels (32-packed in and out): the early
// 3x3 layers of a residual network, whose whole filter is a few tens of kilobytes.
//
// The implicit-GEMM kernels copy, for every tile, the filter rows of the tile's channels and the im2col rows of its
// pixels into LDS: with 64 input channels that is 36 KB of the same weights and 9 x the same activations per tile
// through the 55-64 B/clk a CU's vector-memory path delivers, and that path -- not the matrix pipe -- bounds the layer.
// Here a persistent workgroup (4 waves; tiles of 64 channels x 128 consecutive pixels of one image)
//   * holds the weights of its 64 output channels in REGISTERS, as the A fragments of all 9 * IC / 32 reduction steps
//     (72 VGPRs per 32 input channels; read once per channel tile with coalesced 1 KB copies into LDS, and from there
//     with a padded row pitch that makes the strided fragment reads conflict-free),
//   * copies the input rows a tile needs -- the rows of its pixels plus one above and one below, full width plus one
//     column on each side, zero-filled outside the image by the copy itself -- global -> LDS without a register stage,
//     two tiles ahead of the one being multiplied, into a ring of three patch slots, and
//   * reads every MFMA B fragment straight from the patch: lane (pixel, half) of tap (fh, fw) and channel block cb
//     needs 16 contiguous bytes at patch[row(pixel) + fh][cb][col(pixel) + fw].
// Per tile the copy path moves the patch once (22 KB for 64 channels at 56 x 56) instead of 108 KB.  One barrier per tile;
// "the next patch has landed" is a counted s_waitcnt vmcnt(N), N = the patch copies issued after it.
#include <atomic>

#include "lds_copy.h"

namespace mi355 {
namespace {

constexpr int R4_THREADS = 256;
constexpr int R4_BM = 64, R4_BN = 128;
constexpr int R4_NSLOT = 3;
constexpr int R4_VMCNT0 = 0x0f70;  // s_waitcnt vmcnt(0) with the other counters at their maxima

struct R4Geom {
    int tiles_p;      // pixel tiles per image
    int tiles_n;      // pixel tiles in all: N * tiles_p
    int pw;           // patch row width in pixels: IW + 2
    int cpr;          // 1 KB copies per patch row and channel block
    int slot_bytes;   // one ring slot (a patch; two slots together hold the weight staging area)
    int wpitch;       // bytes between the filter rows of two channels in the staging area: kbytes + 16
    FastDiv div_tp, div_tn, div_wp;
};

// s_waitcnt vmcnt(n) for a wave-uniform n >= 0 (the count is an immediate of the instruction); n > 15 waits as 15
__device__ __forceinline__ void r4_wait_vmcnt(int n) {
    switch (n) {
#define R4_W1(k) case k: wait_vmcnt<k>(); break;
        R4_W1(0) R4_W1(1) R4_W1(2) R4_W1(3) R4_W1(4) R4_W1(5) R4_W1(6) R4_W1(7)
        R4_W1(8) R4_W1(9) R4_W1(10) R4_W1(11) R4_W1(12) R4_W1(13) R4_W1(14)
#undef R4_W1
        default: wait_vmcnt<15>(); break;
    }
}

// KB = 32-byte channel blocks of the input (IC / 32); HZ: the launch has a residual
template <int KB, bool HZ>
__global__ __launch_bounds__(R4_THREADS, 2) void igemm4_kernel(IgemmArgs a, R4Geom g) {
    extern __shared__ __attribute__((aligned(16))) int8_t lds[];
    constexpr int KS = 9 * KB;  // reduction steps of 32 bytes
    const int t = threadIdx.x;
    const int lane = t & 63, w = __builtin_amdgcn_readfirstlane(t >> 6);
    const int l32 = lane & 31, lh = lane >> 5;
    const uint32_t lds0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)lds);
    int* sBias = reinterpret_cast<int*>(lds + R4_NSLOT * g.slot_bytes);

    const int first = blockIdx.x, step = gridDim.x;
    if (first >= a.tiles) return;
    const int count = (a.tiles - 1 - first) / step + 1;  // tiles of this workgroup: first, first + step, ...

    const v4i rs_src = uniform_rsrc(a.src, a.src_bytes);
    const v4i rs_flt = uniform_rsrc(a.flt, a.flt_bytes);

    struct Tile {
        int mt, n, p0, pend, oh0, nrows;  // channel tile, image, first / last pixel in the image, first row, patch rows
    };
    auto decode = [&](int k) __attribute__((always_inline)) -> Tile {
        Tile r;
        const uint32_t tile = (uint32_t)(first + k * step);
        const uint32_t mt = fdiv(tile, g.div_tn), nt = tile - mt * g.tiles_n;
        const uint32_t n = fdiv(nt, g.div_tp), tp = nt - n * g.tiles_p;
        r.mt = (int)mt; r.n = (int)n;
        r.p0 = (int)tp * R4_BN;
        r.pend = min(r.p0 + R4_BN, a.OHW) - 1;
        r.oh0 = (int)fdiv((uint32_t)r.p0, a.div_ow);
        r.nrows = (int)fdiv((uint32_t)r.pend, a.div_ow) - r.oh0 + 3;
        return r;
    };

    // Patch of a tile -> a ring slot.  Patch row j, channel block cb holds input row oh0 - 1 + j, columns -1 .. IW, as
    // 2 * pw pieces of 16 bytes; one copy moves 64 pieces, lanes past the row end are masked off.  The lane part of the
    // address (column, half) does not depend on the tile; the row part is wave-uniform and sits in the scalar offset; a
    // row outside the image is copied with out-of-range lane offsets and arrives as zeros.  Wave w takes the (row,
    // block) pairs w, w + 4, ...  Returns the number of copies this wave issued.
    const int pieces = 2 * g.pw;
    auto lane_off = [&](int c) __attribute__((always_inline)) -> int {
        const int piece = 64 * c + lane, col = (piece >> 1) - 1;
        return (piece < pieces && (unsigned)col < (unsigned)a.IW) ? col * 32 + (piece & 1) * 16 : SENT;
    };
    const int vcol0 = lane_off(0), vcol1 = lane_off(1);
    auto copy_patch = [&](const Tile& tt, int slot) __attribute__((always_inline)) -> int {
        const uint32_t dst = lds0 + (uint32_t)(slot * g.slot_bytes);
        int issued = 0;
        for (int rc = w; rc < tt.nrows * KB; rc += 4) {
            const int j = rc / KB, cb = rc - j * KB;
            const int h = tt.oh0 - 1 + j;
            const bool ok = (unsigned)h < (unsigned)a.IH;
            const int soff = ok ? tt.n * a.src_sn + cb * a.src_scb + h * a.IW * 32 : 0;
            for (int c = 0; c < g.cpr; ++c) {
                const int vo = c == 0 ? vcol0 : c == 1 ? vcol1 : lane_off(c);
                if (64 * c + lane < pieces)
                    lds_copy_row64x16(dst + (uint32_t)(rc * pieces * 16 + c * 1024), ok ? vo : SENT, soff, rs_src);
                ++issued;
            }
        }
        return issued;
    };

    // A fragments of every reduction step: lane (l32, lh) holds bytes 16 * lh .. + 15 of the 32-byte chunk s of channel
    // i * 32 + l32 (chunk s = channel block s / 9, tap s % 9: the order of the filter row itself).  The filter rows of
    // the channel tile (kbytes each, contiguous in memory) are copied into LDS with a row pitch of kbytes + 16, which
    // spreads the 32 rows a fragment read touches over all banks; rows past OC arrive as zeros.
    v4i wr[KS][2];
    auto stage_weights = [&](int mt, uint32_t area) __attribute__((always_inline)) {
        const int rows = min(R4_BM, a.OC - mt * R4_BM);
        const int total = (R4_BM * g.wpitch + 1023) >> 10;
        for (int c = w; c < total; c += 4) {
            const uint32_t q = (uint32_t)(c * 1024 + lane * 16);
            const uint32_t row = fdiv(q, g.div_wp), within = q - row * (uint32_t)g.wpitch;
            const bool ok = (int)row < rows && (int)within < a.kbytes;
            lds_copy64x16(area + (uint32_t)(c * 1024), ok ? (mt * R4_BM + (int)row) * a.kbytes + (int)within : SENT, rs_flt);
        }
    };
    auto read_weights = [&](const int8_t* area) __attribute__((always_inline)) {
#pragma unroll
        for (int s = 0; s < KS; ++s)
#pragma unroll
            for (int i = 0; i < 2; ++i) wr[s][i] = *reinterpret_cast<const v4i*>(area + (i * 32 + l32) * g.wpitch + s * 32 + lh * 16);
    };

    // byte offsets of the 9 * KB fragment positions relative to a lane's base (wave-uniform)
    int koff[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        const int cb = s / 9, tap = s - cb * 9, fh = tap / 3, fw = tap - fh * 3;
        koff[s] = ((fh * KB + cb) * g.pw + fw) * 32;
    }

    // Tiles are numbered channel tile first, so a workgroup's tiles come in runs of one channel tile.  Each run loads its
    // weights once and pipelines its patches; nothing is copied ahead across the end of a run.
    for (int k0 = 0; k0 < count;) {
        Tile tl = decode(k0);
        const int k_end = min(count, ((tl.mt + 1) * g.tiles_n - 1 - first) / step + 1);
        if (k0 > 0) __syncthreads();  // every wave is done with the patches and the bias of the run before
        // the first patch into slot 0, the weights through the space of slots 1 and 2, then the second patch
        (void)copy_patch(tl, 0);
        stage_weights(tl.mt, lds0 + (uint32_t)g.slot_bytes);
        if (t < R4_BM) {
            const int oc = tl.mt * R4_BM + t;
            sBias[t] = (a.has_bias && oc < a.OC) ? a.bias[oc] : 0;
        }
        __builtin_amdgcn_s_waitcnt(R4_VMCNT0);
        __syncthreads();
        read_weights(lds + g.slot_bytes);
        __syncthreads();  // every wave holds its fragments: slots 1 and 2 are free
        Tile tn = tl;  // each tile is decoded once: tn = tile k + 1, decoded when its patch is copied
        if (k0 + 1 < k_end) {
            tn = decode(k0 + 1);
            (void)copy_patch(tn, 1);
        }

        int slot = 0;
        for (int k = k0; k < k_end; ++k) {
            int ahead = 0;  // patch copies issued after those of tile k + 1
            Tile tnn = tn;
            if (k + 2 < k_end) {
                tnn = decode(k + 2);
                ahead = copy_patch(tnn, slot == 0 ? 2 : slot - 1);
            }
            // this lane's pixel and its place in the patch
            const int pc = min(tl.p0 + w * 32 + l32, tl.pend);
            const int oh = (int)fdiv((uint32_t)pc, a.div_ow), ow = pc - oh * a.OW;
            const int8_t* base = lds + slot * g.slot_bytes + (((oh - tl.oh0) * KB) * g.pw + ow) * 32 + lh * 16;
            const int oc_w = tl.mt * R4_BM;
            const int pix_w = tl.n * a.OHW + tl.p0 + w * 32;
            const int m_end = tl.n * a.OHW + tl.pend + 1;
            ZRegs<2, 1> zr;
            if constexpr (HZ) igemm_load_z<32, 2, 1>(a, zr, oc_w, pix_w, l32, lh, m_end);

            v16i acc[2][1];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const v4i b = *reinterpret_cast<const v4i*>(sBias + i * 32 + 8 * q + 4 * lh);
                    acc[i][0][4 * q + 0] = b[0]; acc[i][0][4 * q + 1] = b[1]; acc[i][0][4 * q + 2] = b[2]; acc[i][0][4 * q + 3] = b[3];
                }
            // two B fragments in flight ahead of the MFMAs that consume them
            v4i fb[3];
            fb[0] = *reinterpret_cast<const v4i*>(base + koff[0]);
            fb[1] = *reinterpret_cast<const v4i*>(base + koff[1]);
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                if (s + 2 < KS) fb[(s + 2) % 3] = *reinterpret_cast<const v4i*>(base + koff[s + 2]);
                acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wr[s][0], fb[s % 3], acc[0][0], 0, 0, 0);
                acc[1][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wr[s][1], fb[s % 3], acc[1][0], 0, 0, 0);
            }

            // One barrier per tile, before the epilogue: the next tile's patch has landed (this wave's copies; the
            // barrier covers the other waves') and every wave is done with this tile's slot, which the copies issued at
            // the top of the next iteration overwrite.  Only patch copies are counted, so
            // the wait also covers every older load and store the compiler issued.
            if (k + 1 < k_end) {
                r4_wait_vmcnt(ahead);
                __syncthreads();
            }
            if constexpr (HZ)
                igemm_run_epilogue<32, 2, 1, true>(a, acc, oc_w, pix_w, l32, lh, &zr, -1, 1, 0, m_end);
            else
                igemm_run_epilogue<32, 2, 1>(a, acc, oc_w, pix_w, l32, lh, nullptr, -1, 1, 0, m_end);
            tl = tn;
            tn = tnn;
            slot = slot == 2 ? 0 : slot + 1;
        }
        k0 = k_end;
    }
}

constexpr int kLdsPerCu = 160 * 1024;

struct Cfg4 {
    const char* name;
};
const Cfg4 kCfg4[] = {{"v4_64x128res"}};
constexpr int kNumCfg4 = sizeof(kCfg4) / sizeof(kCfg4[0]);

bool shape_ok(const IgemmArgs& a, int pin, int pout) {
    // 32-packed on both sides, dense, 3x3 / stride 1 / pad 1, 32 or 64 input channels, the fast epilogue
    return pin == 32 && pout == 32 && a.groups == 1 && !a.general && a.sh == 1 && a.sw == 1 && a.FH == 3 && a.FW == 3 &&
           a.ph == 1 && a.pw == 1 && a.OH == a.IH && a.OW == a.IW && (a.kbytes == 288 || a.kbytes == 576) && a.NB > 0;
}

// geometry and LDS of a launch; false when the ring and the bias do not fit twice into the LDS of a CU
bool geometry(const IgemmArgs& a, R4Geom& g, int& lds) {
    g.tiles_p = (a.OHW + R4_BN - 1) / R4_BN;
    g.tiles_n = a.NB * g.tiles_p;
    g.pw = a.IW + 2;
    g.cpr = (2 * g.pw + 63) / 64;
    g.wpitch = a.kbytes + 16;
    const int kb = a.kbytes / 288;
    const int rows_max = (a.OW - 1 + R4_BN - 1) / a.OW + 1 + 2;   // rows 128 consecutive pixels touch, plus one above and below
    // the last copy of a row writes whole 16-byte pieces only for lanes inside the row: a slot is exactly its rows
    int slot = rows_max * kb * g.pw * 32;
    const int wbytes = ((R4_BM * g.wpitch + 1023) >> 10) << 10;   // the staging copies write whole kilobytes
    if (2 * slot < wbytes) slot = (wbytes + 1) / 2;
    g.slot_bytes = (slot + 15) / 16 * 16;
    g.div_tp = make_fastdiv((uint32_t)g.tiles_p);
    g.div_tn = make_fastdiv((uint32_t)g.tiles_n);
    g.div_wp = make_fastdiv((uint32_t)g.wpitch);
    lds = R4_NSLOT * g.slot_bytes + R4_BM * 4;
    return lds <= kLdsPerCu / 2 && (int64_t)g.tiles_n * ((a.OC + R4_BM - 1) / R4_BM) < ((int64_t)1 << 30);
}

template <int KB, bool HZ>
int launch_k(hipStream_t st, IgemmArgs& a, const R4Geom& g, int lds, int cu_count) {
    auto kern = igemm4_kernel<KB, HZ>;
    static std::atomic<int> occ{0};  // zero-initialised; several threads may launch
    if (!occ.load(std::memory_order_relaxed)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsPerCu / 2);
        if (e != hipSuccess) return (int)e;
        occ.store(2, std::memory_order_relaxed);
    }
    if (cu_count <= 0) cu_count = 256;
    // persistent grid: as many workgroups as are resident at once (two per CU)
    int64_t grid = (int64_t)occ.load(std::memory_order_relaxed) * cu_count;
    if (grid > a.tiles) grid = a.tiles;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(R4_THREADS), lds, st, a, g);
    return (int)hipGetLastError();
}

}  // namespace

int igemm4_num_cfgs() { return kNumCfg4; }
const char* igemm4_cfg_name(int cfg) { return cfg >= 0 && cfg < kNumCfg4 ? kCfg4[cfg].name : "?"; }

bool igemm4_can_run(const IgemmArgs& a, int pin, int pout, int cfg) {
    if (cfg != 0 || !shape_ok(a, pin, pout)) return false;
    R4Geom g;
    int lds;
    return geometry(a, g, lds);
}

int launch_igemm4(hipStream_t st, IgemmArgs& a, int pin, int pout, int cfg, int cu_count) {
    R4Geom g;
    int lds;
    if (cfg != 0 || !shape_ok(a, pin, pout) || !geometry(a, g, lds)) return (int)hipErrorInvalidConfiguration;
    a.tiles_m = (a.OC + R4_BM - 1) / R4_BM;
    a.tiles_n = g.tiles_n;
    a.tiles = a.tiles_m * a.tiles_n;
    const bool hz = a.epi.has_z != 0;
    if (a.kbytes == 288) return hz ? launch_k<1, true>(st, a, g, lds, cu_count) : launch_k<1, false>(st, a, g, lds, cu_count);
    return hz ? launch_k<2, true>(st, a, g, lds, cu_count) : launch_k<2, false>(st, a, g, lds, cu_count);
}

}  // namespace mi355
