// Internal declarations shared by the host C-ABI layer and the HIP kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/mi355_convbias.h"
#include "epilogue.h"

namespace mi355 {

// ---- algorithm table ids (order is the ABI of mi355_convbias_algo_name) ----
enum AlgoId {
    ALGO_DIRECT = 0,       // generic one-thread-per-output kernel: every format / mode
    ALGO_IGEMM_MFMA = 1,   // dense implicit GEMM on int8 MFMA (NCHW4 / NCHW32 / mixed)
    ALGO_DEPTHWISE = 2,    // channel-wise, bandwidth bound (NCHW4-packed and NCHW)
    ALGO_C4_MFMA = 3,      // first layers: NCHW4 with 4 input channels, patch-staged MFMA
    ALGO_NCHW_MFMA = 4,    // plain NCHW: relayout into the workspace, the NCHW32 MFMA kernel, relayout back
    ALGO_COUNT = 5
};

// Canonical problem description used by every launcher (derived from mi355_conv_desc)
struct ConvProblem {
    mi355_conv_desc d;
    uint32_t oh, ow;
    uint32_t icpg, ocpg;
    int pin, pout;     // channel pack of src/filter and of dst/bias/z
    bool dw4;          // packed-by-4 channel-wise filter layout
    int64_t src_sn, dst_sn, z_sn;  // batch strides in elements
    EpiParams epi;
};

// The residual table form of the requantisation (epilogue.h): true, the slope and the 256 offsets (indexed by the
// residual byte as an unsigned value; the pointer stays valid for the life of the process) when the host has proved it
// for these scales and this activation.  A hash lookup after the first call for a scale triple.
bool epi_residual_table(const EpiParams& e, float* c, const float** tab);

// ---- launchers (each returns a hipError_t-compatible int; 0 = success) ----
int launch_conv_direct(hipStream_t st, const ConvProblem& p, const int8_t* src, const int8_t* flt,
                       const int32_t* bias, const void* z, void* dst);

// tile_cfg: index into the igemm tile table, -1 = pick by heuristic
int igemm_num_cfgs();
const char* igemm_cfg_name(int cfg);
bool igemm_usable(const ConvProblem& p);
// will_preprocess: the caller will hand exec the filter pre-processed for the chosen tile
int igemm_pick_cfg(const ConvProblem& p, int cu_count, bool will_preprocess = false);
// The tile that runs when tile_cfg is asked for: tile_cfg itself when that kernel can run the problem as it is, else
// the tile the launch code takes in its place (another kernel generation for this packing, a tile that has the general
// epilogue, a ring that fits the LDS).  A choice of the heuristic is replaced silently; a tile the caller forced is not.
int igemm_resolve_cfg(const ConvProblem& p, int tile_cfg);
// flt_preprocessed: flt points to the artefact of launch_igemm_preprocess (only tiles with igemm_preprocessed_bytes > 0)
int launch_conv_igemm(hipStream_t st, const ConvProblem& p, int tile_cfg, int cu_count, const int8_t* src,
                      const int8_t* flt, const int32_t* bias, const int8_t* z, int8_t* dst, bool flt_preprocessed = false);
// weight pre-processing: bytes of the re-tiled filter for this problem and tile (0: the tile reads the reference
// layout only), and the pass that writes it
size_t igemm_preprocessed_bytes(const ConvProblem& p, int tile_cfg);
int launch_igemm_preprocess(hipStream_t st, const ConvProblem& p, const int8_t* flt, int8_t* out);

bool depthwise_usable(const ConvProblem& p);
int launch_conv_depthwise(hipStream_t st, const ConvProblem& p, const int8_t* src, const int8_t* flt,
                          const int32_t* bias, const int8_t* z, int8_t* dst);

bool c4_usable(const ConvProblem& p);
int launch_conv_c4(hipStream_t st, const ConvProblem& p, int cu_count, const int8_t* src, const int8_t* flt,
                   const int32_t* bias, const int8_t* z, int8_t* dst);

// plain NCHW through the caller's workspace (conv_nchw.hip); nchw_mfma_workspace is 0 when the algorithm cannot run
bool nchw_mfma_usable(const ConvProblem& p);
size_t nchw_mfma_workspace(const ConvProblem& p);
int launch_conv_nchw_mfma(hipStream_t st, const ConvProblem& p, int cu_count, const int8_t* src, const int8_t* flt,
                          const int32_t* bias, const int8_t* z, int8_t* dst, void* workspace);

int launch_requant(hipStream_t st, const EpiParams& e, const int32_t* src, const int8_t* z, int8_t* dst, uint64_t count,
                   int cu_count);
int launch_requant8(hipStream_t st, const EpiParams& e, const int8_t* src, const int8_t* z, int8_t* dst, uint64_t count,
                    int cu_count);

// plain streaming kernel: reads read_bytes from src and writes write_bytes to dst in 16-byte accesses (a measuring stick)
int elemwise_q_arity(uint32_t mode);
int launch_elemwise_q(hipStream_t st, const mi355_elemwise_desc& d, const void* s0, const void* s1, const void* s2, void* dst,
                      int cu_count);
int launch_stream_probe(hipStream_t st, const void* src, uint64_t read_bytes, void* dst, uint64_t write_bytes, int cu_count);
int launch_cvt_f32_s8(hipStream_t st, float scale, const float* src, int8_t* dst, uint64_t count, int cu_count);
int launch_cvt_s8_f32(hipStream_t st, float scale, const int8_t* src, float* dst, uint64_t count, int cu_count);

int launch_pooling(hipStream_t st, const mi355_pooling_desc& d, int pack, uint32_t oh, uint32_t ow, const int8_t* src,
                   int8_t* dst, int cu_count);

int launch_relayout(hipStream_t st, const mi355_relayout_desc& d, const uint32_t* oshape, uint32_t ondim,
                    const void* src, void* dst, bool allow_fast);

static inline uint32_t conv_out_size(uint32_t i, uint32_t f, uint32_t dil, uint32_t s, uint32_t p) {
    uint32_t df = (f - 1) * dil + 1;
    return (i + 2 * p - df) / s + 1;
}

// unsigned division by a runtime constant: q = (t + ((x - t) >> s1)) >> s2, t = mulhi(x, m)
struct FastDiv {
    uint32_t m, s1, s2, d;
};

static inline FastDiv make_fastdiv(uint32_t d) {
    FastDiv f;
    f.d = d;
    if (d <= 1) {
        f.m = 0; f.s1 = 0; f.s2 = 0;
        return f;
    }
    uint32_t l = 0;
    while ((1ull << l) < d) ++l;
    f.m = (uint32_t)(((1ull << 32) * ((1ull << l) - d)) / d + 1);
    f.s1 = 1;
    f.s2 = l - 1;
    return f;
}

__device__ __forceinline__ uint32_t fdiv(uint32_t x, const FastDiv& f) {
    uint32_t t = __umulhi(x, f.m);
    return (t + ((x - t) >> f.s1)) >> f.s2;
}

}  // namespace mi355
