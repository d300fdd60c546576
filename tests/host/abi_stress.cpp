// Host-side stress of the C ABI without a GPU: many threads walk random descriptors (valid and invalid) through the
// calls an inference loop makes before a launch -- deduce, query, algorithm and tile usability, pre-processed sizes, the
// epilogue proofs -- and every answer must equal the one a single thread computed first.  Built and run under the host
// sanitizers (make -C tests/host sanitize / tsan): the proof caches, the per-thread descriptor memo and the error
// text are the library's only mutable host state.
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <random>
#include <thread>
#include <vector>

#include "../../include/mi355_convbias.h"

namespace {

struct Answer {
    int st_deduce, st_query, st_pre;
    uint32_t oh, ow;
    mi355_algo algo;
    size_t ws, pre_bytes;
    uint32_t usable_algos, usable_tiles_lo;
    bool operator==(const Answer& o) const {
        return st_deduce == o.st_deduce && st_query == o.st_query && st_pre == o.st_pre && oh == o.oh && ow == o.ow &&
               algo.id == o.algo.id && algo.tile_cfg == o.algo.tile_cfg && algo.reserved == o.algo.reserved && ws == o.ws &&
               pre_bytes == o.pre_bytes && usable_algos == o.usable_algos && usable_tiles_lo == o.usable_tiles_lo;
    }
};

mi355_conv_desc random_desc(std::mt19937& rng, const std::vector<float>& scales) {
    static const uint32_t fmts[] = {MI355_FMT_NCHW, MI355_FMT_NCHW4, MI355_FMT_NCHW32, MI355_FMT_NCHW4_NCHW32,
                                    MI355_FMT_NCHW32_NCHW4, MI355_FMT_NCHW4_NCHW, MI355_FMT_NCHW44, 2 /* no such format */};
    auto pick = [&](uint32_t n) { return (uint32_t)(rng() % n); };
    mi355_conv_desc d;
    memset(&d, 0, sizeof(d));
    d.format = fmts[pick(8)];
    d.nonline = pick(4);                       // incl. SIGMOID, which is refused
    d.mode = pick(8) == 0 ? 1 : 0;
    d.n = 1 + pick(64);
    const uint32_t ch[] = {4, 8, 32, 64, 96, 128, 256, 512, 1024, 30};
    d.ic = ch[pick(10)];
    d.oc = ch[pick(10)];
    d.ih = 1 + pick(57);
    d.iw = 1 + pick(57);
    d.fh = d.fw = 1 + 2 * pick(3);
    if (pick(10) == 0) d.fw = 1 + pick(4);
    d.group = pick(6) == 0 ? (pick(2) ? 2 : d.ic) : 1;
    if (pick(40) == 0) d.group = 0;            // invalid
    d.sparse = d.group > 1 ? MI355_SPARSE_GROUP : MI355_SPARSE_DENSE;
    d.pad_h = d.pad_w = pick(3);
    d.stride_h = d.stride_w = 1 + pick(2);
    d.dilate_h = d.dilate_w = pick(12) == 0 ? 2 : 1;
    d.dst_dtype = pick(8) == 0 ? MI355_DT_QS32 : pick(16) == 0 ? MI355_DT_F32 : MI355_DT_QS8;
    d.bias_mode = pick(8) == 0 ? MI355_BIAS_FULL : pick(8) == 0 ? MI355_BIAS_NONE : MI355_BIAS_BROADCAST_CHANNEL;
    d.has_z = pick(3) == 0;
    d.scale_bias = scales[pick((uint32_t)scales.size())] * scales[pick((uint32_t)scales.size())];
    d.scale_z = scales[pick((uint32_t)scales.size())];
    d.scale_dst = scales[pick((uint32_t)scales.size())];
    if (pick(50) == 0) d.scale_dst = 0.f;      // invalid for a QuantizedS8 dst
    return d;
}

Answer ask(const mi355_conv_desc& d) {
    Answer a;
    memset(&a, 0, sizeof(a));
    a.st_deduce = mi355_convbias_deduce_out(&d, &a.oh, &a.ow);
    a.st_query = mi355_convbias_s8_query(&d, MI355_ALGO_HEURISTIC_PREPROCESS, &a.algo, &a.ws);
    if (a.st_query == MI355_OK) {
        a.st_pre = mi355_convbias_s8_preprocess_size(&d, &a.algo, &a.pre_bytes);
        for (int id = 0; id < mi355_convbias_algo_count(); ++id)
            if (mi355_convbias_algo_usable(&d, id) == 1) a.usable_algos |= 1u << id;
        const int tiles = mi355_igemm_tile_count();
        for (int t = 0; t < tiles && t < 32; ++t)
            if (mi355_igemm_tile_usable(&d, t) == 1) a.usable_tiles_lo |= 1u << t;
    } else {
        // a refused descriptor leaves a message for this thread
        const char* m = mi355_last_error();
        if (!m || !*m) a.st_pre = -1000;
    }
    return a;
}

}  // namespace

int main(int argc, char** argv) {
    const int threads = argc > 1 ? atoi(argv[1]) : 8;
    const int count = argc > 2 ? atoi(argv[2]) : 1500;
    std::mt19937 rng(20240607);
    std::vector<float> scales;
    for (int i = 0; i < 300; ++i) scales.push_back(1e-3f * (1.f + (float)(rng() % 50000) / 1000.f));
    std::vector<mi355_conv_desc> descs;
    for (int i = 0; i < count; ++i) descs.push_back(random_desc(rng, scales));

    // half of the reference answers are computed up front by one thread (the other threads then find the caches warm for
    // those), the other half by whichever thread gets there first
    std::vector<Answer> want(count);
    std::vector<std::atomic<int>> have(count);
    int ok = 0, refused = 0;
    for (int i = 0; i < count; i += 2) {
        want[i] = ask(descs[i]);
        have[i].store(2);
        (want[i].st_query == MI355_OK ? ok : refused)++;
    }
    for (int i = 1; i < count; i += 2) have[i].store(0);
    printf("abi_stress: %d descriptors (%d of the first half accepted, %d refused), %d threads\n", count, ok, refused, threads);
    if (ok < count / 8 || refused < count / 40) {
        printf("the descriptor generator does not exercise both outcomes\n");
        return 1;
    }

    std::atomic<int> bad{0};
    std::vector<std::thread> pool;
    for (int t = 0; t < threads; ++t)
        pool.emplace_back([&, t] {
            std::mt19937 r(1000 + t);
            for (int it = 0; it < 3 * count; ++it) {
                const int i = (int)(r() % (uint32_t)count);
                const Answer a = ask(descs[i]);
                int expect = 0;
                if (have[i].load(std::memory_order_acquire) == 2) {
                    if (!(a == want[i])) bad.fetch_add(1);
                } else if (have[i].compare_exchange_strong(expect, 1)) {
                    want[i] = a;
                    have[i].store(2, std::memory_order_release);
                }
                // the proofs directly, on scales that other threads prove at the same time
                float y = 0.f, c = 0.f, dd = 0.f;
                const float s = scales[r() % scales.size()];
                float y2;
                (void)mi355_epilogue_quotient_form(s, &y, &y2);
                (void)mi355_epilogue_linear_form(s * 1e-2f, s, MI355_NL_RELU, &c, &dd);
                // the residual table form on a few triples that several threads ask for at once: equal answers
                if (r() % 16 == 0) {
                    float tc = 0.f, tab[256];
                    const float sd = scales[r() % 4];
                    const int ok = mi355_epilogue_residual_table(sd * 0.028f, sd * 0.7f, sd, MI355_NL_RELU, &tc, tab);
                    float tc2 = 0.f, tab2[256];
                    const int ok2 = mi355_epilogue_residual_table(sd * 0.028f, sd * 0.7f, sd, MI355_NL_RELU, &tc2, tab2);
                    if (ok != ok2 || (ok == 1 && (tc != tc2 || memcmp(tab, tab2, sizeof(tab)) != 0))) bad.fetch_add(1);
                }
            }
        });
    for (auto& th : pool) th.join();
    if (bad.load()) {
        printf("%d answers differed between threads\n", bad.load());
        return 1;
    }
    printf("ALL OK\n");
    return 0;
}
