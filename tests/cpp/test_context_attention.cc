// The context layer's fused attention (isp_layers::launch_fused_context_attention) by itself, against a float64
// attention written out in this file: ragged batches with history, contexts cut short, grouped and shared key
// heads, query counts that leave a workgroup's last wavefronts or lanes idle, and key counts that end inside a
// tile.  Everything the kernel must not read holds NaN (rows of padded queries, cache rows past a sequence's
// context), and the output starts as NaN, so a leak or a skipped row shows as NaN.
//
//   test_context_attention            (prints one line per case and "passed" or "FAILED")
#include <cstdio>
#include <limits>
#include <numeric>

#include "src/layers/decoder/context_decoder_layer.h"
#include "test_util.h"

struct Case {
    const char* name;
    int head_size, head_num, kv_head_num, max_q, max_seq;
    std::vector<int> lens, hist, ctx_cut;  // ctx = hist + len - ctx_cut
    int max_k_slack;                       // max_k_len = max(ctx) - slack: a max_k_len that cuts the longest context
};

static void run(const Case& c, std::mt19937& gen) {
    using S = uint16_t;
    const int hs = c.head_size, batch = (int)c.lens.size();
    std::vector<int> ctx(batch);
    int max_k = 1;
    for (int b = 0; b < batch; b++) {
        ctx[b] = c.hist[b] + c.lens[b] - c.ctx_cut[b];
        max_k = std::max(max_k, ctx[b]);
    }
    max_k = std::max(1, max_k - c.max_k_slack);
    const int tokens = std::accumulate(c.lens.begin(), c.lens.end(), 0);
    const S nan16 = 0x7e00;
    std::normal_distribution<float> dist(0.f, 1.f);
    // queries [batch, heads, max_q, hs]; keys, values [batch, kv heads, max_seq, hs]
    std::vector<S> q((size_t)batch * c.head_num * c.max_q * hs, nan16);
    std::vector<S> k((size_t)batch * c.kv_head_num * c.max_seq * hs, nan16), v(k.size(), nan16);
    for (int b = 0; b < batch; b++) {
        for (int h = 0; h < c.head_num; h++)
            for (int s = 0; s < c.lens[b]; s++)
                for (int d = 0; d < hs; d++)
                    q[(((size_t)b * c.head_num + h) * c.max_q + s) * hs + d] = Host<half>::to(2.0f * dist(gen));
        for (int h = 0; h < c.kv_head_num; h++)
            for (int s = 0; s < std::min(ctx[b], max_k); s++)
                for (int d = 0; d < hs; d++) {
                    const size_t at = (((size_t)b * c.kv_head_num + h) * c.max_seq + s) * hs + d;
                    k[at] = Host<half>::to(2.0f * dist(gen));
                    v[at] = Host<half>::to(dist(gen));
                }
    }
    std::vector<S> out((size_t)tokens * c.head_num * hs, nan16);
    S *dq = to_device(q), *dk = to_device(k), *dv = to_device(v), *dout = to_device(out);
    int *dh = to_device(c.hist), *dl = to_device(c.lens), *dc = to_device(ctx);
    const float scale = 1.0f / std::sqrt((float)hs);
    isp_layers::launch_fused_context_attention((const half*)dq, (const half*)dk, (const half*)dv, (half*)dout, dh, dl, dc,
                                               batch, c.head_num, c.kv_head_num, hs, c.max_q, max_k, c.max_seq, tokens, scale);
    CHECK(hipDeviceSynchronize());
    auto got = to_host(dout, out.size());

    double worst = 0, peak = 0;
    long long not_finite = 0;
    int first = 0;
    const int group = c.head_num / c.kv_head_num;
    std::vector<double> p, o(hs);
    for (int b = 0; b < batch; b++) {
        for (int s = 0; s < c.lens[b]; s++)
            for (int h = 0; h < c.head_num; h++) {
                const int visible = std::min(std::min(c.hist[b] + s + 1, ctx[b]), max_k);
                const S* qr = &q[(((size_t)b * c.head_num + h) * c.max_q + s) * hs];
                const size_t kv0 = ((size_t)b * c.kv_head_num + h / group) * c.max_seq * hs;
                p.assign(std::max(visible, 0), 0.0);
                double m = -1e300, sum = 0;
                for (int j = 0; j < visible; j++) {
                    double dot = 0;
                    for (int d = 0; d < hs; d++) dot += (double)Host<half>::from(qr[d]) * Host<half>::from(k[kv0 + (size_t)j * hs + d]);
                    p[j] = dot * scale;
                    m = std::max(m, p[j]);
                }
                for (int j = 0; j < visible; j++) sum += (p[j] = std::exp(p[j] - m));
                std::fill(o.begin(), o.end(), 0.0);
                for (int j = 0; j < visible; j++)
                    for (int d = 0; d < hs; d++) o[d] += p[j] / sum * Host<half>::from(v[kv0 + (size_t)j * hs + d]);
                const S* gr = &got[((size_t)(first + s) * c.head_num + h) * hs];
                for (int d = 0; d < hs; d++) {
                    const double g = Host<half>::from(gr[d]);
                    if (!std::isfinite(g)) not_finite++;
                    else worst = std::max(worst, std::fabs(g - o[d]));
                    peak = std::max(peak, std::fabs(o[d]));
                }
            }
        first += c.lens[b];
    }
    // probabilities are rounded to fp16 before the second product (relative 2^-11 each, averaging out over the
    // keys) and the result once more: 2e-3 of the largest output is several times that
    EXPECT(not_finite == 0, "%s: %lld outputs are NaN or infinite (a row skipped, or unwritten memory read)", c.name, not_finite);
    EXPECT(worst <= 2e-3 * peak, "%s: error %g against a largest output of %g", c.name, worst, peak);
    std::printf("%-44s heads of %3d, %d tokens, max_k %d: error %.2e of peak %.2f\n", c.name, hs, tokens, max_k, worst, peak);
    for (void* ptr : {(void*)dq, (void*)dk, (void*)dv, (void*)dout, (void*)dh, (void*)dl, (void*)dc}) CHECK(hipFree(ptr));
}

int main() {
    std::mt19937 gen(20240611);
    const Case cases[] = {
        {"one short sequence", 128, 2, 2, 5, 8, {5}, {0}, {0}, 0},
        {"ragged batch with history, grouped heads", 128, 4, 2, 16, 48, {16, 5, 11}, {0, 9, 30}, {0, 0, 0}, 0},
        {"a context cut short and a max_k_len below it", 128, 4, 4, 16, 48, {16, 7}, {3, 20}, {0, 2}, 1},
        {"two query tiles, the second partly filled", 128, 2, 2, 200, 300, {200, 133}, {0, 70}, {0, 0}, 0},
        {"one key head shared by eight query heads", 128, 8, 1, 130, 130, {129}, {0}, {0}, 0},
        {"a single query over a long history", 128, 4, 2, 1, 1100, {1, 1, 1}, {1000, 63, 64}, {0, 0, 0}, 0},
        {"keys ending exactly at a tile boundary", 128, 2, 1, 64, 128, {64, 64}, {0, 64}, {0, 0}, 0},
        {"an empty sequence inside the batch", 128, 2, 2, 40, 64, {40, 0, 17}, {0, 5, 9}, {0, 0, 0}, 0},
        {"a context of no keys (rows of zeros)", 128, 2, 2, 8, 16, {5, 8}, {0, 0}, {5, 0}, 0},
    };
    try {
        if (!isp_layers::fused_context_attention_supports(128, 32, 8) || !isp_layers::fused_context_attention_supports(64, 32, 8) ||
            isp_layers::fused_context_attention_supports(96, 32, 8) || isp_layers::fused_context_attention_supports(128, 32, 5)) {
            std::printf("FAIL: fused_context_attention_supports\n");
            g_failures++;
        }
        for (const Case& c : cases) {
            run(c, gen);
            Case narrow = c;  // the same case on 64-element heads
            narrow.head_size = 64;
            run(narrow, gen);
        }
    } catch (const std::exception& e) {
        std::printf("exception: %s\n", e.what());
        return 1;
    }
    std::printf("context attention: %s\n", g_failures ? "FAILED" : "passed");
    return g_failures != 0;
}
