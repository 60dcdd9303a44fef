// The C++ host layer on the device: a small decoder with device-generated weights (seeded, so any other caller of
// the library can build the identical model), generate and the continuous-batching scheduler.  Prints one JSON
// object; the Python test that runs this program builds the same model through its own bindings and compares.
#include <cstdio>
#include <map>
#include <memory>

#include "fandhe_rocm_bench.h"
#include "fandhe_safetensors.hpp"

using namespace fandhe;

static void print_rows(const char *key, const std::vector<std::vector<int32_t>> &rows, bool last = false) {
    std::printf("\"%s\": [", key);
    for (size_t r = 0; r < rows.size(); ++r) {
        std::printf("[");
        for (size_t i = 0; i < rows[r].size(); ++i) std::printf("%s%d", i ? ", " : "", rows[r][i]);
        std::printf("]%s", r + 1 < rows.size() ? ", " : "");
    }
    std::printf("]%s\n", last ? "" : ",");
}

// host_gpu_test <checkpoint> <n_layers> <n_heads> <n_kv_heads>: a resident decoder straight from a Llama-style
// safetensors file, then greedy and top-k generation from two fixed prompts.
static int from_checkpoint(int argc, char **argv) {
    if (argc != 5) {
        std::fprintf(stderr, "usage: host_gpu_test [checkpoint n_layers n_heads n_kv_heads]\n");
        return 2;
    }
    Context ctx(0);
    const std::vector<uint8_t> file = st::read_file(argv[1]);
    st::LoadedDecoder m = st::load_decoder(ctx, file.data(), file.size(), (uint32_t)std::atoi(argv[2]), (uint32_t)std::atoi(argv[3]),
                                           (uint32_t)std::atoi(argv[4]), /*max_blocks_per_seq=*/4, /*num_blocks=*/16, /*max_batch=*/4,
                                           128, 16, 1e-5f, 10000.0);
    const std::vector<std::vector<int32_t>> prompts{{3, 1, 4, 1, 5}, {2, 7, 1, 8, 2}};
    std::printf("{\n");
    print_rows("checkpoint_greedy", generate(*m.decoder, prompts, GenerateConfig(20, SamplingStrategy::Greedy())));
    print_rows("checkpoint_top_k", generate(*m.decoder, {prompts[0]}, GenerateConfig(20, SamplingStrategy::TopK(8)).with_seed(21)), true);
    std::printf("}\n");
    return 0;
}

int main(int argc, char **argv) {
    try {
        if (Context::device_count() < 1) {
            std::fprintf(stderr, "host_gpu_test: no gfx950 device\n");
            return 2;
        }
        if (argc > 1) return from_checkpoint(argc, argv);
        Context ctx(0);
        RocmBackendOps ops(ctx);
        fa_decoder_config cfg{};
        cfg.n_layers = 2, cfg.d_model = 256, cfg.n_heads = 4, cfg.n_kv_heads = 2, cfg.head_dim = 128, cfg.d_ffn = 512, cfg.vocab = 1000;
        cfg.block_size = 16, cfg.max_blocks_per_seq = 8, cfg.num_blocks = 48, cfg.max_batch = 8;
        cfg.rms_eps = 1e-5f, cfg.rope_theta = 10000.0;
        const uint64_t D = cfg.d_model, EQ = (uint64_t)cfg.n_heads * cfg.head_dim, EKV = (uint64_t)cfg.n_kv_heads * cfg.head_dim;
        uint64_t seed = 100;
        std::vector<std::unique_ptr<Buffer>> keep;
        std::vector<std::unique_ptr<QWeight>> qkeep;
        auto filled = [&](uint64_t numel, float mean, float std) -> const Buffer & {
            keep.push_back(std::make_unique<Buffer>(Buffer::alloc_uninit(ctx, FA_F32, numel)));
            check(fa_fill_normal(ctx.handle(), keep.back()->handle(), 0, numel, seed++, mean, std));
            return *keep.back();
        };
        auto weight = [&](uint64_t k, uint64_t n) -> const QWeight & {
            const Buffer &w = filled(k * n, 0.0f, 0.05f);
            qkeep.push_back(std::make_unique<QWeight>(QWeight::from_f32(ctx, BufferView{&w, 0}, k, n)));
            return *qkeep.back();
        };
        struct LayerRefs {
            const Buffer *an, *fn;
            const QWeight *wqkv, *wo, *wgu, *wdown;
        };
        std::vector<LayerRefs> layers;
        for (uint32_t l = 0; l < cfg.n_layers; ++l) {
            const Buffer &an = filled(D, 1.0f, 0.1f), &fn = filled(D, 1.0f, 0.1f);
            const QWeight &wqkv = weight(D, EQ + 2 * EKV), &wo = weight(EQ, D), &wgu = weight(D, 2 * (uint64_t)cfg.d_ffn),
                          &wdown = weight(cfg.d_ffn, D);
            layers.push_back({&an, &fn, &wqkv, &wo, &wgu, &wdown});
        }
        const Buffer &embed = filled((uint64_t)cfg.vocab * D, 0.0f, 1.0f), &final_norm = filled(D, 1.0f, 0.1f);
        const QWeight &lm_head = weight(D, cfg.vocab);
        auto wire = [&](Decoder &d) {                             // weights are borrowed: two decoders can share them
            for (uint32_t l = 0; l < cfg.n_layers; ++l)
                d.set_layer(l, *layers[l].an, *layers[l].fn, *layers[l].wqkv, *layers[l].wo, *layers[l].wgu, *layers[l].wdown);
            d.set_head(embed, final_norm, lm_head);
        };
        Decoder dec(ctx, cfg), draft(ctx, cfg);
        wire(dec);
        wire(draft);

        std::printf("{\n");
        // f32 GEMM against the host loop of the reference (k ascending, one fused multiply-add per term)
        {
            const uint64_t m = 5, k = 37, n = 9;
            std::vector<float> a(m * k), b(k * n);
            for (size_t i = 0; i < a.size(); ++i) a[i] = (float)((int)(i * 7 % 13) - 6) * 0.125f;
            for (size_t i = 0; i < b.size(); ++i) b[i] = (float)((int)(i * 5 % 11) - 5) * 0.25f;
            Buffer da = Buffer::upload(ctx, a), db = Buffer::upload(ctx, b);
            const std::vector<float> got = ops.gemm_device(da, db, m, n, k).download<float>();
            bool same = true;
            for (uint64_t i = 0; i < m; ++i)
                for (uint64_t j = 0; j < n; ++j) {
                    float acc = 0.0f;
                    for (uint64_t p = 0; p < k; ++p) acc = std::fma(a[i * k + p], b[p * n + j], acc);
                    same = same && acc == got[i * n + j];
                }
            std::printf("\"gemm_device_bit_exact\": %s,\n", same ? "true" : "false");
        }
        const std::vector<std::vector<int32_t>> prompts{{5, 17, 900, 3, 44}, {1, 2, 3, 4, 5}};
        print_rows("generate_greedy", generate(dec, prompts, GenerateConfig(12, SamplingStrategy::Greedy())));
        print_rows("generate_top_k", generate(dec, {{8, 9, 10}}, GenerateConfig(14, SamplingStrategy::TopK(5)).with_seed(7)));
        print_rows("generate_temperature", generate(dec, prompts, GenerateConfig(10, SamplingStrategy::Temperature(0.8f)).with_seed(3)));

        BatchScheduler<Decoder> sched(dec, SchedulerLimits(3, 16, 40));
        const std::vector<std::pair<std::vector<int32_t>, GenerateConfig>> requests{
            {{5, 17, 900, 3, 44}, GenerateConfig(12, SamplingStrategy::Greedy())},
            {{11, 12}, GenerateConfig(20, SamplingStrategy::TopK(5)).with_seed(7)},
            {{21, 22, 23, 24, 25, 26, 27}, GenerateConfig(16, SamplingStrategy::Temperature(0.8f)).with_seed(3)},
            {{31}, GenerateConfig(9, SamplingStrategy::Greedy())},
            {{41, 42, 43}, GenerateConfig(3, SamplingStrategy::Greedy())},
            {{51, 52, 53, 54}, GenerateConfig(25, SamplingStrategy::Temperature(1.3f)).with_seed(11)},
            {{61, 62}, GenerateConfig(30, SamplingStrategy::TopK(50)).with_seed(13)},
        };
        for (const auto &r : requests) sched.submit(r.first, r.second);
        std::map<uint64_t, std::vector<int32_t>> done;
        for (int it = 0; it < 200 && (sched.queued_len() || sched.active_len()); ++it) {
            sched.step();
            for (auto &f : sched.take_finished()) done[f.first] = f.second;
        }
        const bool clean = sched.take_failed().empty() && sched.queued_len() == 0 && sched.active_len() == 0 &&
                           sched.free_pages() == cfg.num_blocks && done.size() == requests.size();
        std::vector<std::vector<int32_t>> rows;
        for (auto &kv : done) rows.push_back(kv.second);
        print_rows("scheduler", rows);
        std::printf("\"scheduler_prompt_passes\": %llu, \"scheduler_decode_steps\": %llu,\n",
                    (unsigned long long)sched.stats().prompt_passes, (unsigned long long)sched.stats().decode_steps);
        // a request that runs alone equals generate of the same request
        BatchScheduler<Decoder> solo(dec, SchedulerLimits(1, 4, 40));
        solo.submit(requests[1].first, requests[1].second);
        std::vector<std::vector<int32_t>> alone;
        for (int it = 0; it < 100 && (solo.queued_len() || solo.active_len()); ++it) {
            solo.step();
            for (auto &f : solo.take_finished()) alone.push_back(f.second);
        }
        print_rows("scheduler_alone", alone);
        print_rows("generate_same_request", generate(dec, {requests[1].first}, requests[1].second));
        // speculative decoding with a draft that is the target itself: every draft is accepted, in both verification forms
        for (uint64_t k : {4, 9}) {
            const SpeculativeOutput so = generate_speculative(dec, draft, prompts[0], GenerateConfig(24, SamplingStrategy::Greedy()), k);
            std::printf("\"speculative_k%llu\": {\"tokens\": [", (unsigned long long)k);
            for (size_t i = 0; i < so.tokens.size(); ++i) std::printf("%s%d", i ? ", " : "", so.tokens[i]);
            std::printf("], \"rounds\": %llu, \"accepted\": %llu},\n", (unsigned long long)so.rounds, (unsigned long long)so.accepted);
        }
        print_rows("generate_greedy_24", generate(dec, {prompts[0]}, GenerateConfig(24, SamplingStrategy::Greedy())));
        // the sampled form (acceptance on the device), in both verification forms, temperature and top-k
        {
            const std::pair<const char *, GenerateConfig> sampled[] = {
                {"speculative_temperature", GenerateConfig(28, SamplingStrategy::Temperature(0.8f)).with_seed(11)},
                {"speculative_top_k", GenerateConfig(28, SamplingStrategy::TopK(5)).with_seed(7)}};
            for (const auto &sc : sampled)
                for (uint64_t k : {3, 9}) {
                    const SpeculativeOutput so = generate_speculative(dec, draft, prompts[1], sc.second, k);
                    std::printf("\"%s_k%llu\": {\"tokens\": [", sc.first, (unsigned long long)k);
                    for (size_t i = 0; i < so.tokens.size(); ++i) std::printf("%s%d", i ? ", " : "", so.tokens[i]);
                    std::printf("], \"rounds\": %llu, \"accepted\": %llu},\n", (unsigned long long)so.rounds, (unsigned long long)so.accepted);
                }
        }
        // the one-layer cache: two appends, then the last token of every row attends to its five positions
        {
            const uint64_t bs = 4, e = 8, heads = 2, dh = 4, b = 2;
            PagedKvCache cache(ctx, bs, 8, e, FA_F32);
            std::vector<float> k_all, v_all, q(b * e);
            for (size_t i = 0; i < q.size(); ++i) q[i] = 0.25f * (float)((int)(i * 3 % 7) - 3);
            auto chunk = [&](uint64_t l_new, uint64_t t0, std::vector<float> &all, float mul) {
                std::vector<float> x(b * l_new * e);
                for (uint64_t r = 0; r < b; ++r)
                    for (uint64_t t = 0; t < l_new; ++t)
                        for (uint64_t d = 0; d < e; ++d) x[(r * l_new + t) * e + d] = mul * (float)((int)((r * 31 + (t0 + t) * 7 + d * 3) % 11) - 5);
                all.insert(all.end(), x.begin(), x.end());
                return Buffer::upload(ctx, x);
            };
            std::vector<float> k1, v1, k2, v2;
            cache.append(chunk(3, 0, k1, 0.125f), chunk(3, 0, v1, 0.5f), b, 3);
            cache.append(chunk(2, 3, k2, 0.125f), chunk(2, 3, v2, 0.5f), b, 2);
            auto at = [&](const std::vector<float> &c1, const std::vector<float> &c2, uint64_t r, uint64_t t, uint64_t d) {
                return t < 3 ? c1[(r * 3 + t) * e + d] : c2[(r * 2 + (t - 3)) * e + d];
            };
            const std::vector<float> got = cache.attention(Buffer::upload(ctx, q), b, 1, heads, 0, 0.5f).download<float>();
            double worst = 0.0;
            for (uint64_t r = 0; r < b; ++r)
                for (uint64_t h = 0; h < heads; ++h) {
                    double sc[5], mx = -1e30, den = 0.0;
                    for (uint64_t t = 0; t < 5; ++t) {
                        double s = 0.0;
                        for (uint64_t d = 0; d < dh; ++d) s += (double)q[r * e + h * dh + d] * at(k1, k2, r, t, h * dh + d);
                        sc[t] = s * 0.5;
                        mx = std::max(mx, sc[t]);
                    }
                    for (uint64_t t = 0; t < 5; ++t) den += (sc[t] = std::exp(sc[t] - mx));
                    for (uint64_t d = 0; d < dh; ++d) {
                        double o = 0.0;
                        for (uint64_t t = 0; t < 5; ++t) o += sc[t] / den * at(v1, v2, r, t, h * dh + d);
                        worst = std::max(worst, std::fabs(o - (double)got[r * e + h * dh + d]));
                    }
                }
            cache.rewind_to(2);
            const bool state_ok = cache.seq_len() == 2 && cache.num_free_blocks() == 8 - 2 && !cache.is_poisoned();
            std::printf("\"paged_cache_max_abs_err\": %.3e, \"paged_cache_state_ok\": %s,\n", worst, state_ok ? "true" : "false");
        }
        // error behaviour of the boundary reaches the caller as BackendError with the status of the call
        bool rejected = false;
        try {
            dec.set_sequences(std::vector<uint32_t>(cfg.max_blocks_per_seq, 4000), {3});      // page id outside the pool
        } catch (const BackendError &e) {
            rejected = e.status == FA_ERR_INVALID_ARGUMENT;
        }
        std::printf("\"bad_table_rejected\": %s,\n\"scheduler_clean\": %s\n}\n", rejected ? "true" : "false", clean ? "true" : "false");
    } catch (const std::exception &e) {
        std::fprintf(stderr, "host_gpu_test: %s\n", e.what());
        return 1;
    }
    return 0;
}
