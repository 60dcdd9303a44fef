// The C++ host layer on the device: a small decoder with device-generated weights (seeded, so any other caller of
// the library can build the identical model), generate and the continuous-batching scheduler.  Prints one JSON
// object; the Python test that runs this program builds the same model through its own bindings and compares.
#include <cstdio>
#include <map>
#include <memory>

#include "fandhe_rocm.hpp"

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

int main() {
    try {
        if (Context::device_count() < 1) {
            std::fprintf(stderr, "host_gpu_test: no gfx950 device\n");
            return 2;
        }
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
            ops.fill_normal(*keep.back(), seed++, mean, std);
            return *keep.back();
        };
        auto weight = [&](uint64_t k, uint64_t n) -> const QWeight & {
            const Buffer &w = filled(k * n, 0.0f, 0.05f);
            qkeep.push_back(std::make_unique<QWeight>(QWeight::from_f32(ctx, BufferView{&w, 0}, k, n)));
            return *qkeep.back();
        };
        Decoder dec(ctx, cfg);
        for (uint32_t l = 0; l < cfg.n_layers; ++l) {
            const Buffer &an = filled(D, 1.0f, 0.1f), &fn = filled(D, 1.0f, 0.1f);
            const QWeight &wqkv = weight(D, EQ + 2 * EKV), &wo = weight(EQ, D), &wgu = weight(D, 2 * (uint64_t)cfg.d_ffn),
                          &wdown = weight(cfg.d_ffn, D);
            dec.set_layer(l, an, fn, wqkv, wo, wgu, wdown);
        }
        {
            const Buffer &embed = filled((uint64_t)cfg.vocab * D, 0.0f, 1.0f), &norm = filled(D, 1.0f, 0.1f);
            dec.set_head(embed, norm, weight(D, cfg.vocab));
        }

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
