// Host logic of fandhe_rocm.hpp without a device: page allocation order, configuration checks, generate and the
// continuous-batching scheduler over a toy decoder whose next token depends only on a row's own history, so every
// request must come out exactly as if it had run alone, whatever rows it shared steps with.
#include <cstdio>
#include <map>

#include "fandhe_rocm.hpp"

using namespace fandhe;

static int g_checks = 0;
#define CHECK(cond)                                                                    \
    do {                                                                               \
        ++g_checks;                                                                    \
        if (!(cond)) {                                                                 \
            std::fprintf(stderr, "%s:%d: check failed: %s\n", __FILE__, __LINE__, #cond); \
            return 1;                                                                  \
        }                                                                              \
    } while (0)
template <typename F> static bool throws_invalid(F f) {
    try {
        f();
    } catch (const InvalidArgument &) {
        return true;
    }
    return false;
}

struct ToyConfig {
    uint32_t vocab, block_size, max_blocks_per_seq, num_blocks, max_batch;
};

static uint64_t xorshift_star(uint64_t &s) {
    s ^= s >> 12;
    s ^= s << 25;
    s ^= s >> 27;
    return s * 0x2545F4914F6CDD1DULL;
}
// next token of a row: greedy rows follow their last token and length, the others draw once
static int32_t toy_next(int32_t last, uint32_t len, fa_row_sampling &p, uint32_t vocab, int32_t poison) {
    if (last == poison) return -1;                               // "non-finite logits"
    if (p.strategy == FA_SAMPLE_GREEDY) return (int32_t)(((uint64_t)last * 31 + (uint64_t)len * 7 + 3) % vocab);
    const uint64_t r = xorshift_star(p.rng_state);
    const uint32_t span = p.strategy == FA_SAMPLE_TOP_K ? p.top_k : vocab;
    return (int32_t)((r >> 33) % span);
}

class ToyDecoder {
  public:
    explicit ToyDecoder(ToyConfig c, int32_t poison = -2) : cfg_(c), poison_(poison) {}
    const ToyConfig &config() const { return cfg_; }
    void set_sequences(const std::vector<uint32_t> &tables, const std::vector<uint32_t> &lens) {
        if (lens.size() > cfg_.max_batch || tables.size() != lens.size() * cfg_.max_blocks_per_seq)
            throw BackendError(FA_ERR_INVALID_ARGUMENT, "toy: bad tables");
        std::set<uint32_t> used;
        for (uint32_t id : tables) {
            if (id == UINT32_MAX) continue;
            if (id >= cfg_.num_blocks || !used.insert(id).second) throw BackendError(FA_ERR_INVALID_ARGUMENT, "toy: page shared or outside the pool");
        }
        tables_ = tables;
        lens_ = lens;
        tokens_.assign(lens.size(), 0);
        policy_.assign(lens.size(), fa_row_sampling{1, 1.0f, 0, FA_SAMPLE_GREEDY, 0});
        shared_ = false;
    }
    void set_tokens(const std::vector<int32_t> &t) { tokens_ = t; }
    void set_sampling(fa_sampling s, float t, uint64_t k, uint64_t seed) {
        fa_row_sampling p{0, t, (uint32_t)k, (int32_t)s, 0};
        fa_rng_state_from_seed(seed, &p.rng_state);
        policy_.assign(lens_.size(), p);
        shared_ = true;                                          // one generator, rows draw in row order
    }
    void set_row_sampling(const std::vector<fa_row_sampling> &rows) {
        policy_ = rows;
        shared_ = false;
    }
    std::vector<fa_row_sampling> read_row_sampling() const { return policy_; }
    void prefill(const std::vector<int32_t> &tokens, uint32_t l_new) {
        std::vector<std::vector<int32_t>> prompts;
        for (size_t b = 0; b < lens_.size(); ++b) prompts.emplace_back(tokens.begin() + b * l_new, tokens.begin() + (b + 1) * l_new);
        prefill_padded(prompts);
    }
    void prefill_padded(const std::vector<std::vector<int32_t>> &prompts) {
        for (size_t b = 0; b < lens_.size(); ++b) {
            lens_[b] += (uint32_t)prompts[b].size();
            room(b);
            tokens_[b] = pick(b, prompts[b].back());
        }
    }
    void step() {
        for (size_t b = 0; b < lens_.size(); ++b) {
            lens_[b] += 1;
            room(b);
            tokens_[b] = pick(b, tokens_[b]);
        }
    }
    std::vector<int32_t> tokens() const { return tokens_; }

  private:
    void room(size_t b) const {
        const uint32_t need = (lens_[b] + cfg_.block_size - 1) / cfg_.block_size;
        for (uint32_t p = 0; p < need; ++p)
            if (p >= cfg_.max_blocks_per_seq || tables_[b * cfg_.max_blocks_per_seq + p] == UINT32_MAX)
                throw BackendError(FA_ERR_INVALID_ARGUMENT, "toy: a position without a page");
    }
    int32_t pick(size_t b, int32_t last) {
        fa_row_sampling &p = shared_ ? policy_[0] : policy_[b];
        fa_row_sampling mine = policy_[b];
        mine.rng_state = p.rng_state;
        const int32_t t = toy_next(last, lens_[b], mine, cfg_.vocab, poison_);
        p.rng_state = mine.rng_state;
        return t;
    }
    ToyConfig cfg_;
    int32_t poison_;
    std::vector<uint32_t> tables_, lens_;
    std::vector<int32_t> tokens_;
    std::vector<fa_row_sampling> policy_;
    bool shared_ = false;
};

// what a request produces when it runs alone
static std::vector<int32_t> alone(const std::vector<int32_t> &prompt, const GenerateConfig &c, uint32_t vocab) {
    fa_row_sampling p{0, c.temperature, (uint32_t)c.top_k.value_or(0), (int32_t)c.strategy.kind, 0};
    fa_rng_state_from_seed(c.seed, &p.rng_state);
    std::vector<int32_t> t = prompt;
    while (t.size() < c.max_length) t.push_back(toy_next(t.back(), (uint32_t)t.size(), p, vocab, -2));
    return t;
}

int main() {
    // ---- page allocation order: fresh ids ascending, returned ids last in first out
    {
        PageAllocator a(6);
        CHECK((a.take(3) == std::vector<uint32_t>{0, 1, 2}));
        a.give_back({1, 2});
        CHECK(a.free_pages() == 5);
        CHECK((a.take(3) == std::vector<uint32_t>{2, 1, 3}));
        CHECK(throws_invalid([&] { a.take(4); }));
        CHECK(a.free_pages() == 2);
    }
    // ---- configuration checks
    {
        GenerateConfig(8, SamplingStrategy::Greedy()).validate();
        GenerateConfig(8, SamplingStrategy::TopK(3)).validate();
        GenerateConfig(8, SamplingStrategy::Temperature(0.7f)).with_seed(9).validate();
        CHECK(throws_invalid([] { GenerateConfig(8, SamplingStrategy::Greedy()).with_temperature(0.5f).validate(); }));
        CHECK(throws_invalid([] { GenerateConfig(8, SamplingStrategy::TopK(0)).validate(); }));
        CHECK(throws_invalid([] { GenerateConfig(8, SamplingStrategy::Temperature(0.0f)).validate(); }));
        CHECK(throws_invalid([] { GenerateConfig(8, SamplingStrategy::Temperature(NAN)).validate(); }));
        CHECK(throws_invalid([] { GenerateConfig(8, SamplingStrategy::Temperature(0.7f)).with_temperature(0.8f).validate(); }));
        CHECK(throws_invalid([] {
            GenerateConfig c(8, SamplingStrategy::TopK(3));
            c.top_k = 4;
            c.validate();
        }));
        CHECK(throws_invalid([] { GenerateConfig(8, SamplingStrategy::TopK(12)).validate_top_k_le_vocab(11); }));
        CHECK(throws_invalid([] { SchedulerLimits(0, 1, 1); }));
        CHECK(throws_invalid([] { SchedulerLimits(1, 0, 1); }));
        CHECK(throws_invalid([] { SchedulerLimits(1, 1, 0); }));
    }
    // ---- block table: slots follow the pages, rewinding returns pages, the last returned page is reused first
    {
        BlockTable bt(/*max_blocks=*/6, /*block_size=*/4);
        const std::vector<uint32_t> slots = bt.extend_for_append(2, 5);
        CHECK(slots.size() == 10 && std::set<uint32_t>(slots.begin(), slots.end()).size() == 10);
        CHECK(bt.seq_len() == 5 && bt.state().used_blocks == 4 && bt.free_blocks() == 2);
        const std::vector<uint32_t> tables = bt.flatten_tables(3);
        CHECK(tables.size() == 6 && tables[2] == UINT32_MAX && tables[5] == UINT32_MAX);
        for (uint32_t r = 0; r < 2; ++r)
            for (uint32_t t = 0; t < 5; ++t) CHECK(slots[r * 5 + t] == tables[r * 3 + t / 4] * 4 + t % 4);
        BlockTable saved(bt);                                    // a copy is a snapshot
        bool refused = false;
        try {
            bt.extend_for_append(2, 8);                          // 13 positions need 4 pages a row, 8 > 6
        } catch (const BackendError &) {
            refused = true;
        }
        CHECK(refused && bt.seq_len() == 5 && bt.free_blocks() == 2);
        bt.rewind_to(4);
        CHECK(bt.seq_len() == 4 && bt.free_blocks() == 4);
        const uint32_t dropped_last = tables[1 * 3 + 1];         // row 1 gave its second page back last
        CHECK(bt.alloc().value() == dropped_last);
        refused = false;
        try {
            bt.rewind_to(9);
        } catch (const BackendError &) {
            refused = true;
        }
        CHECK(refused);
        CHECK(saved.seq_len() == 5 && saved.free_blocks() == 2);
    }
    const ToyConfig tc{97, 4, 16, 40, 4};
    // ---- generate: rows of a batch share one generator and draw in row order
    {
        ToyDecoder d(tc);
        const std::vector<std::vector<int32_t>> prompts{{5, 6, 7}, {1, 2, 3}, {9, 9, 9}};
        auto out = generate(d, prompts, GenerateConfig(9, SamplingStrategy::Greedy()));
        for (size_t r = 0; r < prompts.size(); ++r) CHECK(out[r] == alone(prompts[r], GenerateConfig(9, SamplingStrategy::Greedy()), tc.vocab));
        auto one = generate(d, {{4, 4}}, GenerateConfig(12, SamplingStrategy::Temperature(0.9f)).with_seed(5));
        CHECK(one[0] == alone({4, 4}, GenerateConfig(12, SamplingStrategy::Temperature(0.9f)).with_seed(5), tc.vocab));
        auto same = generate(d, prompts, GenerateConfig(3, SamplingStrategy::Greedy()));          // nothing to generate
        CHECK(same == prompts);
        CHECK(throws_invalid([&] { generate(d, {{1, 2}, {3}}, GenerateConfig(5, SamplingStrategy::Greedy())); }));
        CHECK(throws_invalid([&] { generate(d, {{}}, GenerateConfig(5, SamplingStrategy::Greedy())); }));
        CHECK(throws_invalid([&] { generate(d, {{1, 2, 3}}, GenerateConfig(2, SamplingStrategy::Greedy())); }));
        CHECK(throws_invalid([&] { generate(d, {{1}, {1}, {1}, {1}, {1}}, GenerateConfig(4, SamplingStrategy::Greedy())); }));   // batch 5 > 4
        CHECK(throws_invalid([&] { generate(d, {{1}}, GenerateConfig(200, SamplingStrategy::Greedy())); }));                  // pages per row
        CHECK(throws_invalid([&] { generate(d, {{1}}, GenerateConfig(5, SamplingStrategy::TopK(98))); }));
    }
    // ---- submit: checks in order, scheduler unchanged on error, ids ascending
    {
        ToyDecoder d(tc);
        CHECK(throws_invalid([&] { BatchScheduler<ToyDecoder>(d, SchedulerLimits(5, 2, 30)); }));   // max_active above max_batch
        BatchScheduler<ToyDecoder> s(d, SchedulerLimits(2, 2, 30));
        CHECK(throws_invalid([&] { s.submit({}, GenerateConfig(5, SamplingStrategy::Greedy())); }));
        CHECK(throws_invalid([&] { s.submit({1, 2, 3}, GenerateConfig(2, SamplingStrategy::Greedy())); }));
        CHECK(throws_invalid([&] { s.submit({1}, GenerateConfig(31, SamplingStrategy::Greedy())); }));
        CHECK(throws_invalid([&] { s.submit({1}, GenerateConfig(5, SamplingStrategy::TopK(0))); }));
        CHECK(s.queued_len() == 0);
        CHECK(s.submit({1}, GenerateConfig(5, SamplingStrategy::Greedy())) == 0);
        CHECK(s.submit({2}, GenerateConfig(5, SamplingStrategy::Greedy())) == 1);
        CHECK(throws_invalid([&] { s.submit({3}, GenerateConfig(5, SamplingStrategy::Greedy())); }));   // queue full
        CHECK(s.queued_len() == 2 && s.active_len() == 0 && s.free_pages() == tc.num_blocks);
    }
    // ---- a mixed run: more requests than rows, fewer pages than all of them need at once
    {
        ToyDecoder d(tc);
        BatchScheduler<ToyDecoder> s(d, SchedulerLimits(4, 64, 64));
        std::map<uint64_t, std::vector<int32_t>> want;
        uint64_t rng = 12345, decode_rows = 0, submitted = 0, prompt_only = 0;
        std::map<uint64_t, std::vector<int32_t>> got;
        std::vector<uint64_t> order;
        auto drain = [&] {
            uint64_t last = 0;
            bool first = true;
            for (auto &f : s.take_finished()) {
                if (!first && f.first < last) return false;      // one iteration reports in request order
                first = false;
                last = f.first;
                got[f.first] = f.second;
            }
            return true;
        };
        for (int wave = 0; wave < 4; ++wave) {
            for (int i = 0; i < 5; ++i) {
                const uint32_t plen = 1 + (uint32_t)(xorshift_star(rng) % 23);
                const uint32_t extra = (uint32_t)(xorshift_star(rng) % 30);
                std::vector<int32_t> prompt;
                for (uint32_t j = 0; j < plen; ++j) prompt.push_back((int32_t)(xorshift_star(rng) % tc.vocab));
                const int kind = (int)(xorshift_star(rng) % 3);
                GenerateConfig c(plen + extra, kind == 0 ? SamplingStrategy::Greedy() : kind == 1 ? SamplingStrategy::TopK(7) : SamplingStrategy::Temperature(0.8f));
                c.with_seed(xorshift_star(rng));
                const uint64_t id = s.submit(prompt, c);
                want[id] = alone(prompt, c, tc.vocab);
                decode_rows += extra > 1 ? extra - 1 : 0;
                prompt_only += extra == 0;
                ++submitted;
            }
            for (int it = 0; it < 3; ++it) {
                s.step();
                CHECK(drain());
                CHECK(s.active_len() <= 4);
            }
        }
        for (int it = 0; it < 400 && (s.queued_len() || s.active_len()); ++it) {
            s.step();
            CHECK(drain());
        }
        CHECK(s.queued_len() == 0 && s.active_len() == 0);
        CHECK(s.take_failed().empty());
        CHECK(got.size() == submitted);
        for (auto &kv : want) CHECK(got[kv.first] == kv.second);
        CHECK(s.free_pages() == tc.num_blocks);
        CHECK(s.stats().decode_rows == decode_rows);
        CHECK(s.stats().prompt_passes >= 1 && s.stats().prompt_passes <= submitted - prompt_only);
    }
    // ---- failures stay with their request
    {
        ToyDecoder d(tc, /*poison=*/50);
        BatchScheduler<ToyDecoder> s(d, SchedulerLimits(4, 16, 40));
        const GenerateConfig g(12, SamplingStrategy::Greedy());
        const uint64_t ok0 = s.submit({1, 2, 3}, g);
        const uint64_t bad_tok = s.submit({1, 200, 3}, g);                       // outside the vocabulary
        const uint64_t bad_k = s.submit({1, 2}, GenerateConfig(12, SamplingStrategy::TopK(98)));
        const uint64_t poisoned = s.submit({7, 50}, g);                          // the toy reports token -1 after 50
        const uint64_t ok1 = s.submit({8, 9}, g);
        std::map<uint64_t, std::vector<int32_t>> got;
        std::map<uint64_t, std::string> failed;
        for (int it = 0; it < 100 && (s.queued_len() || s.active_len()); ++it) {
            s.step();
            for (auto &f : s.take_finished()) got[f.first] = f.second;
            for (auto &f : s.take_failed()) failed[f.first] = f.second;
        }
        CHECK(got.count(ok0) && got[ok0] == alone({1, 2, 3}, g, tc.vocab));
        CHECK(got.count(ok1) && got[ok1] == alone({8, 9}, g, tc.vocab));
        CHECK(failed.count(bad_tok) && failed.count(bad_k) && failed.count(poisoned) && failed.size() == 3);
        CHECK(s.free_pages() == tc.num_blocks);
    }
    std::printf("host_cpu_test: %d checks ok\n", g_checks);
    return 0;
}
