// The C++ safetensors reader (include/fandhe_safetensors.hpp) without a device.  No arguments: format and error
// cases on hand-made files.  With a path: prints every tensor's dtype, shape and the sum / first / last of its
// promoted values as JSON, for the Python test that wrote the file with its own writer.
#include <cinttypes>

#include "fandhe_safetensors.hpp"

using namespace fandhe;
using st::LoadError;

static int g_checks = 0;
#define CHECK(cond)                                                                    \
    do {                                                                               \
        ++g_checks;                                                                    \
        if (!(cond)) {                                                                 \
            std::fprintf(stderr, "%s:%d: check failed: %s\n", __FILE__, __LINE__, #cond); \
            return 1;                                                                  \
        }                                                                              \
    } while (0)

static std::vector<uint8_t> file_of(const std::string &header, const std::vector<uint8_t> &data, int64_t declared = -1) {
    std::vector<uint8_t> f(8);
    const uint64_t n = declared < 0 ? header.size() : (uint64_t)declared;
    for (int i = 0; i < 8; ++i) f[i] = (uint8_t)(n >> (8 * i));
    f.insert(f.end(), header.begin(), header.end());
    f.insert(f.end(), data.begin(), data.end());
    return f;
}
// the kind and (a prefix of) the message of the error a load raises; "" when it succeeds
static std::string error_of(const std::vector<uint8_t> &f, bool typed = true, bool allow_q = false, LoadError::Kind *kind = nullptr) {
    try {
        if (typed)
            st::load_safetensors_typed_from_bytes(f.data(), f.size(), allow_q);
        else
            st::load_safetensors_f32_from_bytes(f.data(), f.size());
    } catch (const LoadError &e) {
        if (kind) *kind = e.kind;
        return e.what();
    }
    return "";
}
static bool starts(const std::string &s, const char *p) { return s.rfind(p, 0) == 0; }

static int summary(const char *path) {
    const std::vector<uint8_t> buf = st::read_file(path);
    const auto typed = st::load_safetensors_typed_from_bytes(buf.data(), buf.size(), true);
    std::printf("{");
    bool first = true;
    for (const auto &kv : typed) {
        const st::TypedTensor &t = kv.second;
        std::printf("%s\n\"%s\": {\"dtype\": \"%s\", \"shape\": [", first ? "" : ",", kv.first.c_str(), t.dtype.c_str());
        first = false;
        for (size_t i = 0; i < t.shape.size(); ++i) std::printf("%s%" PRIu64, i ? ", " : "", t.shape[i]);
        std::printf("], \"nbytes\": %" PRIu64, t.nbytes);
        if (t.dtype != "I8" && t.dtype != "F8_E4M3") {
            const std::vector<float> v = t.to_f32();
            double sum = 0.0;
            for (float x : v) sum += (double)x;
            std::printf(", \"sum\": %.17g", sum);
            if (!v.empty()) std::printf(", \"first\": %.9g, \"last\": %.9g", (double)v.front(), (double)v.back());
        }
        std::printf("}");
    }
    std::printf("\n}\n");
    return 0;
}

int main(int argc, char **argv) {
    if (argc > 1) {
        try {
            return summary(argv[1]);
        } catch (const std::exception &e) {
            std::fprintf(stderr, "host_safetensors_test: %s\n", e.what());
            return 1;
        }
    }
    LoadError::Kind kind;
    // ---- the container
    CHECK(starts(error_of({1, 2, 3}), "HeaderTooSmall"));
    CHECK(starts(error_of(file_of("{}", {}, 5)), "InvalidHeaderLength"));
    CHECK(starts(error_of(file_of("{}", {}, 200000000)), "HeaderTooLarge"));
    CHECK(starts(error_of(file_of("[]", {})), "InvalidHeaderStart"));
    CHECK(starts(error_of(file_of("", {})), "InvalidHeaderStart"));
    CHECK(starts(error_of(file_of("{\xff}", {})), "InvalidHeader"));
    CHECK(starts(error_of(file_of("{\"a\": }", {})), "InvalidHeaderDeserialization"));
    CHECK(starts(error_of(file_of("{\"a\": {\"dtype\": \"F32\", \"shape\": [1]}}", {0, 0, 0, 0})), "InvalidHeaderDeserialization"));
    CHECK(starts(error_of(file_of("{\"a\": {\"dtype\": \"F33\", \"shape\": [1], \"data_offsets\": [0, 4]}}", {0, 0, 0, 0})), "InvalidHeaderDeserialization: unknown dtype"));
    CHECK(starts(error_of(file_of("{\"a\": {\"dtype\": \"F32\", \"shape\": [-1], \"data_offsets\": [0, 4]}}", {0, 0, 0, 0})), "InvalidHeaderDeserialization"));
    CHECK(starts(error_of(file_of("{\"a\": {\"dtype\": \"F32\", \"shape\": [1.5], \"data_offsets\": [0, 4]}}", {0, 0, 0, 0})), "InvalidHeaderDeserialization"));
    CHECK(starts(error_of(file_of("{\"__metadata__\": {\"k\": 3}}", {})), "InvalidHeaderDeserialization: __metadata__"));
    CHECK(error_of(file_of("{\"__metadata__\": {\"k\": \"v\"}}", {})).empty());
    CHECK(error_of(file_of("{}", {})).empty());
    // ---- byte ranges: contiguous from 0, sizes that match, nothing left over
    const std::vector<uint8_t> eight(8, 0);
    CHECK(starts(error_of(file_of("{\"a\": {\"dtype\": \"F32\", \"shape\": [1], \"data_offsets\": [4, 8]}}", eight)), "InvalidOffset(a)"));
    CHECK(starts(error_of(file_of("{\"a\": {\"dtype\": \"F32\", \"shape\": [1], \"data_offsets\": [0, 4]}, "
                                  "\"b\": {\"dtype\": \"F32\", \"shape\": [1], \"data_offsets\": [2, 6]}}", eight)), "InvalidOffset(b)"));
    CHECK(starts(error_of(file_of("{\"a\": {\"dtype\": \"F32\", \"shape\": [3], \"data_offsets\": [0, 8]}}", eight)), "TensorInvalidInfo(a)"));
    CHECK(starts(error_of(file_of("{\"a\": {\"dtype\": \"F32\", \"shape\": [1], \"data_offsets\": [0, 4]}}", eight)), "MetadataIncompleteBuffer"));
    CHECK(starts(error_of(file_of("{\"a\": {\"dtype\": \"F4\", \"shape\": [3], \"data_offsets\": [0, 2]}}", {0, 0})), "MisalignedSlice"));
    CHECK(starts(error_of(file_of("{\"a\": {\"dtype\": \"U8\", \"shape\": [4294967296, 4294967296, 2], \"data_offsets\": [0, 0]}}", {})), "ValidationOverflow"));
    // an empty tensor between two others shares its offset with its successor
    {
        const std::string h = "{\"z\": {\"dtype\": \"F32\", \"shape\": [1], \"data_offsets\": [4, 8]}, "
                              "\"e\": {\"dtype\": \"F32\", \"shape\": [0, 7], \"data_offsets\": [4, 4]}, "
                              "\"a\": {\"dtype\": \"F32\", \"shape\": [1], \"data_offsets\": [0, 4]}}";
        std::vector<uint8_t> data(8, 0);
        const float one = 1.0f, two = 2.0f;
        std::memcpy(&data[0], &one, 4);
        std::memcpy(&data[4], &two, 4);
        const std::vector<uint8_t> f = file_of(h, data);
        const auto t = st::load_safetensors_f32_from_bytes(f.data(), f.size());
        CHECK(t.size() == 3 && t.at("a")[0] == 1.0f && t.at("z")[0] == 2.0f && t.at("e").empty());
    }
    // ---- dtypes: the reference's set promotes exactly as documented; anything else names key and dtype
    {
        // F16: 1.0 (0x3C00), -2.0 (0xC000), smallest subnormal (0x0001), +inf (0x7C00); BF16: 1.5 (0x3FC0), -0.0 (0x8000)
        const std::string h = "{\"b\": {\"dtype\": \"BF16\", \"shape\": [2], \"data_offsets\": [8, 12]}, "
                              "\"h\": {\"dtype\": \"F16\", \"shape\": [2, 2], \"data_offsets\": [0, 8]}, "
                              "\"i\": {\"dtype\": \"I32\", \"shape\": [1], \"data_offsets\": [12, 16]}, "
                              "\"l\": {\"dtype\": \"I64\", \"shape\": [1], \"data_offsets\": [16, 24]}, "
                              "\"d\": {\"dtype\": \"F64\", \"shape\": [1], \"data_offsets\": [24, 32]}, "
                              "\"o\": {\"dtype\": \"BOOL\", \"shape\": [3], \"data_offsets\": [32, 35]}}";
        std::vector<uint8_t> data{0x00, 0x3C, 0x00, 0xC0, 0x01, 0x00, 0x00, 0x7C, 0xC0, 0x3F, 0x00, 0x80};
        const int32_t i32 = -7;
        const int64_t i64 = (1LL << 40) + 1;
        const double f64 = 0.1;
        data.resize(35);
        std::memcpy(&data[12], &i32, 4);
        std::memcpy(&data[16], &i64, 8);
        std::memcpy(&data[24], &f64, 8);
        data[32] = 1, data[33] = 0, data[34] = 1;
        std::vector<uint8_t> f = file_of(h, data);
        const auto t = st::load_safetensors_typed_from_bytes(f.data(), f.size());
        const std::vector<float> hv = t.at("h").to_f32(), bv = t.at("b").to_f32();
        CHECK(hv[0] == 1.0f && hv[1] == -2.0f && hv[2] == 5.9604644775390625e-8f && std::isinf(hv[3]) && hv[3] > 0);
        CHECK(bv[0] == 1.5f && bv[1] == 0.0f && std::signbit(bv[1]));
        CHECK(t.at("i").to_f32()[0] == -7.0f && t.at("l").to_f32()[0] == 1099511627776.0f && t.at("d").to_f32()[0] == 0.1f);
        CHECK((t.at("o").to_f32() == std::vector<float>{1.0f, 0.0f, 1.0f}));
        CHECK(starts(error_of(f, /*typed=*/false, false, &kind), "unsupported dtype (key=b): BF16") && kind == LoadError::UnsupportedDtype);
        f[f.size() - 2] = 2;                                      // a BOOL byte other than 0 / 1
        CHECK(starts(error_of(f, true, false, &kind), "BOOL tensor holds a value other than 0 / 1 (key=o, index=1): 2") && kind == LoadError::InvalidBoolValue);
    }
    {
        const std::vector<uint8_t> f = file_of("{\"q\": {\"dtype\": \"I8\", \"shape\": [2], \"data_offsets\": [0, 2]}, "
                                               "\"u\": {\"dtype\": \"U8\", \"shape\": [1], \"data_offsets\": [2, 3]}}", {1, 2, 3});
        CHECK(starts(error_of(f, true, false, &kind), "unsupported dtype (key=q): I8") && kind == LoadError::UnsupportedDtype);
        CHECK(starts(error_of(f, true, true, &kind), "unsupported dtype (key=u): U8"));     // quantized types allowed: U8 still is not one
        st::validate_safetensors_layout_from_bytes(f.data(), f.size());                       // the layout itself is fine
    }
    // ---- require_keys: all missing keys at once
    {
        const std::vector<uint8_t> f = file_of("{\"model.norm.weight\": {\"dtype\": \"F32\", \"shape\": [1], \"data_offsets\": [0, 4]}}", {0, 0, 0, 0});
        const auto t = st::load_safetensors_typed_from_bytes(f.data(), f.size());
        bool caught = false;
        try {
            st::require_keys(t, st::llama_decoder_keys(1));
        } catch (const LoadError &e) {
            caught = e.kind == LoadError::MissingKeys && e.keys.size() == 11 && e.keys[0] == "model.embed_tokens.weight";
        }
        CHECK(caught);
        CHECK(st::llama_decoder_keys(2).size() == 3 + 2 * 9);
        bool io = false;
        try {
            st::read_file("/nonexistent/file.safetensors");
        } catch (const LoadError &e) {
            io = e.kind == LoadError::Io;
        }
        CHECK(io);
    }
    std::printf("host_safetensors_test: %d checks ok\n", g_checks);
    return 0;
}
