// The knob-file loader of libmoe355 (csrc/config.cpp) driven through its C entry points in a process built with
// AddressSanitizer and UndefinedBehaviorSanitizer (host code only; tests/test_host_sanitizers.py builds and runs it).
// Inputs: the reference's own file, every malformed and out-of-domain text the Python tests use, truncated and
// oversized texts, tiny and absent error buffers, a missing file.  Any sanitizer report fails the run; the few
// results checked here only make sure the calls were not optimised away.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "moe355.h"

static int failures = 0;
#define CHECK(cond)                                                        \
    do {                                                                   \
        if (!(cond)) { std::fprintf(stderr, "check failed: %s (line %d)\n", #cond, __LINE__); ++failures; } \
    } while (0)

static const char* kReference =
    "{\n  \"capacity_factor\": 1,\n  \"drop_tokens\": 0,\n  \"expert_top_k\": 1,\n  \"is_training\": 0,\n  \"hidden_act\": 0,\n"
    "  \"hidden_size\": 1024,\n  \"intermediate_size\": 4096,\n  \"micro_batch\": 4,\n  \"num_experts\": 1,\n"
    "  \"sequence_len\": 2048,\n  \"torch_dtype\": 0\n}\n";

int main(int argc, char** argv) {
    moe_config c;
    char err[256];
    CHECK(moe_config_default(&c) == MOE_OK);
    CHECK(moe_config_validate(&c, err, sizeof err) == MOE_OK);
    CHECK(moe_config_from_json_string(kReference, &c, err, sizeof err) == MOE_OK);
    CHECK(moe_config_tokens(&c) == 4 * 2048 && c.hidden_size == 1024);
    int64_t cap = 0;
    CHECK(moe_config_capacity(&c, &cap) == MOE_OK && cap == 8192);

    // every prefix of the reference file (truncated input), with error buffers of every small size and none at all
    const std::string ref(kReference);
    for (size_t n = 0; n < ref.size(); ++n) {
        const std::string cut = ref.substr(0, n);
        char small[8];
        for (size_t e = 0; e <= sizeof small; ++e) (void)moe_config_from_json_string(cut.c_str(), &c, e ? small : nullptr, e);
    }
    const char* bad[] = {"", "[]", "{", "{\"a\" 1}", "{\"hidden_size\": }", "{\"hidden_size\": 64,}", "{} x", "{\"a\": \"unterminated",
                         "{\"a\": {\"b\": [1, 2, {\"c\": \"}\"}]}}", "{\"hidden_size\": 1e999}", "{\"hidden_size\": -1e999}",
                         "{\"hidden_size\": nan}", "{\"\\u0041\": 1}", "{\"a\\\"b\": 1}", "{\"x\": tru}", "{\"x\": true, \"y\": false, \"z\": null}"};
    for (const char* t : bad) (void)moe_config_from_json_string(t, &c, err, sizeof err);
    // out-of-domain and huge values, duplicate keys, a very long key and a very deep nest
    std::vector<std::string> texts;
    const char* keys[] = {"capacity_factor", "drop_tokens", "expert_top_k", "is_training", "hidden_act", "hidden_size", "intermediate_size",
                          "micro_batch", "num_experts", "sequence_len", "torch_dtype", "gate_fn", "norm_topk_prob"};
    const char* values[] = {"0", "-1", "1.5", "3000000000", "-3000000000", "1e30", "0.000001", "64", "true"};
    for (const char* k : keys)
        for (const char* v : values) {
            std::string t = ref.substr(0, ref.rfind('}'));
            t += std::string(", \"") + k + "\": " + v + "}";
            texts.push_back(t);
        }
    texts.push_back("{\"" + std::string(100000, 'k') + "\": 1}");
    texts.push_back(std::string(5000, '[') + std::string(5000, ']'));
    texts.push_back("{\"a\": " + std::string(2000, '{') + std::string(2000, '}') + "}");
    for (const std::string& t : texts) (void)moe_config_from_json_string(t.c_str(), &c, err, sizeof err);
    // sizes whose product would overflow 32 bits must not overflow in tokens / capacity
    moe_config big;
    moe_config_default(&big);
    big.micro_batch = 2000000000; big.sequence_len = 2000000000; big.expert_top_k = 16; big.num_experts = 16;
    big.capacity_factor = 1e300;
    (void)moe_config_validate(&big, err, sizeof err);
    (void)moe_config_tokens(&big);
    (void)moe_config_capacity(&big, &cap);
    CHECK(moe_config_from_json_file("/nonexistent/aristos_config.json", &c, err, sizeof err) == MOE_ERR_BAD_CONFIG);
    if (argc > 1) CHECK(moe_config_from_json_file(argv[1], &c, err, sizeof err) == MOE_OK);
    CHECK(moe_config_from_json_string(nullptr, &c, err, sizeof err) != MOE_OK);
    CHECK(moe_config_from_json_string(kReference, nullptr, err, sizeof err) != MOE_OK);
    for (int s = -2; s < 12; ++s) CHECK(moe_status_string(s) != nullptr && std::strlen(moe_status_string(s)) > 0);
    CHECK(moe_version() == MOE355_VERSION);
    std::printf("config loader under sanitizers: %d failed checks\n", failures);
    return failures ? 1 : 0;
}
