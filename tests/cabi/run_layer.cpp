// A C++ caller of the C ABI with no Python in the process: what a maintainer of the reference would write in place
// of the driver in main.cu.  Reads the knob file and raw operand files, runs moe_forward on a stream of its own,
// writes the output and the routing result.
//
//   run_layer <config.json> <directory>
//     reads  x.bin gate_w.bin w_up.bin [w_gate.bin] w_down.bin        (row-major, storage dtype of the config)
//     writes out.bin topk_idx.bin slot.bin expert_count.bin
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "moe355.h"

#define HIP_OK(x)                                                                         \
    do {                                                                                  \
        hipError_t e_ = (x);                                                              \
        if (e_ != hipSuccess) {                                                           \
            fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));                       \
            return 2;                                                                     \
        }                                                                                 \
    } while (0)
#define MOE_OK_OR_DIE(x)                                                                  \
    do {                                                                                  \
        int rc_ = (x);                                                                    \
        if (rc_ != MOE_OK) {                                                              \
            fprintf(stderr, "%s: %s\n", #x, moe_status_string(rc_));                      \
            return 3;                                                                     \
        }                                                                                 \
    } while (0)

static bool read_file(const std::string& path, std::vector<char>* out, bool required) {
    FILE* f = fopen(path.c_str(), "rb");
    if (!f) {
        if (required) fprintf(stderr, "cannot open %s\n", path.c_str());
        return false;
    }
    fseek(f, 0, SEEK_END);
    const long n = ftell(f);
    fseek(f, 0, SEEK_SET);
    out->resize((size_t)n);
    const size_t got = fread(out->data(), 1, (size_t)n, f);
    fclose(f);
    return got == (size_t)n;
}

static bool write_file(const std::string& path, const void* p, size_t n) {
    FILE* f = fopen(path.c_str(), "wb");
    if (!f) return false;
    const size_t put = fwrite(p, 1, n, f);
    fclose(f);
    return put == n;
}

static int upload(const std::string& path, size_t expect, bool required, void** dev) {
    *dev = nullptr;
    std::vector<char> host;
    if (!read_file(path, &host, required)) return required ? 1 : 0;
    if (host.size() != expect) {
        fprintf(stderr, "%s: %zu bytes, expected %zu\n", path.c_str(), host.size(), expect);
        return 1;
    }
    if (hipMalloc(dev, expect) != hipSuccess) return 1;
    return hipMemcpy(*dev, host.data(), expect, hipMemcpyHostToDevice) == hipSuccess ? 0 : 1;
}

int main(int argc, char** argv) {
    if (argc != 3) {
        fprintf(stderr, "usage: %s <config.json> <directory>\n", argv[0]);
        return 1;
    }
    const std::string dir = std::string(argv[2]) + "/";
    moe_config cfg;
    char err[256];
    int rc = moe_config_from_json_file(argv[1], &cfg, err, sizeof err);
    if (rc != MOE_OK) {
        fprintf(stderr, "config: %s (%s)\n", err, moe_status_string(rc));
        return 3;
    }
    if (cfg.torch_dtype != 0 && cfg.torch_dtype != 2) {
        fprintf(stderr, "this caller handles fp32 and bf16 layers\n");
        return 1;
    }
    const int64_t S = moe_config_tokens(&cfg);
    const size_t es = cfg.torch_dtype == 0 ? 4 : 2;
    const size_t H = (size_t)cfg.hidden_size, I = (size_t)cfg.intermediate_size, E = (size_t)cfg.num_experts;
    const size_t k = (size_t)cfg.expert_top_k;

    moe_weights w = {};
    void *x, *gate_w, *w_up, *w_gate, *w_down;
    if (upload(dir + "x.bin", (size_t)S * H * es, true, &x)) return 1;
    if (upload(dir + "gate_w.bin", E * H * es, true, &gate_w)) return 1;
    if (upload(dir + "w_up.bin", E * I * H * es, true, &w_up)) return 1;
    if (upload(dir + "w_gate.bin", E * I * H * es, cfg.hidden_act == 2, &w_gate)) return 1;
    if (upload(dir + "w_down.bin", E * H * I * es, true, &w_down)) return 1;
    w.gate_w = gate_w;
    w.w_up = w_up;
    w.w_gate = w_gate;
    w.w_down = w_down;

    moe_handle* h = nullptr;
    MOE_OK_OR_DIE(moe_create(&cfg, &h));
    size_t ws_bytes = 0;
    MOE_OK_OR_DIE(moe_workspace_bytes(&cfg, &ws_bytes));
    void *ws, *out;
    HIP_OK(hipMalloc(&ws, ws_bytes));
    HIP_OK(hipMalloc(&out, (size_t)S * H * es));
    moe_routing_out r = {};
    HIP_OK(hipMalloc((void**)&r.topk_idx, (size_t)S * k * 4));
    HIP_OK(hipMalloc((void**)&r.topk_w, (size_t)S * k * 4));
    HIP_OK(hipMalloc((void**)&r.slot, (size_t)S * k * 4));
    HIP_OK(hipMalloc((void**)&r.expert_count, E * 4));
    HIP_OK(hipMalloc((void**)&r.expert_offset, E * 4));
    HIP_OK(hipMalloc((void**)&r.token_indices, (size_t)S * k * 4));
    hipStream_t st;
    HIP_OK(hipStreamCreate(&st));

    // a workspace that is one byte short must be refused before anything is launched
    if (moe_forward(h, x, &w, out, &r, ws, ws_bytes - 1, st) != MOE_ERR_WORKSPACE) {
        fprintf(stderr, "short workspace was not refused\n");
        return 4;
    }
    // the per-task trace of the queue kernel: a buffer of the caller's, one record per tile of the call that follows
    void* trace = nullptr;
    const size_t trace_bytes = moe_task_trace_bytes(1 << 14);
    HIP_OK(hipMalloc(&trace, trace_bytes));
    MOE_OK_OR_DIE(moe_set_task_trace(h, trace, trace_bytes));
    MOE_OK_OR_DIE(moe_forward(h, x, &w, out, &r, ws, ws_bytes, st));
    HIP_OK(hipStreamSynchronize(st));
    int64_t t0 = 0, t1 = 0;
    MOE_OK_OR_DIE(moe_get_task_counts(h, ws, st, &t0, &t1));
    int64_t traced = 0;
    int32_t mode = 0;
    MOE_OK_OR_DIE(moe_get_ffn_mode(h, &mode));
    {
        std::vector<moe_task_record> rec(1 << 14);
        MOE_OK_OR_DIE(moe_get_task_trace(h, st, rec.data(), (int64_t)rec.size(), &traced));
        if (mode == MOE_FFN_PERSISTENT && traced != t0 + t1) {
            fprintf(stderr, "trace holds %lld records for %lld tasks\n", (long long)traced, (long long)(t0 + t1));
            return 6;
        }
        for (int64_t i = 0; i < traced; ++i)
            if (rec[i].end_us < rec[i].start_us || rec[i].phase < 0 || rec[i].phase > 1) {
                fprintf(stderr, "bad trace record %lld\n", (long long)i);
                return 6;
            }
    }
    MOE_OK_OR_DIE(moe_set_task_trace(h, nullptr, 0));

    std::vector<char> host((size_t)S * H * es);
    HIP_OK(hipMemcpy(host.data(), out, host.size(), hipMemcpyDeviceToHost));
    if (!write_file(dir + "out.bin", host.data(), host.size())) return 5;
    std::vector<int32_t> ints((size_t)S * k);
    HIP_OK(hipMemcpy(ints.data(), r.topk_idx, ints.size() * 4, hipMemcpyDeviceToHost));
    if (!write_file(dir + "topk_idx.bin", ints.data(), ints.size() * 4)) return 5;
    HIP_OK(hipMemcpy(ints.data(), r.slot, ints.size() * 4, hipMemcpyDeviceToHost));
    if (!write_file(dir + "slot.bin", ints.data(), ints.size() * 4)) return 5;
    std::vector<int32_t> counts(E);
    HIP_OK(hipMemcpy(counts.data(), r.expert_count, E * 4, hipMemcpyDeviceToHost));
    if (!write_file(dir + "expert_count.bin", counts.data(), E * 4)) return 5;

    printf("ok tokens=%lld tasks=%lld+%lld traced=%lld version=%d\n", (long long)S, (long long)t0, (long long)t1,
           (long long)traced, moe_version());
    moe_destroy(h);
    return 0;
}
