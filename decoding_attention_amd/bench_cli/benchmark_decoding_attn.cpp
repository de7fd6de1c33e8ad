// Command-line benchmark of the decoding-attention C-ABI on one MI355X.
//
// Takes the flags of the reference's benchmark executable (benchmarks/cpp/benchmark_decoding_attn.cpp:12-27:
// -b -sq -sk -hq -hk -d -dv -is_causal -is_alibi -is_bf16 -warmup_iterations -profiling_iterations
// -sleep_duration -enable_check -cpu_procs -gpu_rank, in gflags spelling) and writes the reference's log lines to
// stderr (csrc/common/logging.h:38-42, csrc/common/tester.h:95-110,288-292), so that the reference's log parsers
// (tools/performance/cpp/performance.py) read its output unchanged.  One extra flag, -seed, fixes the inputs.
//
// Host code only: the work is done by da_decoding_attn() from libdecoding_attn_hip.so.  -enable_check compares the
// GPU output with a plain fp32 attention loop kept in this file; that loop is a checker and nothing else uses it.
#include <hip/hip_runtime_api.h>
#include <omp.h>
#include <sys/syscall.h>
#include <time.h>
#include <unistd.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <random>
#include <string>
#include <vector>

#include "decoding_attn_hip.h"

namespace {

const char* now_text() {
    static char text[64];
    const time_t raw = time(nullptr);
    text[strftime(text, sizeof(text), "%Y-%m-%d %H:%M:%S", localtime(&raw))] = '\0';
    return text;
}

const char* file_tail(const char* path) {
    const char* slash = strrchr(path, '/');
    return slash ? slash + 1 : path;
}

// "[DA date time pid:tid file:line function] message": seven space-separated fields precede the message, which is
// what the log parsers count on.
#define DLOG(format, ...)                                                                                         \
    fprintf(stderr, "[DA %s %d:%ld %s:%d %s] " format "\n", now_text(), (int)getpid(), (long)syscall(SYS_gettid), \
            file_tail(__FILE__), __LINE__, __FUNCTION__, ##__VA_ARGS__)

#define HIP_OK(call)                                                                        \
    do {                                                                                    \
        const hipError_t status_ = (call);                                                  \
        if (status_ != hipSuccess) {                                                        \
            DLOG("HIP runtime error: %s (%s)", hipGetErrorString(status_), #call);          \
            exit(EXIT_FAILURE);                                                             \
        }                                                                                   \
    } while (0)

// ---------------------------------------------------------------------------------------------------------------
// flags

struct Flag {
    const char* name;
    bool is_bool;
    unsigned* u;
    bool* b;
    const char* help;
};

struct Options {
    unsigned b = 2, sq = 1, sk = 256, hq = 32, hk = 32, d = 128, dv = 128;
    bool is_causal = false, is_alibi = false, is_bf16 = false;
    unsigned warmup_iterations = 1, profiling_iterations = 10, sleep_duration = 100;
    bool enable_check = false;
    unsigned cpu_procs = (unsigned)omp_get_num_procs(), gpu_rank = 0, seed = 0;
    bool seed_given = false;
};

std::vector<Flag> flag_table(Options& o) {
    return {
        {"b", false, &o.b, nullptr, "batch size"},
        {"sq", false, &o.sq, nullptr, "q seq len (decoding: 1)"},
        {"sk", false, &o.sk, nullptr, "kv seq len"},
        {"hq", false, &o.hq, nullptr, "q head num"},
        {"hk", false, &o.hk, nullptr, "kv head num"},
        {"d", false, &o.d, nullptr, "head dim"},
        {"dv", false, &o.dv, nullptr, "head dim v"},
        {"is_causal", true, nullptr, &o.is_causal, "causal mask (meaningless for one query token; must be false)"},
        {"is_alibi", true, nullptr, &o.is_alibi, "enable alibi"},
        {"is_bf16", true, nullptr, &o.is_bf16, "data type of q, k, v and o"},
        {"warmup_iterations", false, &o.warmup_iterations, nullptr, "warmup iteration numbers and average the result"},
        {"profiling_iterations", false, &o.profiling_iterations, nullptr,
         "profiling iteration numbers and average the result"},
        {"sleep_duration", false, &o.sleep_duration, nullptr, "sleep_milliseconds between profiling"},
        {"enable_check", true, nullptr, &o.enable_check, "check the GPU result against the CPU result"},
        {"cpu_procs", false, &o.cpu_procs, nullptr, "processor num used of CPU"},
        {"gpu_rank", false, &o.gpu_rank, nullptr, "the used GPU rank"},
        {"seed", false, &o.seed, nullptr, "seed of the random inputs (default: from the random device)"},
    };
}

bool parse_bool(const std::string& text, bool* out) {
    if (text == "true" || text == "1" || text == "t" || text == "yes" || text == "y") return *out = true, true;
    if (text == "false" || text == "0" || text == "f" || text == "no" || text == "n") return *out = false, true;
    return false;
}

// gflags spelling: -name=value, --name=value, -name value; booleans also as -name and -noname.
bool parse_flags(int argc, char** argv, Options& o) {
    const std::vector<Flag> table = flag_table(o);
    for (int i = 1; i < argc; ++i) {
        std::string arg = argv[i];
        if (arg == "-help" || arg == "--help" || arg == "-h") {
            for (const Flag& f : table) fprintf(stdout, "  -%s (%s) type: %s\n", f.name, f.help, f.is_bool ? "bool" : "uint32");
            exit(0);
        }
        if (arg.size() < 2 || arg[0] != '-') {
            fprintf(stderr, "ERROR: unexpected argument '%s'\n", arg.c_str());
            return false;
        }
        arg = arg.substr(arg[1] == '-' ? 2 : 1);
        std::string name = arg, value;
        bool has_value = false;
        const size_t eq = arg.find('=');
        if (eq != std::string::npos) {
            name = arg.substr(0, eq);
            value = arg.substr(eq + 1);
            has_value = true;
        }
        const Flag* hit = nullptr;
        bool negated = false;
        for (const Flag& f : table)
            if (name == f.name) hit = &f;
        if (!hit && name.rfind("no", 0) == 0)
            for (const Flag& f : table)
                if (f.is_bool && name.substr(2) == f.name) hit = &f, negated = true;
        if (!hit) {
            fprintf(stderr, "ERROR: unknown command line flag '%s'\n", name.c_str());
            return false;
        }
        if (hit->is_bool) {
            if (negated) {
                *hit->b = false;
            } else if (!has_value) {
                *hit->b = true;
            } else if (!parse_bool(value, hit->b)) {
                fprintf(stderr, "ERROR: illegal value '%s' specified for bool flag '%s'\n", value.c_str(), hit->name);
                return false;
            }
            continue;
        }
        if (!has_value) {
            if (i + 1 >= argc) {
                fprintf(stderr, "ERROR: flag '%s' is missing its argument\n", hit->name);
                return false;
            }
            value = argv[++i];
        }
        char* end = nullptr;
        const unsigned long parsed = strtoul(value.c_str(), &end, 10);
        if (value.empty() || *end != '\0' || value[0] == '-' || parsed > 0xfffffffful) {
            fprintf(stderr, "ERROR: illegal value '%s' specified for uint32 flag '%s'\n", value.c_str(), hit->name);
            return false;
        }
        *hit->u = (unsigned)parsed;
        if (hit->u == &o.seed) o.seed_given = true;
    }
    return true;
}

// ---------------------------------------------------------------------------------------------------------------
// 16-bit element types on the host

uint16_t to_f16(float x) {
    uint32_t bits;
    memcpy(&bits, &x, 4);
    const uint32_t sign = (bits >> 16) & 0x8000u;
    bits &= 0x7fffffffu;
    if (bits >= 0x7f800000u) return (uint16_t)(sign | (bits > 0x7f800000u ? 0x7e00u : 0x7c00u));
    if (bits >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);  // rounds to infinity
    if (bits < 0x38800000u) {                                   // subnormal half or zero
        if (bits < 0x33000000u) return (uint16_t)sign;
        const int shift = 126 - (int)(bits >> 23);  // 14..24
        const uint32_t mant = (bits & 0x7fffffu) | 0x800000u;
        uint32_t half = mant >> shift;
        const uint32_t rem = mant & ((1u << shift) - 1), mid = 1u << (shift - 1);
        if (rem > mid || (rem == mid && (half & 1))) ++half;
        return (uint16_t)(sign | half);
    }
    uint32_t half = (bits - 0x38000000u) >> 13;
    const uint32_t rem = bits & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1))) ++half;
    return (uint16_t)(sign | half);
}

float from_f16(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f, mant = h & 0x3ffu, bits;
    if (exp == 0) {
        if (mant == 0) {
            bits = sign;
        } else {
            int e = -1;
            do {
                mant <<= 1;
                ++e;
            } while (!(mant & 0x400u));
            bits = sign | ((uint32_t)(112 - e) << 23) | ((mant & 0x3ffu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (mant << 13);
    } else {
        bits = sign | ((exp + 112) << 23) | (mant << 13);
    }
    float x;
    memcpy(&x, &bits, 4);
    return x;
}

uint16_t to_bf16(float x) {
    uint32_t bits;
    memcpy(&bits, &x, 4);
    if ((bits & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((bits >> 16) | 0x40u);
    return (uint16_t)((bits + 0x7fffu + ((bits >> 16) & 1)) >> 16);
}

float from_bf16(uint16_t h) {
    const uint32_t bits = (uint32_t)h << 16;
    float x;
    memcpy(&x, &bits, 4);
    return x;
}

// A tensor of 16-bit elements with a host copy and a device copy, filled with uniform(-1, 1) values like the
// reference's test tensors (csrc/common/tensor.h:31-36,117-119).
struct Tensor16 {
    std::vector<uint16_t> host;
    uint16_t* dev = nullptr;

    Tensor16(size_t n, const char* name, bool bf16, std::default_random_engine& engine) : host(n) {
        std::uniform_real_distribution<float> uniform(-1.0f, 1.0f);
        for (size_t i = 0; i < n; ++i) host[i] = bf16 ? to_bf16(uniform(engine)) : to_f16(uniform(engine));
        HIP_OK(hipMalloc((void**)&dev, n * sizeof(uint16_t)));
        HIP_OK(hipMemcpy(dev, host.data(), n * sizeof(uint16_t), hipMemcpyHostToDevice));
        DLOG("%s: %zu, cpu: %p, gpu: %p", name, n, (void*)host.data(), (void*)dev);
    }
    ~Tensor16() {
        if (dev) (void)hipFree(dev);
    }
    Tensor16(const Tensor16&) = delete;
    Tensor16& operator=(const Tensor16&) = delete;
    void fetch() { HIP_OK(hipMemcpy(host.data(), dev, host.size() * sizeof(uint16_t), hipMemcpyDeviceToHost)); }
};

// Checker for -enable_check: attention for one query token per sequence in fp32, softmax normalised before the
// product with V, result rounded to the element type (the arithmetic of csrc/common/tester.h:133-259).
void check_attention(const Options& o, const std::vector<uint16_t>& q, const std::vector<uint16_t>& k,
                     const std::vector<uint16_t>* v, std::vector<uint16_t>& out) {
    const bool bf16 = o.is_bf16;
    auto load = [bf16](uint16_t x) { return bf16 ? from_bf16(x) : from_f16(x); };
    const size_t v_row = (size_t)o.hk * (v ? o.dv : o.d);  // V aliases the head of each K row when absent
    const std::vector<uint16_t>& vals = v ? *v : k;
    const float scale = 1.0f / std::sqrt((float)o.d);
    const unsigned ratio = o.hq / o.hk;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (unsigned b = 0; b < o.b; ++b) {
        for (unsigned h = 0; h < o.hq; ++h) {
            const unsigned hk = h / ratio;
            const uint16_t* qrow = &q[((size_t)b * o.hq + h) * o.d];
            std::vector<float> p(o.sk);
            const float slope = o.is_alibi ? 1.0f / std::exp2(8.0f * (float)(h + 1) / (float)o.hq) : 0.0f;
            float top = -INFINITY;
            for (unsigned j = 0; j < o.sk; ++j) {
                const uint16_t* krow = &k[(((size_t)b * o.sk + j) * o.hk + hk) * o.d];
                float dot = 0.0f;
                for (unsigned t = 0; t < o.d; ++t) dot += load(qrow[t]) * load(krow[t]);
                p[j] = dot * scale + slope * ((float)j - (float)(o.sk - 1));
                top = std::max(top, p[j]);
            }
            float sum = 0.0f;
            for (unsigned j = 0; j < o.sk; ++j) sum += (p[j] = std::exp(p[j] - top));
            for (unsigned j = 0; j < o.sk; ++j) p[j] /= sum;
            uint16_t* orow = &out[((size_t)b * o.hq + h) * o.dv];
            for (unsigned t = 0; t < o.dv; ++t) {
                float acc = 0.0f;
                for (unsigned j = 0; j < o.sk; ++j)
                    acc += p[j] * load(vals[((size_t)b * o.sk + j) * v_row + (size_t)hk * (v ? o.dv : o.d) + t]);
                orow[t] = bf16 ? to_bf16(acc) : to_f16(acc);
            }
        }
    }
}

struct Timer {
    hipStream_t stream;
    hipEvent_t t0, t1;
    explicit Timer(hipStream_t s) : stream(s) {
        HIP_OK(hipEventCreate(&t0));
        HIP_OK(hipEventCreate(&t1));
    }
    ~Timer() {
        (void)hipEventDestroy(t0);
        (void)hipEventDestroy(t1);
    }
    void start() { HIP_OK(hipEventRecord(t0, stream)); }
    float stop_ms() {
        float ms = 0.0f;
        HIP_OK(hipEventRecord(t1, stream));
        HIP_OK(hipEventSynchronize(t1));
        HIP_OK(hipEventElapsedTime(&ms, t0, t1));
        return ms;
    }
};

void run_case(const Options& o, hipStream_t stream) {
    std::random_device device;
    std::default_random_engine engine{o.seed_given ? o.seed : device()};
    const size_t total_q = (size_t)o.b * o.sq, total_k = (size_t)o.b * o.sk;
    Tensor16 q(total_q * o.hq * o.d, "Tensor Q", o.is_bf16, engine);
    Tensor16 k(total_k * o.hk * o.d, "Tensor K", o.is_bf16, engine);
    // as in the reference's tester (csrc/common/tester.h:64-69): a separate V only when d == dv, else V = K[..., :dv]
    std::unique_ptr<Tensor16> v;
    if (o.d == o.dv) v.reset(new Tensor16(total_k * o.hk * o.dv, "Tensor V", o.is_bf16, engine));
    Tensor16 out(total_q * o.hq * o.dv, "Tensor O", o.is_bf16, engine);
    std::vector<uint16_t> expect;

    std::vector<int32_t> cu(o.b + 1);
    for (unsigned i = 0; i <= o.b; ++i) cu[i] = (int32_t)((size_t)i * o.sk);
    int32_t* cu_dev = nullptr;
    HIP_OK(hipMalloc((void**)&cu_dev, cu.size() * sizeof(int32_t)));
    HIP_OK(hipMemcpy(cu_dev, cu.data(), cu.size() * sizeof(int32_t), hipMemcpyHostToDevice));
    DLOG("Tensor cu_seq_k: %zu, cpu: %p, gpu: %p", cu.size(), (void*)cu.data(), (void*)cu_dev);

    if (o.enable_check) {
        expect.resize(out.host.size());
        const double t0 = omp_get_wtime();
        check_attention(o, q.host, k.host, v ? &v->host : nullptr, expect);
        DLOG("MHA CPU use: %.3f ms", (omp_get_wtime() - t0) * 1e3);
    }

    auto call = [&] {
        const int rc = da_decoding_attn(q.dev, k.dev, v ? v->dev : nullptr, out.dev, cu_dev, o.sk, o.b, o.hq, o.hk, o.d,
                                        o.dv, o.is_alibi, o.is_bf16, stream);
        if (rc != DA_OK) {
            DLOG("da_decoding_attn failed (%d): %s", rc, da_last_error());
            exit(EXIT_FAILURE);
        }
    };

    const char* name = "Decoding-Attention";
    DLOG("----------------- Evaluating %s -----------------", name);
    usleep(o.sleep_duration * 1000);
    HIP_OK(hipMemsetAsync(out.dev, 0, out.host.size() * sizeof(uint16_t), stream));

    Timer timer(stream);
    timer.start();
    for (unsigned i = 0; i < o.warmup_iterations; ++i) call();
    DLOG("Warm up time: %.3f ms", (double)timer.stop_ms() / (double)std::max(1u, o.warmup_iterations));

    if (o.enable_check) {
        out.fetch();
        double worst = 0.0, mean = 0.0;
        for (size_t i = 0; i < expect.size(); ++i) {
            const float a = o.is_bf16 ? from_bf16(out.host[i]) : from_f16(out.host[i]);
            const float e = o.is_bf16 ? from_bf16(expect[i]) : from_f16(expect[i]);
            const double diff = std::fabs((double)a - (double)e);
            worst = std::max(worst, diff);
            mean += diff;
        }
        DLOG("Max diff: %f, avg diff: %f", worst, mean / (double)expect.size());
    }

    timer.start();
    for (unsigned i = 0; i < o.profiling_iterations; ++i) call();
    const double ms = (double)timer.stop_ms() / (double)std::max(1u, o.profiling_iterations);
    // the reference's accounting (csrc/common/tester.h:270-276): 2 (d + dv) flops per (query head, key); Q, K and O
    // bytes, V left out
    const double work = (double)o.b * o.sq * o.sk * o.hq * (double)(o.d + o.dv) * 2.0;
    const double bytes = ((double)o.b * o.sq * o.hq * o.d + (double)o.b * o.sk * o.hk * o.d +
                          (double)o.b * o.sq * o.hq * o.dv) * 2.0;
    const double tflops = work * 1e-12 / (ms * 1e-3), gbps = bytes * 1e-9 / (ms * 1e-3);
    DLOG("%s exit, profiling time: %.4f ms (%.2f%%), throughput: %.4f TFLOPS (%.2f%%), bandwidth: %.3f GB/s (%.2f%%)",
         name, ms, 100.0, tflops, 100.0, gbps, 100.0);
    (void)hipFree(cu_dev);
}

}  // namespace

int main(int argc, char** argv) {
    Options o;
    if (!parse_flags(argc, argv, o)) return EXIT_FAILURE;
    if (o.sq != 1 || o.is_causal) {
        fprintf(stderr, "ERROR: decoding attention takes one query token per sequence: -sq must be 1 and -is_causal false\n");
        return EXIT_FAILURE;
    }
    omp_set_num_threads((int)std::max(1u, o.cpu_procs));
    HIP_OK(hipSetDevice((int)o.gpu_rank));

    hipDeviceProp_t prop;
    HIP_OK(hipGetDeviceProperties(&prop, (int)o.gpu_rank));
    // (one device line; the reference's plot tools read only the `exit, profiling time` line of run_case)
    DLOG("Decoding Attention on GPU %u: %s (%s), %d compute units, wavefront %d, %zu KiB LDS per compute unit, %.0f GiB; "
         "%u CPU threads; library version %d",
         o.gpu_rank, prop.name, prop.gcnArchName, prop.multiProcessorCount, prop.warpSize,
         prop.maxSharedMemoryPerMultiProcessor / 1024, (double)prop.totalGlobalMem / (double)(1ull << 30), o.cpu_procs,
         da_version());

    hipStream_t stream = nullptr;
    DLOG("DMHA: Softmax (Q (%u x %u x %u x %u) * K^T (%u x %u x %u x %u)) * V (%u x %u x %u x %u) = O (%u x %u x %u x %u)",
         o.b, o.sq, o.hq, o.d, o.b, o.sk, o.hk, o.d, o.b, o.sk, o.hk, o.dv, o.b, o.sq, o.hq, o.dv);
    DLOG("Profiling: is causal: %d, stream: %p, is alibi: %d, is bf16: %d, warmup iterations: %u, profiling iterations: "
         "%u, sleep duration: %u ms, enable check: %d",
         o.is_causal, (void*)stream, o.is_alibi, o.is_bf16, o.warmup_iterations, o.profiling_iterations,
         o.sleep_duration, o.enable_check);

    run_case(o, stream);
    DLOG("Done");
    return 0;
}
