// allreduce <NUM_BYTES> <ALG> <ITERS> <DELAY> [--flags]
//
// Command-line driver with the contract of the reference benchmark binaries
// (main() of stragglar/allreduce_8GPU.cu:907-1094 and allreduce_4GPU.cu
// :401-625; usage in README.md:33): same four positional arguments, same CSV
// on stdout, same self-check, same exit behaviour.  It emulates all n ranks on
// one MI355X and talks to the device only through the C ABI in sar.h.
//
// Optional flags after the four positionals (the reference fixes these at
// compile time or has no counterpart):
//   --ranks N          emulated ranks (default 8; the reference builds one binary per n)
//   --dtype T          f32 (default) | f16 | bf16
//   --schedule FILE    StragglAR table in the synthesizers' text format
//                      (default: the table the reference hard-codes for n=4/8, else
//                      $SAR_SCHEDULE_DIR or <exe>/../schedules/stragglar_n<N>.txt)
//   --init MODE        reference (default: rank i <- i+base, self-check on) | uniform | normal
//   --seed S           seed of --init uniform/normal (default 0)
//   --base B           constant of rank 0 for --init reference (default 1 for n=8, 0 for n=4, as the reference)
//   --graph 0|1        replay the rounds as one hipGraph instead of launching them one by one (default 0:
//                      on this software stack a replayed node costs more than an eager launch)
//   --report           also print, to stderr, the bytes the timed part sends to memory, the rate and its fraction of
//                      the 8 TB/s HBM peak, and the rows' algorithmic bytes and rate
//   --executor 0|1|2   0 = one launch per round, 1 = the column kernel (one launch per schedule), 2 = the library's
//                      choice (default)
//   --sequence 0|1     1 (default): every timed iteration runs directly behind the same step on a second set of rank
//                      buffers (untimed), as in a sequence of AllReduces: it starts with that step's last stores still
//                      in the 256 MB Infinity Cache and pays for pushing them out, as the next would for its own.
//                      0: behind the fill alone, as the reference times it (its GPUs have no such cache; here a step
//                      with cached stores is then timed 3 to 12 % too fast)
//   --nocheck          skip the final "all ranks hold the same" check: for a --schedule that times a part of a
//                      table (a row list of the exchanges alone, say) and is no AllReduce
#include <cerrno>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>
#include <string>
#include <vector>

#include <unistd.h>

#include "sar.h"

namespace {

[[noreturn]] void die(const char* what) {
    // CHECK_CUDA / CHECK_NCCL of the reference: print and exit(EXIT_FAILURE)
    printf("SAR error: %s: '%s'\n", what, sar_last_error());
    exit(EXIT_FAILURE);
}
#define CHECK_SAR(call) do { if ((call) != SAR_OK) die(#call); } while (0)

std::string exe_dir() {
    char buf[4096];
    ssize_t n = readlink("/proc/self/exe", buf, sizeof(buf) - 1);
    if (n <= 0) return ".";
    buf[n] = 0;
    std::string s(buf);
    size_t p = s.rfind('/');
    return p == std::string::npos ? "." : s.substr(0, p);
}

bool read_file(const std::string& path, std::string* out) {
    std::ifstream f(path, std::ios::binary);
    if (!f) return false;
    std::ostringstream ss; ss << f.rdbuf(); *out = ss.str();
    return true;
}

float half_bits_to_float(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 0x1fu, man = h & 0x3ffu, u;
    if (exp == 0) { float v = std::ldexp((float)man, -24); memcpy(&u, &v, 4); u |= sign; }
    else if (exp == 31) u = sign | 0x7f800000u | (man << 13);
    else u = sign | ((exp + 112u) << 23) | (man << 13);
    float f; memcpy(&f, &u, 4); return f;
}

float load_elem(const void* p, size_t i, int dtype) {
    if (dtype == SAR_F32) return ((const float*)p)[i];
    uint16_t h = ((const uint16_t*)p)[i];
    if (dtype == SAR_F16) return half_bits_to_float(h);
    uint32_t u = (uint32_t)h << 16; float f; memcpy(&f, &u, 4); return f;
}

}  // namespace

int main(int argc, char* argv[]) {
    // positional arguments first, optional --flags after them
    int npos = 0;
    while (1 + npos < argc && strncmp(argv[1 + npos], "--", 2) != 0) ++npos;
    if (argc < 5 || npos != 4) {
        fprintf(stderr, "Usage: %s <bufferSize> <algorithm> <numIters> <sleepTimeMs>\n", argv[0]);
        exit(EXIT_FAILURE);
    }
    size_t bytes = (size_t)strtoull(argv[1], NULL, 10);
    const char* alg = argv[2];
    int numIters = atoi(argv[3]);
    float sleepTime = (float)atof(argv[4]);

    int numRanks = 8, dtype = SAR_F32, use_graph = 0, base = -1, report = 0, executor = -1, check = 1, sequence = 1;
    unsigned long long seed = 0;
    std::string schedule_path, init = "reference";
    for (int i = 5; i < argc; ++i) {
        std::string a = argv[i];
        auto need = [&](const char* name) -> const char* {
            if (i + 1 >= argc) { fprintf(stderr, "%s needs a value\n", name); exit(EXIT_FAILURE); }
            return argv[++i];
        };
        if (a == "--ranks") numRanks = atoi(need("--ranks"));
        else if (a == "--dtype") {
            std::string t = need("--dtype");
            if (t == "f32") dtype = SAR_F32; else if (t == "f16") dtype = SAR_F16; else if (t == "bf16") dtype = SAR_BF16;
            else { fprintf(stderr, "Invalid dtype: %s\n", t.c_str()); exit(EXIT_FAILURE); }
        }
        else if (a == "--schedule") schedule_path = need("--schedule");
        else if (a == "--init") init = need("--init");
        else if (a == "--seed") seed = strtoull(need("--seed"), NULL, 10);
        else if (a == "--base") base = atoi(need("--base"));
        else if (a == "--graph") use_graph = atoi(need("--graph"));
        else if (a == "--report") report = 1;
        else if (a == "--executor") executor = atoi(need("--executor"));      // 0 one launch per round, 1 column kernel, 2 the library's choice
        else if (a == "--sequence") sequence = atoi(need("--sequence"));
        else if (a == "--nocheck") check = 0;                                  // a --schedule that is not an AllReduce (timing parts of a table)
        else { fprintf(stderr, "Unknown option: %s\n", a.c_str()); exit(EXIT_FAILURE); }
    }
    if (strcmp(alg, "ring") != 0 && strcmp(alg, "rhd") != 0 && strcmp(alg, "direct") != 0 && strcmp(alg, "stragglar") != 0) {
        fprintf(stderr, "Invalid algorithm: %s\n", alg);
        exit(EXIT_FAILURE);
    }
    if (init != "reference" && init != "uniform" && init != "normal") {
        fprintf(stderr, "Invalid init mode: %s\n", init.c_str());
        exit(EXIT_FAILURE);
    }
    if (numRanks < 3 || numRanks > SAR_MAX_RANKS) {
        fprintf(stderr, "Invalid rank count: %d\n", numRanks);
        exit(EXIT_FAILURE);
    }
    if (base < 0) base = (numRanks == 4) ? 0 : 1;   // allreduce_4GPU.cu fills rank i with i, allreduce_8GPU.cu with i+1
    const int es = dtype == SAR_F32 ? 4 : 2;
    const size_t size = bytes / (size_t)es;          // elements per rank, as bytes / sizeof(float) in the reference
    if (size == 0) { fprintf(stderr, "Buffer too small: %zu bytes\n", bytes); exit(EXIT_FAILURE); }

    // the schedule (host only, so a bad table is reported before any device work)
    sar_schedule* main_sched = NULL; sar_schedule* prework = NULL;
    if (strcmp(alg, "stragglar") == 0) {
        std::string text;
        if (!schedule_path.empty()) {
            if (!read_file(schedule_path, &text)) { fprintf(stderr, "Cannot read schedule: %s\n", schedule_path.c_str()); exit(EXIT_FAILURE); }
        } else if (numRanks != 4 && numRanks != 8) {
            const char* dir = getenv("SAR_SCHEDULE_DIR");
            std::string name = "/stragglar_n" + std::to_string(numRanks) + ".txt";
            std::string p1 = dir ? std::string(dir) + name : std::string(), p2 = exe_dir() + "/../schedules" + name;
            if (!(dir && read_file(p1, &text)) && !read_file(p2, &text)) {
                fprintf(stderr, "No StragglAR table for %d ranks: pass --schedule FILE (synthesizer output)\n", numRanks);
                exit(EXIT_FAILURE);
            }
        }
        if (text.empty()) CHECK_SAR(sar_schedule_builtin("stragglar", numRanks, &main_sched));
        else CHECK_SAR(sar_schedule_parse(text.data(), text.size(), numRanks, &main_sched));
        if (sleepTime >= 0) CHECK_SAR(sar_schedule_builtin("prework_rs", numRanks, &prework));
    } else {
        CHECK_SAR(sar_schedule_builtin(alg, numRanks, &main_sched));
        if (sleepTime >= 0 && strcmp(alg, "direct") == 0) CHECK_SAR(sar_schedule_builtin("prework_ar", numRanks, &prework));
    }
    char why[512];
    if (sar_schedule_validate(main_sched, why, sizeof(why)) != SAR_OK) { printf("SAR error: invalid schedule: '%s'\n", why); exit(EXIT_FAILURE); }

    // Check GPUs (allreduce_8GPU.cu:932-937; one device carries every rank here)
    int nGPUs = 0;
    if (sar_device_count(&nGPUs) != SAR_OK || nGPUs < 1) {
        printf("Need at least %d GPUs\n", 1);
        return -1;
    }

    sar_ctx* ctx = NULL;
    CHECK_SAR(sar_create(0, &ctx));
    if (sleepTime >= 0) {
        int64_t ticks = 0;
        CHECK_SAR(sar_sleep_ticks(ctx, sleepTime, &ticks));
        printf("Sleep cycles: %ld\n", (long)ticks);
    }
    if (executor >= 0) {
        sar_tuning_t tune;
        CHECK_SAR(sar_get_tuning(ctx, &tune));
        tune.executor = executor;
        CHECK_SAR(sar_set_tuning(ctx, &tune));
    }
    CHECK_SAR(sar_alloc_ranks(ctx, numRanks, (uint64_t)size * es, dtype));
    CHECK_SAR(sar_prepare(ctx, prework, main_sched, use_graph));
    sar_stats_t st;
    CHECK_SAR(sar_stats(ctx, &st));

    // the step before every timed one, on rank buffers of its own (--sequence)
    sar_ctx* before = NULL;
    if (sequence) {
        CHECK_SAR(sar_create(0, &before));
        sar_tuning_t tune;
        CHECK_SAR(sar_get_tuning(ctx, &tune));
        CHECK_SAR(sar_set_tuning(before, &tune));
        if (sar_alloc_ranks(before, numRanks, (uint64_t)size * es, dtype) != SAR_OK) {
            fprintf(stderr, "no room for a second set of rank buffers (%s): every iteration is timed behind the fill alone\n", sar_last_error());
            sar_destroy(before); before = NULL;
        } else {
            CHECK_SAR(sar_prepare(before, prework, main_sched, 0));
        }
    }
    int before_runs = 0;
    auto step_before = [&]() {
        if (!before) return;
        if (before_runs++ % 8 == 0)                      // sums of sums grow: fresh values before they overflow
            for (int r = 0; r < numRanks; ++r) CHECK_SAR(sar_fill_uniform(before, r, 101 + r, -6e-5, 6e-5));
        CHECK_SAR(sar_run(before, sleepTime, NULL));      // the same launches as the timed step
    };

    auto fill = [&]() {
        if (init == "reference") { CHECK_SAR(sar_fill_reference_pattern(ctx, alg, sleepTime, base)); return; }
        for (int r = 0; r < numRanks; ++r) {
            if (init == "uniform") CHECK_SAR(sar_fill_uniform(ctx, r, seed, -1.0, 1.0));
            else CHECK_SAR(sar_fill_normal(ctx, r, seed, 0.0, 1e-3));
        }
    };

    // warm-up (the reference exchanges chunks 10 times before timing, :993-1006)
    fill();
    for (int i = 0; i < 2; ++i) CHECK_SAR(sar_run(ctx, -1.f, NULL));

    printf("algorithm,buffer_size_bytes,iteration,delay,runtime_ms,BW(GB/s)\n");
    double sum_ms = 0; double min_ms = 1e30;
    for (int iter = 0; iter < numIters + 1; ++iter) {
        fill();
        step_before();
        float ms = 0.f;
        CHECK_SAR(sar_run(ctx, sleepTime, &ms));
        if (iter == 0) continue;
        float bw;
        if (sleepTime > 0) bw = (float)size * es / 1024.0 / 1024.0 / 1024.0 * 1000.0 / (ms - sleepTime);
        else bw = (float)size * es / 1024.0 / 1024.0 / 1024.0 * 1000.0 / ms;
        printf("%s,%zu,%d,%.3f,%.3f,%.3f\n", alg, (size_t)size * es, iter, sleepTime, ms, bw);
        double net = ms - (sleepTime > 0 ? sleepTime : 0);
        sum_ms += net; if (net < min_ms) min_ms = net;
    }
    if (report && numIters > 0) {
        // what the timed part of an iteration (runtime - delay) moves: the schedule, and the pre-work too when nobody is
        // late (delay 0: it runs in front of the schedule; with a delay it runs beside the straggler's absence)
        const bool with_prework = sleepTime == 0 && st.prework_bytes > 0;
        const bool one_launch = with_prework && st.fused_prework;
        const double algorithmic = (double)st.algorithmic_bytes + (with_prework ? (double)st.prework_bytes : 0.0);
        const double on_chip = one_launch ? (double)st.fused_forwarded_bytes + (double)st.fused_elided_store_bytes
                                          : (double)st.forwarded_bytes + (double)st.elided_store_bytes;
        const double to_memory = algorithmic - on_chip;
        double mean = sum_ms / numIters;
        fprintf(stderr, "# bytes_to_memory=%.0f mean_ms=%.4f min_ms=%.4f memory_GBps=%.1f (best %.1f) frac_of_8TBps=%.3f algorithmic_bytes=%.0f algorithmic_GBps=%.1f launches=%d graph=%d\n",
                to_memory, mean, min_ms, to_memory / mean / 1e6, to_memory / min_ms / 1e6, to_memory / mean / 1e6 / 8000.0, algorithmic, algorithmic / mean / 1e6,
                one_launch ? 1 : st.main_launches + (with_prework ? st.prework_launches : 0), st.uses_graph);
        fprintf(stderr, "# executor=%s components=%d column_threads=%d value_slots=%d taken_from_LDS_bytes=%.0f stores_left_out_bytes=%.0f prework=%s ranks_in_two_hbm_regions=%d\n",
                st.executor ? "column" : "rounds", st.col_components, st.col_block, st.col_slots,
                one_launch ? (double)st.fused_forwarded_bytes : (double)st.forwarded_bytes, one_launch ? (double)st.fused_elided_store_bytes : (double)st.elided_store_bytes,
                one_launch ? "in the same launch" : with_prework ? "in front of the schedule" : st.prework_bytes > 0 ? "beside the delay (not in these figures)" : "none",
                st.arena_spread);
    }

    // result check (allreduce_8GPU.cu:1069-1077 asserts 36.0; allreduce_4GPU.cu:593-603 prints mismatches)
    int failures = 0;
    if (init == "reference") {
        float expect = 0.f;
        for (int i = 0; i < numRanks; ++i) expect += (float)(i + base);
        std::vector<char> hostOut((size_t)size * es);
        for (int r = 0; r < numRanks; ++r) {
            CHECK_SAR(sar_download(ctx, r, 0, hostOut.data(), (uint64_t)size * es));
            for (size_t i = 0; i < size; ++i) {
                float v = load_elem(hostOut.data(), i, dtype);
                if (v != expect) {
                    if (failures < 16) printf("Rank %d, idx %zu, val %.3f\n", r, i, v);
                    ++failures;
                }
            }
        }
        if (failures && numRanks != 4) {
            // assert(hostOut[i] == 36.0) in the 8-rank reference: abort
            fflush(stdout);
            fprintf(stderr, "%s: Assertion `hostOut[i] == %.1f' failed (%d elements differ).\n", argv[0], expect, failures);
            abort();
        }
    } else if (check) {
        // the tail of size mod parts elements is never moved (chunk = size / (numRanks-1), :901)
        int same = 0, parts = sar_schedule_parts(main_sched);
        CHECK_SAR(sar_ranks_identical(ctx, (uint64_t)(size / parts) * parts, &same));
        if (!same) { printf("Rank buffers differ after the AllReduce\n"); failures = 1; }
    }

    sar_schedule_free(main_sched);
    sar_schedule_free(prework);
    sar_destroy(before);
    sar_destroy(ctx);
    for (int i = 0; i < numRanks; ++i) printf("Rank %d, done\n", i);
    return (failures && init != "reference") ? EXIT_FAILURE : 0;
}
