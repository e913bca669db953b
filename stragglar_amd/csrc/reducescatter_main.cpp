// reducescatter <NUM_BYTES> <ITERS> [--ranks N] [--dtype T]
//
// Times the pre-work alone: the in-place ReduceScatter among the n-1 ranks
// that are on time.  Same contract as the reference's stand-alone
// stragglar/reducescatter.cu (:36-132): two positional arguments, rank i
// filled with i+1 before every iteration, iteration 0 unreported, rows
// "<bytes>,<iter>,<ms>,<GiB/s>" without a header.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

#include "sar.h"

#define CHECK_SAR(call) do { if ((call) != SAR_OK) { printf("SAR error: %s: '%s'\n", #call, sar_last_error()); exit(EXIT_FAILURE); } } while (0)

int main(int argc, char* argv[]) {
    int npos = 0;
    while (1 + npos < argc && strncmp(argv[1 + npos], "--", 2) != 0) ++npos;
    if (argc < 3 || npos != 2) {
        fprintf(stderr, "Usage: %s <bufferSize> <numIters>\n", argv[0]);
        exit(EXIT_FAILURE);
    }
    size_t bytes = (size_t)strtoull(argv[1], NULL, 10);
    int numIters = atoi(argv[2]);
    int numRanks = 8, dtype = SAR_F32;
    for (int i = 3; i < argc; ++i) {
        std::string a = argv[i];
        if (a == "--ranks" && i + 1 < argc) numRanks = atoi(argv[++i]);
        else if (a == "--dtype" && i + 1 < argc) {
            std::string t = argv[++i];
            if (t == "f32") dtype = SAR_F32; else if (t == "f16") dtype = SAR_F16; else if (t == "bf16") dtype = SAR_BF16;
            else { fprintf(stderr, "Invalid dtype: %s\n", t.c_str()); exit(EXIT_FAILURE); }
        } else { fprintf(stderr, "Unknown option: %s\n", a.c_str()); exit(EXIT_FAILURE); }
    }
    if (numRanks < 3 || numRanks > SAR_MAX_RANKS) { fprintf(stderr, "Invalid rank count: %d\n", numRanks); exit(EXIT_FAILURE); }
    const int es = dtype == SAR_F32 ? 4 : 2;
    const size_t size = bytes / (size_t)es;
    if (size == 0) { fprintf(stderr, "Buffer too small: %zu bytes\n", bytes); exit(EXIT_FAILURE); }

    int nGPUs = 0;
    if (sar_device_count(&nGPUs) != SAR_OK || nGPUs < 1) {
        printf("Need at least %d GPUs\n", 1);
        return -1;
    }
    sar_schedule* rs = NULL;
    CHECK_SAR(sar_schedule_builtin("prework_rs", numRanks, &rs));
    sar_ctx* ctx = NULL;
    CHECK_SAR(sar_create(0, &ctx));
    CHECK_SAR(sar_alloc_ranks(ctx, numRanks, (uint64_t)size * es, dtype));
    CHECK_SAR(sar_prepare(ctx, NULL, rs, 0));
    for (int iter = 0; iter < numIters + 1; ++iter) {
        for (int i = 0; i < numRanks; ++i) CHECK_SAR(sar_fill_const(ctx, i, 0, size, (double)(i + 1)));
        float ms = 0.f;
        CHECK_SAR(sar_run(ctx, -1.f, &ms));
        if (iter == 0) continue;
        float bw = (float)size * es / 1024.0 / 1024.0 / 1024.0 * 1000.0 / ms;
        printf("%zu,%d,%.3f,%.3f\n", (size_t)size * es, iter, ms, bw);
    }
    sar_schedule_free(rs);
    sar_destroy(ctx);
    return 0;
}
