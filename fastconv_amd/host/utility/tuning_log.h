// Append-only text log of tuning results, one CSV line per (algorithm, layer
// shape, batch): the role of ./gemm_log/linux_tuning_log in the reference
// (convLayer/im2colConv.cpp:66-92 lookup, :202-222 append), keyed by the full
// layer geometry instead of (M, N, K).
#pragma once

#include <string>

struct TuningKey {
    const char *algo;   // "winograd_zc", "winograd_blocked", "im2col"
    int n, c, h, w, k, kh, kw, sh, sw, pt, pb, pl, pr;
};

struct TuningEntry {
    int config;      // tile-shape id of the GEMM stage / implicit GEMM
    int option;      // winograd_zc: filter transform offline (1) / online (0);
                     // winograd_blocked: 2 * images per block + the same flag; im2col: unused
    double ms;       // best time per Forward
};

const char *tuning_log_path();
bool tuning_log_lookup(const TuningKey &key, TuningEntry *entry);
bool tuning_log_append(const TuningKey &key, const TuningEntry &entry);
