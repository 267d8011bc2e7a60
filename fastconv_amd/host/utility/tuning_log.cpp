#include "tuning_log.h"

#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/stat.h>

const char *tuning_log_path() {
    const char *env = getenv("FASTCONV_TUNING_LOG");
    return env ? env : "./gemm_log/mi355x_tuning_log";
}

static void key_string(const TuningKey &k, char *buf, size_t len) {
    snprintf(buf, len, "%s,%d,%d,%d,%d,%d,%d,%d,%d,%d,%d,%d,%d,%d", k.algo, k.n, k.c, k.h, k.w, k.k, k.kh, k.kw, k.sh,
             k.sw, k.pt, k.pb, k.pl, k.pr);
}

bool tuning_log_lookup(const TuningKey &key, TuningEntry *entry) {
    FILE *fp = fopen(tuning_log_path(), "r");
    if (!fp) return false;
    char want[256], line[512];
    key_string(key, want, sizeof want);
    const size_t wl = strlen(want);
    bool found = false;
    while (fgets(line, sizeof line, fp)) {
        if (strncmp(line, want, wl) != 0 || line[wl] != ',') continue;
        TuningEntry e;
        if (sscanf(line + wl + 1, "%d,%d,%lf", &e.config, &e.option, &e.ms) == 3) {
            *entry = e;      // the last matching line wins: the log is append-only
            found = true;
        }
    }
    fclose(fp);
    return found;
}

bool tuning_log_append(const TuningKey &key, const TuningEntry &entry) {
    const char *path = tuning_log_path();
    if (!getenv("FASTCONV_TUNING_LOG")) mkdir("./gemm_log", 0775);
    FILE *fp = fopen(path, "a");
    if (!fp) {
        fprintf(stderr, "Warning: cannot append to tuning log %s\n", path);
        return false;
    }
    char ks[256];
    key_string(key, ks, sizeof ks);
    fprintf(fp, "%s,%d,%d,%.6f\n", ks, entry.config, entry.option, entry.ms);
    fclose(fp);
    return true;
}
