#include "helper.h"

#include <math.h>

float diff(float *arr1, float *arr2, int len) {
    long num = 0;
    double dif = 0.0;
    for (int i = 0; i < len; ++i) {
        const float err = fabsf(arr1[i] - arr2[i]);
        if (err > 1e-5f) {
            dif += err;
            num++;
        }
    }
    const float r = num == 0 ? 0.f : (float)(dif / num);
    LOGD("The difference is %.5f\n", r);
    return r;
}

float diff(float *arr1, float *arr2, int M, int N) {
    long num = 0;
    float dif = 0.0f;
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j) {
            const float err = fabsf(arr1[i * N + j] - arr2[i * N + j]);
            if (err > 1e-4) {
                dif += err;
                num++;
                LOGD("Error position (%d, %d), value %.4f, %.4f\n", i, j, arr1[i * N + j], arr2[i * N + j]);
            }
        }
    const float r = num == 0 ? 0.f : dif / num;
    LOGD("The difference is %.5f\n", r);
    return r;
}

double max_rel_err(const float *y, const float *ref, size_t len) {
    double maxerr = 0.0, maxref = 0.0;
    for (size_t i = 0; i < len; i++) {
        const double e = fabs((double)y[i] - (double)ref[i]);
        if (!(e <= maxerr)) maxerr = e;
        const double a = fabs((double)ref[i]);
        if (a > maxref) maxref = a;
    }
    return maxref > 0.0 ? maxerr / maxref : maxerr;
}

static double elapsed_ms(const timespec &a, const timespec &b) {
    return (b.tv_sec - a.tv_sec) * 1000.0 + (b.tv_nsec - a.tv_nsec) / 1000000.0;
}

void Timer::startBench() { clock_gettime(CLOCK_MONOTONIC, &start); }

void Timer::accumBench() {
    clock_gettime(CLOCK_MONOTONIC, &stop);
    accumulate += elapsed_ms(start, stop);
}

void Timer::printBench(const char *comment, int fold) { LOGD("%s %lfms\n", comment, accumulate / fold); }

void Timer::endBench(const char *comment) {
    clock_gettime(CLOCK_MONOTONIC, &stop);
    LOGD("%s %lfms\n", comment, elapsed_ms(start, stop));
}

double Timer::endBench(double fold) {
    clock_gettime(CLOCK_MONOTONIC, &stop);
    return elapsed_ms(start, stop) / fold;
}

void Timer::endBench(const char *comment, double fold) {
    clock_gettime(CLOCK_MONOTONIC, &stop);
    printf("%s time: %lfms\n", comment, elapsed_ms(start, stop) / fold);
}
