#include "device.h"

#include <stdio.h>
#include <stdlib.h>

namespace fastconv {

static size_t g_pool_bytes = 0;

void Device::Configure(size_t bytes) { g_pool_bytes = bytes; }

Device &Device::Get() {
    static Device dev;
    return dev;
}

Device::Device() : ctx_(NULL), pool_(NULL) {
    int rc = fc_init(0, &ctx_);
    if (rc != FC_OK) {
        fprintf(stderr, "Error: cannot open GPU 0: %s. This build has no CPU path.\n", fc_status_string(rc));
        exit(EXIT_FAILURE);
    }
    size_t bytes = g_pool_bytes ? g_pool_bytes : ((size_t)8 << 30);
    if (const char *env = getenv("FASTCONV_POOL_BYTES")) {
        const unsigned long long v = strtoull(env, NULL, 10);
        if (v > 0) bytes = (size_t)v;
    }
    rc = fc_pool_create(ctx_, bytes, &pool_);
    if (rc != FC_OK) {
        fprintf(stderr, "Error: cannot allocate the %zu-byte device arena: %s\n", bytes, fc_last_error(ctx_));
        exit(EXIT_FAILURE);
    }
}

Device::~Device() {
    if (pool_) fc_pool_destroy(pool_);
    if (ctx_) fc_destroy(ctx_);
}

void Device::Check(int status, const char *what) {
    if (status == FC_OK) return;
    fprintf(stderr, "Error: %s failed: %s\n", what, fc_last_error(ctx_));
    exit(EXIT_FAILURE);
}

void *Device::Alloc(size_t bytes, const char *what) {
    void *p = NULL;
    const int rc = fc_pool_alloc(pool_, bytes, &p);
    if (rc != FC_OK || p == NULL) {
        fprintf(stderr, "Buffer is NULL (%s, %zu bytes): %s\n", what, bytes, fc_last_error(ctx_));
        exit(EXIT_FAILURE);
    }
    return p;
}

size_t Device::Mark() {
    size_t m = 0;
    Check(fc_pool_mark(pool_, &m), "fc_pool_mark");
    return m;
}

void Device::Release(size_t mark) { Check(fc_pool_release(pool_, mark), "fc_pool_release"); }

}  // namespace fastconv
