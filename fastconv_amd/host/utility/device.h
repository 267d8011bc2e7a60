// Process-wide GPU state of the host layers: one fc_context (one stream) and
// one arena, the single hipMalloc that backs every device buffer of every layer
// and both memory pools.  The reference has no such object (its layers malloc);
// this is where its process-wide OpenMP state (conv_layer.h:31) went.
#pragma once

#include <stddef.h>

#include "fastconv_hip.h"

namespace fastconv {

class Device {
   public:
    // Arena size used when the first layer is built: FASTCONV_POOL_BYTES if set,
    // else `bytes` from Configure(), else 8 GiB.
    static void Configure(size_t bytes);
    static Device &Get();

    fc_context *ctx() { return ctx_; }
    fc_pool *pool() { return pool_; }

    // exit(EXIT_FAILURE) with the library's message on any error, as the
    // reference does on a NULL buffer (convLayer/winoF63ConvZC.cpp:203-206).
    void *Alloc(size_t bytes, const char *what);
    void Check(int status, const char *what);
    size_t Mark();
    void Release(size_t mark);

   private:
    Device();
    ~Device();
    fc_context *ctx_;
    fc_pool *pool_;
};

}  // namespace fastconv
