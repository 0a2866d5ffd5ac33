// api_internal.h -- what the translation units behind the C ABI (api.hip, api_ops.hip) share: the context and tensor
// objects, the error helpers and the context lock.
#pragma once

#include "../../include/rllama_hip.h"
#include "kernels.h"

#include <hip/hip_runtime.h>

#include <mutex>

namespace rlh {
// records the calling thread's error text (rlh_last_error) and returns `code`
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int set_error(int code, const char *msg);
} // namespace rlh

#define HIP_TRY(expr)                                                                                          \
    do {                                                                                                       \
        hipError_t _e = (expr);                                                                                \
        if (_e != hipSuccess) {                                                                                \
            return rlh::fail(_e == hipErrorOutOfMemory ? RLH_ERR_OOM : RLH_ERR_HIP, "%s failed: %s (%s:%d)",   \
                             #expr, hipGetErrorString(_e), __FILE__, __LINE__);                                \
        }                                                                                                      \
    } while (0)

// Work memory of the op-level entry points that need more than their operands (rlh_attn_decode, rlh_argmax_greedy):
// allocated on first use, kept until rlh_shutdown.
struct OpScratch {
    rlh::DecodeState *state = nullptr;
    float *attn_ws = nullptr;      // partial triples of a split sequence
    size_t attn_ws_floats = 0;
    unsigned *tickets = nullptr;   // [kOpMaxHeads]
    int32_t *token = nullptr;      // one id
    void *gemm_ws = nullptr;       // partial sums of products cut along K (kOpGemmWsBytes), as the forward's prompt path has
};
constexpr size_t kOpGemmWsBytes = (size_t)64 << 20;
constexpr int kOpMaxHeads = 1024;

struct rlh_ctx {
    int device = 0;
    int verbose = 0;
    hipStream_t stream = nullptr;
    hipDeviceProp_t prop;
    std::recursive_mutex mu;
    OpScratch ops;
    void *noalloc_scratch = nullptr; // this device's address of the library's static work memory (api_ops.hip)
};

struct rlh_tensor {
    rlh_ctx *ctx = nullptr;
    void *p = nullptr;
    int rows = 0, cols = 0, dtype = RLH_F16;
    size_t esize() const { return dtype == RLH_F16 ? 2 : 4; }
    size_t count() const { return (size_t)rows * cols; }
};

struct rlh_event {
    rlh_ctx *ctx = nullptr;
    hipEvent_t ev = nullptr;
};

struct CtxLock {
    std::lock_guard<std::recursive_mutex> g;
    explicit CtxLock(rlh_ctx *c) : g(c->mu) { (void)hipSetDevice(c->device); }
};

namespace rlh {
void ops_release(rlh_ctx *ctx); // frees the op-level work memory (rlh_shutdown)
// looks up the context's device address of the static work memory of rlh_attn_decode_noalloc; rlh_init calls it with the
// device current
int noalloc_setup(rlh_ctx *ctx);
// how many blocks per head the decode attention uses at sequence length T
int attn_splits_rule(int T, int single_max, int chunk, int max_splits);
} // namespace rlh
