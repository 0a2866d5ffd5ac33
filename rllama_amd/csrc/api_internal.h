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

// The library's switches.  Read from the environment (RLLAMA_HIP_<NAME>) once, when the context is made, and changed
// afterwards only through rlh_set_option under the context lock: no launch path reads the environment.
struct Tunables {
    rlh::GemmTune gemm{};
    int gemv_burst_fixed = 0;      // GEMV_BURST=0: single-row products always issue bursts of 8 loads per lane
    int attn_chunk = -1;           // ATTN_CHUNK: positions per workgroup of a split sequence: N >= 16, 0 = 128, -1 = about one workgroup per compute unit
    int attn_single_max = 384;     // ATTN_SINGLE_MAX=N: longest sequence one workgroup per head handles alone
    int attn_merge_mode = 2;       // ATTN_MERGE=0: the pieces of a split sequence are combined by a second launch; 2: inside the kernel
    int attn_lds = 0;              // ATTN_LDS=1: cache rows staged through LDS (comparison form)
    int prefill_attn_gemm = 0;     // PREFILL_ATTN=gemm: multi-token attention as two batched GEMMs around a softmax kernel
    int prefill_attn_order = 2;    // PREFILL_ATTN_ORDER=0/1/2: launch order of the query blocks of the one-kernel attention
    int decode_graph = 0;          // DECODE_GRAPH=1: greedy decode loops replay one captured HIP graph per token
    int decode_fold = 1;           // DECODE_FOLD=0: embedding row and greedy pick as launches of their own instead of inside the first and last product of a token step
};

namespace rlh {
// applies NAME=value (value nullptr: back to the default); false if the name or the value is not known
bool tunables_set(Tunables &t, const char *name, const char *value);
void tunables_from_env(Tunables &t);
} // namespace rlh

struct rlh_ctx {
    int device = 0;
    int verbose = 0;
    hipStream_t stream = nullptr;
    hipDeviceProp_t prop;
    std::recursive_mutex mu;
    OpScratch ops;
    Tunables tun;
    unsigned tun_version = 0;        // bumped by rlh_set_option: captured decode steps of an older version are dropped
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
int attn_splits_rule(int T, int n_heads, int compute_units, int single_max, int chunk, int max_splits);
} // namespace rlh
