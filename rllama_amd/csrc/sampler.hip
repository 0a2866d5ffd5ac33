// sampler.hip -- TokenSampler::sample (Noeda/rllama src/token_sampler.rs:83-174) on host logits.  Host code only: the
// reference samples on the CPU from the logits forward() returns, and so does this (the greedy case has a device
// argmax in misc.hip).  The arithmetic is fp32 in the reference's order; the top-k cut uses a partial sort instead
// of sorting the whole vocabulary.
#include "../../include/rllama_hip.h"

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <vector>

namespace rlh {
int set_error(int code, const char *msg); // api.hip
}

extern "C" void rlh_sampler_default(rlh_sampler_params *p) {
    if (!p) return;
    p->temperature = 0.2f; // token_sampler.rs:20-29
    p->top_p = 1.0f;
    p->top_k = 1;
    p->repetition_penalty = 0.8f;
}

namespace {

struct Cand {
    int32_t id;
    float p;
};

// descending by probability, NaN last (token_sampler.rs:131-145); equal probabilities by ascending id
inline bool before(const Cand &a, const Cand &b) {
    const bool an = std::isnan(a.p), bn = std::isnan(b.p);
    if (an || bn) return an == bn ? a.id < b.id : bn;
    if (a.p != b.p) return a.p > b.p;
    return a.id < b.id;
}

// probabilities of the whole vocabulary -> the candidates after both cuts; returns their mass
float cut(std::vector<Cand> &c, const rlh_sampler_params &sp) {
    const size_t k = sp.top_k < 0 ? 0 : std::min<size_t>((size_t)sp.top_k, c.size());
    std::partial_sort(c.begin(), c.begin() + (ptrdiff_t)k, c.end(), before);
    c.resize(k); // :147
    float acc = 0.0f;
    for (size_t i = 0; i < c.size(); i++) { // :148-155
        acc += c[i].p;
        if (acc >= sp.top_p) {
            c.resize(i + 1);
            break;
        }
    }
    float total = 0.0f;
    for (const Cand &x : c) total += x.p; // :156-159
    return total;
}

int candidates(const float *logits, int vocab, const rlh_sampler_params &sp, const int32_t *existing, int n_existing, std::vector<Cand> &c, float *total) {
    if (!logits || vocab < 1 || n_existing < 0 || (n_existing > 0 && !existing)) return rlh::set_error(RLH_ERR_INVALID, "sampler: bad argument");
    const float inv_t = sp.temperature > 0.0f ? 1.0f / sp.temperature : 1.0f; // :99-102
    const bool scale = sp.temperature > 0.0f;
    // Token 0 is the only one the penalty, "maximum" and shift loops reach (they run over the rows of a 1 x vocab tensor,
    // :105, :113, :121): l0 * penalty^count - (that same value) = 0 whenever it is finite, NaN otherwise.
    float l0 = scale ? logits[0] * inv_t : logits[0];
    if (sp.repetition_penalty != 1.0f) {
        int count = 0;
        for (int i = 0; i < n_existing; i++) count += existing[i] == 0;
        if (count > 0) l0 = l0 * powf(sp.repetition_penalty, (float)count);
    }
    const float maxv = l0 > -INFINITY ? l0 : -INFINITY;
    l0 = l0 - maxv;
    c.resize((size_t)vocab);
    float sum = 0.0f; // softmax of tensor.rs:479-494: no maximum subtracted, sequential fp32 sum
    for (int i = 0; i < vocab; i++) {
        const float e = expf(i == 0 ? l0 : (scale ? logits[i] * inv_t : logits[i]));
        c[(size_t)i] = {i, e};
        sum += e;
    }
    for (Cand &x : c) x.p = x.p / sum;
    *total = cut(c, sp);
    return RLH_OK;
}

} // namespace

extern "C" int rlh_sample_candidates(const float *logits, int vocab, const rlh_sampler_params *p, const int32_t *existing_tokens, int n_existing,
                                     int32_t *out_ids, float *out_probs, int cap, int *n_out, float *total_p) {
    if (!p || !out_ids || !out_probs || !n_out || !total_p || cap < 0) return rlh::set_error(RLH_ERR_INVALID, "rlh_sample_candidates: NULL argument");
    std::vector<Cand> c;
    float total = 0.0f;
    const int rc = candidates(logits, vocab, *p, existing_tokens, n_existing, c, &total);
    if (rc != RLH_OK) return rc;
    if (c.size() > (size_t)cap) return rlh::set_error(RLH_ERR_INVALID, "rlh_sample_candidates: more candidates than the output arrays hold");
    for (size_t i = 0; i < c.size(); i++) {
        out_ids[i] = c[i].id;
        out_probs[i] = c[i].p;
    }
    *n_out = (int)c.size();
    *total_p = total;
    return RLH_OK;
}

extern "C" int rlh_sample(const float *logits, int vocab, const rlh_sampler_params *p, const int32_t *existing_tokens, int n_existing, float u,
                          int32_t *token, float *prob) {
    if (!p || !token || !(u >= 0.0f && u <= 1.0f)) return rlh::set_error(RLH_ERR_INVALID, "rlh_sample: bad argument (u must be in [0, 1])");
    std::vector<Cand> c;
    float total = 0.0f;
    const int rc = candidates(logits, vocab, *p, existing_tokens, n_existing, c, &total);
    if (rc != RLH_OK) return rc;
    const float draw = total > 0.0f ? u * total : 0.0f; // :160-165
    float acc = 0.0f;
    for (const Cand &x : c) { // :166-172
        acc += x.p;
        if (acc >= draw) {
            *token = x.id;
            if (prob) *prob = x.p / total;
            return RLH_OK;
        }
    }
    *token = 0; // :173
    if (prob) *prob = 0.0f;
    return RLH_OK;
}
