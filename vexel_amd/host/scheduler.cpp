// Continuous-batching scheduler above the model runtime: the step of inference/scheduler/scheduler.go:166-483
// (collectReady, formBatches, runDecodeStep, runBatchedPrefill) with the Sequence bookkeeping of
// inference/scheduler/sequence.go, and the token sampler of inference/pkg/sampler/sampler.go.
//
// Differences from the reference, each deliberate:
//  * Batch membership and order. The reference iterates a Go map (scheduler.go:213-219), so which ready sequences
//    form a batch, and in what order, changes from run to run. Here sequences are taken in ascending id.
//  * Chunked prefill. With prefill_chunk > 0 a prompt is fed in pieces of that many tokens, one piece per step, so
//    that long prompts interleave with other sequences' decode steps; 0 feeds the whole prompt at once as
//    runBatchedPrefill does. Later pieces attend through the f16 pool (runtime/block.go:875-895), so logits after
//    the prompt depend on the piece size, as they would in the reference.
//  * A finished sequence that the scheduler drops on its own (no caller removed it first) releases its KV blocks;
//    the reference only forgets it (scheduler.go:182-187), after which RemoveSequence cannot find it any more.
//  * Sampled requests draw their uniform numbers from a SplitMix64 stream seeded per sequence, not from Go's
//    math/rand (whose generator table is no part of the reference's tree). Greedy requests (temperature 0) use the
//    device argmax; in decode steps sampled requests are sampled on the device too (vh_sample_last_logits, the
//    same sums in the same order), so logits move to the host only for the token that follows a prompt.
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <map>
#include <numeric>
#include <string>
#include <vector>

#include "vexel_host.h"

extern "C" void vh_set_error(const char *text);

namespace {

int sfail(const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    vh_set_error(buf);
    return VH_ERR;
}

struct Seq {  // scheduler.Sequence (sequence.go:39-71)
    std::vector<int32_t> prompt, generated;
    int prompt_pos = 0, position = 0;
    int state = VH_SEQ_PENDING;
    int max_tokens = 0;  // 0 = the scheduler's limit
    bool sampled = false;
    float temperature = 0.f, top_p = 0.f;
    int top_k = 0;
    uint64_t rng = 0;

    bool prefill_complete() const { return prompt_pos >= (int)prompt.size(); }  // sequence.go:205-207
    bool reached_max(int global_max) const {                                      // sequence.go:196-202
        const int limit = max_tokens > 0 ? max_tokens : global_max;
        return limit > 0 && (int)generated.size() >= limit;
    }
};

float next_uniform(uint64_t *state) {  // SplitMix64, top 24 bits: [0, 1)
    uint64_t z = (*state += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return (float)(z >> 40) * (1.0f / 16777216.0f);
}

}  // namespace

struct vh_scheduler {
    vh_model *m = nullptr;
    vh_sched_config cfg{};
    vh_config mc{};
    std::map<int64_t, Seq> seqs;  // ascending id: the batch order
    std::vector<float> logits;    // host staging
};

extern "C" {

// sampler.Argmax (sampler.go:80-91): first index of the strict maximum; NaN never wins.
int vh_argmax(const float *logits, int n) {
    float best = -3.40282346638528859811704183484516925e+38f;
    int idx = 0;
    for (int i = 0; i < n; i++)
        if (logits[i] > best) {
            best = logits[i];
            idx = i;
        }
    return idx;
}

// Sampler.Sample (sampler.go:48-77) with the uniform draw r in [0, 1) given by the caller. Where probabilities tie at
// the nucleus cutoff the lower index is kept first (the reference's sort is not stable, so its choice among equal
// probabilities is unspecified).
int vh_sample(const float *logits, int n, float temperature, int top_k, float top_p, float r) {
    if (!logits || n <= 0) return -1;
    if (temperature == 0.f) return vh_argmax(logits, n);
    std::vector<float> probs((size_t)n);
    // softmax of logits / temperature (sampler.go:94-116)
    float mx = -3.40282346638528859811704183484516925e+38f;
    for (int i = 0; i < n; i++) {
        probs[i] = logits[i] / temperature;
        if (probs[i] > mx) mx = probs[i];
    }
    float sum = 0.f;
    for (int i = 0; i < n; i++) {
        probs[i] = (float)exp((double)(probs[i] - mx));
        sum += probs[i];
    }
    for (int i = 0; i < n; i++) probs[i] /= sum;
    if (top_k > 0 && top_k < n) {  // sampler.go:119-144
        std::vector<float> sorted(probs);
        std::nth_element(sorted.begin(), sorted.begin() + (top_k - 1), sorted.end(), std::greater<float>());
        const float threshold = sorted[top_k - 1];
        float s = 0.f;
        for (int i = 0; i < n; i++) {
            if (probs[i] < threshold) probs[i] = 0.f;
            else s += probs[i];
        }
        if (s > 0.f)
            for (int i = 0; i < n; i++) probs[i] /= s;
    }
    if (top_p > 0.f && top_p < 1.0f) {  // sampler.go:147-188
        std::vector<int> order((size_t)n);
        std::iota(order.begin(), order.end(), 0);
        std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return probs[a] > probs[b]; });
        float cum = 0.f;
        int cutoff = n;
        for (int i = 0; i < n; i++) {
            cum += probs[order[i]];
            if (cum > top_p) {
                cutoff = i + 1;
                break;
            }
        }
        std::vector<char> keep((size_t)n, 0);
        for (int i = 0; i < cutoff; i++) keep[order[i]] = 1;
        float s = 0.f;
        for (int i = 0; i < n; i++) {
            if (!keep[i]) probs[i] = 0.f;
            else s += probs[i];
        }
        if (s > 0.f)
            for (int i = 0; i < n; i++) probs[i] /= s;
    }
    float cum = 0.f;  // sampleFromProbs (sampler.go:191-203)
    for (int i = 0; i < n; i++) {
        cum += probs[i];
        if (r < cum) return i;
    }
    return n - 1;
}

int vh_sched_create(vh_model *m, const vh_sched_config *cfg, vh_scheduler **out) {
    if (!m || !cfg || !out) return sfail("vh_sched_create: null argument");
    if (cfg->max_batch_size < 1 || cfg->prefill_chunk < 0) return sfail("vh_sched_create: bad configuration");
    vh_scheduler *s = new vh_scheduler;
    s->m = m;
    s->cfg = *cfg;
    vh_model_get_config(m, &s->mc);
    if (cfg->max_batch_size > s->mc.max_batch)
        return delete s, sfail("max_batch_size %d exceeds the model's max_batch %d", cfg->max_batch_size, s->mc.max_batch);
    if (cfg->prefill_chunk > s->mc.max_batch)
        return delete s, sfail("prefill_chunk %d exceeds the model's max_batch %d (rows of its activation buffers)",
                               cfg->prefill_chunk, s->mc.max_batch);
    *out = s;
    return VH_OK;
}

void vh_sched_destroy(vh_scheduler *s) { delete s; }

// Scheduler.AddSequence (scheduler.go:645-677) for an already tokenized prompt; the KV sequence is created with it.
int vh_sched_add_sequence(vh_scheduler *s, int64_t seq_id, const int32_t *prompt, int n, int max_tokens) {
    if (!s || n < 0 || (n > 0 && !prompt)) return sfail("vh_sched_add_sequence: bad arguments");
    if (s->seqs.count(seq_id)) return sfail("sequence %lld already exists", (long long)seq_id);
    for (int i = 0; i < n; i++)
        if (prompt[i] < 0 || prompt[i] >= s->mc.vocab) return sfail("prompt token %d out of range", prompt[i]);
    if (vh_pool_create_sequence(s->m, seq_id) != VH_OK) return VH_ERR;
    Seq q;
    q.prompt.assign(prompt, prompt + n);
    q.max_tokens = max_tokens;
    s->seqs[seq_id] = q;
    return VH_OK;
}

// Per-request sampling (Sequence.SetSamplingParams, sequence.go:150-160): temperature 0 keeps the request greedy.
int vh_sched_set_sampling(vh_scheduler *s, int64_t seq_id, float temperature, int top_k, float top_p, uint64_t seed) {
    if (!s || !s->seqs.count(seq_id)) return sfail("unknown sequence");
    Seq &q = s->seqs[seq_id];
    q.sampled = temperature > 0.f;
    q.temperature = temperature;
    q.top_k = top_k;
    q.top_p = top_p;
    q.rng = seed;
    return VH_OK;
}

// Scheduler.RemoveSequence (scheduler.go:679-699): forgets the sequence and frees its KV blocks.
int vh_sched_remove_sequence(vh_scheduler *s, int64_t seq_id) {
    if (!s) return sfail("null scheduler");
    auto it = s->seqs.find(seq_id);
    if (it == s->seqs.end()) return VH_OK;
    s->seqs.erase(it);
    if (vh_pool_has_sequence(s->m, seq_id) > 0) return vh_pool_delete_sequence(s->m, seq_id);
    return VH_OK;
}

int vh_sched_sequence_count(const vh_scheduler *s) { return s ? (int)s->seqs.size() : 0; }

int vh_sched_state(const vh_scheduler *s, int64_t seq_id) {
    if (!s) return -1;
    auto it = s->seqs.find(seq_id);
    return it == s->seqs.end() ? -1 : it->second.state;
}

int vh_sched_position(const vh_scheduler *s, int64_t seq_id) {
    if (!s) return -1;
    auto it = s->seqs.find(seq_id);
    return it == s->seqs.end() ? -1 : it->second.position;
}

// Copies up to cap generated tokens; returns how many the sequence has, -1 if unknown.
int vh_sched_generated(const vh_scheduler *s, int64_t seq_id, int32_t *out, int cap) {
    if (!s) return -1;
    auto it = s->seqs.find(seq_id);
    if (it == s->seqs.end()) return -1;
    const std::vector<int32_t> &g = it->second.generated;
    for (int i = 0; i < (int)g.size() && i < cap; i++) out[i] = g[i];
    return (int)g.size();
}

// One Scheduler.step (scheduler.go:166-201). *tokens_out = tokens generated in this step (may be NULL).
int vh_sched_step(vh_scheduler *s, int *tokens_out) {
    if (!s) return sfail("null scheduler");
    if (tokens_out) *tokens_out = 0;
    const int V = s->mc.vocab;
    // collectReady + formBatches (scheduler.go:203-243): ready sequences in id order, at most max_batch_size
    std::vector<int64_t> batch;
    for (auto &kv : s->seqs) {
        const int st = kv.second.state;
        if ((st == VH_SEQ_PENDING || st == VH_SEQ_PREFILL || st == VH_SEQ_DECODING) && (int)batch.size() < s->cfg.max_batch_size)
            batch.push_back(kv.first);
    }
    if (batch.empty()) {  // scheduler.go:178-191: finished sequences are dropped when nothing else is left to run
        for (auto it = s->seqs.begin(); it != s->seqs.end();) {
            if (it->second.state != VH_SEQ_FINISHED) {
                ++it;
                continue;
            }
            // (the reference forgets such a sequence without releasing its KV blocks, and its RemoveSequence
            // then no longer finds it: the blocks are released here)
            if (vh_pool_has_sequence(s->m, it->first) > 0 && vh_pool_delete_sequence(s->m, it->first) != VH_OK) return VH_ERR;
            it = s->seqs.erase(it);
        }
        return VH_OK;
    }
    auto is_stop = [&](int tok) { return tok == s->cfg.eos_token; };  // scheduler.go:110-116 (primary EOS)
    vh_arch arch;
    vh_model_get_architecture(s->m, &arch);
    auto pick = [&](Seq &q, float *row, int device_argmax) {
        if (!q.sampled) return device_argmax >= 0 ? device_argmax : vh_argmax(row, V);
        if (arch.final_softcap > 0.f) {  // model.go:336-350 on the host copy (scheduler.go:772-773)
            const double cap = (double)arch.final_softcap, inv_cap = 1.0 / cap;
            for (int i = 0; i < V; i++) row[i] = (float)(cap * tanh((double)row[i] * inv_cap));
        }
        return vh_sample(row, V, q.temperature, q.top_k, q.top_p, next_uniform(&q.rng));
    };
    int produced = 0;
    // prefill (scheduler.go:255-274, 483-552): a pending sequence with prompt left is fed before any decode
    for (int64_t id : batch) {
        Seq &q = s->seqs[id];
        if ((q.state != VH_SEQ_PENDING && q.state != VH_SEQ_PREFILL) || q.prompt.empty() || q.prefill_complete()) continue;
        const int left = (int)q.prompt.size() - q.prompt_pos;
        const int n = s->cfg.prefill_chunk > 0 ? std::min(left, s->cfg.prefill_chunk) : left;
        s->logits.resize((size_t)V);
        if (vh_prefill(s->m, q.prompt.data() + q.prompt_pos, n, id, q.prompt_pos, 0, s->logits.data()) != VH_OK) return VH_ERR;
        q.prompt_pos += n;
        q.position = q.prompt_pos;  // SetPrefillComplete (sequence.go:211-214) once the last piece is in
        if (!q.prefill_complete()) {
            q.state = VH_SEQ_PREFILL;
            continue;
        }
        const int tok = pick(q, s->logits.data(), -1);  // the first generated token comes from the prompt's last logits
        q.generated.push_back(tok);
        produced++;
        q.state = is_stop(tok) ? VH_SEQ_FINISHED : VH_SEQ_DECODING;  // scheduler.go:530-551 (no length check here)
    }
    // decode (scheduler.go:276-303): everything that is decoding now, the just-prefilled sequences included
    std::vector<int64_t> ids;
    std::vector<int32_t> tokens, positions;
    bool need_logits = false;
    for (int64_t id : batch) {
        Seq &q = s->seqs[id];
        if (!(q.state == VH_SEQ_DECODING || (q.state == VH_SEQ_PENDING && q.prefill_complete()))) continue;
        int tok = 1, pos = 0;  // BOS fallback (scheduler.go:293-296)
        if (!q.generated.empty()) {  // Sequence.NextInputToken (sequence.go:116-133)
            tok = q.generated.back();
            pos = q.position;
        }
        ids.push_back(id);
        tokens.push_back(tok);
        positions.push_back(pos);
        need_logits = need_logits || q.sampled;
    }
    if (!ids.empty()) {
        const int b = (int)ids.size();
        std::vector<int32_t> am((size_t)b);
        if (vh_decode_batched(s->m, tokens.data(), ids.data(), positions.data(), b, nullptr, am.data()) != VH_OK) return VH_ERR;
        if (need_logits) {  // sampled requests: the sampler runs on the device, on the logits the step left there
            std::vector<float> temp((size_t)b, 0.f), tp((size_t)b, 0.f), uni((size_t)b, 0.f);
            std::vector<int32_t> tk((size_t)b, 0);
            for (int i = 0; i < b; i++) {
                Seq &q = s->seqs[ids[i]];
                if (!q.sampled) continue;  // temperature 0: the greedy choice
                temp[i] = q.temperature, tk[i] = q.top_k, tp[i] = q.top_p, uni[i] = next_uniform(&q.rng);
            }
            if (vh_sample_last_logits(s->m, b, temp.data(), tk.data(), tp.data(), uni.data(), am.data()) != VH_OK) return VH_ERR;
        }
        for (int i = 0; i < b; i++) {  // scheduler.go:404-456
            Seq &q = s->seqs[ids[i]];
            q.position++;  // AdvancePosition (the prompt is complete here)
            if (q.state == VH_SEQ_PENDING) q.state = VH_SEQ_DECODING;
            const int tok = am[i];
            q.generated.push_back(tok);
            produced++;
            if (is_stop(tok) || q.reached_max(s->cfg.max_tokens)) q.state = VH_SEQ_FINISHED;
        }
    }
    if (tokens_out) *tokens_out = produced;
    return VH_OK;
}

}  // extern "C"
