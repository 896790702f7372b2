// Host-side block selection for eviction (no device code): ADAPTIVE_RKV block calculator, KVCrush steps and
// their C entry points.
#include "pa_select.h"

#include <algorithm>
#include <numeric>
#include <queue>
#include <string>

#include "../../include/pa_amd.h"

namespace pa {

namespace {
struct Scored {
    double score;
    size_t block;
    bool operator<(const Scored& r) const { return score < r.score; }
};
}  // namespace

std::set<size_t> RkvBlockCalculator::diversity_block_set(size_t max_kept, const double* scores, size_t n,
                                                         size_t* kept) const {
    std::priority_queue<Scored> by_score;
    double total = 0.0;
    for (size_t i = 0; i < n; ++i) {
        total += scores[i];
        by_score.push({scores[i], i});
    }
    const double wanted = total * attention_mass;
    double have = 0.0;
    size_t taken = 0;
    while (have < wanted && !by_score.empty() && taken < max_kept) {
        have += by_score.top().score;
        by_score.pop();
        ++taken;
    }
    std::set<size_t> others;
    for (; !by_score.empty(); by_score.pop()) others.insert(by_score.top().block);
    *kept = taken;
    return others;
}

bool RkvBlockCalculator::filtered_block_diversity(const double* unfiltered, size_t n_values, size_t eviction_size,
                                                  const std::set<size_t>& set, std::vector<double>& out) const {
    if (block_size == 0 || eviction_size % block_size) return false;
    const size_t rows = eviction_size / block_size;
    if (n_values != rows * eviction_size || set.size() * block_size > n_values) return false;
    out.assign(rows, 0.0);
    const double denom = (double)(set.size() * block_size);
    for (size_t r = 0; r < rows; ++r) {
        const double* row = unfiltered + r * eviction_size;
        double acc = 0.0;
        for (size_t b : set) {  // ascending block order, each block summed on its own first
            if (b >= rows) continue;  // counted in the mean's size, as a set member without columns
            double part = 0.0;
            for (size_t j = 0; j < block_size; ++j) part += row[b * block_size + j];
            acc += part;
        }
        out[r] = acc / denom;
    }
    return true;
}

std::set<size_t> RkvBlockCalculator::most_diverse_blocks(size_t left, const std::set<size_t>& set,
                                                         const double* filtered) const {
    std::priority_queue<Scored> by_diversity;
    for (size_t b : set) by_diversity.push({filtered[b], b});
    std::set<size_t> out;
    while (out.size() < left && !by_diversity.empty()) {
        out.insert(by_diversity.top().block);
        by_diversity.pop();
    }
    return out;
}

void KvCrushSelector::init(size_t budget_, int32_t anchor_mode_, size_t seed, size_t block_size_) {
    budget = budget_;
    anchor_mode = anchor_mode_;
    block_size = block_size_;
    rng = std::mt19937(seed);
}

std::vector<uint8_t> KvCrushSelector::indicators(size_t n_tokens, const double* scores) const {
    std::vector<size_t> order(n_tokens);
    std::iota(order.begin(), order.end(), 0);
    const size_t half = n_tokens / 2;
    std::partial_sort(order.begin(), order.begin() + half, order.end(),
                      [scores](size_t i, size_t j) { return scores[i] > scores[j]; });
    std::vector<uint8_t> bits(n_tokens, 0);
    for (size_t i = 0; i < half; ++i) bits[order[i]] = 1;
    return bits;
}

bool KvCrushSelector::anchor_point(size_t n_tokens, const uint8_t* ind, std::vector<uint8_t>& anchor) {
    anchor.assign(block_size, 0);
    switch (anchor_mode) {
    case ANCHOR_RANDOM: {
        std::uniform_int_distribution<int> coin(0, 1);
        std::generate(anchor.begin(), anchor.end(), [&]() { return (uint8_t)coin(rng); });
        return true;
    }
    case ANCHOR_ZEROS:
        return true;
    case ANCHOR_ONES:
        std::fill(anchor.begin(), anchor.end(), (uint8_t)1);
        return true;
    case ANCHOR_MEAN: {  // majority bit per in-block position
        const size_t blocks = n_tokens / block_size;
        for (size_t pos = 0; pos < block_size; ++pos) {
            size_t ones = 0;
            for (size_t b = 0; b < blocks; ++b) ones += ind[b * block_size + pos];
            anchor[pos] = (double)ones / (double)blocks > 0.5 ? 1 : 0;
        }
        return true;
    }
    case ANCHOR_ALTERNATING:
        for (size_t i = 0; i < block_size; ++i) anchor[i] = (uint8_t)(i % 2);
        return true;
    default:
        return false;
    }
}

std::vector<size_t> KvCrushSelector::hamming(size_t n_tokens, const uint8_t* ind, const uint8_t* anchor) const {
    const size_t blocks = n_tokens / block_size;
    std::vector<size_t> dist(blocks, 0);
    for (size_t b = 0; b < blocks; ++b)
        for (size_t j = 0; j < block_size; ++j) dist[b] += ind[b * block_size + j] != anchor[j] ? 1 : 0;
    return dist;
}

std::vector<size_t> KvCrushSelector::representative(const size_t* distances, size_t n_blocks,
                                                    const std::vector<size_t>& eligible) const {
    std::vector<uint8_t> is_eligible(n_blocks, 0);
    for (size_t b : eligible)
        if (b < n_blocks) is_eligible[b] = 1;
    std::vector<size_t> cand;
    cand.reserve(eligible.size());
    for (size_t b = 0; b < n_blocks; ++b)
        if (is_eligible[b]) cand.push_back(b);
    std::sort(cand.begin(), cand.end(), [distances](size_t a, size_t b) { return distances[a] < distances[b]; });
    const size_t keep = std::min(cand.size(), budget);
    std::vector<size_t> out;
    if (keep == 0) return out;
    const size_t stride = cand.size() / keep;
    for (size_t i = 0; i < keep; ++i)
        if (i * stride < cand.size()) out.push_back(cand[i * stride]);
    return out;
}

std::vector<size_t> KvCrushSelector::blocks_to_retain(size_t n_tokens, const std::vector<size_t>& evicted,
                                                      const double* scores) {
    const std::vector<uint8_t> bits = indicators(n_tokens, scores);
    std::vector<uint8_t> anchor;
    if (!anchor_point(n_tokens, bits.data(), anchor)) return {};
    const std::vector<size_t> dist = hamming(n_tokens, bits.data(), anchor.data());
    return representative(dist.data(), dist.size(), evicted);
}

}  // namespace pa

struct pa_kvcrush {
    pa::KvCrushSelector sel;
    std::string error;
};

namespace {
thread_local std::string g_select_error;

int32_t fail(pa_kvcrush* k, int32_t code, const char* msg) {
    if (k) k->error = msg; else g_select_error = msg;
    return code;
}
}  // namespace

extern "C" {

const char* pa_select_last_error(void) { return g_select_error.c_str(); }

int32_t pa_adaptive_rkv_diversity_block_set(double attention_mass, uint64_t max_num_blocks_kept,
                                            const double* block_scores, uint64_t num_blocks, uint64_t* set_out,
                                            uint64_t* set_count, uint64_t* num_blocks_kept) {
    if ((num_blocks && (!block_scores || !set_out)) || !set_count || !num_blocks_kept)
        return fail(nullptr, PA_INVALID_C_PARAM, "null argument");
    try {
        const pa::RkvBlockCalculator calc{attention_mass, 1};
        size_t kept = 0;
        const std::set<size_t> rest = calc.diversity_block_set(max_num_blocks_kept, block_scores, num_blocks, &kept);
        std::copy(rest.begin(), rest.end(), set_out);
        *set_count = rest.size();
        *num_blocks_kept = kept;
        return PA_OK;
    } catch (const std::exception& e) {
        return fail(nullptr, PA_UNKNOWN_EXCEPTION, e.what());
    }
}

int32_t pa_adaptive_rkv_filtered_block_diversity(uint64_t block_size, const double* unfiltered, uint64_t num_values,
                                                 uint64_t eviction_size, const uint64_t* set, uint64_t set_count,
                                                 double* out) {
    if (!unfiltered || !out || (set_count && !set)) return fail(nullptr, PA_INVALID_C_PARAM, "null argument");
    try {
        const pa::RkvBlockCalculator calc{0.0, (size_t)block_size};
        std::vector<double> r;
        if (!calc.filtered_block_diversity(unfiltered, num_values, eviction_size, std::set<size_t>(set, set + set_count), r))
            return fail(nullptr, PA_PARAMETER_MISMATCH,
                        "diversity must hold eviction_size / block_size rows of eviction_size values, eviction_size a "
                        "multiple of block_size, and the set must name blocks inside it");
        std::copy(r.begin(), r.end(), out);
        return PA_OK;
    } catch (const std::exception& e) {
        return fail(nullptr, PA_UNKNOWN_EXCEPTION, e.what());
    }
}

int32_t pa_adaptive_rkv_most_diverse_blocks(uint64_t num_blocks_left_to_fill, const uint64_t* set, uint64_t set_count,
                                            const double* filtered, uint64_t num_filtered, uint64_t* out,
                                            uint64_t* out_count) {
    if (!out_count || (set_count && (!set || !filtered || !out))) return fail(nullptr, PA_INVALID_C_PARAM, "null argument");
    if (num_blocks_left_to_fill > set_count)
        return fail(nullptr, PA_PARAMETER_MISMATCH, "more blocks left to fill than the diversity set holds");
    for (uint64_t i = 0; i < set_count; ++i)
        if (set[i] >= num_filtered) return fail(nullptr, PA_OUT_OF_BOUNDS, "set names a block without a diversity value");
    try {
        const pa::RkvBlockCalculator calc{0.0, 1};
        const std::set<size_t> r = calc.most_diverse_blocks(num_blocks_left_to_fill, std::set<size_t>(set, set + set_count), filtered);
        std::copy(r.begin(), r.end(), out);
        *out_count = r.size();
        return PA_OK;
    } catch (const std::exception& e) {
        return fail(nullptr, PA_UNKNOWN_EXCEPTION, e.what());
    }
}

int32_t pa_kvcrush_create(uint64_t budget, int32_t anchor_point_mode, uint64_t rng_seed, uint64_t block_size,
                          pa_kvcrush** out) {
    if (!out) return fail(nullptr, PA_INVALID_C_PARAM, "out is null");
    *out = nullptr;
    if (block_size == 0) return fail(nullptr, PA_PARAMETER_MISMATCH, "block_size must be non-zero");
    if (anchor_point_mode < pa::ANCHOR_RANDOM || anchor_point_mode > pa::ANCHOR_ALTERNATING)
        return fail(nullptr, PA_PARAMETER_MISMATCH, "Invalid anchor point type");
    pa_kvcrush* k = new (std::nothrow) pa_kvcrush();
    if (!k) return fail(nullptr, PA_NOT_ALLOCATED, "host allocation failed");
    k->sel.init(budget, anchor_point_mode, rng_seed, block_size);
    *out = k;
    return PA_OK;
}

void pa_kvcrush_destroy(pa_kvcrush* k) { delete k; }
const char* pa_kvcrush_last_error(const pa_kvcrush* k) { return k ? k->error.c_str() : g_select_error.c_str(); }

int32_t pa_kvcrush_create_indicators(pa_kvcrush* k, uint64_t num_tokens, const double* layer_scores, uint64_t num_scores,
                                     uint8_t* indicators_out) {
    if (!k) return PA_INVALID_C_PARAM;
    if (num_tokens && (!layer_scores || !indicators_out)) return fail(k, PA_INVALID_C_PARAM, "null argument");
    if (num_scores < num_tokens) return fail(k, PA_OUT_OF_BOUNDS, "fewer scores than tokens in the evictable blocks");
    try {
        const std::vector<uint8_t> bits = k->sel.indicators(num_tokens, layer_scores);
        std::copy(bits.begin(), bits.end(), indicators_out);
        return PA_OK;
    } catch (const std::exception& e) {
        return fail(k, PA_UNKNOWN_EXCEPTION, e.what());
    }
}

int32_t pa_kvcrush_create_anchor_point(pa_kvcrush* k, uint64_t num_tokens, const uint8_t* indicators, uint8_t* anchor_out) {
    if (!k) return PA_INVALID_C_PARAM;
    if (!anchor_out || (num_tokens && !indicators)) return fail(k, PA_INVALID_C_PARAM, "null argument");
    try {
        std::vector<uint8_t> anchor;
        if (!k->sel.anchor_point(num_tokens, indicators, anchor)) return fail(k, PA_PARAMETER_MISMATCH, "Invalid anchor point type");
        std::copy(anchor.begin(), anchor.end(), anchor_out);
        return PA_OK;
    } catch (const std::exception& e) {
        return fail(k, PA_UNKNOWN_EXCEPTION, e.what());
    }
}

int32_t pa_kvcrush_hamming_distances(pa_kvcrush* k, uint64_t num_tokens, const uint8_t* indicators, const uint8_t* anchor,
                                     uint64_t* distances_out) {
    if (!k) return PA_INVALID_C_PARAM;
    if (!anchor || (num_tokens && (!indicators || !distances_out))) return fail(k, PA_INVALID_C_PARAM, "null argument");
    try {
        const std::vector<size_t> d = k->sel.hamming(num_tokens, indicators, anchor);
        std::copy(d.begin(), d.end(), distances_out);
        return PA_OK;
    } catch (const std::exception& e) {
        return fail(k, PA_UNKNOWN_EXCEPTION, e.what());
    }
}

int32_t pa_kvcrush_representative_blocks(pa_kvcrush* k, const uint64_t* distances, uint64_t num_blocks,
                                         const uint64_t* eligible, uint64_t num_eligible, uint64_t* out,
                                         uint64_t* out_count) {
    if (!k) return PA_INVALID_C_PARAM;
    if (!out_count || (num_blocks && !distances) || (num_eligible && (!eligible || !out)))
        return fail(k, PA_INVALID_C_PARAM, "null argument");
    try {
        std::vector<size_t> d(distances, distances + num_blocks);
        const std::vector<size_t> r = k->sel.representative(d.data(), d.size(), std::vector<size_t>(eligible, eligible + num_eligible));
        std::copy(r.begin(), r.end(), out);
        *out_count = r.size();
        return PA_OK;
    } catch (const std::exception& e) {
        return fail(k, PA_UNKNOWN_EXCEPTION, e.what());
    }
}

int32_t pa_kvcrush_blocks_to_retain(pa_kvcrush* k, uint64_t num_tokens, const uint64_t* evicted, uint64_t num_evicted,
                                    const double* layer_scores, uint64_t num_scores, uint64_t* out, uint64_t* out_count) {
    if (!k) return PA_INVALID_C_PARAM;
    if (!out_count || (num_evicted && (!evicted || !out)) || (num_tokens && !layer_scores))
        return fail(k, PA_INVALID_C_PARAM, "null argument");
    if (num_scores < num_tokens) return fail(k, PA_OUT_OF_BOUNDS, "fewer scores than tokens in the evictable blocks");
    try {
        const std::vector<size_t> r = k->sel.blocks_to_retain(num_tokens, std::vector<size_t>(evicted, evicted + num_evicted), layer_scores);
        std::copy(r.begin(), r.end(), out);
        *out_count = r.size();
        return PA_OK;
    } catch (const std::exception& e) {
        return fail(k, PA_UNKNOWN_EXCEPTION, e.what());
    }
}

}  // extern "C"
