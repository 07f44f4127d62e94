// Test infrastructure only: exposes the reference's own host-compilable combine reduction
// (csrc/backends/ascend/elastic/combine_state.hpp, `combine_reduce_origin_records`, compiled from the
// reference tree where it lies) through a C interface so that tests can run it on their own inputs.
// Built by oracle/Makefile into oracle/_ref/, only when the reference tree is present.
#include <cstdint>

#include "csrc/backends/ascend/elastic/combine_state.hpp"

using namespace deep_ep::ascend::elastic;

namespace {

struct Record {
    CombineRecordHeader header{};
    const float* activations = nullptr;      // [hidden]
    const float* routing_weights = nullptr;  // [num_topk]
};

struct Range {
    const Record* records = nullptr;
    std::uint64_t count = 0;
};

struct Records {
    const Range* ranges;
    std::uint64_t record_count(std::uint64_t contributor_rank) const { return ranges[contributor_rank].count; }
    CombineOriginRecordView record_at(std::uint64_t contributor_rank, std::uint64_t slot, std::uint64_t hidden) const {
        const Record& r = ranges[contributor_rank].records[slot];
        return {r.header, r.activations[hidden], r.routing_weights};
    }
};

}  // namespace

// One origin token.  Contributions are listed per contributor rank: for rank r, `counts[r]` records starting
// at `offsets[r]`; record i carries lane `lanes[i]` and `hidden` fp32 activations (bf16 values widened).
// route[k] is the token's expert id per lane (-1 = none).  Returns the fp32 result of column `column`.
extern "C" float ref_combine_reduce_column(int num_ranks, const int* offsets, const int* counts, const int* lanes,
                                           const float* activations, int hidden, const std::int64_t* route,
                                           int num_topk, int num_experts, int column, float bias0, float bias1) {
    const std::int32_t origin_token = 0;   // `route` holds this one token's lanes
    Record records[64];
    Range ranges[16];
    const float no_weights[32] = {};
    if (num_ranks > 16) return 0.0f / 0.0f;
    for (int r = 0; r < num_ranks; ++r) {
        for (int i = offsets[r]; i < offsets[r] + counts[r]; ++i) {
            records[i].header = CombineRecordHeader{kCombineRecordAbiVersion, sizeof(CombineRecordHeader),
                                                    origin_token, r, lanes[i], lanes[i]};
            records[i].activations = activations + static_cast<std::int64_t>(i) * hidden;
            records[i].routing_weights = no_weights;
        }
        ranges[r] = Range{records + offsets[r], static_cast<std::uint64_t>(counts[r])};
    }
    const Records source{ranges};
    return combine_reduce_origin_records(source, num_ranks, origin_token, route, num_topk, num_experts, num_experts / num_ranks,
                                         false, false, column, bias0, bias1, nullptr);
}
