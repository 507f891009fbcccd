// Exercises the C++ host mirror without a GPU: the pure-CPU grouping and the struct layouts.
#include <cassert>
#include <cstdio>
#include <cstddef>

#include "../turbo-fieldfare_amd/host/tf_host.hpp"

int main() {
    static_assert(sizeof(tf::MoEExpertOffsets) == 36, "ExpertOffsets layout");
    static_assert(sizeof(tf::PrefillTokenExpertPair) == 16, "pair layout");
    static_assert(sizeof(tf::PrefillGroupedRoutedMoEStreamedParams) == 128, "streamed params layout");
    static_assert(offsetof(tf_prefill_streamed_params, local_expert) == 28, "localExpert0 offset");
    static_assert(offsetof(tf_prefill_streamed_params, gate_W_off) == 92, "gateWOff offset");
    static_assert(offsetof(tf_prefill_streamed_params, down_b_off) == 124, "downBOff offset");
    // PrefillMoEGroupingTests.swift:6-56
    const uint32_t rows[12][4] = {{0, 3, 0, 10}, {0, 1, 1, 11}, {0, 4, 2, 12}, {1, 1, 0, 13}, {1, 3, 1, 14}, {1, 2, 2, 15},
                                  {2, 4, 0, 16}, {2, 3, 1, 17}, {2, 1, 2, 18}, {3, 5, 0, 19}, {3, 1, 1, 20}, {3, 4, 2, 21}};
    std::vector<tf::PrefillTokenExpertPair> pairs;
    for (int i = 11; i >= 0; --i) pairs.push_back({rows[i][0], rows[i][1], rows[i][2], rows[i][3]});
    const auto g = tf::PrefillMoEGrouping::groupTokenExpertPairs(pairs, 4, 3, 6, 2);
    const uint32_t want_e[12] = {1, 1, 1, 1, 2, 3, 3, 3, 4, 4, 4, 5};
    for (int i = 0; i < 12; ++i) assert(g.sortedPairs[i].expert == want_e[i]);
    assert(g.groups.size() == 5 && g.tiles.size() == 3);
    assert(g.perExpertOffsets[0] == 0xFFFFFFFFu && g.perExpertOffsets[5] == 11 && g.perExpertCounts[1] == 4);
    assert(g.tiles[1].group_start == 2 && g.tiles[1].pair_start == 5 && g.tiles[1].pair_count == 6);
    assert(g.maxPairsPerExpert() == 4 && g.maxPairsPerTile() == 6 && g.maxLiveExpertsPerTile() == 2);
    bool threw = false;
    try {
        tf::PrefillMoEGrouping::groupTokenExpertPairs({{0, 0, 0, 1}}, 1, 1, 1, 17);
    } catch (const tf::Error &e) {
        threw = e.status == TF_ERR_GROUP_INVALID_TILE_EXPERT_COUNT;
    }
    assert(threw);
    std::puts("host mirror ok");
    return 0;
}
