// Drives the C++ layout reader from the command line for the CPU tests:
//   gturbo_layout_check <model directory>      prints a summary of packed_experts/layout.json, or "error: <field>: <reason>"
#include <cstdio>

#include "../turbo-fieldfare_amd/host/tf_gturbo.hpp"

int main(int argc, char **argv) {
    if (argc != 2) return 2;
    try {
        const tf::gturbo::PackedExpertsLayout layout = tf::gturbo::loadLayout(argv[1]);
        std::printf("stride %llu layers %d experts %d\n", (unsigned long long)layout.expertStride, layout.numLayers, layout.expertsPerLayer);
        for (const auto &l : layout.layers) {
            std::printf("layer %d file %s ranks", l.layer, l.file.c_str());
            for (const uint32_t r : layout.physicalRanks(l.layer)) std::printf(" %u", r);
            std::printf("\n");
            try {
                const tf::MoEExpertOffsets o = layout.routedExpertOffsets(l.layer);
                std::printf("offsets %u %u %u %u %u %u %u %u %u\n", o.gate_W_off, o.gate_s_off, o.gate_b_off, o.up_W_off, o.up_s_off, o.up_b_off,
                            o.down_W_off, o.down_s_off, o.down_b_off);
            } catch (const tf::gturbo::FormatError &e) {
                std::printf("offsets-error: %s\n", e.what());
            }
        }
        const auto &t = layout.expert(0, 0).subTensors;
        for (const auto &kv : t) std::printf("tensor %s %llu %llu %s bits %d\n", kv.first.c_str(), (unsigned long long)kv.second.offset,
                                             (unsigned long long)kv.second.size, kv.second.dtype.c_str(), kv.second.bits);
    } catch (const tf::gturbo::FormatError &e) {
        std::printf("error: %s\n", e.what());
        return 1;
    }
    return 0;
}
