// Drives the C++ resident-index reader from the command line for the CPU tests:
//   gturbo_resident_check <model_weights.bin> [tensor name ...]
// prints the header, every entry in name order and the TensorView of each named tensor, or "error: <detail>".
#include <cstdio>

#include "../turbo-fieldfare_amd/host/tf_gturbo.hpp"

int main(int argc, char **argv) {
    if (argc < 2) return 2;
    try {
        const tf::gturbo::ResidentIndex index = tf::gturbo::loadResidentIndex(argv[1]);
        std::printf("header %llu %llu %llu\n", (unsigned long long)index.header.indexSize, (unsigned long long)index.header.residentSize,
                    (unsigned long long)index.header.entryCount);
        for (const auto &kv : index.entries) {
            const tf::gturbo::ResidentIndexEntry &e = kv.second;
            std::printf("entry %s dtype %u weights %llu+%llu shape %u %u %u %u scales %llu+%llu biases %llu+%llu\n", e.name.c_str(), e.dtype,
                        (unsigned long long)e.fileOffset, (unsigned long long)e.sizeBytes, e.shape[0], e.shape[1], e.shape[2], e.shape[3],
                        (unsigned long long)e.scaleOffset, (unsigned long long)e.scaleSize, (unsigned long long)e.biasOffset,
                        (unsigned long long)e.biasSize);
        }
        for (int i = 2; i < argc; ++i) {
            try {
                const std::string name = argv[i];
                const tf::gturbo::TensorView v = name == "@sharedExpertGate0" ? index.sharedExpertGate(0)
                                                 : name == "@router1"         ? index.router(1)
                                                 : name == "@lmHead"          ? index.lmHead()
                                                                              : index.resident(name);
                std::printf("view %s %llu %llu %llu %llu %llu %llu\n", argv[i], (unsigned long long)v.offset, (unsigned long long)v.length,
                            (unsigned long long)v.scaleOffset, (unsigned long long)v.scaleLength, (unsigned long long)v.biasOffset,
                            (unsigned long long)v.biasLength);
            } catch (const tf::gturbo::ModelError &e) {
                std::printf("view-error %d: %s\n", (int)e.kind, e.what());
            }
        }
    } catch (const tf::gturbo::ModelError &e) {
        std::printf("error %d: %s\n", (int)e.kind, e.what());
        return 1;
    } catch (const tf::gturbo::FormatError &e) {
        std::printf("format-error: %s\n", e.what());
        return 1;
    }
    return 0;
}
