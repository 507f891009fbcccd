// File -> HBM uploads: one packed-experts layer file into a resident pool in logical expert order, and a byte range of a
// file (the resident payload of model_weights.bin) into one allocation.
#include <errno.h>
#include <fcntl.h>
#include <string.h>
#include <sys/stat.h>
#include <unistd.h>

#include <vector>

#include "tf_context.hpp"

using namespace tfk;

namespace {

struct Fd {
    int fd = -1;
    ~Fd() {
        if (fd >= 0) close(fd);
    }
};

struct Pinned {
    void *p = nullptr;
    ~Pinned() {
        if (p) (void)hipHostFree(p);
    }
};

struct Event {
    hipEvent_t e = nullptr;
    ~Event() {
        if (e) (void)hipEventDestroy(e);
    }
};

// reads exactly n bytes at `offset`; false on error or a short file
bool read_exact(int fd, void *dst, size_t n, uint64_t offset) {
    uint8_t *out = static_cast<uint8_t *>(dst);
    while (n > 0) {
        const ssize_t got = pread(fd, out, n, (off_t)offset);
        if (got < 0 && errno == EINTR) continue;
        if (got <= 0) return false;
        out += got;
        offset += (uint64_t)got;
        n -= (size_t)got;
    }
    return true;
}

}  // namespace

extern "C" {

int32_t tf_upload_packed_experts_layer(tf_ctx *ctx, tf_stream stream, const char *layer_file_path, uint64_t expert_stride,
                                       uint32_t num_experts, const uint32_t *physical_rank, void *device_pool) {
    TF_REQUIRE(ctx, ctx && layer_file_path && device_pool, TF_ERR_INVALID_ARGUMENT, "upload_packed_experts_layer: null argument");
    TF_REQUIRE(ctx, num_experts > 0 && expert_stride > 0 && expert_stride % 16 == 0, TF_ERR_INVALID_ARGUMENT,
               "upload_packed_experts_layer: expert stride must be a positive multiple of 16 and the layer non-empty");
    TF_REQUIRE(ctx, expert_stride <= (1ull << 32), TF_ERR_INVALID_ARGUMENT, "upload_packed_experts_layer: expert stride above 4 GiB");
    if (physical_rank) {
        std::vector<bool> seen(num_experts, false);
        for (uint32_t e = 0; e < num_experts; ++e) {
            TF_REQUIRE(ctx, physical_rank[e] < num_experts && !seen[physical_rank[e]], TF_ERR_INVALID_ARGUMENT,
                       "upload_packed_experts_layer: physical ranks are not a permutation (expert %u)", e);
            seen[physical_rank[e]] = true;
        }
    }
    Fd file;
    file.fd = open(layer_file_path, O_RDONLY | O_CLOEXEC | O_NONBLOCK);
    TF_REQUIRE(ctx, file.fd >= 0, TF_ERR_INVALID_ARGUMENT, "upload_packed_experts_layer: cannot open %s: %s", layer_file_path, strerror(errno));
    struct stat st;
    TF_REQUIRE(ctx, fstat(file.fd, &st) == 0 && S_ISREG(st.st_mode), TF_ERR_INVALID_ARGUMENT, "upload_packed_experts_layer: %s is not a regular file",
               layer_file_path);
    TF_REQUIRE(ctx, (uint64_t)st.st_size == (uint64_t)num_experts * expert_stride, TF_ERR_DIMENSION_MISMATCH,
               "upload_packed_experts_layer: %s holds %llu bytes, expected %u experts of %llu", layer_file_path, (unsigned long long)st.st_size,
               num_experts, (unsigned long long)expert_stride);
    // two pinned staging buffers: the file read of one expert overlaps the copy of the previous one
    Pinned staging[2];
    Event done[2];
    for (int i = 0; i < 2; ++i) {
        if (hipHostMalloc(&staging[i].p, expert_stride, hipHostMallocDefault) != hipSuccess) return fail(ctx, TF_ERR_OUT_OF_MEMORY, "upload_packed_experts_layer: no pinned staging memory");
        if (hipEventCreateWithFlags(&done[i].e, hipEventDisableTiming) != hipSuccess) return fail(ctx, TF_ERR_DEVICE, "upload_packed_experts_layer: event creation failed");
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    bool in_use[2] = {false, false};
    for (uint32_t e = 0; e < num_experts; ++e) {
        const int slot = (int)(e & 1u);
        if (in_use[slot] && hipEventSynchronize(done[slot].e) != hipSuccess) return fail(ctx, TF_ERR_DEVICE, "upload_packed_experts_layer: copy failed");
        const uint64_t rank = physical_rank ? physical_rank[e] : e;
        if (!read_exact(file.fd, staging[slot].p, expert_stride, rank * expert_stride)) {
            (void)hipStreamSynchronize(s);
            return fail(ctx, TF_ERR_DEVICE, "upload_packed_experts_layer: short read from %s at expert %u", layer_file_path, e);
        }
        hipError_t err = hipMemcpyAsync(static_cast<uint8_t *>(device_pool) + (uint64_t)e * expert_stride, staging[slot].p, expert_stride,
                                        hipMemcpyHostToDevice, s);
        if (err == hipSuccess) err = hipEventRecord(done[slot].e, s);
        if (err != hipSuccess) {
            (void)hipStreamSynchronize(s);
            return fail(ctx, TF_ERR_DEVICE, "upload_packed_experts_layer: %s", hipGetErrorString(err));
        }
        in_use[slot] = true;
    }
    // the staging buffers are released on return
    const hipError_t err = hipStreamSynchronize(s);
    if (err != hipSuccess) return fail(ctx, TF_ERR_DEVICE, "upload_packed_experts_layer: %s", hipGetErrorString(err));
    return TF_OK;
}

int32_t tf_upload_file_region(tf_ctx *ctx, tf_stream stream, const char *file_path, uint64_t file_offset, uint64_t bytes,
                              void *device_dst) {
    TF_REQUIRE(ctx, ctx && file_path && device_dst, TF_ERR_INVALID_ARGUMENT, "upload_file_region: null argument");
    TF_REQUIRE(ctx, bytes > 0 && file_offset <= (uint64_t)INT64_MAX && bytes <= UINT64_MAX - file_offset, TF_ERR_INVALID_ARGUMENT,
               "upload_file_region: empty or overflowing range");
    Fd file;
    file.fd = open(file_path, O_RDONLY | O_CLOEXEC | O_NONBLOCK);
    TF_REQUIRE(ctx, file.fd >= 0, TF_ERR_INVALID_ARGUMENT, "upload_file_region: cannot open %s: %s", file_path, strerror(errno));
    struct stat st;
    TF_REQUIRE(ctx, fstat(file.fd, &st) == 0 && S_ISREG(st.st_mode) && st.st_size >= 0, TF_ERR_INVALID_ARGUMENT,
               "upload_file_region: %s is not a regular file", file_path);
    // ResidentBuffer.init's bound (ResidentBuffer.swift:37-41)
    TF_REQUIRE(ctx, file_offset + bytes <= (uint64_t)st.st_size, TF_ERR_DIMENSION_MISMATCH,
               "upload_file_region: range [%llu, %llu) exceeds the %llu bytes of %s", (unsigned long long)file_offset,
               (unsigned long long)(file_offset + bytes), (unsigned long long)st.st_size, file_path);
    constexpr uint64_t kChunk = 16ull << 20;
    const uint64_t chunk = bytes < kChunk ? bytes : kChunk;
    Pinned staging[2];
    Event done[2];
    for (int i = 0; i < 2; ++i) {
        if (hipHostMalloc(&staging[i].p, chunk, hipHostMallocDefault) != hipSuccess) return fail(ctx, TF_ERR_OUT_OF_MEMORY, "upload_file_region: no pinned staging memory");
        if (hipEventCreateWithFlags(&done[i].e, hipEventDisableTiming) != hipSuccess) return fail(ctx, TF_ERR_DEVICE, "upload_file_region: event creation failed");
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    bool in_use[2] = {false, false};
    int slot = 0;
    for (uint64_t pos = 0; pos < bytes; pos += chunk, slot ^= 1) {
        const uint64_t n = bytes - pos < chunk ? bytes - pos : chunk;
        if (in_use[slot] && hipEventSynchronize(done[slot].e) != hipSuccess) return fail(ctx, TF_ERR_DEVICE, "upload_file_region: copy failed");
        if (!read_exact(file.fd, staging[slot].p, n, file_offset + pos)) {
            (void)hipStreamSynchronize(s);
            return fail(ctx, TF_ERR_DEVICE, "upload_file_region: short read from %s at byte %llu", file_path, (unsigned long long)(file_offset + pos));
        }
        hipError_t err = hipMemcpyAsync(static_cast<uint8_t *>(device_dst) + pos, staging[slot].p, n, hipMemcpyHostToDevice, s);
        if (err == hipSuccess) err = hipEventRecord(done[slot].e, s);
        if (err != hipSuccess) {
            (void)hipStreamSynchronize(s);
            return fail(ctx, TF_ERR_DEVICE, "upload_file_region: %s", hipGetErrorString(err));
        }
        in_use[slot] = true;
    }
    const hipError_t err = hipStreamSynchronize(s);   // the staging buffers are released on return
    if (err != hipSuccess) return fail(ctx, TF_ERR_DEVICE, "upload_file_region: %s", hipGetErrorString(err));
    return TF_OK;
}

}  // extern "C"
