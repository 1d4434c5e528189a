// `.aeon` expert container reader and the load-time pipeline that turns its payloads into
// HBM-resident experts in the wave64 packing. Host code; the only device work is the repack
// kernel the layout file provides.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cerrno>
#include <cstring>
#include <vector>

#include "common.hpp"

struct aeon_expert_catalog {
    uint32_t version = 0;
    uint32_t layers = 0;
    uint32_t experts_per_layer = 0;
    uint64_t payload_bytes = 0;
    std::vector<uint64_t> offsets;  // [layers * experts_per_layer]
    int fd = -1;
    const uint8_t* base = nullptr;
    size_t file_bytes = 0;
};

namespace aeon355 {

namespace {

constexpr size_t kIndexHeaderBytes = 32;
constexpr size_t kIndexEntryBytes = 16;
constexpr char kIndexMagic[12] = {'A', 'E', 'O', 'N', '_', 'E', 'X', 'P', 'E', 'R', 'T', 'S'};

uint32_t read_u32(const uint8_t* p) {
    uint32_t v;
    std::memcpy(&v, p, sizeof v);
    return v;
}
uint64_t read_u64(const uint8_t* p) {
    uint64_t v;
    std::memcpy(&v, p, sizeof v);
    return v;
}

int read_whole_file(const char* path, std::vector<uint8_t>* out) {
    const int fd = ::open(path, O_RDONLY);
    AEON_REQUIRE(fd >= 0, AEON_ERR_IO, "cannot open expert index %s: %s", path, std::strerror(errno));
    struct stat st;
    if (::fstat(fd, &st) != 0) {
        ::close(fd);
        set_error("cannot stat expert index %s", path);
        return AEON_ERR_IO;
    }
    out->resize(static_cast<size_t>(st.st_size));
    size_t got = 0;
    while (got < out->size()) {
        const ssize_t n = ::read(fd, out->data() + got, out->size() - got);
        if (n <= 0) break;
        got += static_cast<size_t>(n);
    }
    ::close(fd);
    AEON_REQUIRE(got == out->size(), AEON_ERR_IO, "incomplete read of expert index %s", path);
    return AEON_OK;
}

size_t round_up(size_t v, size_t to) { return (v + to - 1) / to * to; }

// Slot layout of the resident pool: [W1 packed | W1 scale | W3 packed | W3 scale | W2 packed |
// W2 scale], each sub-tensor 256-byte aligned, the slot 4096-byte aligned.
struct SlotLayout {
    size_t offset[6];
    size_t bytes;
};

SlotLayout slot_layout(int hidden, int intermediate, int scale_group) {
    const size_t sizes[6] = {
        aeon_a64_packed_bytes(intermediate, hidden), aeon_a64_scale_bytes(intermediate, hidden, scale_group),
        aeon_a64_packed_bytes(intermediate, hidden), aeon_a64_scale_bytes(intermediate, hidden, scale_group),
        aeon_a64_packed_bytes(hidden, intermediate), aeon_a64_scale_bytes(hidden, intermediate, scale_group)};
    SlotLayout l{};
    size_t at = 0;
    for (int i = 0; i < 6; ++i) {
        l.offset[i] = at;
        at += round_up(sizes[i], 256);
    }
    l.bytes = round_up(at, 4096);
    return l;
}

int check_expert_shape(int hidden, int intermediate, const char* who) {
    AEON_REQUIRE(hidden > 0 && intermediate > 0 && hidden % 256 == 0 && intermediate % 256 == 0,
                 AEON_ERR_INVALID_ARGUMENT,
                 "%s: hidden and intermediate must be positive multiples of 256 (the swizzle's "
                 "8x4 and 4x8 blocks of 32 columns, the packing's 128-column groups); got %d, %d",
                 who, hidden, intermediate);
    return AEON_OK;
}

}  // namespace

}  // namespace aeon355

using namespace aeon355;

extern "C" int aeon_expert_catalog_open(const char* index_path, const char* experts_path,
                                        uint32_t expected_version, uint32_t sector_size,
                                        aeon_expert_catalog** out) {
    const char* who = "aeon_expert_catalog_open";
    AEON_REQUIRE(index_path && experts_path && out, AEON_ERR_INVALID_ARGUMENT, "%s: null argument", who);
    AEON_REQUIRE(expected_version != 0 && sector_size != 0 && (sector_size & (sector_size - 1)) == 0,
                 AEON_ERR_INVALID_ARGUMENT,
                 "%s: the artifact specification is incomplete (version %u, sector size %u)", who,
                 expected_version, sector_size);
    *out = nullptr;
    std::vector<uint8_t> index;
    if (int rc = read_whole_file(index_path, &index)) return rc;
    AEON_REQUIRE(index.size() >= kIndexHeaderBytes, AEON_ERR_IO, "%s: expert index too small for its header", who);
    AEON_REQUIRE(std::memcmp(index.data(), kIndexMagic, sizeof kIndexMagic) == 0, AEON_ERR_IO,
                 "%s: invalid expert index magic", who);
    aeon_expert_catalog c;
    c.version = read_u32(index.data() + 12);
    AEON_REQUIRE(c.version == expected_version, AEON_ERR_IO,
                 "%s: unexpected expert index version %u, expected %u", who, c.version, expected_version);
    c.layers = read_u32(index.data() + 16);
    c.experts_per_layer = read_u32(index.data() + 20);
    c.payload_bytes = read_u64(index.data() + 24);
    AEON_REQUIRE(c.layers > 0 && c.experts_per_layer > 0 && c.payload_bytes > 0, AEON_ERR_IO,
                 "%s: empty expert catalog (%u layers x %u experts x %llu bytes)", who, c.layers,
                 c.experts_per_layer, static_cast<unsigned long long>(c.payload_bytes));
    const uint64_t total = static_cast<uint64_t>(c.layers) * c.experts_per_layer;
    AEON_REQUIRE(total <= (SIZE_MAX - kIndexHeaderBytes) / kIndexEntryBytes, AEON_ERR_IO,
                 "%s: expert catalog is too large", who);
    AEON_REQUIRE(index.size() >= kIndexHeaderBytes + total * kIndexEntryBytes, AEON_ERR_IO,
                 "%s: expert index has incomplete entries (%zu bytes for %llu experts)", who,
                 index.size(), static_cast<unsigned long long>(total));

    c.fd = ::open(experts_path, O_RDONLY);
    AEON_REQUIRE(c.fd >= 0, AEON_ERR_IO, "%s: cannot open experts file %s: %s", who, experts_path,
                 std::strerror(errno));
    struct stat st;
    if (::fstat(c.fd, &st) != 0 || st.st_size <= 0) {
        ::close(c.fd);
        set_error("%s: cannot stat experts file %s (or it is empty)", who, experts_path);
        return AEON_ERR_IO;
    }
    c.file_bytes = static_cast<size_t>(st.st_size);
    c.offsets.resize(total);
    for (uint64_t i = 0; i < total; ++i) {
        const uint8_t* entry = index.data() + kIndexHeaderBytes + i * kIndexEntryBytes;
        const uint64_t offset = read_u64(entry);
        const uint64_t length = read_u64(entry + 8);
        if (length != c.payload_bytes || offset % sector_size != 0 || offset > c.file_bytes ||
            c.payload_bytes > c.file_bytes - offset) {
            ::close(c.fd);
            set_error("%s: expert index entry %llu is invalid (offset %llu, length %llu, payload %llu, "
                      "file %zu bytes, sector %u)", who, static_cast<unsigned long long>(i),
                      static_cast<unsigned long long>(offset), static_cast<unsigned long long>(length),
                      static_cast<unsigned long long>(c.payload_bytes), c.file_bytes, sector_size);
            return AEON_ERR_IO;
        }
        c.offsets[i] = offset;
    }
    void* base = ::mmap(nullptr, c.file_bytes, PROT_READ, MAP_SHARED, c.fd, 0);
    if (base == MAP_FAILED) {
        ::close(c.fd);
        set_error("%s: cannot map experts file %s: %s", who, experts_path, std::strerror(errno));
        return AEON_ERR_IO;
    }
    c.base = static_cast<const uint8_t*>(base);
    *out = new aeon_expert_catalog(std::move(c));
    return AEON_OK;
}

extern "C" void aeon_expert_catalog_close(aeon_expert_catalog* catalog) {
    if (catalog == nullptr) return;
    if (catalog->base != nullptr) ::munmap(const_cast<uint8_t*>(catalog->base), catalog->file_bytes);
    if (catalog->fd >= 0) ::close(catalog->fd);
    delete catalog;
}

extern "C" int aeon_expert_catalog_info(const aeon_expert_catalog* catalog, uint32_t* layers,
                                        uint32_t* experts_per_layer, uint64_t* payload_bytes,
                                        uint32_t* version) {
    AEON_REQUIRE(catalog != nullptr, AEON_ERR_INVALID_ARGUMENT, "aeon_expert_catalog_info: null catalog");
    if (layers) *layers = catalog->layers;
    if (experts_per_layer) *experts_per_layer = catalog->experts_per_layer;
    if (payload_bytes) *payload_bytes = catalog->payload_bytes;
    if (version) *version = catalog->version;
    return AEON_OK;
}

extern "C" int aeon_expert_catalog_payload(const aeon_expert_catalog* catalog, uint32_t layer,
                                           uint32_t expert, const void** payload, uint64_t* bytes) {
    const char* who = "aeon_expert_catalog_payload";
    AEON_REQUIRE(catalog != nullptr && payload != nullptr, AEON_ERR_INVALID_ARGUMENT, "%s: null argument", who);
    AEON_REQUIRE(layer < catalog->layers && expert < catalog->experts_per_layer, AEON_ERR_OUT_OF_RANGE,
                 "%s: invalid expert index L%u E%u (catalog is %u x %u)", who, layer, expert,
                 catalog->layers, catalog->experts_per_layer);
    const uint64_t slot = static_cast<uint64_t>(layer) * catalog->experts_per_layer + expert;
    *payload = catalog->base + catalog->offsets[slot];
    if (bytes) *bytes = catalog->payload_bytes;
    return AEON_OK;
}

extern "C" int aeon_payload_layout_for(int hidden, int intermediate, aeon_payload_layout* out) {
    if (int rc = check_expert_shape(hidden, intermediate, "aeon_payload_layout_for")) return rc;
    AEON_REQUIRE(out != nullptr, AEON_ERR_INVALID_ARGUMENT, "aeon_payload_layout_for: null output");
    const size_t weights = static_cast<size_t>(hidden) * intermediate;
    const size_t packed = weights / 2;           // two int4 per byte
    const size_t scale = weights / 32 * 2;       // one fp16 per 32 columns
    out->w1_packed = 0;
    out->w1_scale = out->w1_packed + packed;
    out->w2_packed = out->w1_scale + scale;
    out->w2_scale = out->w2_packed + packed;
    out->w3_packed = out->w2_scale + scale;
    out->w3_scale = out->w3_packed + packed;
    out->total = out->w3_scale + scale;
    return AEON_OK;
}

extern "C" size_t aeon_a64_slot_bytes(int hidden, int intermediate, int scale_group) {
    if (hidden <= 0 || intermediate <= 0 || hidden % 128 != 0 || intermediate % 128 != 0) return 0;
    if (scale_group != 128 && scale_group != 32) return 0;
    return slot_layout(hidden, intermediate, scale_group).bytes;
}

extern "C" int aeon_a64_slot_views(void* d_slot, int hidden, int intermediate, int scale_group,
                                   aeon_a64_expert* out) {
    AEON_REQUIRE(d_slot != nullptr && out != nullptr, AEON_ERR_INVALID_ARGUMENT, "aeon_a64_slot_views: null argument");
    AEON_REQUIRE(hidden > 0 && intermediate > 0 && hidden % 128 == 0 && intermediate % 128 == 0,
                 AEON_ERR_INVALID_ARGUMENT, "aeon_a64_slot_views: the wave64 packing needs multiples of 128 "
                 "(hidden=%d intermediate=%d)", hidden, intermediate);
    AEON_REQUIRE(scale_group == 128 || scale_group == 32, AEON_ERR_INVALID_ARGUMENT,
                 "aeon_a64_slot_views: scale_group must be 128 or 32, not %d", scale_group);
    const SlotLayout l = slot_layout(hidden, intermediate, scale_group);
    char* base = static_cast<char*>(d_slot);
    out->w1_packed = base + l.offset[0];
    out->w1_scale = base + l.offset[1];
    out->w3_packed = base + l.offset[2];
    out->w3_scale = base + l.offset[3];
    out->w2_packed = base + l.offset[4];
    out->w2_scale = base + l.offset[5];
    return AEON_OK;
}

namespace {

// Everything the loader allocates, released on every exit path.
struct LoadResources {
    void* staged[2] = {nullptr, nullptr};
    int* d_mismatch = nullptr;
    hipStream_t stream[2] = {nullptr, nullptr};
    hipEvent_t repacked[2] = {nullptr, nullptr};
    ~LoadResources() {
        for (int i = 0; i < 2; ++i) {
            if (repacked[i]) (void)hipEventDestroy(repacked[i]);
            if (stream[i]) (void)hipStreamDestroy(stream[i]);
            if (staged[i]) (void)hipFree(staged[i]);
        }
        if (d_mismatch) (void)hipFree(d_mismatch);
    }
};

}  // namespace

extern "C" int aeon_resident_load_layer(const aeon_expert_catalog* catalog, uint32_t layer,
                                        uint32_t first, uint32_t count, int hidden,
                                        int intermediate, int scale_group, void* d_pool,
                                        size_t pool_bytes, aeon_a64_expert* h_table) {
    const char* who = "aeon_resident_load_layer";
    AEON_REQUIRE(catalog != nullptr && d_pool != nullptr && h_table != nullptr, AEON_ERR_INVALID_ARGUMENT,
                 "%s: null argument", who);
    if (int rc = check_expert_shape(hidden, intermediate, who)) return rc;
    AEON_REQUIRE(scale_group == 128 || scale_group == 32, AEON_ERR_INVALID_ARGUMENT,
                 "%s: scale_group must be 128 or 32, not %d", who, scale_group);
    AEON_REQUIRE(layer < catalog->layers && first <= catalog->experts_per_layer &&
                     count <= catalog->experts_per_layer - first,
                 AEON_ERR_OUT_OF_RANGE, "%s: experts [%u, %u) of layer %u are outside the %u x %u catalog",
                 who, first, first + count, layer, catalog->layers, catalog->experts_per_layer);
    aeon_payload_layout payload;
    if (int rc = aeon_payload_layout_for(hidden, intermediate, &payload)) return rc;
    AEON_REQUIRE(payload.total == catalog->payload_bytes, AEON_ERR_INVALID_ARGUMENT,
                 "%s: an expert of shape (%d, %d) is %zu bytes in the container's layout, the catalog's "
                 "payloads are %llu", who, hidden, intermediate, payload.total,
                 static_cast<unsigned long long>(catalog->payload_bytes));
    const SlotLayout slot = slot_layout(hidden, intermediate, scale_group);
    AEON_REQUIRE(pool_bytes >= static_cast<size_t>(count) * slot.bytes, AEON_ERR_INVALID_ARGUMENT,
                 "%s: pool of %zu bytes cannot hold %u slots of %zu", who, pool_bytes, count, slot.bytes);
    if (count == 0) return AEON_OK;

    LoadResources r;
    for (int i = 0; i < 2; ++i) {
        AEON_HIP(hipMalloc(&r.staged[i], payload.total));
        AEON_HIP(hipStreamCreateWithFlags(&r.stream[i], hipStreamNonBlocking));
        AEON_HIP(hipEventCreateWithFlags(&r.repacked[i], hipEventDisableTiming));
    }
    AEON_HIP(hipMalloc(reinterpret_cast<void**>(&r.d_mismatch), sizeof(int)));
    AEON_HIP(hipMemset(r.d_mismatch, 0, sizeof(int)));

    // Expert i uses staging buffer and stream i%2. The copy reads the file mapping directly
    // (pageable memory: the runtime stages it and returns once the bytes are on their way), so
    // while one expert is being re-swizzled on the device the host is already paging in and
    // copying the next.
    const size_t sub_offset[3] = {payload.w1_packed, payload.w3_packed, payload.w2_packed};
    const size_t sub_scale[3] = {payload.w1_scale, payload.w3_scale, payload.w2_scale};
    for (uint32_t i = 0; i < count; ++i) {
        const int b = static_cast<int>(i & 1);
        if (i >= 2) AEON_HIP(hipEventSynchronize(r.repacked[b]));  // buffers of expert i-2 are free
        const uint64_t entry = static_cast<uint64_t>(layer) * catalog->experts_per_layer + first + i;
        AEON_HIP(hipMemcpyAsync(r.staged[b], catalog->base + catalog->offsets[entry], payload.total,
                                hipMemcpyHostToDevice, r.stream[b]));
        char* d_slot = static_cast<char*>(d_pool) + static_cast<size_t>(i) * slot.bytes;
        if (int rc = aeon_a64_slot_views(d_slot, hidden, intermediate, scale_group, &h_table[i])) return rc;
        void* dst_packed[3] = {const_cast<void*>(h_table[i].w1_packed), const_cast<void*>(h_table[i].w3_packed),
                               const_cast<void*>(h_table[i].w2_packed)};
        void* dst_scale[3] = {const_cast<void*>(h_table[i].w1_scale), const_cast<void*>(h_table[i].w3_scale),
                              const_cast<void*>(h_table[i].w2_scale)};
        const char* src = static_cast<const char*>(r.staged[b]);
        for (int m = 0; m < 3; ++m) {
            const bool down = m == 2;  // W2 is [hidden][intermediate] with the (8, 4) swizzle
            if (int rc = aeon_a64_repack_device(src + sub_offset[m], src + sub_scale[m],
                                                down ? hidden : intermediate, down ? intermediate : hidden,
                                                down ? 8 : 4, down ? 4 : 8, scale_group, dst_packed[m],
                                                dst_scale[m], r.d_mismatch, r.stream[b])) {
                return rc;
            }
        }
        AEON_HIP(hipEventRecord(r.repacked[b], r.stream[b]));
    }
    AEON_HIP(hipStreamSynchronize(r.stream[0]));
    AEON_HIP(hipStreamSynchronize(r.stream[1]));
    int found = 0;
    AEON_HIP(hipMemcpy(&found, r.d_mismatch, sizeof(int), hipMemcpyDeviceToHost));
    // One scale per 128 columns only holds a payload whose four group-32 scales agree there: a
    // pool built from any other payload would compute with wrong weights, so it is an error, and
    // the pool's contents are not to be used.
    AEON_REQUIRE(found == 0, AEON_ERR_INVALID_ARGUMENT,
                 "%s: %d 128-column groups of layer %u carry four different group-32 scales; load with "
                 "scale_group 32 to keep them", who, found, layer);
    return AEON_OK;
}
