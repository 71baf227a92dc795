// Minimal reader for contiguous HDF5 datasets.  See util.h for the subset it accepts.
#include "util.h"

#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <string>
#include <vector>

namespace {

struct Failure {
    const char *text;
};

struct File {
    std::vector<unsigned char> bytes;

    const unsigned char *at(uint64_t offset, uint64_t length) const {
        if (offset > bytes.size() || length > bytes.size() - offset) throw Failure{"read_hdf5: structure points outside the file"};
        return bytes.data() + offset;
    }
    uint64_t u(uint64_t offset, int width) const {  // little-endian unsigned
        const unsigned char *p = at(offset, (uint64_t)width);
        uint64_t v = 0;
        for (int i = width - 1; i >= 0; --i) v = (v << 8) | p[i];
        return v;
    }
    bool tagged(uint64_t offset, const char *four) const { return memcmp(at(offset, 4), four, 4) == 0; }
};

struct Dataset {
    int rank = -1;
    uint64_t dims[2] = {1, 1};
    int type_class = -1, type_size = 0;
    bool type_signed = false, type_big_endian = false;
    bool have_layout = false;
    uint64_t address = 0, size = 0;
};

// Version 1 object header: 16-byte prefix, then 8-byte aligned messages, possibly continued elsewhere.
Dataset parse_object_header(const File &f, uint64_t address) {
    if (f.u(address, 1) != 1) throw Failure{"read_hdf5: only version 1 object headers are supported"};
    Dataset d;
    struct Block { uint64_t begin, end; };
    std::vector<Block> blocks;
    blocks.push_back({address + 16, address + 16 + f.u(address + 8, 4)});
    for (size_t b = 0; b < blocks.size() && b < 64; ++b) {
        uint64_t p = blocks[b].begin;
        while (p + 8 <= blocks[b].end) {
            const uint64_t type = f.u(p, 2), size = f.u(p + 2, 2), body = p + 8;
            if (type == 0x0001) {  // dataspace
                const uint64_t version = f.u(body, 1), rank = f.u(body + 1, 1);
                if (version != 1 && version != 2) throw Failure{"read_hdf5: unknown dataspace version"};
                if (rank < 1 || rank > 2) throw Failure{"read_hdf5: only one- and two-dimensional datasets are supported"};
                const uint64_t first = body + (version == 1 ? 8 : 4);
                d.rank = (int)rank;
                for (uint64_t i = 0; i < rank; ++i) d.dims[i] = f.u(first + 8 * i, 8);
            } else if (type == 0x0003) {  // datatype
                const uint64_t class_and_version = f.u(body, 1), bits0 = f.u(body + 1, 1);
                d.type_class = (int)(class_and_version & 15);
                d.type_big_endian = (bits0 & 1) != 0;
                d.type_signed = (bits0 & 8) != 0;
                d.type_size = (int)f.u(body + 4, 4);
            } else if (type == 0x0008) {  // data layout
                if (f.u(body, 1) != 3) throw Failure{"read_hdf5: only version 3 data layouts are supported"};
                if (f.u(body + 1, 1) != 1) throw Failure{"read_hdf5: only contiguous datasets are supported (this one is compact or chunked)"};
                d.address = f.u(body + 2, 8);
                d.size = f.u(body + 10, 8);
                d.have_layout = true;
            } else if (type == 0x000b) {  // filter pipeline
                throw Failure{"read_hdf5: filtered (compressed) datasets are not supported"};
            } else if (type == 0x0010) {  // continuation
                const uint64_t where = f.u(body, 8), length = f.u(body + 8, 8);
                blocks.push_back({where, where + length});
            }
            p = body + size;
        }
    }
    if (d.rank < 0 || d.type_class < 0 || !d.have_layout) throw Failure{"read_hdf5: object is not a dataset"};
    return d;
}

// Walks the group B-tree (node type 0) down to its symbol nodes and returns the object header
// address of `name`, or UINT64_MAX.
uint64_t find_in_group(const File &f, uint64_t node, uint64_t heap_data, const std::string &name, int depth) {
    if (depth > 16 || !f.tagged(node, "TREE")) throw Failure{"read_hdf5: malformed group B-tree"};
    if (f.u(node + 4, 1) != 0) throw Failure{"read_hdf5: malformed group B-tree"};
    const uint64_t level = f.u(node + 5, 1), used = f.u(node + 6, 2);
    uint64_t p = node + 8 + 16 + 8;  // past the sibling pointers and key 0
    for (uint64_t i = 0; i < used; ++i, p += 16) {
        const uint64_t child = f.u(p, 8);
        if (level > 0) {
            const uint64_t hit = find_in_group(f, child, heap_data, name, depth + 1);
            if (hit != UINT64_MAX) return hit;
            continue;
        }
        if (!f.tagged(child, "SNOD")) throw Failure{"read_hdf5: malformed symbol node"};
        const uint64_t symbols = f.u(child + 6, 2);
        for (uint64_t s = 0; s < symbols; ++s) {
            const uint64_t entry = child + 8 + 40 * s;
            const uint64_t name_at = heap_data + f.u(entry, 8);
            const char *text = (const char *)f.at(name_at, 1);
            const size_t room = f.bytes.size() - (size_t)name_at;
            if (strnlen(text, room) == name.size() && memcmp(text, name.data(), name.size()) == 0) return f.u(entry + 8, 8);
        }
    }
    return UINT64_MAX;
}

float element(const File &f, const Dataset &d, uint64_t index) {
    const uint64_t p = d.address + index * (uint64_t)d.type_size;
    if (d.type_class == 1) {
        if (d.type_size == 4) { uint32_t v = (uint32_t)f.u(p, 4); float out; memcpy(&out, &v, 4); return out; }
        uint64_t v = f.u(p, 8); double out; memcpy(&out, &v, 8); return (float)out;
    }
    uint64_t v = f.u(p, d.type_size);
    if (d.type_signed && d.type_size < 8 && (v >> (8 * d.type_size - 1))) v |= ~0ULL << (8 * d.type_size);
    return d.type_signed ? (float)(int64_t)v : (float)v;
}

void read_dataset(const char *filepath, const char *tag, long long *rows, long long *cols, float **data) {
    File f;
    FILE *in = fopen(filepath, "rb");
    if (!in) throw Failure{"read_hdf5: cannot open the file"};
    unsigned char chunk[65536];
    size_t got;
    while ((got = fread(chunk, 1, sizeof(chunk), in)) > 0) f.bytes.insert(f.bytes.end(), chunk, chunk + got);
    fclose(in);
    static const unsigned char kSignature[8] = {0x89, 'H', 'D', 'F', '\r', '\n', 0x1a, '\n'};
    if (f.bytes.size() < 96 || memcmp(f.bytes.data(), kSignature, 8) != 0) throw Failure{"read_hdf5: not an HDF5 file"};
    if (f.u(8, 1) != 0) throw Failure{"read_hdf5: only superblock version 0 is supported"};
    if (f.u(13, 1) != 8 || f.u(14, 1) != 8) throw Failure{"read_hdf5: only 8-byte offsets and lengths are supported"};
    // superblock: 24 bytes of versions and sizes, four addresses, then the root group's symbol entry
    const uint64_t root = 24 + 32;
    if (f.u(root + 16, 4) != 1) throw Failure{"read_hdf5: root group without a cached B-tree (new-style group?)"};
    const uint64_t btree = f.u(root + 24, 8), heap = f.u(root + 32, 8);
    if (!f.tagged(heap, "HEAP")) throw Failure{"read_hdf5: malformed local heap"};
    const uint64_t heap_data = f.u(heap + 24, 8);
    std::string name = tag ? tag : "Default";
    while (!name.empty() && name[0] == '/') name.erase(0, 1);
    if (name.find('/') != std::string::npos) throw Failure{"read_hdf5: datasets inside sub-groups are not supported"};
    const uint64_t header = find_in_group(f, btree, heap_data, name, 0);
    if (header == UINT64_MAX) throw Failure{"read_hdf5: no dataset of that name in the file"};
    const Dataset d = parse_object_header(f, header);
    if (d.type_big_endian) throw Failure{"read_hdf5: big-endian data is not supported"};
    const bool floating = d.type_class == 1 && (d.type_size == 4 || d.type_size == 8);
    const bool integer = d.type_class == 0 && (d.type_size == 1 || d.type_size == 2 || d.type_size == 4 || d.type_size == 8);
    if (!floating && !integer) throw Failure{"read_hdf5: only float32, float64 and integer data are supported"};
    const uint64_t count = d.dims[0] * d.dims[1];
    if (d.dims[0] > 0x7fffffffULL || d.dims[1] > 0x7fffffffULL) throw Failure{"read_hdf5: dimension too large"};
    if (d.size != count * (uint64_t)d.type_size) throw Failure{"read_hdf5: dataset size does not match its shape"};
    if (count) f.at(d.address, d.size);  // range check once
    float *out = (float *)malloc(count ? count * sizeof(float) : 1);
    if (!out) throw Failure{"read_hdf5: out of memory"};
    if (d.type_class == 1 && d.type_size == 4) {
        if (count) memcpy(out, f.at(d.address, d.size), d.size);
    } else {
        for (uint64_t i = 0; i < count; ++i) out[i] = element(f, d, i);
    }
    *rows = (long long)d.dims[0];
    *cols = (long long)d.dims[1];
    *data = out;
}

}  // namespace

Matrix *read_hdf5(const char *filepath) { return read_hdf5(filepath, "/Default"); }

Matrix *read_hdf5(const char *filepath, const char *tag) {
    long long rows = 0, cols = 0;
    float *data = nullptr;
    try {
        read_dataset(filepath, tag, &rows, &cols, &data);
    } catch (const Failure &why) {
        printf("%s (%s)\n", why.text, filepath);
        throw why.text;
    }
    Matrix *out = empty_cpu(0, 0);
    free(out->data);
    out->rows = (int)rows;
    out->cols = (int)cols;
    out->size = rows * cols;
    out->bytes = (size_t)out->size * sizeof(float);
    out->data = data;
    return out;
}

extern "C" int cn_facade_read_hdf5(const char *filepath, const char *tag, long long *rows, long long *cols,
                                   float **data, const char **error_text) {
    try {
        read_dataset(filepath, tag, rows, cols, data);
    } catch (const Failure &why) {
        if (error_text) *error_text = why.text;
        return 1;
    }
    return 0;
}
