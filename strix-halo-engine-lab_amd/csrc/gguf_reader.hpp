// GGUF v3 container reader and the tensor map of one MoE layer (host code; no device call).
// The container follows the published GGUF layout: "GGUF", version u32, tensor count u64, key/value count u64, the
// key/value entries, the tensor infos (name, rank, extents fastest first, ggml type, offset relative to the data
// section), zero padding up to general.alignment (default 32), the tensor data. Admission follows the reference reader
// (include/strix/gguf_reader.hpp, src/gguf_reader.cpp:22-90,130-260,296-360): version 3 only, bounded counts and string
// lengths, lower-case dotted keys without duplicates, booleans 0 / 1, rank 1..4 with non-zero extents, known tensor types,
// alignment a non-zero multiple of 8, zero padding, aligned offsets, every tensor inside the file, no two tensors overlapping.
// Storage geometry is pinned for the types this library computes with and the plain ones (F32, F16, BF16, Q8_0, Q5_1,
// Q4_K, Q5_K, Q6_K and the other K / legacy block formats of ggml); a type without a pinned geometry is refused.
// The layer map resolves blk.<L>.ffn_gate_exps / ffn_up_exps / ffn_down_exps / ffn_gate_inp / ffn_norm (and the optional
// shared expert ffn_*_shexp) as the reference's prepared-MoE admission names them (src/qwen_moe_prepared.cpp:104-119,
// src/weight/adapters/qwen.cpp:8) and checks shapes and types against each other.
#pragma once
#include <cstdio>
#include <cstring>
#include <string>
#include <unordered_set>
#include <vector>
#include <algorithm>

namespace strix950 {

struct GgufValue {
    std::string key;
    uint32_t type = 0;                     // GGUF metadata value type 0..12
    bool has_u = false, has_i = false, has_f = false, has_b = false, has_s = false;
    uint64_t u = 0;
    int64_t i = 0;
    double f = 0;
    bool b = false;
    std::string s;
    uint32_t array_type = 0;
    uint64_t array_length = 0;
};
struct GgufTensor {
    std::string name;
    std::vector<uint64_t> dims;
    uint32_t type = 0;
    uint64_t relative = 0, absolute = 0, bytes = 0;
};
struct GgufFile {
    uint64_t file_size = 0, alignment = 32, data_offset = 0;
    std::vector<GgufValue> metadata;
    std::vector<GgufTensor> tensors;
    std::string error;
};

// {block elements, block bytes} of a ggml tensor type, {0, 0} when not pinned here
inline void gguf_geometry(uint32_t type, uint64_t& elements, uint64_t& bytes) {
    static const struct { uint32_t type; uint64_t elements, bytes; } table[] = {
        {0, 1, 4}, {1, 1, 2}, {2, 32, 18}, {3, 32, 20}, {6, 32, 22}, {7, 32, 24}, {8, 32, 34}, {9, 32, 36},
        {10, 256, 84}, {11, 256, 110}, {12, 256, 144}, {13, 256, 176}, {14, 256, 210}, {15, 256, 292},
        {24, 1, 1}, {25, 1, 2}, {26, 1, 4}, {27, 1, 8}, {28, 1, 8}, {30, 1, 2}};
    elements = bytes = 0;
    for (const auto& row : table)
        if (row.type == type) { elements = row.elements; bytes = row.bytes; }
}

class GgufParser {
public:
    GgufParser(FILE* f, uint64_t size, GgufFile& out) : f_(f), size_(size), out_(out) {}
    bool run() {
        char magic[4];
        if (!bytes(magic, 4)) return false;
        if (std::memcmp(magic, "GGUF", 4) != 0) return fail("invalid GGUF magic");
        uint32_t version; uint64_t tensor_count, kv_count;
        if (!get(version)) return false;
        if (version != 3) return fail("only GGUF v3 little-endian is supported");
        if (!get(tensor_count) || !get(kv_count)) return false;
        if (tensor_count > 1000000ULL) return fail("tensor count exceeds configured limit");
        if (kv_count > 1000000ULL) return fail("metadata count exceeds configured limit");
        std::unordered_set<std::string> keys, names;
        for (uint64_t n = 0; n < kv_count; ++n) {
            GgufValue v;
            if (!string(v.key, 65535)) return false;
            if (!valid_key(v.key)) return fail("invalid GGUF metadata key");
            if (!value_type(v.type) || !value(v.type, &v, 0)) return false;
            if (!keys.insert(v.key).second) return fail("duplicate GGUF metadata key");
            out_.metadata.push_back(std::move(v));
        }
        for (const GgufValue& v : out_.metadata)
            if (v.key == "general.alignment") {
                if (!v.has_u) return fail("general.alignment must be an unsigned integer");
                out_.alignment = v.u;
            }
        if (out_.alignment == 0 || out_.alignment % 8 != 0) return fail("general.alignment must be a non-zero multiple of 8");
        for (uint64_t n = 0; n < tensor_count; ++n) {
            GgufTensor t;
            if (!string(t.name, 64)) return false;
            if (t.name.empty()) return fail("tensor name cannot be empty");
            uint32_t rank;
            if (!get(rank)) return false;
            if (rank == 0 || rank > 4) return fail("tensor dimension count is invalid");
            for (uint32_t d = 0; d < rank; ++d) {
                uint64_t extent;
                if (!get(extent)) return false;
                if (extent == 0) return fail("tensor dimensions must be non-zero");
                t.dims.push_back(extent);
            }
            if (!get(t.type)) return false;
            if (!valid_type(t.type)) return fail("unsupported or removed GGML tensor type");
            if (!get(t.relative)) return false;
            if (!names.insert(t.name).second) return fail("duplicate GGUF tensor name");
            out_.tensors.push_back(std::move(t));
        }
        const uint64_t rem = at_ % out_.alignment;
        out_.data_offset = rem == 0 ? at_ : at_ + (out_.alignment - rem);
        if (out_.data_offset > size_) return fail("aligned tensor-data offset exceeds file size");
        while (at_ < out_.data_offset) {
            uint8_t pad;
            if (!get(pad)) return false;
            if (pad != 0) return fail("GGUF padding must contain zero bytes");
        }
        for (GgufTensor& t : out_.tensors) {
            if (t.relative % out_.alignment != 0) return fail("tensor offset is not aligned");
            if (t.relative > UINT64_MAX - out_.data_offset) return fail("GGUF size arithmetic overflow");
            t.absolute = out_.data_offset + t.relative;
            if (t.absolute > size_) return fail("tensor offset exceeds file size");
            uint64_t block_elements, block_bytes;
            gguf_geometry(t.type, block_elements, block_bytes);
            if (block_elements == 0) return fail("GGML tensor type has no pinned storage geometry");
            if (t.dims[0] % block_elements != 0) return fail("tensor row is not divisible by its quantization block size");
            uint64_t n = t.dims[0] / block_elements;
            if (!mul(n, block_bytes)) return false;
            for (size_t d = 1; d < t.dims.size(); ++d)
                if (!mul(n, t.dims[d])) return false;
            t.bytes = n;
            if (t.bytes > size_ - t.absolute) return fail("tensor data range exceeds file size");
        }
        std::vector<const GgufTensor*> ordered;
        for (const GgufTensor& t : out_.tensors) ordered.push_back(&t);
        std::sort(ordered.begin(), ordered.end(), [](const GgufTensor* a, const GgufTensor* b) { return a->absolute < b->absolute; });
        for (size_t n = 1; n < ordered.size(); ++n)
            if (ordered[n - 1]->absolute + ordered[n - 1]->bytes > ordered[n]->absolute) return fail("GGUF tensor data ranges overlap");
        return true;
    }

private:
    bool fail(const char* what) { out_.error = what; return false; }
    bool bytes(void* to, size_t n) {
        if (n > size_ - at_) return fail("unexpected end of GGUF file");
        if (n != 0 && std::fread(to, 1, n, f_) != n) return fail("failed to read GGUF bytes");
        at_ += n;
        return true;
    }
    bool skip(uint64_t n) {                        // pass over n bytes unread: one bounds check, one seek
        if (n > size_ - at_) return fail("unexpected end of GGUF file");
        if (n != 0 && fseeko(f_, static_cast<off_t>(n), SEEK_CUR) != 0) return fail("failed to read GGUF bytes");
        at_ += n;
        return true;
    }
    static uint32_t scalar_bytes(uint32_t type) {  // 0 for the types that are no fixed-size scalars (string, array)
        switch (type) {
        case 0: case 1: case 7: return 1U;
        case 2: case 3: return 2U;
        case 4: case 5: case 6: return 4U;
        case 10: case 11: case 12: return 8U;
        default: return 0U;
        }
    }
    // the elements of an array whose values nobody asked for: scalars in one step (booleans are still checked, in blocks),
    // strings by their length fields
    bool skip_elements(uint32_t element, uint64_t length, uint32_t depth) {
        if (element == 7U) {
            uint8_t block[4096];
            for (uint64_t done = 0; done < length;) {
                const size_t n = static_cast<size_t>(length - done < sizeof block ? length - done : sizeof block);
                if (!bytes(block, n)) return false;
                for (size_t i = 0; i < n; ++i)
                    if (block[i] > 1) return fail("GGUF boolean must be zero or one");
                done += n;
            }
            return true;
        }
        if (const uint32_t unit = scalar_bytes(element)) {
            uint64_t total = length;
            return mul(total, unit) && skip(total);
        }
        if (element == 8U) {
            for (uint64_t n = 0; n < length; ++n) {
                uint64_t len;
                if (!get(len)) return false;
                if (len > 64ULL * 1024ULL * 1024ULL) return fail("GGUF string exceeds configured limit");
                if (!skip(len)) return false;
            }
            return true;
        }
        for (uint64_t n = 0; n < length; ++n)
            if (!value(element, nullptr, depth + 1U)) return false;
        return true;
    }
    template <class T> bool get(T& v) {            // little-endian scalar (the hosts this library runs on are little-endian)
        return bytes(&v, sizeof(T));
    }
    bool mul(uint64_t& a, uint64_t b) {
        if (b != 0 && a > UINT64_MAX / b) return fail("GGUF size arithmetic overflow");
        a *= b;
        return true;
    }
    bool string(std::string& s, uint64_t limit) {
        uint64_t n;
        if (!get(n)) return false;
        if (n > limit || n > 64ULL * 1024ULL * 1024ULL) return fail("GGUF string exceeds configured limit");
        s.resize(static_cast<size_t>(n));
        return bytes(s.data(), s.size());
    }
    bool value_type(uint32_t& t) {
        if (!get(t)) return false;
        if (t > 12U) return fail("unknown GGUF metadata value type");
        return true;
    }
    template <class T> bool scalar_u(GgufValue* o) { T v; if (!get(v)) return false; if (o) { o->has_u = true; o->u = v; } return true; }
    template <class T> bool scalar_i(GgufValue* o) { T v; if (!get(v)) return false; if (o) { o->has_i = true; o->i = v; } return true; }
    bool value(uint32_t type, GgufValue* o, uint32_t depth) {
        switch (type) {
        case 0: return scalar_u<uint8_t>(o);
        case 1: return scalar_i<int8_t>(o);
        case 2: return scalar_u<uint16_t>(o);
        case 3: return scalar_i<int16_t>(o);
        case 4: return scalar_u<uint32_t>(o);
        case 5: return scalar_i<int32_t>(o);
        case 6: { float v; if (!get(v)) return false; if (o) { o->has_f = true; o->f = v; } return true; }
        case 7: { uint8_t v; if (!get(v)) return false; if (v > 1) return fail("GGUF boolean must be zero or one"); if (o) { o->has_b = true; o->b = v == 1; } return true; }
        case 8: { std::string s; if (!string(s, 64ULL * 1024ULL * 1024ULL)) return false; if (o) { o->has_s = true; o->s = std::move(s); } return true; }
        case 9: {
            if (depth >= 8U) return fail("GGUF array nesting exceeds configured limit");
            uint32_t element; uint64_t length;
            if (!value_type(element) || !get(length)) return false;
            if (length > 100000000ULL - array_elements_) return fail("GGUF arrays exceed configured element limit");
            array_elements_ += length;
            if (o) { o->array_type = element; o->array_length = length; }
            return skip_elements(element, length, depth);
        }
        case 10: return scalar_u<uint64_t>(o);
        case 11: return scalar_i<int64_t>(o);
        default: { double v; if (!get(v)) return false; if (o) { o->has_f = true; o->f = v; } return true; }
        }
    }
    static bool valid_key(const std::string& key) {
        if (key.empty() || key.front() == '.' || key.back() == '.') return false;
        bool previous_dot = false;
        for (const char symbol : key) {
            const unsigned char c = static_cast<unsigned char>(symbol);
            const bool ok = (c >= 'a' && c <= 'z') || (c >= '0' && c <= '9') || c == '_' || c == '.';
            if (!ok || (c == '.' && previous_dot)) return false;
            previous_dot = c == '.';
        }
        return true;
    }
    // ggml type ids in use; 4, 5 (Q4_2, Q4_3) and 31..33, 36..38 (the repacked Q4_0 / IQ4_NL forms) were removed upstream
    static bool valid_type(uint32_t type) {
        if (type > 39U) return false;
        switch (type) {
        case 4: case 5: case 31: case 32: case 33: case 36: case 37: case 38: return false;
        default: return true;
        }
    }
    FILE* f_;
    uint64_t size_, at_ = 0, array_elements_ = 0;
    GgufFile& out_;
};

inline const GgufTensor* gguf_find(const GgufFile& g, const std::string& name) {
    for (const GgufTensor& t : g.tensors)
        if (t.name == name) return &t;
    return nullptr;
}
inline void gguf_export(const GgufTensor& t, mi355_gguf_tensor& out) {
    out = mi355_gguf_tensor{};
    out.name = t.name.c_str();
    out.n_dims = static_cast<uint32_t>(t.dims.size());
    for (size_t d = 0; d < t.dims.size(); ++d) out.dims[d] = t.dims[d];
    out.ggml_type = t.type; out.offset = t.absolute; out.bytes = t.bytes;
}

}  // namespace strix950

using namespace strix950;

extern "C" {

void* mi355_gguf_open(const char* path) {
    if (!path) { fail(MI355_E_INVALID_ARGUMENT, "gguf: null path"); return nullptr; }
    FILE* f = std::fopen(path, "rb");
    if (!f) { fail(MI355_E_INVALID_ARGUMENT, "cannot open GGUF file"); return nullptr; }
    GgufFile* g = new GgufFile{};
    bool ok = std::fseek(f, 0, SEEK_END) == 0;
    const long size = ok ? std::ftell(f) : -1L;
    ok = ok && size >= 0 && std::fseek(f, 0, SEEK_SET) == 0;
    if (ok) {
        g->file_size = static_cast<uint64_t>(size);
        ok = GgufParser(f, g->file_size, *g).run();
    } else g->error = "cannot size GGUF file";
    std::fclose(f);
    if (!ok) {
        fail(MI355_E_INVALID_ARGUMENT, g->error.c_str());
        delete g;
        return nullptr;
    }
    return g;
}
void mi355_gguf_close(void* file) { delete static_cast<GgufFile*>(file); }
uint64_t mi355_gguf_tensor_count(const void* file) { return file ? static_cast<const GgufFile*>(file)->tensors.size() : 0; }
uint64_t mi355_gguf_metadata_count(const void* file) { return file ? static_cast<const GgufFile*>(file)->metadata.size() : 0; }
uint64_t mi355_gguf_alignment(const void* file) { return file ? static_cast<const GgufFile*>(file)->alignment : 0; }
uint64_t mi355_gguf_data_offset(const void* file) { return file ? static_cast<const GgufFile*>(file)->data_offset : 0; }

int32_t mi355_gguf_tensor_at(const void* file, uint64_t index, mi355_gguf_tensor* out) {
    const GgufFile* g = static_cast<const GgufFile*>(file);
    STRIX_REQUIRE(g && out && index < g->tensors.size(), "gguf: tensor index out of range");
    gguf_export(g->tensors[index], *out);
    return MI355_OK;
}
int32_t mi355_gguf_find_tensor(const void* file, const char* name, mi355_gguf_tensor* out) {
    const GgufFile* g = static_cast<const GgufFile*>(file);
    STRIX_REQUIRE(g && name && out, "gguf: null argument");
    const GgufTensor* t = gguf_find(*g, name);
    STRIX_REQUIRE(t != nullptr, "gguf: no tensor of that name");
    gguf_export(*t, *out);
    return MI355_OK;
}
// kind: 0 unsigned (also booleans), 1 signed, 2 floating, 3 string (text receives the pointer, valid until close)
int32_t mi355_gguf_metadata(const void* file, const char* key, uint32_t* kind, uint64_t* u, int64_t* i, double* f, const char** text) {
    const GgufFile* g = static_cast<const GgufFile*>(file);
    STRIX_REQUIRE(g && key && kind, "gguf: null argument");
    for (const GgufValue& v : g->metadata)
        if (v.key == key) {
            if (v.has_u || v.has_b) { *kind = 0; if (u) *u = v.has_u ? v.u : (v.b ? 1U : 0U); }
            else if (v.has_i) { *kind = 1; if (i) *i = v.i; }
            else if (v.has_f) { *kind = 2; if (f) *f = v.f; }
            else if (v.has_s) { *kind = 3; if (text) *text = v.s.c_str(); }
            else { *kind = 4; if (u) *u = v.array_length; }       // an array: its length
            return MI355_OK;
        }
    return fail(MI355_E_INVALID_ARGUMENT, "gguf: no metadata entry of that key");
}

int32_t mi355_gguf_moe_layer(const void* file, uint32_t layer, mi355_gguf_moe_layer_map* out) {
    const GgufFile* g = static_cast<const GgufFile*>(file);
    STRIX_REQUIRE(g && out, "gguf: null argument");
    const std::string prefix = "blk." + std::to_string(layer) + ".";
    const GgufTensor* gate = gguf_find(*g, prefix + "ffn_gate_exps.weight");
    const GgufTensor* up = gguf_find(*g, prefix + "ffn_up_exps.weight");
    const GgufTensor* down = gguf_find(*g, prefix + "ffn_down_exps.weight");
    const GgufTensor* router = gguf_find(*g, prefix + "ffn_gate_inp.weight");
    STRIX_REQUIRE(gate && up && down && router, "gguf moe layer: ffn_gate_exps / ffn_up_exps / ffn_down_exps / ffn_gate_inp not all present");
    // extents fastest first: gate / up [hidden][ffn][experts], down [ffn][hidden][experts], router [hidden][experts]
    STRIX_REQUIRE(gate->dims.size() == 3 && up->dims == gate->dims && up->type == gate->type && up->bytes == gate->bytes,
                  "gguf moe layer: gate and up expert tensors must be rank 3 with the same shape and type");
    const uint64_t hidden = gate->dims[0], ffn = gate->dims[1], experts = gate->dims[2];
    STRIX_REQUIRE(down->dims.size() == 3 && down->dims[0] == ffn && down->dims[1] == hidden && down->dims[2] == experts,
                  "gguf moe layer: the down expert tensor must be [ffn][hidden][experts]");
    STRIX_REQUIRE(router->type == 0 && router->dims.size() == 2 && router->dims[0] == hidden && router->dims[1] == experts,
                  "gguf moe layer: the router must be an F32 [hidden][experts] tensor");
    STRIX_REQUIRE(gate->type == MI355_TYPE_Q4_K || gate->type == MI355_TYPE_Q5_K || gate->type == MI355_TYPE_Q8_0,
                  "gguf moe layer: gate / up experts must be Q4_K, Q5_K or Q8_0");
    if (!(down->type == MI355_TYPE_Q4_K || down->type == MI355_TYPE_Q5_K || down->type == MI355_TYPE_Q6_K || down->type == MI355_TYPE_Q8_0 || down->type == MI355_TYPE_Q5_1))
        return fail(MI355_E_UNSUPPORTED, "gguf moe layer: down experts must be Q4_K, Q5_K, Q6_K, Q8_0 or Q5_1");
    STRIX_REQUIRE(hidden <= 0xffffffffULL && ffn <= 0xffffffffULL && experts <= kRouteMaxExperts, "gguf moe layer: geometry beyond this library's");
    *out = mi355_gguf_moe_layer_map{};
    gguf_export(*gate, out->gate); gguf_export(*up, out->up); gguf_export(*down, out->down); gguf_export(*router, out->router);
    out->hidden = static_cast<uint32_t>(hidden); out->ffn = static_cast<uint32_t>(ffn); out->experts = static_cast<uint32_t>(experts);
    out->gate_type = gate->type; out->down_type = down->type;
    const auto optional = [&](const char* name, mi355_gguf_tensor& slot, std::initializer_list<uint64_t> shape, bool any_type) {
        const GgufTensor* t = gguf_find(*g, prefix + name);
        if (!t) return true;
        if (t->dims != std::vector<uint64_t>(shape) || (!any_type && t->type != 0)) return false;
        gguf_export(*t, slot);
        return true;
    };
    STRIX_REQUIRE(optional("ffn_norm.weight", out->norm, {hidden}, false), "gguf moe layer: ffn_norm must be an F32 [hidden] tensor");
    STRIX_REQUIRE(optional("exp_probs_b.bias", out->router_bias, {experts}, false), "gguf moe layer: exp_probs_b must be an F32 [experts] tensor");
    const GgufTensor* sg = gguf_find(*g, prefix + "ffn_gate_shexp.weight");
    if (sg) {
        STRIX_REQUIRE(sg->dims.size() == 2 && sg->dims[0] == hidden, "gguf moe layer: the shared expert's gate must be [hidden][shared ffn]");
        const uint64_t sffn = sg->dims[1];
        STRIX_REQUIRE(optional("ffn_gate_shexp.weight", out->shared_gate, {hidden, sffn}, true) && optional("ffn_up_shexp.weight", out->shared_up, {hidden, sffn}, true) &&
                      optional("ffn_down_shexp.weight", out->shared_down, {sffn, hidden}, true) && out->shared_up.bytes != 0 && out->shared_down.bytes != 0 &&
                      out->shared_up.ggml_type == out->shared_gate.ggml_type,
                      "gguf moe layer: the shared expert needs gate / up [hidden][shared ffn] of one type and down [shared ffn][hidden]");
        out->shared_ffn = static_cast<uint32_t>(sffn);
        STRIX_REQUIRE(optional("ffn_gate_inp_shexp.weight", out->shared_router, {hidden}, false), "gguf moe layer: ffn_gate_inp_shexp must be an F32 [hidden] tensor");
    }
    return MI355_OK;
}

}  // extern "C"
