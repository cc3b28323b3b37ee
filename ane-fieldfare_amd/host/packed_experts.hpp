// Reader of the packed routed-expert files of an installed checkpoint: `packed_experts/layout.json` plus one
// `layer_NN.bin` per layer, each `expertsPerLayer` blobs of `expertStride` bytes. It stands where the
// reference has GTurboPackedExpertsLayoutCodec + GTurboV1StructuralValidator
// (Sources/ANEFieldfareImportedFormat/GTurboPackedExpertsLayoutV1.swift:3-188), PackedExpertsLayoutReader
// (Infrastructure/ModelIO/PackedExpertsLayout.swift:52-89), Model.routedExpertOffsets
// (Runtime/Inference/ModelExpertIO.swift:11-30) and MappedExpertLayer
// (Infrastructure/Streaming/MappedExpertLayer.swift:41-140). The reference maps every layer file and binds
// expert pages to the GPU on demand; here each layer file is mapped once, copied into the HBM arena and
// unmapped: after uploadPackedExperts() every expert is resident and no call touches storage again.
//
// Header-only, C++17, no dependencies beyond the C ABI; the parsing and validation half needs no GPU.
#pragma once

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cctype>
#include <cstdint>
#include <fstream>
#include <map>
#include <memory>
#include <set>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "fieldfare_host.hpp"

namespace fieldfare {

// GTurboFormatError (GTurboFormatV1.swift:24-37): "<field>: <reason>"
struct GTurboFormatError : std::runtime_error {
    enum Kind { invalid, overflow, truncated } kind;
    std::string field;
    GTurboFormatError(Kind k, const std::string &f, const std::string &reason)
        : std::runtime_error(f + ": " + reason), kind(k), field(f) {}
};

constexpr uint64_t kGTurboAlignmentBytes = 16384;   // GTurboFormatV1.alignmentBytes (GTurboFormatV1.swift:7)

struct SubTensorEntry {       // GTurboSubTensorV1 / SubTensorEntry (PackedExpertsLayout.swift:4-10)
    uint64_t offset = 0;      // relative to the expert blob's start
    uint64_t size = 0;
    std::string dtype;        // "U32" | "BF16"
    std::vector<uint32_t> shape;
    int bits = 0;             // 0 = absent
};

struct ExpertEntry {          // PackedExpertsLayout.swift:12-33
    int expert = 0;           // logical id used by the router
    int physicalRank = 0;     // position of the blob inside the layer file
    uint64_t offset = 0;      // byte offset of the blob in the layer file (= physicalRank * expertStride)
    uint64_t size = 0;
    std::map<std::string, SubTensorEntry> subTensors;
};

struct LayerLayout {
    int layer = 0;
    std::string file;         // basename, e.g. "layer_00.bin"
    std::vector<ExpertEntry> experts;   // sorted by logical id after decoding
};

struct PackedExpertsLayout {
    uint64_t expertStride = 0;
    int numLayers = 0;
    int expertsPerLayer = 0;
    std::vector<LayerLayout> layers;    // sorted by layer after decoding

    const ExpertEntry &expert(int layer, int e) const { return layers.at(layer).experts.at(e); }

    // Model.routedExpertOffsets (ModelExpertIO.swift:11-30): the nine sub-tensor offsets, read from expert 0
    ffmoe_offsets routedExpertOffsets(int layer) const {
        const ExpertEntry &ex = expert(layer, 0);
        auto off = [&](const char *role) -> uint32_t {
            auto it = ex.subTensors.find(role);
            if (it == ex.subTensors.end() || it->second.offset > 0xFFFFFFFFull)
                throw std::runtime_error(std::string("invalid routed expert metadata for role ") + role);
            return (uint32_t)it->second.offset;
        };
        return ffmoe_offsets{off("gate"), off("gate_scales"), off("gate_biases"), off("up"),  off("up_scales"),
                             off("up_biases"), off("down"), off("down_scales"), off("down_biases")};
    }
    // Model.routedExpertPhysicalOffsets (ModelExpertIO.swift:32-34)
    std::vector<uint64_t> routedExpertPhysicalOffsets(int layer) const {
        std::vector<uint64_t> out;
        for (const ExpertEntry &e : layers.at(layer).experts) out.push_back(e.offset);
        return out;
    }
};

namespace detail {

// A JSON value, just enough for layout.json: objects, arrays, strings, unsigned integers, null.
struct Json {
    enum Type { null_, number, string, array, object, boolean } type = null_;
    uint64_t u = 0;
    bool negative_or_fraction = false;
    std::string s;
    std::vector<Json> items;
    std::vector<std::pair<std::string, Json>> members;
    const Json *find(const std::string &key) const {
        for (const auto &m : members)
            if (m.first == key) return &m.second;
        return nullptr;
    }
};

class JsonParser {
public:
    explicit JsonParser(const std::string &text) : t_(text) {}
    Json parse() {
        Json v = value();
        ws();
        if (p_ != t_.size()) fail("trailing characters");
        return v;
    }

private:
    const std::string &t_;
    size_t p_ = 0;
    int depth_ = 0;
    [[noreturn]] void fail(const std::string &why) const {
        throw GTurboFormatError(GTurboFormatError::invalid, "packed_experts/layout.json", why + " at byte " + std::to_string(p_));
    }
    void ws() {
        while (p_ < t_.size() && (t_[p_] == ' ' || t_[p_] == '\n' || t_[p_] == '\t' || t_[p_] == '\r')) ++p_;
    }
    char peek() {
        ws();
        if (p_ >= t_.size()) throw GTurboFormatError(GTurboFormatError::truncated, "packed_experts/layout.json", "truncated");
        return t_[p_];
    }
    void expect(char c) {
        if (peek() != c) fail(std::string("expected '") + c + "'");
        ++p_;
    }
    Json value() {
        if (++depth_ > 64) fail("nesting too deep");
        Json v;
        const char c = peek();
        if (c == '{') {
            v.type = Json::object;
            ++p_;
            if (peek() == '}') { ++p_; --depth_; return v; }
            for (;;) {
                std::string key = str();
                expect(':');
                v.members.emplace_back(std::move(key), value());
                if (peek() == ',') { ++p_; continue; }
                expect('}');
                break;
            }
        } else if (c == '[') {
            v.type = Json::array;
            ++p_;
            if (peek() == ']') { ++p_; --depth_; return v; }
            for (;;) {
                v.items.push_back(value());
                if (peek() == ',') { ++p_; continue; }
                expect(']');
                break;
            }
        } else if (c == '"') {
            v.type = Json::string;
            v.s = str();
        } else if (c == '-' || std::isdigit((unsigned char)c)) {
            v.type = Json::number;
            if (c == '-') { v.negative_or_fraction = true; ++p_; }
            bool any = false;
            while (p_ < t_.size() && std::isdigit((unsigned char)t_[p_])) {
                const uint64_t d = (uint64_t)(t_[p_] - '0');
                if (v.u > (UINT64_MAX - d) / 10) throw GTurboFormatError(GTurboFormatError::overflow, "packed_experts/layout.json", "arithmetic overflow");
                v.u = v.u * 10 + d;
                any = true;
                ++p_;
            }
            if (!any) fail("bad number");
            while (p_ < t_.size() && (t_[p_] == '.' || t_[p_] == 'e' || t_[p_] == 'E' || t_[p_] == '+' || t_[p_] == '-' ||
                                      std::isdigit((unsigned char)t_[p_]))) {
                v.negative_or_fraction = true;
                ++p_;
            }
        } else if (t_.compare(p_, 4, "null") == 0) {
            p_ += 4;
        } else if (t_.compare(p_, 4, "true") == 0) {
            v.type = Json::boolean; v.u = 1; p_ += 4;
        } else if (t_.compare(p_, 5, "false") == 0) {
            v.type = Json::boolean; p_ += 5;
        } else {
            fail("unexpected character");
        }
        --depth_;
        return v;
    }
    std::string str() {
        expect('"');
        std::string out;
        for (;;) {
            if (p_ >= t_.size()) throw GTurboFormatError(GTurboFormatError::truncated, "packed_experts/layout.json", "truncated");
            const char c = t_[p_++];
            if (c == '"') break;
            if (c != '\\') { out.push_back(c); continue; }
            if (p_ >= t_.size()) fail("bad escape");
            const char e = t_[p_++];
            switch (e) {
                case '"': out.push_back('"'); break;
                case '\\': out.push_back('\\'); break;
                case '/': out.push_back('/'); break;
                case 'b': out.push_back('\b'); break;
                case 'f': out.push_back('\f'); break;
                case 'n': out.push_back('\n'); break;
                case 'r': out.push_back('\r'); break;
                case 't': out.push_back('\t'); break;
                case 'u': {
                    if (p_ + 4 > t_.size()) fail("bad escape");
                    unsigned cp = 0;
                    for (int i = 0; i < 4; ++i) {
                        const char h = t_[p_++];
                        cp = cp * 16 + (std::isdigit((unsigned char)h) ? h - '0' : (std::tolower((unsigned char)h) - 'a' + 10));
                        if (!std::isxdigit((unsigned char)h)) fail("bad escape");
                    }
                    if (cp < 0x80) out.push_back((char)cp);
                    else if (cp < 0x800) { out.push_back((char)(0xC0 | (cp >> 6))); out.push_back((char)(0x80 | (cp & 0x3F))); }
                    else { out.push_back((char)(0xE0 | (cp >> 12))); out.push_back((char)(0x80 | ((cp >> 6) & 0x3F))); out.push_back((char)(0x80 | (cp & 0x3F))); }
                    break;
                }
                default: fail("bad escape");
            }
        }
        return out;
    }
};

inline uint64_t requireU64(const Json &obj, const char *key, const std::string &where) {
    const Json *v = obj.find(key);
    if (!v || v->type != Json::number || v->negative_or_fraction)
        throw GTurboFormatError(GTurboFormatError::invalid, "packed_experts/layout.json", where + "." + key + ": expected an unsigned integer");
    return v->u;
}
inline int requireInt(const Json &obj, const char *key, const std::string &where) {
    const uint64_t u = requireU64(obj, key, where);
    if (u > 0x7FFFFFFFull) throw GTurboFormatError(GTurboFormatError::invalid, "packed_experts/layout.json", where + "." + key + ": out of range");
    return (int)u;
}
// nil when the key is absent or null
inline int optionalInt(const Json &obj, const char *key, const std::string &where, bool &present) {
    const Json *v = obj.find(key);
    present = v && v->type != Json::null_;
    return present ? requireInt(obj, key, where) : 0;
}
inline uint64_t checkedAdd(uint64_t a, uint64_t b, const std::string &field) {
    if (a > UINT64_MAX - b) throw GTurboFormatError(GTurboFormatError::overflow, field, "arithmetic overflow");
    return a + b;
}
inline uint64_t checkedMultiply(uint64_t a, uint64_t b, const std::string &field) {
    if (a != 0 && b > UINT64_MAX / a) throw GTurboFormatError(GTurboFormatError::overflow, field, "arithmetic overflow");
    return a * b;
}

// GTurboPathValidator.validateBasename (GTurboFormatV1.swift:52-79): a safe, canonical, slash-free name
inline void validateBasename(const std::string &name, const std::string &field) {
    if (name.empty() || name[0] == '/' || name.find('\0') != std::string::npos)
        throw GTurboFormatError(GTurboFormatError::invalid, field, "unsafe relative path");
    size_t start = 0;
    for (;;) {
        const size_t slash = name.find('/', start);
        const std::string comp = name.substr(start, slash == std::string::npos ? std::string::npos : slash - start);
        if (comp.empty() || comp == "." || comp == "..")
            throw GTurboFormatError(GTurboFormatError::invalid, field, "non-canonical path");
        if (slash == std::string::npos) break;
        start = slash + 1;
    }
    if (name.find('/') != std::string::npos) throw GTurboFormatError(GTurboFormatError::invalid, field, "expected basename");
}
// appleFilesystemKey (GTurboFormatV1.swift:53-56) for the ASCII names the format uses: case-folded
inline std::string filesystemKey(std::string s) {
    for (char &c : s) c = (char)std::tolower((unsigned char)c);
    return s;
}

}  // namespace detail

struct PackedExpertsLayoutReader {
    static constexpr uint64_t defaultMaxBytes = 16ull * 1024 * 1024;   // PackedExpertsLayout.swift:53

    // GTurboPackedExpertsLayoutCodec.decode + GTurboV1StructuralValidator.validate
    // (GTurboPackedExpertsLayoutV1.swift:66-161), then the sort of PackedExpertsLayoutReader.decode
    // (PackedExpertsLayout.swift:68-88): layers by index, experts by logical id.
    static PackedExpertsLayout decode(const std::string &jsonText) {
        using namespace detail;
        const Json root = JsonParser(jsonText).parse();
        if (root.type != Json::object) throw GTurboFormatError(GTurboFormatError::invalid, "packed_experts/layout.json", "expected an object");
        PackedExpertsLayout out;
        out.expertStride = requireU64(root, "expertStride", "layout");
        out.numLayers = requireInt(root, "numLayers", "layout");
        out.expertsPerLayer = requireInt(root, "expertsPerLayer", "layout");
        const Json *layers = root.find("layers");
        if (!layers || layers->type != Json::array) throw GTurboFormatError(GTurboFormatError::invalid, "packed_experts/layout.json", "layout.layers: expected an array");
        if (out.numLayers <= 0 || out.expertsPerLayer <= 0 || out.expertStride == 0 || out.expertStride % kGTurboAlignmentBytes != 0 ||
            (int)layers->items.size() != out.numLayers)
            throw GTurboFormatError(GTurboFormatError::invalid, "layout", "invalid dimensions or stride");
        std::set<int> layerIDs;
        std::set<std::string> layerFiles;
        for (const Json &lj : layers->items) {
            if (lj.type != Json::object) throw GTurboFormatError(GTurboFormatError::invalid, "layout.layers", "expected an object");
            LayerLayout layer;
            layer.layer = requireInt(lj, "layer", "layout.layers[]");
            const Json *file = lj.find("file");
            const Json *experts = lj.find("experts");
            if (!file || file->type != Json::string || !experts || experts->type != Json::array)
                throw GTurboFormatError(GTurboFormatError::invalid, "layout.layers", "missing file or experts");
            layer.file = file->s;
            if (layer.layer >= out.numLayers || !layerIDs.insert(layer.layer).second)
                throw GTurboFormatError(GTurboFormatError::invalid, "layout.layers", "duplicate or invalid layer");
            const std::string lf = "layout.layers[" + std::to_string(layer.layer) + "]";
            validateBasename(layer.file, lf + ".file");
            const std::string key = filesystemKey(layer.file);
            if (key == "layout.json") throw GTurboFormatError(GTurboFormatError::invalid, lf + ".file", "reserved packed-expert filename");
            if (!layerFiles.insert(key).second) throw GTurboFormatError(GTurboFormatError::invalid, lf + ".file", "duplicate layer filename");
            if ((int)experts->items.size() != out.expertsPerLayer)
                throw GTurboFormatError(GTurboFormatError::invalid, lf + ".experts", "wrong expert count");
            std::set<int> logicalIDs, physicalRanks;
            std::set<uint64_t> offsets;
            int explicitIDs = 0;
            for (const Json &ej : experts->items) {
                if (ej.type != Json::object) throw GTurboFormatError(GTurboFormatError::invalid, lf + ".experts", "expected an object");
                const Json *id = ej.find("expert");
                if (id && id->type != Json::null_) ++explicitIDs;
            }
            if (explicitIDs != 0 && explicitIDs != out.expertsPerLayer)
                throw GTurboFormatError(GTurboFormatError::invalid, lf + ".experts", "expert ids must be either all explicit or all positional");
            int position = 0;
            for (const Json &ej : experts->items) {
                ExpertEntry ex;
                bool hasID = false, hasRank = false;
                const int id = optionalInt(ej, "expert", lf + ".experts[]", hasID);
                const int rank = optionalInt(ej, "physicalRank", lf + ".experts[]", hasRank);
                ex.expert = hasID ? id : position;
                ex.physicalRank = hasRank ? rank : ex.expert;
                ex.offset = requireU64(ej, "offset", lf + ".experts[]");
                ex.size = requireU64(ej, "size", lf + ".experts[]");
                if (ex.expert >= out.expertsPerLayer || ex.physicalRank >= out.expertsPerLayer || !logicalIDs.insert(ex.expert).second ||
                    !physicalRanks.insert(ex.physicalRank).second || !offsets.insert(ex.offset).second)
                    throw GTurboFormatError(GTurboFormatError::invalid, lf + ".experts", "duplicate or invalid expert mapping");
                const std::string ef = "expert[" + std::to_string(ex.expert) + "]";
                if (ex.offset != checkedMultiply((uint64_t)ex.physicalRank, out.expertStride, "expert.offset") || ex.size != out.expertStride)
                    throw GTurboFormatError(GTurboFormatError::invalid, ef, "offset or size does not match physical rank");
                const Json *tensors = ej.find("tensors");
                if (!tensors || tensors->type != Json::object) throw GTurboFormatError(GTurboFormatError::invalid, ef + ".tensors", "expected an object");
                struct Range { uint64_t start, end; std::string name; };
                std::vector<Range> ranges;
                for (const auto &m : tensors->members) {
                    const std::string tf = ef + ".tensors." + m.first;
                    if (m.second.type != Json::object) throw GTurboFormatError(GTurboFormatError::invalid, tf, "expected an object");
                    SubTensorEntry st;
                    st.offset = requireU64(m.second, "offset", tf);
                    st.size = requireU64(m.second, "size", tf);
                    const Json *dtype = m.second.find("dtype");
                    const Json *shape = m.second.find("shape");
                    if (!dtype || dtype->type != Json::string || !shape || shape->type != Json::array)
                        throw GTurboFormatError(GTurboFormatError::invalid, tf, "invalid dtype or shape");
                    st.dtype = dtype->s;
                    bool shapeOK = !shape->items.empty();
                    for (const Json &dim : shape->items) {
                        if (dim.type != Json::number || dim.negative_or_fraction || dim.u == 0 || dim.u > 0xFFFFFFFFull) { shapeOK = false; break; }
                        st.shape.push_back((uint32_t)dim.u);
                    }
                    bool hasBits = false;
                    st.bits = optionalInt(m.second, "bits", tf, hasBits);
                    if ((st.dtype != "U32" && st.dtype != "BF16") || m.first.empty() || st.size == 0 || !shapeOK ||
                        (hasBits && (st.bits <= 0 || st.bits > 32)))
                        throw GTurboFormatError(GTurboFormatError::invalid, tf, "invalid dtype or shape");
                    const uint64_t end = checkedAdd(st.offset, st.size, "tensor." + m.first + ".range");
                    if (end > ex.size) throw GTurboFormatError(GTurboFormatError::invalid, tf, "range exceeds expert blob");
                    if (!ex.subTensors.emplace(m.first, st).second) throw GTurboFormatError(GTurboFormatError::invalid, tf, "duplicate tensor name");
                    ranges.push_back({st.offset, end, m.first});
                }
                std::sort(ranges.begin(), ranges.end(), [](const Range &a, const Range &b) { return a.start == b.start ? a.end < b.end : a.start < b.start; });
                for (size_t i = 0; i + 1 < ranges.size(); ++i)
                    if (ranges[i].end > ranges[i + 1].start)
                        throw GTurboFormatError(GTurboFormatError::invalid, ef + ".tensors", "overlapping ranges " + ranges[i].name + " and " + ranges[i + 1].name);
                layer.experts.push_back(std::move(ex));
                ++position;
            }
            std::sort(layer.experts.begin(), layer.experts.end(), [](const ExpertEntry &a, const ExpertEntry &b) { return a.expert < b.expert; });
            out.layers.push_back(std::move(layer));
        }
        std::sort(out.layers.begin(), out.layers.end(), [](const LayerLayout &a, const LayerLayout &b) { return a.layer < b.layer; });
        return out;
    }

    static PackedExpertsLayout read(const std::string &checkpointDir, uint64_t maxBytes = defaultMaxBytes) {
        const std::string path = checkpointDir + "/packed_experts/layout.json";
        std::ifstream in(path, std::ios::binary);
        if (!in) throw std::runtime_error("cannot open " + path);
        std::ostringstream ss;
        ss << in.rdbuf();
        const std::string text = ss.str();
        if (text.size() > maxBytes) throw GTurboFormatError(GTurboFormatError::invalid, "packed_experts/layout.json", "larger than the reader's limit");
        return decode(text);
    }
};

// MappedExpertLayerError (MappedExpertLayer.swift:6-33)
struct MappedExpertLayerError : std::runtime_error {
    enum Kind { mapFailed, sizeMismatch, misaligned, expertOutOfRange } kind;
    MappedExpertLayerError(Kind k, const std::string &m) : std::runtime_error(m), kind(k) {}
};

// One layer file mapped read-only (MappedExpertLayer.init, MappedExpertLayer.swift:83-140): the same size and
// alignment checks; the experts are plain pointers into the mapping instead of no-copy GPU buffers.
class MappedExpertLayer {
public:
    MappedExpertLayer(const std::string &path, int expertCount, uint64_t expertBytes, const std::vector<uint64_t> &expertOffsets)
        : expertCount_(expertCount), expertBytes_(expertBytes), offsets_(expertOffsets) {
        if ((int)expertOffsets.size() != expertCount) throw std::invalid_argument("one offset per expert");
        const uint64_t page = (uint64_t)sysconf(_SC_PAGESIZE);
        if (expertBytes == 0 || expertBytes % page != 0)
            throw MappedExpertLayerError(MappedExpertLayerError::misaligned, "expert layout is not page aligned: expert stride " +
                                                                                std::to_string(expertBytes) + ", page " + std::to_string(page));
        fd_ = ::open(path.c_str(), O_RDONLY | O_CLOEXEC);
        if (fd_ < 0) throw MappedExpertLayerError(MappedExpertLayerError::mapFailed, "mmap(" + path + ") failed: errno " + std::to_string(errno));
        struct stat info {};
        uint64_t maxOffset = 0;
        for (uint64_t o : expertOffsets) maxOffset = std::max(maxOffset, o);
        const uint64_t required = maxOffset + expertBytes;
        if (fstat(fd_, &info) != 0 || (uint64_t)info.st_size < required) {
            const uint64_t actual = (uint64_t)info.st_size;
            ::close(fd_);
            throw MappedExpertLayerError(MappedExpertLayerError::sizeMismatch, "expert file size mismatch: expected " + std::to_string(required) +
                                                                                  ", got " + std::to_string(actual));
        }
        for (uint64_t o : expertOffsets)
            if (o % page != 0) {
                ::close(fd_);
                throw MappedExpertLayerError(MappedExpertLayerError::misaligned, "expert layout is not page aligned: expert offset " +
                                                                                    std::to_string(o) + ", page " + std::to_string(page));
            }
        bytes_ = (required + page - 1) / page * page;
        void *raw = mmap(nullptr, bytes_, PROT_READ, MAP_SHARED, fd_, 0);
        if (raw == MAP_FAILED) {
            ::close(fd_);
            throw MappedExpertLayerError(MappedExpertLayerError::mapFailed, "mmap(" + path + ") failed: errno " + std::to_string(errno));
        }
        base_ = static_cast<const uint8_t *>(raw);
    }
    ~MappedExpertLayer() {
        if (base_) munmap(const_cast<uint8_t *>(base_), bytes_);
        if (fd_ >= 0) ::close(fd_);
    }
    MappedExpertLayer(const MappedExpertLayer &) = delete;
    MappedExpertLayer &operator=(const MappedExpertLayer &) = delete;
    int expertCount() const { return expertCount_; }
    uint64_t expertBytes() const { return expertBytes_; }
    const uint8_t *base() const { return base_; }
    const uint8_t *expert(int e) const {
        if (e < 0 || e >= expertCount_) throw MappedExpertLayerError(MappedExpertLayerError::expertOutOfRange, "expert " + std::to_string(e) + " is out of range");
        return base_ + offsets_[e];
    }

private:
    int expertCount_;
    uint64_t expertBytes_;
    std::vector<uint64_t> offsets_;
    int fd_ = -1;
    const uint8_t *base_ = nullptr;
    size_t bytes_ = 0;
};

// The nine sub-tensors of a routed expert must have the byte sizes the context's shape implies.
inline void checkRoutedExpertTensors(const ExpertEntry &ex, const ffmoe_shape &sh) {
    const uint64_t guW = (uint64_t)sh.f * sh.d / 2, guS = (uint64_t)sh.f * (sh.d / 64) * 2;
    const uint64_t dnW = (uint64_t)sh.d * sh.f / 2, dnS = (uint64_t)sh.d * (sh.f / 64) * 2;
    const struct { const char *role; uint64_t size; const char *dtype; } want[9] = {
        {"gate", guW, "U32"}, {"gate_scales", guS, "BF16"}, {"gate_biases", guS, "BF16"}, {"up", guW, "U32"},    {"up_scales", guS, "BF16"},
        {"up_biases", guS, "BF16"}, {"down", dnW, "U32"},   {"down_scales", dnS, "BF16"}, {"down_biases", dnS, "BF16"}};
    for (const auto &w : want) {
        auto it = ex.subTensors.find(w.role);
        if (it == ex.subTensors.end())
            throw GTurboFormatError(GTurboFormatError::invalid, "expert[" + std::to_string(ex.expert) + "].tensors", std::string("missing ") + w.role);
        if (it->second.size != w.size || it->second.dtype != w.dtype || (it->second.bits != 0 && w.dtype[0] == 'U' && it->second.bits != 4))
            throw GTurboFormatError(GTurboFormatError::invalid, "expert[" + std::to_string(ex.expert) + "].tensors." + w.role,
                                    "size, dtype or bits do not match d = " + std::to_string(sh.d) + ", f = " + std::to_string(sh.f));
    }
}

// Loads every layer named by the layout into the context's arena. A layer whose experts sit at their logical
// positions with the offsets of expert 0 goes up as one copy of the mapped file; any other layer (reordered
// physical ranks, per-expert tensor offsets) goes up expert by expert. Returns the bytes read from storage.
inline uint64_t uploadPackedExperts(Context &ctx, const std::string &checkpointDir, const PackedExpertsLayout &layout) {
    const ffmoe_shape &sh = ctx.shape();
    if ((uint32_t)layout.numLayers != sh.n_layers || (uint32_t)layout.expertsPerLayer != sh.n_experts)
        throw GTurboFormatError(GTurboFormatError::invalid, "manifest/layout", "dimension mismatch");
    uint64_t total = 0;
    for (const LayerLayout &layer : layout.layers) {
        for (const ExpertEntry &ex : layer.experts) checkRoutedExpertTensors(ex, sh);
        const std::string path = checkpointDir + "/packed_experts/" + layer.file;
        MappedExpertLayer mapped(path, layout.expertsPerLayer, layout.expertStride, layout.routedExpertPhysicalOffsets(layer.layer));
        const ffmoe_offsets first = layout.routedExpertOffsets(layer.layer);
        bool uniform = true;
        for (const ExpertEntry &ex : layer.experts) {
            uniform = uniform && ex.physicalRank == ex.expert;
            const char *roles[9] = {"gate", "gate_scales", "gate_biases", "up", "up_scales", "up_biases", "down", "down_scales", "down_biases"};
            const uint32_t offs[9] = {first.gate_w, first.gate_s, first.gate_b, first.up_w, first.up_s, first.up_b, first.down_w, first.down_s, first.down_b};
            for (int i = 0; i < 9; ++i) uniform = uniform && ex.subTensors.at(roles[i]).offset == offs[i];
        }
        if (uniform) {
            ctx.uploadLayer((uint32_t)layer.layer, mapped.base(), layout.expertStride, first);
        } else {
            for (const ExpertEntry &ex : layer.experts) {
                const uint8_t *blob = mapped.expert(ex.expert);
                auto proj = [&](const char *w, const char *s, const char *b) {
                    return ffmoe_projection{blob + ex.subTensors.at(w).offset, reinterpret_cast<const uint16_t *>(blob + ex.subTensors.at(s).offset),
                                            reinterpret_cast<const uint16_t *>(blob + ex.subTensors.at(b).offset)};
                };
                const ffmoe_projection g = proj("gate", "gate_scales", "gate_biases"), u = proj("up", "up_scales", "up_biases"),
                                       dn = proj("down", "down_scales", "down_biases");
                char *err = nullptr;
                check(ffmoe_upload_expert_parts(ctx.raw(), (uint32_t)layer.layer, (uint32_t)ex.expert, &g, &u, &dn, 0, &err), err);
            }
        }
        total += (uint64_t)layout.expertsPerLayer * layout.expertStride;
    }
    return total;
}

}  // namespace fieldfare
