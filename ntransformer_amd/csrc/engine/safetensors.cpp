// engine/safetensors.cpp -- see safetensors.h
#include "safetensors.h"
#include "../../../include/ntk.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>
#include <cstdio>
#include <fstream>
#include <sstream>

namespace nt {

static bool read_file(const std::string& path, std::string& out) {
    std::ifstream f(path, std::ios::binary);
    if (!f) return false;
    std::ostringstream ss;
    ss << f.rdbuf();
    out = ss.str();
    return true;
}

static size_t dtype_bytes(const std::string& d) {
    if (d == "BF16" || d == "F16" || d == "I16" || d == "U16") return 2;
    if (d == "F32" || d == "I32" || d == "U32") return 4;
    if (d == "F64" || d == "I64" || d == "U64") return 8;
    if (d == "I8" || d == "U8" || d == "BOOL") return 1;
    return 0;
}

ModelFolder::~ModelFolder() {
    if (map_) munmap(map_, map_bytes_);
}

bool ModelFolder::looks_like(const std::string& path) {
    struct stat st;
    if (stat(path.c_str(), &st) != 0 || !S_ISDIR(st.st_mode)) return false;
    return stat((path + "/config.json").c_str(), &st) == 0;
}

std::string ModelFolder::architecture_of(const std::string& path) {
    std::string txt;
    if (!read_file(path + "/config.json", txt)) return "";
    Json j;
    if (!j.parse(txt.data(), txt.size())) return "";
    return j.at("architecture").is_string() ? j.at("architecture").str : "";
}

int ModelFolder::open(const std::string& dir) {
    std::string txt;
    if (!read_file(dir + "/config.json", txt)) { err_ = "cannot read " + dir + "/config.json"; return NTK_E_IO; }
    if (!config_.parse(txt.data(), txt.size()) || !config_.is_object()) { err_ = "config.json is not a JSON object"; return NTK_E_FORMAT; }
    const std::string path = dir + "/model.safetensors";
    const int fd = ::open(path.c_str(), O_RDONLY);
    if (fd < 0) { err_ = "cannot open " + path; return NTK_E_IO; }
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size < 8) { ::close(fd); err_ = "model.safetensors is too short"; return NTK_E_FORMAT; }
    map_bytes_ = (size_t)st.st_size;
    map_ = mmap(nullptr, map_bytes_, PROT_READ, MAP_PRIVATE, fd, 0);
    ::close(fd);
    if (map_ == MAP_FAILED) { map_ = nullptr; err_ = "cannot map " + path; return NTK_E_IO; }
    const uint8_t* base = (const uint8_t*)map_;
    uint64_t hlen = 0;
    for (int i = 7; i >= 0; --i) hlen = (hlen << 8) | base[i];
    if (hlen > map_bytes_ - 8) { err_ = "safetensors header runs past the file"; return NTK_E_FORMAT; }
    Json header;
    if (!header.parse((const char*)base + 8, (size_t)hlen) || !header.is_object()) { err_ = "safetensors header is not a JSON object"; return NTK_E_FORMAT; }
    const uint8_t* data = base + 8 + hlen;
    const size_t data_bytes = map_bytes_ - 8 - (size_t)hlen;
    for (const auto& kv : header.obj) {
        if (kv.first == "__metadata__") continue;
        const Json& m = kv.second;
        StTensor t;
        t.dtype = m.at("dtype").str;
        for (const auto& d : m.at("shape").arr) t.shape.push_back(d.integer());
        const auto& off = m.at("data_offsets").arr;
        if (off.size() != 2) { err_ = "tensor " + kv.first + ": no data_offsets"; return NTK_E_FORMAT; }
        const uint64_t a = (uint64_t)off[0].integer(), b = (uint64_t)off[1].integer();
        const size_t eb = dtype_bytes(t.dtype);
        if (b < a || b > data_bytes || eb == 0 || (uint64_t)t.numel() * eb != b - a) { err_ = "tensor " + kv.first + ": offsets do not fit its shape"; return NTK_E_FORMAT; }
        t.data = data + a;
        t.nbytes = (size_t)(b - a);
        tensors_.emplace(kv.first, std::move(t));
    }
    return NTK_OK;
}

const StTensor* ModelFolder::tensor(const std::string& name) const {
    auto it = tensors_.find(name);
    return it == tensors_.end() ? nullptr : &it->second;
}

}  // namespace nt
