// safetensors.h — read-only view of a .safetensors file: an 8-byte little-endian header length, that many bytes of JSON (tensor name -> dtype, shape,
// data_offsets relative to the end of the header), then the tensor bytes.  The file is mapped, nothing is copied; every offset is checked against the file.
#pragma once

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdint>
#include <map>
#include <string>
#include <vector>

#include "json.h"

namespace mi355 {

struct SafeTensor {
    std::string dtype;
    std::vector<int64_t> shape;
    const uint8_t *data = nullptr;
    size_t bytes = 0;
    int64_t numel() const { int64_t n = 1; for (int64_t d : shape) n *= d; return n; }
};

class SafeTensorsFile {
  public:
    SafeTensorsFile() = default;
    SafeTensorsFile(const SafeTensorsFile &) = delete;
    SafeTensorsFile &operator=(const SafeTensorsFile &) = delete;
    ~SafeTensorsFile() {
        if (map_ && map_ != MAP_FAILED) munmap(map_, size_);
        if (fd_ >= 0) close(fd_);
    }
    // "" on success, else what is wrong with the file
    std::string open(const std::string &path) {
        fd_ = ::open(path.c_str(), O_RDONLY);
        if (fd_ < 0) return "cannot open " + path;
        struct stat st;
        if (fstat(fd_, &st) != 0 || st.st_size < 8) return path + ": too short for a safetensors header";
        size_ = (size_t)st.st_size;
        map_ = mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd_, 0);
        if (map_ == MAP_FAILED) { map_ = nullptr; return "cannot map " + path; }
        const uint8_t *p = (const uint8_t *)map_;
        uint64_t hl = 0;
        for (int i = 7; i >= 0; i--) hl = (hl << 8) | p[i];
        if (hl > size_ - 8 || hl > (1ull << 30)) return path + ": header length out of range";
        Json head;
        std::string jerr;
        if (!Json::parse(std::string((const char *)p + 8, (size_t)hl), head, &jerr) || !head.is_object()) return path + ": header is not a JSON object (" + jerr + ")";
        const uint8_t *base = p + 8 + hl;
        const size_t room = size_ - 8 - (size_t)hl;
        for (const auto &kv : head.members()) {
            if (kv.first == "__metadata__") continue;
            const Json &t = kv.second;
            SafeTensor st2;
            st2.dtype = t["dtype"].as_string();
            for (const Json &d : t["shape"].items()) { if (d.as_int(-1) < 0) return path + ": negative dimension in " + kv.first; st2.shape.push_back(d.as_int()); }
            const Json &off = t["data_offsets"];
            if (!off.is_array() || off.size() != 2) return path + ": " + kv.first + " has no data_offsets";
            const int64_t a = off.at(0).as_int(-1), b = off.at(1).as_int(-1);
            if (a < 0 || b < a || (uint64_t)b > room) return path + ": " + kv.first + " lies outside the file";
            const int es = st2.dtype == "BF16" || st2.dtype == "F16" ? 2 : st2.dtype == "F32" || st2.dtype == "I32" ? 4 : st2.dtype == "F64" || st2.dtype == "I64" ? 8 : 0;
            if (!es) return path + ": " + kv.first + " has unsupported dtype " + st2.dtype;
            st2.data = base + a;
            st2.bytes = (size_t)(b - a);
            if ((uint64_t)st2.numel() * (uint64_t)es != st2.bytes) return path + ": " + kv.first + " shape does not match its byte range";
            tensors_[kv.first] = st2;
        }
        return "";
    }
    const SafeTensor *find(const std::string &name) const {
        auto it = tensors_.find(name);
        return it == tensors_.end() ? nullptr : &it->second;
    }
    const std::map<std::string, SafeTensor> &tensors() const { return tensors_; }
    size_t file_bytes() const { return size_; }

  private:
    int fd_ = -1;
    void *map_ = nullptr;
    size_t size_ = 0;
    std::map<std::string, SafeTensor> tensors_;
};

}  // namespace mi355
