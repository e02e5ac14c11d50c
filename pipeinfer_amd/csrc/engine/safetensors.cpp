#include "safetensors.h"
#include "json.h"

#include <cstring>
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

namespace pi {

safetensors_file::~safetensors_file() { if (map_) munmap(map_, map_len_); }

bool safetensors_file::open(const std::string & path, std::string & err) {
    const int fd = ::open(path.c_str(), O_RDONLY);
    if (fd < 0) { err = "cannot open " + path; return false; }
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size < 8) { close(fd); err = path + " is not a safetensors file (too short)"; return false; }
    map_len_ = (size_t) st.st_size;
    map_ = mmap(nullptr, map_len_, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (map_ == MAP_FAILED) { map_ = nullptr; err = "mmap of " + path + " failed"; return false; }
    file_bytes = map_len_;
    const uint8_t * base = (const uint8_t *) map_;
    uint64_t hlen = 0;
    for (int i = 7; i >= 0; i--) hlen = (hlen << 8) | base[i];
    if (hlen > map_len_ - 8) { err = path + ": header length beyond the end of the file"; return false; }
    json head;
    if (!json::parse(std::string((const char *) base + 8, (size_t) hlen), head, err)) { err = path + ": header: " + err; return false; }
    if (!head.is_obj()) { err = path + ": header is not an object"; return false; }
    const uint8_t * data = base + 8 + hlen;
    const size_t data_len = map_len_ - 8 - (size_t) hlen;
    for (const auto & kv : head.obj) {
        if (kv.first == "__metadata__") continue;
        const json * dt = kv.second.find("dtype"), * sh = kv.second.find("shape"), * off = kv.second.find("data_offsets");
        if (!dt || !dt->is_str() || !sh || !sh->is_arr() || !off || !off->is_arr() || off->arr.size() != 2) { err = path + ": malformed entry for tensor " + kv.first; return false; }
        st_tensor t;
        t.dtype = dt->str;
        for (const json & d : sh->arr) t.shape.push_back((int64_t) d.num);
        const uint64_t a = (uint64_t) off->arr[0].num, b = (uint64_t) off->arr[1].num;
        if (a > b || b > data_len) { err = path + ": tensor " + kv.first + " lies outside the file"; return false; }
        t.data = data + a; t.nbytes = (size_t) (b - a);
        const size_t esz = t.dtype == "BF16" || t.dtype == "F16" ? 2 : t.dtype == "F32" || t.dtype == "I32" ? 4 : t.dtype == "F64" || t.dtype == "I64" ? 8 : 1;
        if ((size_t) t.elements() * esz != t.nbytes) { err = path + ": tensor " + kv.first + " has " + std::to_string(t.nbytes) + " bytes for its shape and type"; return false; }
        tensors[kv.first] = std::move(t);
    }
    return true;
}

}  // namespace pi
