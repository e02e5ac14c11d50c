// Reader of a safetensors file: 8-byte little-endian header length, that many bytes of JSON (name -> dtype, shape, data_offsets), then the tensor bytes.  The file is mapped,
// not copied; tensors point into the mapping.
#pragma once

#include <cstdint>
#include <map>
#include <string>
#include <vector>

namespace pi {

struct st_tensor {
    std::string dtype;                     // "BF16", "F32", "F16", "I32", ...
    std::vector<int64_t> shape;
    const uint8_t * data = nullptr;
    size_t nbytes = 0;
    int64_t elements() const { int64_t n = 1; for (int64_t d : shape) n *= d; return n; }
};

class safetensors_file {
public:
    ~safetensors_file();
    bool open(const std::string & path, std::string & err);
    const st_tensor * tensor(const std::string & name) const { auto it = tensors.find(name); return it == tensors.end() ? nullptr : &it->second; }
    std::map<std::string, st_tensor> tensors;
    size_t file_bytes = 0;
private:
    void * map_ = nullptr; size_t map_len_ = 0;
};

}  // namespace pi
