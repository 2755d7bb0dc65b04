// safetensors_lite.h — reads a .safetensors file: 8 bytes little-endian header length, that many bytes of JSON
// (name -> {dtype, shape, data_offsets}), then the tensors' bytes.  The file is memory-mapped; nothing in it is executed.
#ifndef SAFETENSORS_LITE_H
#define SAFETENSORS_LITE_H
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

#include "json_lite.h"

struct st_tensor {
    std::string name, dtype;  // "BF16", "F32", "F16", "I32", ...
    std::vector<int64_t> shape;
    const uint8_t * data = nullptr;
    size_t size = 0;
    int64_t numel() const {
        int64_t n = 1;
        for (int64_t d : shape) n *= d;
        return n;
    }
};

struct st_file {
    void * map = nullptr;
    size_t map_size = 0;
    std::vector<st_tensor> tensors;
    ~st_file() {
        if (map) munmap(map, map_size);
    }
    const st_tensor * find(const std::string & name) const {
        for (auto & t : tensors)
            if (t.name == name) return &t;
        return nullptr;
    }
    static size_t dtype_size(const std::string & d) {
        if (d == "F64" || d == "I64" || d == "U64") return 8;
        if (d == "F32" || d == "I32" || d == "U32") return 4;
        if (d == "BF16" || d == "F16" || d == "I16" || d == "U16") return 2;
        if (d == "I8" || d == "U8" || d == "BOOL" || d == "F8_E4M3" || d == "F8_E5M2") return 1;
        return 0;
    }
    // nullptr (with a message on stderr) when the file is missing, truncated or inconsistent
    static st_file * open(const char * path) {
        const int fd = ::open(path, O_RDONLY);
        if (fd < 0) { fprintf(stderr, "safetensors: cannot open %s\n", path); return nullptr; }
        struct stat sb;
        if (fstat(fd, &sb) != 0 || sb.st_size < 8) { close(fd); fprintf(stderr, "safetensors: %s is too short\n", path); return nullptr; }
        st_file * f = new st_file();
        f->map_size = (size_t) sb.st_size;
        f->map = mmap(nullptr, f->map_size, PROT_READ, MAP_PRIVATE, fd, 0);
        close(fd);
        if (f->map == MAP_FAILED) { f->map = nullptr; delete f; fprintf(stderr, "safetensors: mmap of %s failed\n", path); return nullptr; }
        const uint8_t * p = (const uint8_t *) f->map;
        uint64_t hlen = 0;
        for (int i = 7; i >= 0; --i) hlen = (hlen << 8) | p[i];
        if (hlen > f->map_size - 8) { delete f; fprintf(stderr, "safetensors: %s: header length beyond the file\n", path); return nullptr; }
        json_value head;
        if (!json_parser::parse((const char *) p + 8, (size_t) hlen, head) || head.kind != json_value::OBJ) {
            delete f;
            fprintf(stderr, "safetensors: %s: header is not a JSON object\n", path);
            return nullptr;
        }
        const uint8_t * base = p + 8 + hlen;
        const size_t data_size = f->map_size - 8 - (size_t) hlen;
        for (auto & kv : head.obj) {
            if (kv.first == "__metadata__") continue;
            const json_value * dt = kv.second.get("dtype"), * sh = kv.second.get("shape"), * off = kv.second.get("data_offsets");
            if (!dt || !sh || !off || dt->kind != json_value::STR || sh->kind != json_value::ARR || off->kind != json_value::ARR || off->arr.size() != 2) {
                delete f;
                fprintf(stderr, "safetensors: %s: malformed entry %s\n", path, kv.first.c_str());
                return nullptr;
            }
            st_tensor t;
            t.name = kv.first;
            t.dtype = dt->str;
            for (auto & d : sh->arr) t.shape.push_back((int64_t) d.number(0));
            const uint64_t a = (uint64_t) off->arr[0].number(0), b = (uint64_t) off->arr[1].number(0);
            if (b < a || b > data_size || (uint64_t) t.numel() * dtype_size(t.dtype) != b - a) {
                delete f;
                fprintf(stderr, "safetensors: %s: tensor %s does not fit its byte range\n", path, kv.first.c_str());
                return nullptr;
            }
            t.data = base + a;
            t.size = (size_t) (b - a);
            f->tensors.push_back(std::move(t));
        }
        return f;
    }
};
#endif
