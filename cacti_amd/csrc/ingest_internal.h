// What the checkpoint readers (safetensors, torch pickle archives) share: one table of named tensors
// over memory-mapped files.  TensorsDir (src/util/safetensor.rs:34-43) and PickleDir
// (src/util/safepickle.rs:36-44) hold the same fields: file paths, names in order of appearance, a
// sorted name set and a name -> (file, tensor) map.
#pragma once
#include <stdint.h>
#include <sys/mman.h>
#include <unistd.h>

#include <map>
#include <string>
#include <vector>

namespace cacti {

struct TensorEntry {
    std::string dtype;                  // safetensors spelling: "F16", "BF16", "F32", ...
    std::vector<int64_t> shape;
    int file = 0;
    uint64_t off = 0, eoff = 0;         // absolute byte range in the file
};

struct MappedFile {
    std::string path;
    int fd = -1;
    void *base = nullptr;
    size_t size = 0;
};

size_t ingest_dtype_bytes(const std::string &d);

// opens and maps `path` read-only into `mf`; a status of include/cacti_hip_runtime.h
int ingest_map_file(const std::string &path, size_t min_size, const char *who, MappedFile *mf);

}  // namespace cacti

struct cacti_tensors_dir {
    std::string path;
    std::vector<cacti::MappedFile> files;
    std::vector<std::string> serial_key;                        // order of appearance
    std::map<std::string, cacti::TensorEntry> tensors;          // byte-wise sorted names (BTreeMap<SmolStr, ..>)
    std::vector<const std::string *> sorted;                    // index -> name

    ~cacti_tensors_dir()
    {
        for (cacti::MappedFile &f : files) {
            if (f.base && f.base != MAP_FAILED) munmap(f.base, f.size);
            if (f.fd >= 0) close(f.fd);
        }
    }
};
