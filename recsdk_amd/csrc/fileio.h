// Plain local-file helpers of the checkpoint code (what the reference's LocalFileSystem does for raw array files:
// training/tf_rec_v1/src/core/file_system/local_file_system/local_file_system.cpp).
#ifndef RECSDK_CSRC_FILEIO_H
#define RECSDK_CSRC_FILEIO_H

#include <errno.h>
#include <fcntl.h>
#include <string.h>
#include <sys/stat.h>
#include <sys/types.h>
#include <unistd.h>

#include <string>
#include <vector>

#include "common.h"

namespace recsdk {

// mkdir -p of the directory part of `path` (LocalFileSystem::CreateFileDir / CreateDir, mode 0750)
inline bool make_parent_dirs(const std::string& path)
{
    for (size_t i = 1; i < path.size(); ++i) {
        if (path[i] != '/') {
            continue;
        }
        const std::string dir = path.substr(0, i);
        if (mkdir(dir.c_str(), 0750) != 0 && errno != EEXIST) {
            return false;
        }
    }
    return true;
}

inline int64_t file_size_of(const std::string& path)
{
    struct stat st;
    if (stat(path.c_str(), &st) != 0) {
        return -1;
    }
    return (int64_t)st.st_size;
}

inline bool write_all(int fd, const void* data, size_t bytes)
{
    const char* p = static_cast<const char*>(data);
    while (bytes > 0) {
        const ssize_t w = write(fd, p, bytes);
        if (w < 0) {
            if (errno == EINTR) {
                continue;
            }
            return false;
        }
        p += w;
        bytes -= (size_t)w;
    }
    return true;
}

inline bool read_all_at(int fd, void* data, size_t bytes, int64_t offset)
{
    char* p = static_cast<char*>(data);
    while (bytes > 0) {
        const ssize_t r = pread(fd, p, bytes, offset);
        if (r < 0 && errno == EINTR) {
            continue;
        }
        if (r <= 0) {
            return false;
        }
        p += r;
        offset += r;
        bytes -= (size_t)r;
    }
    return true;
}

// Create (truncate) `path`, parents included, and write the bytes.  Returns a RECSDK_* code.
inline int write_file(const std::string& path, const void* data, size_t bytes)
{
    if (!make_parent_dirs(path)) {
        set_error("Create directory for %s failed: %s", path.c_str(), strerror(errno));
        return RECSDK_EIO;
    }
    const int fd = open(path.c_str(), O_RDWR | O_CREAT | O_TRUNC, 0640);
    if (fd == -1) {
        set_error("Open file %s to write failed.", path.c_str());
        return RECSDK_EIO;
    }
    const bool ok = write_all(fd, data, bytes);
    close(fd);
    if (!ok) {
        set_error("Error writing to local file %s, please check the disk space or file permissions!", path.c_str());
        return RECSDK_EIO;
    }
    return RECSDK_OK;
}

// Whole file into `out` (elements of `elem` bytes; a size that is no multiple of it is an error).
inline int read_file(const std::string& path, size_t elem, std::vector<char>* out)
{
    const int64_t size = file_size_of(path);
    if (size < 0) {
        set_error("Failed to open read file: %s.", path.c_str());
        return RECSDK_EIO;
    }
    if (elem > 1 && size % (int64_t)elem != 0) {
        set_error("Data is missing or incomplete in load file: %s.", path.c_str());
        return RECSDK_EIO;
    }
    out->resize((size_t)size);
    const int fd = open(path.c_str(), O_RDONLY);
    if (fd == -1) {
        set_error("Failed to open read file: %s.", path.c_str());
        return RECSDK_EIO;
    }
    const bool ok = size == 0 || read_all_at(fd, out->data(), (size_t)size, 0);
    close(fd);
    if (!ok) {
        set_error("Failed to read file path: %s.", path.c_str());
        return RECSDK_EIO;
    }
    return RECSDK_OK;
}

}  // namespace recsdk

#endif
