// Host helpers of the operator surface: logging, status check, raw binary file I/O.
// Counterpart of the reference's utils/utils.h:22-117 with acl* replaced by the cch_* C ABI.
#ifndef CATCCOS_HOST_UTILS_H
#define CATCCOS_HOST_UTILS_H

#include <fcntl.h>
#include <sys/file.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cerrno>
#include <cstdio>
#include <cstring>
#include <string>

#include "catccos_hip.h"

// The strings "[ERROR]" and "error num:" are what the reference's run_all_examples.sh greps for.
#define INFO_LOG(fmt, ...) fprintf(stdout, "[INFO] " fmt "\n", ##__VA_ARGS__)
#define WARN_LOG(fmt, ...) fprintf(stdout, "[WARN] " fmt "\n", ##__VA_ARGS__)
#define ERROR_LOG(fmt, ...) fprintf(stdout, "[ERROR] " fmt "\n", ##__VA_ARGS__)

// Like the reference's ACL_CHECK: report and carry on; callers that must stop test the code.
#define CCH_CHECK(call)                                                                              \
    do {                                                                                             \
        int cch_status_ = (call);                                                                    \
        if (cch_status_ != CCH_OK)                                                                   \
            fprintf(stderr, "%s:%d cchError:%d %s\n", __FILE__, __LINE__, cch_status_, cch_last_error()); \
    } while (0)

// Reads a whole regular file into `buffer`; fails if it is missing, empty or larger than the buffer.
inline bool ReadFile(const std::string &filePath, void *buffer, size_t bufferSize, size_t *bytesRead = nullptr)
{
    struct stat st;
    if (stat(filePath.c_str(), &st) != 0) {
        ERROR_LOG("Failed to get file %s", filePath.c_str());
        return false;
    }
    if (!S_ISREG(st.st_mode)) {
        ERROR_LOG("%s is not a file, please enter a file.", filePath.c_str());
        return false;
    }
    const size_t size = static_cast<size_t>(st.st_size);
    if (size == 0) {
        ERROR_LOG("File size is 0");
        return false;
    }
    if (size > bufferSize) {
        ERROR_LOG("File size is larger than buffer size.");
        return false;
    }
    FILE *f = fopen(filePath.c_str(), "rb");
    if (!f) {
        ERROR_LOG("Open file failed. path = %s.", filePath.c_str());
        return false;
    }
    const size_t got = fread(buffer, 1, size, f);
    fclose(f);
    if (bytesRead) *bytesRead = got;
    return got == size;
}

// Writes `size` bytes at `offset` under an exclusive flock: several ranks may fill slices of one file.
inline bool WriteFile(const std::string &filePath, const void *buffer, size_t size, size_t offset = 0)
{
    if (buffer == nullptr) {
        ERROR_LOG("Write file failed. Buffer is nullptr.");
        return false;
    }
    const int fd = open(filePath.c_str(), O_RDWR | O_CREAT, 0666);
    if (fd == -1) {
        ERROR_LOG("Open file failed. path = %s", filePath.c_str());
        return false;
    }
    bool ok = true;
    if (flock(fd, LOCK_EX) == -1) {
        fprintf(stderr, "Failed to acquire lock: %s\n", strerror(errno));
        ok = false;
    } else {
        if (pwrite(fd, buffer, size, static_cast<off_t>(offset)) != static_cast<ssize_t>(size)) {
            fprintf(stderr, "Failed to write to file: %s\n", strerror(errno));
            ok = false;
        }
        flock(fd, LOCK_UN);
    }
    close(fd);
    return ok;
}

#endif  // CATCCOS_HOST_UTILS_H
