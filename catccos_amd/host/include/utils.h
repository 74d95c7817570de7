// Logging macros and raw .bin file helpers of the host plugin layer.
// Mirrors the helper set of the reference's utils/utils.h:24-140 (INFO_LOG/WARN_LOG/ERROR_LOG, ReadFile,
// ReadFileOrThrow, WriteFile with an exclusive lock and a byte offset) on plain POSIX.
#ifndef UTILS_H
#define UTILS_H

#include <fcntl.h>
#include <sys/file.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cerrno>
#include <climits>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <iostream>
#include <stdexcept>
#include <string>

#include "mx_runtime.h"

#define INFO_LOG(fmt, args...) fprintf(stdout, "[INFO] " fmt "\n", ##args)
#define WARN_LOG(fmt, args...) fprintf(stdout, "[WARN] " fmt "\n", ##args)
#define ERROR_LOG(fmt, args...) fprintf(stdout, "[ERROR] " fmt "\n", ##args)

// Reads exactly bufferSize bytes; a missing, empty or differently sized file is an error.
inline bool ReadFile(const std::string& filePath, void* buffer, size_t bufferSize)
{
    struct stat info {};
    if (stat(filePath.c_str(), &info) != 0) {
        ERROR_LOG("Failed to get file");
        return false;
    }
    if (!S_ISREG(info.st_mode)) {
        ERROR_LOG("%s is not a file, please enter a file.", filePath.c_str());
        return false;
    }
    if (info.st_size == 0) {
        ERROR_LOG("File size is 0");
        return false;
    }
    if (static_cast<size_t>(info.st_size) != bufferSize) {
        ERROR_LOG("File size does not match buffer size.");
        return false;
    }
    std::ifstream in(filePath, std::ios::binary);
    if (!in) {
        ERROR_LOG("Open file failed. path = %s.", filePath.c_str());
        return false;
    }
    in.read(static_cast<char*>(buffer), static_cast<std::streamsize>(bufferSize));
    if (static_cast<size_t>(in.gcount()) != bufferSize) {
        ERROR_LOG("Failed to read the complete file.");
        return false;
    }
    return true;
}

inline void ReadFileOrThrow(const std::string& filePath, void* buffer, size_t bufferSize)
{
    if (!ReadFile(filePath, buffer, bufferSize)) {
        throw std::runtime_error("Failed to read file: " + filePath);
    }
}

// Writes size bytes at byte `offset` under an exclusive flock, so several ranks can fill one file.
inline bool WriteFile(const std::string& filePath, const void* buffer, size_t size, size_t offset = 0)
{
    if (buffer == nullptr) {
        ERROR_LOG("Write file failed. Buffer is nullptr.");
        return false;
    }
    const int fd = open(filePath.c_str(), O_RDWR | O_CREAT, 0666);
    if (fd < 0) {
        ERROR_LOG("Open file failed. path = %s", filePath.c_str());
        return false;
    }
    bool ok = false;
    if (flock(fd, LOCK_EX) != 0) {
        std::cerr << "Failed to acquire lock: " << strerror(errno) << std::endl;
    } else {
        const ssize_t written = pwrite(fd, buffer, size, static_cast<off_t>(offset));
        if (written == static_cast<ssize_t>(size)) {
            ok = true;
        } else if (written < 0) {
            std::cerr << "Failed to write to file: " << strerror(errno) << std::endl;
        } else {
            std::cerr << "Incomplete file write: " << written << " of " << size << " bytes" << std::endl;
        }
        flock(fd, LOCK_UN);
    }
    close(fd);
    return ok;
}

#endif  // UTILS_H
