// The metadata wire format of the reference (src/utils/serdes/serdes.cpp:23-169), so that a
// blob made by getLocalMD here is one the reference's loadRemoteMD parses and vice versa:
//
//   "nixlSerDes|"  then, per item:  tag bytes | length (8 bytes, host order) | payload | '|'
//
// Items are read back in the order they were written; a reader names the tag it expects and
// gets an empty string / NIXL_ERR_MISMATCH when the next item carries another one.
#ifndef NIXL_AMD_AGENT_SERDES_H
#define NIXL_AMD_AGENT_SERDES_H

#include <cstdint>
#include <cstring>
#include <string>

#include "common/nixl_log.h"
#include "nixl_types.h"

class nixlSerDes {
public:
    nixlSerDes() : bytes_(kHeader), cursor_(bytes_.size()) {}

    nixl_status_t
    addStr(const std::string &tag, const std::string &str) {
        return addBuf(tag, str.data(), static_cast<ssize_t>(str.size()));
    }

    nixl_status_t
    addBuf(const std::string &tag, const void *buf, ssize_t len) {
        if (len < 0 || (len > 0 && !buf)) return NIXL_ERR_INVALID_PARAM;
        const uint64_t n = static_cast<uint64_t>(len);
        bytes_.append(tag);
        bytes_.append(reinterpret_cast<const char *>(&n), sizeof(n));
        bytes_.append(static_cast<const char *>(buf), static_cast<size_t>(len));
        bytes_.push_back('|');
        return NIXL_SUCCESS;
    }

    // Payload of the next item, which must carry `tag`; empty on any mismatch.  Only the
    // "msg" item may legitimately be empty (serdes.cpp:75-77).
    std::string
    getStr(const std::string &tag) {
        uint64_t n = 0;
        if (!peek(tag, n)) return "";
        const size_t at = cursor_ + tag.size() + sizeof(n);
        if (bytes_.size() - at < n + 1) {
            NIXL_ERROR << "deserialization of tag '" << tag << "' failed: incomplete data";
            return "";
        }
        cursor_ = at + n + 1;
        return bytes_.substr(at, n);
    }

    // Length of the next item's payload, or -1.
    ssize_t
    getBufLen(const std::string &tag) const {
        uint64_t n = 0;
        return peek(tag, n) ? static_cast<ssize_t>(n) : -1;
    }

    nixl_status_t
    getBuf(const std::string &tag, void *buf, ssize_t len) {
        uint64_t n = 0;
        if (!peek(tag, n) || len < 0 || static_cast<uint64_t>(len) != n) return NIXL_ERR_MISMATCH;
        const size_t at = cursor_ + tag.size() + sizeof(n);
        if (bytes_.size() - at < n + 1) return NIXL_ERR_MISMATCH;
        std::memcpy(buf, bytes_.data() + at, n);
        cursor_ = at + n + 1;
        return NIXL_SUCCESS;
    }

    std::string
    exportStr() const {
        return bytes_;
    }

    nixl_status_t
    importStr(const std::string &blob) {
        if (blob.compare(0, std::strlen(kHeader), kHeader) != 0) {
            NIXL_ERROR << "deserialization failed: missing nixlSerDes header";
            return NIXL_ERR_MISMATCH;
        }
        bytes_ = blob;
        cursor_ = std::strlen(kHeader);
        return NIXL_SUCCESS;
    }

private:
    static constexpr const char *kHeader = "nixlSerDes|";

    bool
    peek(const std::string &tag, uint64_t &n) const {
        if (bytes_.size() < cursor_ + tag.size() + sizeof(n)) return false;
        if (std::memcmp(bytes_.data() + cursor_, tag.data(), tag.size()) != 0) return false;
        std::memcpy(&n, bytes_.data() + cursor_ + tag.size(), sizeof(n));
        return true;
    }

    std::string bytes_;
    size_t cursor_;
};

#endif
