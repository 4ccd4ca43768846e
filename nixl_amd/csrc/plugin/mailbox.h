// Notification mailbox of the HIP backend: a bounded multi-producer, single-consumer ring in
// POSIX shared memory.  Producers are engines of other processes (and their threads), the
// consumer is the engine that created the mailbox.  Header-only, no GPU code: the ring is
// tested on the CPU from several threads and processes.
#ifndef NIXL_AMD_HIP_MAILBOX_H
#define NIXL_AMD_HIP_MAILBOX_H

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <cstdint>
#include <cstring>
#include <deque>
#include <string>
#include <utility>

namespace nixl_amd_hip {

constexpr uint32_t kMailboxSlots = 256;
constexpr uint32_t kMailboxSlotBytes = 4096 - 16;
constexpr uint32_t kMailboxMagic = 0x584f424du; // "MBOX"

// Cell sequence numbers as in Vyukov's bounded queue.  A message is the sender's agent name
// followed by the payload.  A producer that dies between claiming a cell and publishing it
// leaves that cell unpublished: the consumer stops there (messages behind it are not lost,
// but not delivered either) until the mailbox is recreated.
struct Mailbox {
    struct Cell {
        std::atomic<uint64_t> sequence;
        uint32_t senderLen;
        uint32_t msgLen;
        char data[kMailboxSlotBytes];
    };
    std::atomic<uint32_t> magic;
    std::atomic<uint64_t> head; // next position to write
    std::atomic<uint64_t> tail; // next position to read
    Cell cells[kMailboxSlots];

    // false: the message does not fit a slot, or the ring is full (the owner has not drained it)
    bool
    push(const std::string &sender, const std::string &msg) {
        if (sender.size() + msg.size() > kMailboxSlotBytes) return false;
        uint64_t pos = head.load(std::memory_order_relaxed);
        for (;;) {
            Cell &c = cells[pos % kMailboxSlots];
            const uint64_t seq = c.sequence.load(std::memory_order_acquire);
            const int64_t dif = static_cast<int64_t>(seq) - static_cast<int64_t>(pos);
            if (dif == 0) {
                if (head.compare_exchange_weak(pos, pos + 1, std::memory_order_relaxed)) {
                    c.senderLen = static_cast<uint32_t>(sender.size());
                    c.msgLen = static_cast<uint32_t>(msg.size());
                    std::memcpy(c.data, sender.data(), sender.size());
                    std::memcpy(c.data + sender.size(), msg.data(), msg.size());
                    c.sequence.store(pos + 1, std::memory_order_release);
                    return true;
                }
            } else if (dif < 0) {
                return false;
            } else {
                pos = head.load(std::memory_order_relaxed);
            }
        }
    }

    // One consumer at a time (the owner serialises its callers).  false: nothing to read.
    bool
    pop(std::string &sender, std::string &msg) {
        const uint64_t pos = tail.load(std::memory_order_relaxed);
        Cell &c = cells[pos % kMailboxSlots];
        if (c.sequence.load(std::memory_order_acquire) != pos + 1) return false;
        // lengths come from another process: never read past the slot
        const uint32_t sl = std::min(c.senderLen, kMailboxSlotBytes), ml = std::min(c.msgLen, kMailboxSlotBytes - sl);
        sender.assign(c.data, sl);
        msg.assign(c.data + sl, ml);
        tail.store(pos + 1, std::memory_order_relaxed);
        c.sequence.store(pos + kMailboxSlots, std::memory_order_release);
        return true;
    }
};

// The sending side of one peer's mailbox: messages that find the ring full wait here, in
// order, and go out when the peer has drained some (flush, which every later send also does
// first).  The reference queues notifications without loss; a full ring must not lose one
// either.  Not thread-safe: the owner serialises its callers.
class MailboxSender {
public:
    static constexpr size_t kMaxBacklog = 65536; // messages; beyond that the peer is taken to be gone

    enum class Result { kSent, kQueued, kTooLong, kBacklogFull };

    explicit MailboxSender(Mailbox *box = nullptr) : box_(box) {}

    Mailbox *
    box() const {
        return box_;
    }

    Result
    send(const std::string &sender, const std::string &msg) {
        if (sender.size() + msg.size() > kMailboxSlotBytes) return Result::kTooLong;
        flush();
        if (backlog_.empty() && box_->push(sender, msg)) return Result::kSent;
        if (backlog_.size() >= kMaxBacklog) return Result::kBacklogFull;
        backlog_.emplace_back(sender, msg);
        return Result::kQueued;
    }

    // Moves waiting messages into the ring while it takes them; true when none is left.
    bool
    flush() {
        while (!backlog_.empty() && box_->push(backlog_.front().first, backlog_.front().second))
            backlog_.pop_front();
        return backlog_.empty();
    }

    size_t
    waiting() const {
        return backlog_.size();
    }

private:
    Mailbox *box_;
    std::deque<std::pair<std::string, std::string>> backlog_;
};

// Creates (O_EXCL) or opens the shared-memory object `name` and maps it; nullptr on failure.
inline Mailbox *
mapMailbox(const std::string &name, bool create) {
    static_assert(std::atomic<uint64_t>::is_always_lock_free, "the mailbox needs lock-free 64-bit atomics");
    const int fd = shm_open(name.c_str(), create ? (O_RDWR | O_CREAT | O_EXCL) : O_RDWR, 0600);
    if (fd < 0) return nullptr;
    if (create && ftruncate(fd, sizeof(Mailbox)) != 0) {
        close(fd);
        shm_unlink(name.c_str());
        return nullptr;
    }
    struct stat st {};
    if (fstat(fd, &st) != 0 || static_cast<size_t>(st.st_size) < sizeof(Mailbox)) {
        close(fd);
        return nullptr;
    }
    void *mem = mmap(nullptr, sizeof(Mailbox), PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
    close(fd);
    if (mem == MAP_FAILED) return nullptr;
    auto *m = static_cast<Mailbox *>(mem);
    if (create) {
        for (uint32_t i = 0; i < kMailboxSlots; ++i)
            m->cells[i].sequence.store(i, std::memory_order_relaxed);
        m->head.store(0, std::memory_order_relaxed);
        m->tail.store(0, std::memory_order_relaxed);
        m->magic.store(kMailboxMagic, std::memory_order_release);
    } else if (m->magic.load(std::memory_order_acquire) != kMailboxMagic) {
        munmap(mem, sizeof(Mailbox));
        return nullptr;
    }
    return m;
}

inline void
unmapMailbox(Mailbox *m) {
    if (m) munmap(m, sizeof(Mailbox));
}

} // namespace nixl_amd_hip

#endif
