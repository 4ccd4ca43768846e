// The notification mailbox of the HIP backend (nixl_amd/csrc/plugin/mailbox.h) without a GPU:
// several producer threads of this process and one producer in a child process push numbered
// messages into one ring; the consumer must see every message exactly once, each producer's
// messages in the order they were sent, and bytes intact.  Also: a full ring refuses, a message
// longer than a slot is refused, a second creation of the same name fails, a foreign object is
// not taken for a mailbox.  Prints "OK".
#include <sys/wait.h>

#include <cstdio>
#include <cstdlib>
#include <map>
#include <thread>
#include <vector>

#include "mailbox.h"

using namespace nixl_amd_hip;

#define CHECK(x)                                                      \
    do {                                                              \
        if (!(x)) {                                                   \
            std::fprintf(stderr, "%s:%d: %s failed\n", __FILE__, __LINE__, #x); \
            return 1;                                                 \
        }                                                             \
    } while (0)

static std::string
payload(int producer, int i) {
    std::string s = std::to_string(producer) + ":" + std::to_string(i) + ":";
    s.append(static_cast<size_t>((producer * 131 + i * 7) % 600), static_cast<char>('a' + (i % 26)));
    return s;
}

static void
produce(Mailbox *m, int producer, int count) {
    const std::string name = "p" + std::to_string(producer);
    for (int i = 0; i < count; ++i)
        while (!m->push(name, payload(producer, i)))
            std::this_thread::yield(); // full: the consumer is behind
}

int
main() {
    const std::string name = "/nixl_amd_mailbox_check_" + std::to_string(getpid());
    shm_unlink(name.c_str());
    Mailbox *m = mapMailbox(name, true);
    CHECK(m != nullptr);
    CHECK(mapMailbox(name, true) == nullptr); // the name is taken
    std::string sender, msg;
    CHECK(!m->pop(sender, msg)); // empty

    // limits
    CHECK(!m->push("a", std::string(kMailboxSlotBytes, 'x'))); // one byte too long with the sender's name
    CHECK(m->push("a", std::string(kMailboxSlotBytes - 1, 'x')));
    CHECK(m->pop(sender, msg) && sender == "a" && msg.size() == kMailboxSlotBytes - 1);
    for (uint32_t i = 0; i < kMailboxSlots; ++i)
        CHECK(m->push("f", std::to_string(i)));
    CHECK(!m->push("f", "one too many")); // full
    for (uint32_t i = 0; i < kMailboxSlots; ++i)
        CHECK(m->pop(sender, msg) && msg == std::to_string(i));
    CHECK(!m->pop(sender, msg));

    // a sender whose messages find the ring full keeps them, in order, and delivers them late
    {
        nixl_amd_hip::MailboxSender out(m);
        using Result = nixl_amd_hip::MailboxSender::Result;
        const uint32_t total = kMailboxSlots + 300;
        for (uint32_t i = 0; i < total; ++i) {
            const Result r = out.send("s", std::to_string(i));
            CHECK(r == (i < kMailboxSlots ? Result::kSent : Result::kQueued));
        }
        CHECK(out.waiting() == 300 && !out.flush()); // still full: nothing moves
        CHECK(out.send("s", std::string(kMailboxSlotBytes, 'x')) == Result::kTooLong);
        uint32_t next = 0;
        for (int round = 0; next < total; ++round) {
            CHECK(round < 10);
            while (m->pop(sender, msg)) {
                CHECK(sender == "s" && msg == std::to_string(next));
                ++next;
            }
            out.flush(); // room again: the waiting messages follow, oldest first
        }
        CHECK(out.waiting() == 0 && out.send("s", "after") == Result::kSent);
        CHECK(m->pop(sender, msg) && msg == "after" && !m->pop(sender, msg));
    }

    // producers: threads 0..3 here, producer 4 in a child process that maps the ring by name
    constexpr int kThreads = 4, kCount = 20000;
    const pid_t child = fork();
    CHECK(child >= 0);
    if (child == 0) {
        Mailbox *theirs = mapMailbox(name, false);
        if (!theirs) _exit(2);
        produce(theirs, kThreads, kCount);
        _exit(0);
    }
    std::vector<std::thread> threads;
    for (int p = 0; p < kThreads; ++p)
        threads.emplace_back(produce, m, p, kCount);
    std::map<std::string, int> next;
    long received = 0;
    const long expected = static_cast<long>(kThreads + 1) * kCount;
    while (received < expected) {
        if (!m->pop(sender, msg)) {
            std::this_thread::yield();
            continue;
        }
        const int producer = std::atoi(sender.c_str() + 1);
        int &i = next[sender];
        if (msg != payload(producer, i)) {
            std::fprintf(stderr, "producer %s: message %d arrived as '%.40s'\n", sender.c_str(), i, msg.c_str());
            return 1;
        }
        ++i;
        ++received;
    }
    for (auto &t : threads)
        t.join();
    int status = 0;
    CHECK(waitpid(child, &status, 0) == child && WIFEXITED(status) && WEXITSTATUS(status) == 0);
    CHECK(!m->pop(sender, msg));
    CHECK(next.size() == kThreads + 1);

    // something else under a name is not a mailbox
    unmapMailbox(m);
    shm_unlink(name.c_str());
    CHECK(mapMailbox(name, false) == nullptr);
    const int fd = shm_open(name.c_str(), O_RDWR | O_CREAT, 0600);
    CHECK(fd >= 0 && ftruncate(fd, sizeof(Mailbox)) == 0);
    close(fd);
    CHECK(mapMailbox(name, false) == nullptr); // zero-filled: no magic
    shm_unlink(name.c_str());
    std::puts("OK");
    return 0;
}
