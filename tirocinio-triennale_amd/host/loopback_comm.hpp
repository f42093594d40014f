// An in-process communicator for allreduce_ring.hpp: the ranks are host threads of one process
// that share one GPU, and a message is a device-to-device copy into the buffer the receiver has
// posted.  It exists so that the ring schedule can be run and checked on a single GPU; a real
// deployment implements homcomp::RingComm over MPI or RCCL instead.
//
// Matching follows MPI's rule for one (source, tag) pair: receives are matched in the order in
// which they were posted.  send() blocks until the receiver has posted the receive (rendezvous),
// which the ring never turns into a deadlock because every rank posts before it sends.
#pragma once

#include <hip/hip_runtime.h>

#include <condition_variable>
#include <cstdint>
#include <memory>
#include <mutex>
#include <vector>

#include "allreduce_ring.hpp"

namespace homcomp {

class LoopbackWorld {
public:
    explicit LoopbackWorld(int size) : ranks_((size_t)size)
    {
        for (int r = 0; r < size; ++r) comms_.emplace_back(new Comm(*this, r));
    }
    int size() const { return (int)ranks_.size(); }
    RingComm &comm(int rank) { return *comms_[(size_t)rank]; }

private:
    enum { kRequests = 3 };   // two MPI_Irecv requests and the receive half of MPI_Sendrecv
    struct Posted {
        void *buf = nullptr;
        size_t capacity = 0, bytes = 0;
        int from = -1;
        uint64_t seq = 0;
        bool posted = false, done = false, truncated = false;
    };
    struct Mailbox {
        std::mutex mu;
        std::condition_variable cv;
        Posted req[kRequests];
        uint64_t next_seq = 1;
    };

    class Comm : public RingComm {
    public:
        Comm(LoopbackWorld &w, int rank) : w_(w), rank_(rank) {}
        int rank() const override { return rank_; }
        int size() const override { return w_.size(); }
        int irecv(void *d_buf, size_t capacity, int from, int request) override
        {
            return w_.post(rank_, d_buf, capacity, from, request);
        }
        int send(const void *d_buf, size_t bytes, int to) override { return w_.deliver(rank_, d_buf, bytes, to); }
        int wait(int request, size_t *bytes) override { return w_.complete(rank_, request, bytes); }
        int sendrecv(const void *d_send, size_t send_bytes, int to, void *d_recv, size_t capacity, int from,
                     size_t *bytes) override
        {
            int rc = w_.post(rank_, d_recv, capacity, from, kRequests - 1);
            if (rc == 0) rc = w_.deliver(rank_, d_send, send_bytes, to);
            if (rc == 0) rc = w_.complete(rank_, kRequests - 1, bytes);
            return rc;
        }

    private:
        LoopbackWorld &w_;
        int rank_;
    };

    int post(int me, void *buf, size_t capacity, int from, int request)
    {
        if (request < 0 || request >= kRequests || from < 0 || from >= size()) return 1;
        Mailbox &m = ranks_[(size_t)me];
        {
            std::lock_guard<std::mutex> lock(m.mu);
            Posted &p = m.req[request];
            if (p.posted) return 1;   // the request is still in use
            p = Posted();
            p.buf = buf;
            p.capacity = capacity;
            p.from = from;
            p.seq = m.next_seq++;
            p.posted = true;
        }
        m.cv.notify_all();
        return 0;
    }

    int deliver(int me, const void *buf, size_t bytes, int to)
    {
        if (to < 0 || to >= size()) return 1;
        Mailbox &m = ranks_[(size_t)to];
        std::unique_lock<std::mutex> lock(m.mu);
        Posted *p = nullptr;
        m.cv.wait(lock, [&] {
            p = nullptr;
            for (Posted &q : m.req)
                if (q.posted && !q.done && q.from == me && (!p || q.seq < p->seq)) p = &q;
            return p != nullptr;
        });
        p->truncated = bytes > p->capacity;
        p->bytes = p->truncated ? p->capacity : bytes;
        const bool ok = hipMemcpy(p->buf, buf, p->bytes, hipMemcpyDeviceToDevice) == hipSuccess;
        p->done = true;
        const bool truncated = p->truncated;
        lock.unlock();
        m.cv.notify_all();
        return ok && !truncated ? 0 : 1;
    }

    int complete(int me, int request, size_t *bytes)
    {
        if (request < 0 || request >= kRequests) return 1;
        Mailbox &m = ranks_[(size_t)me];
        std::unique_lock<std::mutex> lock(m.mu);
        Posted &p = m.req[request];
        if (!p.posted) return 1;
        m.cv.wait(lock, [&] { return p.done; });
        *bytes = p.bytes;
        const bool truncated = p.truncated;
        p = Posted();
        return truncated ? 1 : 0;
    }

    std::vector<Mailbox> ranks_;
    std::vector<std::unique_ptr<Comm>> comms_;
};

}  // namespace homcomp
