#include "transport.h"

#include <chrono>
#include <condition_variable>
#include <deque>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <tuple>

#include "ring_abi.h"

namespace mpic {
namespace {

// MPI_REQUIRES_OK, ring.h:36-39: any failing MPI call ends the collective
// with this message.
Status MpiFailure(const char* call, int step, int code) {
  return errors::Unknown("MPI operation failed unexpectedly. [" + std::string(call) + " at ring step " +
                         std::to_string(step) + " returned " + std::to_string(code) + "]");
}
#define MPI_REQUIRES_OK(call, name, step)            \
  do {                                               \
    const int mpi_rc_ = (call);                      \
    if (mpi_rc_ != 0) return MpiFailure((name), (step), mpi_rc_); \
  } while (0)

Status DeviceFailure(int rc, const char* what) {
  std::string msg = std::string(what) + ": " + ring_status_string(rc);
  if (rc == RING_ERR_HIP) msg += " (hipError " + std::to_string(ring_last_hip_error()) + ")";
  return errors::Unknown(msg);
}
#define DEVICE_REQUIRES_OK(call, what)                       \
  do {                                                       \
    const int ring_rc_ = (call);                             \
    if (ring_rc_ != RING_OK) return DeviceFailure(ring_rc_, (what)); \
  } while (0)

struct Piece {
  size_t offset, count;  // elements, relative to the segment
};

// A segment of `elems` elements in `chunks` pieces, sized like the ring's own
// segments: elems / chunks each, the first elems % chunks one more. A function
// of the segment size only, so sender and receiver cut a segment alike.
std::vector<Piece> PiecesOf(size_t elems, int chunks) {
  std::vector<Piece> p(static_cast<size_t>(chunks));
  const size_t q = elems / static_cast<size_t>(chunks), rem = elems % static_cast<size_t>(chunks);
  size_t at = 0;
  for (size_t c = 0; c < p.size(); c++) {
    p[c] = Piece{at, q + (c < rem ? 1 : 0)};
    at += p[c].count;
  }
  return p;
}

// One event per piece, marking the accumulate that produced it.
class PieceEvents {
 public:
  ~PieceEvents() {
    for (void* e : events_) ring_event_destroy(e);
  }
  int Create(int n) {
    for (int i = 0; i < n; i++) {
      void* e = nullptr;
      const int rc = ring_event_create(&e);
      if (rc != RING_OK) return rc;
      events_.push_back(e);
    }
    return RING_OK;
  }
  void* operator[](size_t i) const { return events_[i]; }
  bool empty() const { return events_.empty(); }

 private:
  std::vector<void*> events_;
};

// Receives posted and not yet waited for. A wait consumes its request whether
// it succeeds or not; whatever is still outstanding when the collective ends
// early is cancelled, so the transport stops touching the caller's buffers.
class Requests {
 public:
  Requests(const mpic_transport* t, int n) : t_(t), reqs_(static_cast<size_t>(n), nullptr) {}
  ~Requests() {
    for (void* r : reqs_)
      if (r && t_ && t_->cancel) t_->cancel(t_->user, r);
  }
  Requests(const Requests&) = delete;
  Requests& operator=(const Requests&) = delete;
  void** slot(int c) { return &reqs_[static_cast<size_t>(c)]; }
  bool pending(int c) const { return reqs_[static_cast<size_t>(c)] != nullptr; }
  int Wait(int c) {
    void* r = reqs_[static_cast<size_t>(c)];
    reqs_[static_cast<size_t>(c)] = nullptr;
    return t_->wait(t_->user, r);
  }
  void swap(Requests& other) { reqs_.swap(other.reqs_); }

 private:
  const mpic_transport* t_;
  std::vector<void*> reqs_;
};

inline char* At(void* base, size_t elems, size_t esz) { return static_cast<char*>(base) + elems * esz; }
inline void* OrNull(char* p, size_t count) { return count ? p : nullptr; }

Status CheckTransport(const mpic_transport* t, int n) {
  if (n > 1 && (!t || !t->irecv || !t->send || !t->wait))
    return errors::InvalidArgument("a ring of more than one rank needs a transport with irecv, send and wait");
  return Status::OK();
}

}  // namespace

Status RingAllreduceTransport(int n, int r, DataType dt, const void* input, void* output, void* temp,
                              size_t temp_elements, size_t count, const mpic_transport* t, void* stream,
                              const RingOptions& opts) {
  int code = 0;
  Status s = RingDataType(dt, &code);
  if (!s.ok()) return s;
  if (n < 1 || r < 0 || r >= n) return errors::InvalidArgument("rank out of range for the ring");
  if (opts.chunks < 1 || opts.chunks > 16 || opts.divisor < 0) return errors::InvalidArgument("bad ring options");
  s = CheckTransport(t, n);
  if (!s.ok()) return s;
  if (count && (!input || !output)) return errors::InvalidArgument("null tensor with a non-zero element count");
  const size_t esz = ring_dtype_size(code);
  const int chunks = opts.chunks, divisor = opts.divisor;

  std::vector<size_t> sizes(static_cast<size_t>(n)), starts(static_cast<size_t>(n));
  DEVICE_REQUIRES_OK(ring_segment_table(count, n, sizes.data(), starts.data()), "ring_segment_table");
  const size_t max_seg = sizes[0];
  if (n > 1 && max_seg && (!temp || temp_elements < max_seg))
    return errors::InvalidArgument("the temp buffer is smaller than the largest segment");

  // ring.h:146-148
  if (n == 1) {
    if (divisor > 0 && count) {
      ring_row row{output, input, nullptr, count};
      DEVICE_REQUIRES_OK(ring_apply_rows_avg(&row, 1, nullptr, divisor, code, stream), "ring_apply_rows_avg");
    } else if (input != output && count) {
      DEVICE_REQUIRES_OK(ring_copy_bytes(output, input, count * esz, stream), "ring_copy_bytes");
    }
    DEVICE_REQUIRES_OK(ring_stream_synchronize(stream), "ring_stream_synchronize");
    return Status::OK();
  }
  if (input != output && count)
    DEVICE_REQUIRES_OK(ring_copy_bytes(output, input, count * esz, stream), "ring_copy_bytes");
  // the first send reads the copy (the reference's copy is synchronous, ring.cu.cc:41-47)
  DEVICE_REQUIRES_OK(ring_stream_synchronize(stream), "ring_stream_synchronize");

  // ring.h:169-173
  const int recv_from = (r - 1 + n) % n;
  const int send_to = (r + 1) % n;

  // With pieces, an event per piece orders "accumulated" before "forwarded";
  // with whole segments the stream is synchronised after every accumulate, as
  // the reference's AccumulateTensorData does (ring.cu.cc:69).
  const bool pieces = chunks > 1;
  const bool two_halves = pieces && temp_elements >= 2 * max_seg;
  PieceEvents done;
  if (pieces) DEVICE_REQUIRES_OK(done.Create(chunks), "ring_event_create");
  Requests requests(t, chunks);

  // ring.h:183-205: at step i send segment (r-i), receive segment (r-i-1) into
  // temp and add it into the buffer.
  for (int i = 0; i < n - 1; i++) {
    const size_t send_seg = static_cast<size_t>(((r - i) % n + n) % n);
    const size_t recv_seg = static_cast<size_t>(((r - i - 1) % n + n) % n);
    const std::vector<Piece> send_pieces = PiecesOf(sizes[send_seg], chunks);
    const std::vector<Piece> recv_pieces = PiecesOf(sizes[recv_seg], chunks);
    char* half = At(temp, two_halves ? static_cast<size_t>(i % 2) * max_seg : 0, esz);
    // One temp for all steps: the previous step's accumulates must have read
    // it before a neighbour may write it again. With two halves the half of
    // step i-2 is free: every one of that step's accumulates was waited for
    // before its piece was sent at step i-1.
    if (pieces && !two_halves && i > 0)
      DEVICE_REQUIRES_OK(ring_stream_synchronize(stream), "ring_stream_synchronize");
    for (int c = 0; c < chunks; c++) {
      const Piece& p = recv_pieces[static_cast<size_t>(c)];
      MPI_REQUIRES_OK(t->irecv(t->user, OrNull(At(half, p.offset, esz), p.count), p.count * esz, recv_from,
                               kTagTensor, requests.slot(c)),
                      "MPI_Irecv", i);
    }
    for (int c = 0; c < chunks; c++) {
      const Piece& p = send_pieces[static_cast<size_t>(c)];
      // what is sent at step i > 0 is what was accumulated at step i-1
      if (two_halves && i > 0)
        DEVICE_REQUIRES_OK(ring_event_synchronize(done[static_cast<size_t>(c)]), "ring_event_synchronize");
      MPI_REQUIRES_OK(t->send(t->user, OrNull(At(output, starts[send_seg] + p.offset, esz), p.count),
                              p.count * esz, send_to, kTagTensor),
                      "MPI_Send", i);
    }
    for (int c = 0; c < chunks; c++) {
      const Piece& p = recv_pieces[static_cast<size_t>(c)];
      MPI_REQUIRES_OK(requests.Wait(c), "MPI_Wait", i);
      if (p.count) {
        char* dst = At(output, starts[recv_seg] + p.offset, esz);
        // the last step completes the segment this rank owns: the average's divide rides on it
        ring_row row{dst, At(half, p.offset, esz), dst, p.count};
        DEVICE_REQUIRES_OK(ring_apply_rows_avg(&row, 1, nullptr, i == n - 2 ? divisor : 0, code, stream),
                           "ring_apply_rows_avg");
      }
      if (pieces) DEVICE_REQUIRES_OK(ring_event_record(done[static_cast<size_t>(c)], stream), "ring_event_record");
    }
    if (!pieces) DEVICE_REQUIRES_OK(ring_stream_synchronize(stream), "ring_stream_synchronize");
  }
  // single temp with pieces: the per-step synchronisation above covered every
  // step but the last
  if (pieces && !two_halves) DEVICE_REQUIRES_OK(ring_stream_synchronize(stream), "ring_stream_synchronize");

  // ring.h:211-225: at step i send segment (r-i+1), receive segment (r-i)
  // straight into the buffer (MPI_Sendrecv = receive posted, send, wait). A
  // piece is forwarded once it has arrived; the wait for step i's pieces is
  // therefore made at step i+1, just before each is sent on.
  Requests previous(t, chunks);
  for (int i = 0; i < n - 1; i++) {
    const size_t send_seg = static_cast<size_t>(((r - i + 1) % n + n) % n);
    const size_t recv_seg = static_cast<size_t>(((r - i) % n + n) % n);
    const std::vector<Piece> send_pieces = PiecesOf(sizes[send_seg], chunks);
    const std::vector<Piece> recv_pieces = PiecesOf(sizes[recv_seg], chunks);
    for (int c = 0; c < chunks; c++) {
      const Piece& p = recv_pieces[static_cast<size_t>(c)];
      MPI_REQUIRES_OK(t->irecv(t->user, OrNull(At(output, starts[recv_seg] + p.offset, esz), p.count),
                               p.count * esz, recv_from, kTagTensor, requests.slot(c)),
                      "MPI_Sendrecv", i);
    }
    for (int c = 0; c < chunks; c++) {
      const Piece& p = send_pieces[static_cast<size_t>(c)];
      if (i == 0) {
        // the owned segment: its last accumulate must have finished
        if (two_halves)
          DEVICE_REQUIRES_OK(ring_event_synchronize(done[static_cast<size_t>(c)]), "ring_event_synchronize");
      } else {
        MPI_REQUIRES_OK(previous.Wait(c), "MPI_Sendrecv", i - 1);
      }
      MPI_REQUIRES_OK(t->send(t->user, OrNull(At(output, starts[send_seg] + p.offset, esz), p.count),
                              p.count * esz, send_to, kTagTensor),
                      "MPI_Sendrecv", i);
    }
    previous.swap(requests);
  }
  for (int c = 0; c < chunks; c++) {
    if (previous.pending(c)) MPI_REQUIRES_OK(previous.Wait(c), "MPI_Sendrecv", n - 2);
  }
  return Status::OK();
}

Status RingAllgatherTransport(int n, int r, DataType dt, const void* input, const std::vector<size_t>& rows,
                              size_t elems_per_row, void* output, const mpic_transport* t, void* stream,
                              const RingOptions& opts) {
  int code = 0;
  Status s = RingDataType(dt, &code);
  if (!s.ok()) return s;
  if (n < 1 || r < 0 || r >= n || rows.size() != static_cast<size_t>(n))
    return errors::InvalidArgument("rank or sizes do not match the ring");
  if (opts.chunks < 1 || opts.chunks > 16 || opts.divisor < 0) return errors::InvalidArgument("bad ring options");
  s = CheckTransport(t, n);
  if (!s.ok()) return s;
  const size_t esz = ring_dtype_size(code);
  const int chunks = opts.chunks;
  std::vector<size_t> starts(static_cast<size_t>(n));
  DEVICE_REQUIRES_OK(ring_allgather_table(rows.data(), n, elems_per_row, starts.data()), "ring_allgather_table");
  auto elems = [&](size_t seg) { return elems_per_row * rows[seg]; };

  // ring.h:263-266: own slice to its offset (divided on the way, if asked)
  const size_t own = elems(static_cast<size_t>(r));
  if (own) {
    if (!input || !output) return errors::InvalidArgument("null tensor with a non-zero element count");
    ring_row row{At(output, starts[static_cast<size_t>(r)], esz), input, nullptr, own};
    DEVICE_REQUIRES_OK(ring_apply_rows_avg(&row, 1, nullptr, opts.divisor, code, stream), "ring_apply_rows_avg");
  }
  DEVICE_REQUIRES_OK(ring_stream_synchronize(stream), "ring_stream_synchronize");
  if (n == 1) return Status::OK();
  if (!output) {
    size_t total = 0;
    for (size_t k = 0; k < rows.size(); k++) total += elems(k);
    if (total) return errors::InvalidArgument("null output with a non-zero element count");
  }

  const int recv_from = (r - 1 + n) % n;
  const int send_to = (r + 1) % n;
  // ring.h:279-298: at step i send segment (r-i), receive segment (r-i-1).
  Requests requests(t, chunks), previous(t, chunks);
  for (int i = 0; i < n - 1; i++) {
    const size_t send_seg = static_cast<size_t>(((r - i) % n + n) % n);
    const size_t recv_seg = static_cast<size_t>(((r - i - 1) % n + n) % n);
    const std::vector<Piece> send_pieces = PiecesOf(elems(send_seg), chunks);
    const std::vector<Piece> recv_pieces = PiecesOf(elems(recv_seg), chunks);
    for (int c = 0; c < chunks; c++) {
      const Piece& p = recv_pieces[static_cast<size_t>(c)];
      MPI_REQUIRES_OK(t->irecv(t->user, OrNull(At(output, starts[recv_seg] + p.offset, esz), p.count),
                               p.count * esz, recv_from, kTagTensor, requests.slot(c)),
                      "MPI_Sendrecv", i);
    }
    for (int c = 0; c < chunks; c++) {
      const Piece& p = send_pieces[static_cast<size_t>(c)];
      if (i > 0) {
        MPI_REQUIRES_OK(previous.Wait(c), "MPI_Sendrecv", i - 1);
      }
      MPI_REQUIRES_OK(t->send(t->user, OrNull(At(output, starts[send_seg] + p.offset, esz), p.count),
                              p.count * esz, send_to, kTagTensor),
                      "MPI_Sendrecv", i);
    }
    previous.swap(requests);
  }
  for (int c = 0; c < chunks; c++) {
    if (previous.pending(c)) MPI_REQUIRES_OK(previous.Wait(c), "MPI_Sendrecv", n - 2);
  }
  return Status::OK();
}

}  // namespace mpic

// =============================================================================
// Loopback transport: virtual ranks of one process, one thread each.
// =============================================================================

namespace {

constexpr int kLoopbackTimeout = 1;   // a blocking call gave up waiting for its peer
constexpr int kLoopbackTruncate = 2;  // the message is longer than the posted receive (MPI_ERR_TRUNCATE)
constexpr int kLoopbackDevice = 3;    // the device copy failed
constexpr int kLoopbackArgument = 4;

struct PostedReceive {
  void* buf = nullptr;
  size_t bytes = 0;
  std::tuple<int, int, int> key;  // (source, destination, tag): the queue it waits in
  bool done = false;
  int status = 0;
};

struct LoopbackEndpoint {
  mpic_loopback* world = nullptr;
  int rank = 0;
  void* stream = nullptr;  // this rank's sends copy on it
};

}  // namespace

struct mpic_loopback {
  int n = 0;
  std::chrono::duration<double> timeout{30.0};
  std::mutex mu;
  std::condition_variable cv;
  // receives posted and not yet matched, per (source, destination, tag), in order
  std::map<std::tuple<int, int, int>, std::deque<std::shared_ptr<PostedReceive>>> posted;
  std::vector<std::unique_ptr<LoopbackEndpoint>> endpoints;
};

namespace {

// A wall-clock deadline: waits on it go through pthread_cond_timedwait, which
// ThreadSanitizer models (it does not model the steady-clock wait of wait_for).
std::chrono::system_clock::time_point Deadline(const mpic_loopback* w) {
  return std::chrono::system_clock::now() +
         std::chrono::duration_cast<std::chrono::system_clock::duration>(w->timeout);
}

// Takes a receive nobody will wait for out of its queue. If a sender has already
// claimed it, its copy is under way: wait (bounded) until that has finished, so
// that on return the buffer is no longer written.
void Withdraw(mpic_loopback* w, const std::shared_ptr<PostedReceive>& p, std::unique_lock<std::mutex>* lock) {
  if (p->done) return;
  auto& queue = w->posted[p->key];
  for (auto it = queue.begin(); it != queue.end(); ++it) {
    if (it->get() == p.get()) {
      queue.erase(it);
      return;
    }
  }
  w->cv.wait_until(*lock, Deadline(w), [&] { return p->done; });
}

int LoopbackIrecv(void* user, void* buf, size_t bytes, int source, int tag, void** request) {
  LoopbackEndpoint* ep = static_cast<LoopbackEndpoint*>(user);
  mpic_loopback* w = ep->world;
  if (!request || source < 0 || source >= w->n || (bytes && !buf)) return kLoopbackArgument;
  auto p = std::make_shared<PostedReceive>();
  p->buf = buf;
  p->bytes = bytes;
  p->key = std::make_tuple(source, ep->rank, tag);
  {
    std::lock_guard<std::mutex> guard(w->mu);
    w->posted[p->key].push_back(p);
  }
  w->cv.notify_all();
  *request = new std::shared_ptr<PostedReceive>(p);
  return 0;
}

int LoopbackSend(void* user, const void* buf, size_t bytes, int dest, int tag) {
  LoopbackEndpoint* ep = static_cast<LoopbackEndpoint*>(user);
  mpic_loopback* w = ep->world;
  if (dest < 0 || dest >= w->n || (bytes && !buf)) return kLoopbackArgument;
  std::shared_ptr<PostedReceive> p;
  {
    std::unique_lock<std::mutex> lock(w->mu);
    auto& queue = w->posted[std::make_tuple(ep->rank, dest, tag)];
    if (!w->cv.wait_until(lock, Deadline(w), [&] { return !queue.empty(); })) return kLoopbackTimeout;
    p = queue.front();
    queue.pop_front();
  }
  int status = 0;
  if (bytes > p->bytes) {
    status = kLoopbackTruncate;
  } else if (bytes) {
    // the endpoint's copy stream is made by the first message that carries data
    if (!ep->stream && ring_stream_create(&ep->stream) != RING_OK) ep->stream = nullptr;
    if (!ep->stream || ring_copy_bytes(p->buf, buf, bytes, ep->stream) != RING_OK || ring_stream_synchronize(ep->stream) != RING_OK)
      status = kLoopbackDevice;
  }
  {
    std::lock_guard<std::mutex> guard(w->mu);
    p->status = status;
    p->done = true;
  }
  w->cv.notify_all();
  return status;
}

int LoopbackWait(void* user, void* request) {
  LoopbackEndpoint* ep = static_cast<LoopbackEndpoint*>(user);
  mpic_loopback* w = ep->world;
  if (!request) return kLoopbackArgument;
  std::unique_ptr<std::shared_ptr<PostedReceive>> holder(static_cast<std::shared_ptr<PostedReceive>*>(request));
  std::shared_ptr<PostedReceive> p = *holder;
  std::unique_lock<std::mutex> lock(w->mu);
  if (w->cv.wait_until(lock, Deadline(w), [&] { return p->done; })) return p->status;
  Withdraw(w, p, &lock);
  return kLoopbackTimeout;
}

// MPI_Cancel + MPI_Request_free for a receive that will not be waited for.
int LoopbackCancel(void* user, void* request) {
  LoopbackEndpoint* ep = static_cast<LoopbackEndpoint*>(user);
  mpic_loopback* w = ep->world;
  if (!request) return kLoopbackArgument;
  std::unique_ptr<std::shared_ptr<PostedReceive>> holder(static_cast<std::shared_ptr<PostedReceive>*>(request));
  std::unique_lock<std::mutex> lock(w->mu);
  Withdraw(w, *holder, &lock);
  return 0;
}

}  // namespace

extern "C" {

int mpic_loopback_create(int n, double timeout_seconds, mpic_loopback** loopback) {
  if (n < 1 || !loopback || !(timeout_seconds > 0)) return MPIC_INVALID_ARGUMENT;
  mpic_loopback* w = new mpic_loopback;
  w->n = n;
  w->timeout = std::chrono::duration<double>(timeout_seconds);
  w->endpoints.resize(static_cast<size_t>(n));
  *loopback = w;
  return MPIC_OK;
}

int mpic_loopback_destroy(mpic_loopback* w) {
  if (!w) return MPIC_OK;
  for (auto& ep : w->endpoints)
    if (ep && ep->stream) ring_stream_destroy(ep->stream);
  delete w;
  return MPIC_OK;
}

int mpic_loopback_endpoint(mpic_loopback* w, int rank, mpic_transport* transport) {
  if (!w || !transport || rank < 0 || rank >= w->n) return MPIC_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> guard(w->mu);
  auto& ep = w->endpoints[static_cast<size_t>(rank)];
  if (!ep) {
    ep.reset(new LoopbackEndpoint);
    ep->world = w;
    ep->rank = rank;
  }
  transport->user = ep.get();
  transport->irecv = LoopbackIrecv;
  transport->send = LoopbackSend;
  transport->wait = LoopbackWait;
  transport->cancel = LoopbackCancel;
  return MPIC_OK;
}

}  // extern "C"
