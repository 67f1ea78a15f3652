// The ring of ring.h over a transport that supplies the reference's MPI
// point-to-point calls for device buffers, and an in-process transport between
// virtual ranks driven by threads.
#ifndef MPIC_TRANSPORT_H_
#define MPIC_TRANSPORT_H_

#include <cstddef>
#include <vector>

#include "framework.h"
#include "mpi_collectives.h"
#include "ring_driver.h"

namespace mpic {

// ring.h:19
constexpr int kTagTensor = 12;

// ring.h:136-228 for rank r of n. opts.chunks pieces per segment.
Status RingAllreduceTransport(int n, int r, DataType dt, const void* input, void* output, void* temp,
                              size_t temp_elements, size_t count, const mpic_transport* transport, void* stream,
                              const RingOptions& opts);

// ring.h:236-301 for rank r of n.
Status RingAllgatherTransport(int n, int r, DataType dt, const void* input, const std::vector<size_t>& rows,
                              size_t elems_per_row, void* output, const mpic_transport* transport, void* stream,
                              const RingOptions& opts);

}  // namespace mpic
#endif  // MPIC_TRANSPORT_H_
