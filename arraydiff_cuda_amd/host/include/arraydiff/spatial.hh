// Spatial2DComm: the host-side halo "communicator".
//
// Same five-call surface and the same recorded-argument protocol as the reference
// (include/arraydiff/spatial.hh:15-87, src/spatial.cc:10-245): InitAll wires the ranks of a
// num_w x num_h grid (rank = r_w + num_w * r_h); group_start bumps the epoch and clears the
// buffer slot; halo_exchange / halo_reduce only record; group_end checks that every peer has
// recorded for this epoch and a non-NULL buffer, then enqueues THIS rank's share on
// conn.stream().  Differences: a peer that has not recorded makes group_end return
// ADH_EPROTOCOL instead of spinning forever on a volatile (src/spatial.cc:59-70); a NULL peer
// buffer or an unsupported grid / format / type returns an error code instead of assert(0)
// (src/spatial.cc:71-73,132-134,195-200); any K <= 16 is served where the reference had 1x2
// and 1x4 only; the kernels behind it are the C ABI's adh_halo_*_nchw_rank.
#ifndef ARRAYDIFF_SPATIAL_HH
#define ARRAYDIFF_SPATIAL_HH

#include "arraydiff/context.hh"

#include <cstddef>
#include <cstdint>

#define ARRAYDIFF_MAX_PEERS 16

namespace arraydiff {

enum Spatial2DOperation { SPATIAL2D_OP_HXEXCH = 0, SPATIAL2D_OP_HXREDUCE = 1 };
enum Spatial2DTensorFormat { SPATIAL2D_TENSOR_NCHW = 0, SPATIAL2D_TENSOR_NHWC = 1 };
enum Spatial2DDataType {
  SPATIAL2D_DATA_FLOAT = 0,
  SPATIAL2D_DATA_DOUBLE = 1,
  SPATIAL2D_DATA_HALF = 2,
  SPATIAL2D_DATA_BFLOAT16 = 3,  // not in the reference
};

// returned by group_end on top of the C ABI's codes
#define ADH_EPROTOCOL (-16)

struct Spatial2DArg {
  Spatial2DOperation operation;
  Spatial2DTensorFormat tensor_format;
  Spatial2DDataType data_type;
  uint32_t halo_pad, base_width, base_height, num_channels, batch_size;
  void *buffer;
  uint64_t epoch;
};

class Spatial2DComm {
public:
  static int InitAll(Spatial2DComm *comms, uint32_t num_w_ranks, uint32_t num_h_ranks);

  Spatial2DComm() : rank(0), rank_w(0), rank_h(0), num_ranks(0), num_w_ranks(0), num_h_ranks(0), epoch(0) {
    arg.buffer = nullptr;
    arg.epoch = 0;
  }

  void group_start();
  int group_end(GPUConn &conn);
  void halo_exchange(void *buf, uint32_t halo_pad, uint32_t base_width, uint32_t base_height,
                     uint32_t num_channels, uint32_t batch_size, Spatial2DTensorFormat tensor_format,
                     Spatial2DDataType data_type);
  void halo_reduce(void *buf, uint32_t halo_pad, uint32_t base_width, uint32_t base_height,
                   uint32_t num_channels, uint32_t batch_size, Spatial2DTensorFormat tensor_format,
                   Spatial2DDataType data_type);

  // One launch for all ranks of the group, for callers that hold every rank (HaloExch2DOp):
  // requires every rank to have recorded the same call for the same epoch.
  static int group_end_all(Spatial2DComm *comms, GPUConn &conn);

  uint32_t rank, rank_w, rank_h, num_ranks, num_w_ranks, num_h_ranks;
  uint64_t epoch;
  Spatial2DArg arg;
  Spatial2DComm *peer_comms[ARRAYDIFF_MAX_PEERS];

private:
  void record(Spatial2DOperation op, void *buf, uint32_t halo_pad, uint32_t base_width, uint32_t base_height,
              uint32_t num_channels, uint32_t batch_size, Spatial2DTensorFormat tensor_format,
              Spatial2DDataType data_type);
  int check_group(void **bufs, int *dtype) const;
};

}  // namespace arraydiff

#endif
