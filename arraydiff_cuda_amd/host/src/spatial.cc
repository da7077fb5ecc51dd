// Spatial2DComm: recorded-argument protocol and dispatch to the C ABI.
// Behaviour after the reference's src/spatial.cc:10-245 (see include/arraydiff/spatial.hh for
// the differences: error codes instead of a spin-wait and asserts, any K <= 16, one-launch
// group_end_all).  No device call happens before every check has passed.
#include "arraydiff/spatial.hh"

#include "adh_capi.h"

namespace arraydiff {

int Spatial2DComm::InitAll(Spatial2DComm *comms, uint32_t num_w_ranks, uint32_t num_h_ranks) {
  if (!comms) return ADH_ENULL;
  const uint64_t n = (uint64_t)num_w_ranks * num_h_ranks;
  if (n == 0 || n > ARRAYDIFF_MAX_PEERS) return ADH_EINVAL;
  // rank = r_w + num_w * r_h (src/spatial.cc:32-44); no peer-access setup: one device
  for (uint32_t r_h = 0; r_h < num_h_ranks; ++r_h)
    for (uint32_t r_w = 0; r_w < num_w_ranks; ++r_w) {
      Spatial2DComm &c = comms[r_w + num_w_ranks * r_h];
      c.rank = r_w + num_w_ranks * r_h;
      c.rank_w = r_w;
      c.rank_h = r_h;
      c.num_ranks = (uint32_t)n;
      c.num_w_ranks = num_w_ranks;
      c.num_h_ranks = num_h_ranks;
      c.epoch = 0;
      c.arg.buffer = nullptr;
      c.arg.epoch = 0;
      for (uint32_t r2 = 0; r2 < n; ++r2) c.peer_comms[r2] = &comms[r2];
    }
  return ADH_OK;
}

void Spatial2DComm::group_start() {
  ++epoch;
  arg.buffer = nullptr;
}

void Spatial2DComm::record(Spatial2DOperation op, void *buf, uint32_t halo_pad, uint32_t base_width,
                           uint32_t base_height, uint32_t num_channels, uint32_t batch_size,
                           Spatial2DTensorFormat tensor_format, Spatial2DDataType data_type) {
  arg.operation = op;
  arg.tensor_format = tensor_format;
  arg.data_type = data_type;
  arg.halo_pad = halo_pad;
  arg.base_width = base_width;
  arg.base_height = base_height;
  arg.num_channels = num_channels;
  arg.batch_size = batch_size;
  arg.buffer = buf;
  arg.epoch = epoch;
}

void Spatial2DComm::halo_exchange(void *buf, uint32_t halo_pad, uint32_t base_width, uint32_t base_height,
                                  uint32_t num_channels, uint32_t batch_size, Spatial2DTensorFormat tensor_format,
                                  Spatial2DDataType data_type) {
  record(SPATIAL2D_OP_HXEXCH, buf, halo_pad, base_width, base_height, num_channels, batch_size, tensor_format,
         data_type);
}

void Spatial2DComm::halo_reduce(void *buf, uint32_t halo_pad, uint32_t base_width, uint32_t base_height,
                                uint32_t num_channels, uint32_t batch_size, Spatial2DTensorFormat tensor_format,
                                Spatial2DDataType data_type) {
  record(SPATIAL2D_OP_HXREDUCE, buf, halo_pad, base_width, base_height, num_channels, batch_size, tensor_format,
         data_type);
}

// Every peer recorded for my epoch, with a buffer, and a combination that exists.
int Spatial2DComm::check_group(void **bufs, int *dtype) const {
  if (num_ranks == 0) return ADH_EINVAL;  // InitAll was not run
  for (uint32_t r = 0; r < num_ranks; ++r)
    if (peer_comms[r]->arg.epoch != epoch) return ADH_EPROTOCOL;
  for (uint32_t r = 0; r < num_ranks; ++r) {
    if (!peer_comms[r]->arg.buffer) return ADH_ENULL;
    bufs[r] = peer_comms[r]->arg.buffer;
  }
  if (arg.tensor_format != SPATIAL2D_TENSOR_NCHW) return ADH_EUNIMPL;
  if (arg.data_type == SPATIAL2D_DATA_FLOAT) *dtype = ADH_F32;
  else if (arg.data_type == SPATIAL2D_DATA_BFLOAT16) *dtype = ADH_BF16;
  else return ADH_EUNIMPL;
  if (arg.operation != SPATIAL2D_OP_HXEXCH && arg.operation != SPATIAL2D_OP_HXREDUCE) return ADH_EUNIMPL;
  return ADH_OK;
}

int Spatial2DComm::group_end(GPUConn &conn) {
  void *bufs[ARRAYDIFF_MAX_PEERS];
  int dtype = ADH_F32;
  int e = check_group(bufs, &dtype);
  if (e) return e;
  if (arg.operation == SPATIAL2D_OP_HXEXCH)
    return adh_halo_exchange_nchw_rank(dtype, num_w_ranks, num_h_ranks, rank, arg.halo_pad, arg.base_width,
                                       arg.base_height, arg.num_channels, arg.batch_size, bufs, conn.stream());
  return adh_halo_reduce_nchw_rank(dtype, num_w_ranks, num_h_ranks, rank, arg.halo_pad, arg.base_width,
                                   arg.base_height, arg.num_channels, arg.batch_size, bufs, conn.stream());
}

int Spatial2DComm::group_end_all(Spatial2DComm *comms, GPUConn &conn) {
  if (!comms) return ADH_ENULL;
  Spatial2DComm &c0 = comms[0];
  void *bufs[ARRAYDIFF_MAX_PEERS];
  int dtype = ADH_F32;
  int e = c0.check_group(bufs, &dtype);
  if (e) return e;
  for (uint32_t r = 1; r < c0.num_ranks; ++r) {
    const Spatial2DArg &a = comms[r].arg, &b = c0.arg;
    if (comms[r].epoch != c0.epoch) return ADH_EPROTOCOL;
    if (a.operation != b.operation || a.tensor_format != b.tensor_format || a.data_type != b.data_type ||
        a.halo_pad != b.halo_pad || a.base_width != b.base_width || a.base_height != b.base_height ||
        a.num_channels != b.num_channels || a.batch_size != b.batch_size)
      return ADH_EINVAL;
  }
  const Spatial2DArg &a = c0.arg;
  if (a.operation == SPATIAL2D_OP_HXEXCH)
    return adh_halo_exchange_nchw(dtype, c0.num_w_ranks, c0.num_h_ranks, a.halo_pad, a.base_width, a.base_height,
                                  a.num_channels, a.batch_size, bufs, conn.stream());
  return adh_halo_reduce_nchw(dtype, c0.num_w_ranks, c0.num_h_ranks, a.halo_pad, a.base_width, a.base_height,
                              a.num_channels, a.batch_size, bufs, conn.stream());
}

}  // namespace arraydiff
