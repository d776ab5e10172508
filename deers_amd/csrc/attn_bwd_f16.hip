// Fused causal attention backward, f16 storage / f32 accumulate, gfx950.
//
// Replaces the reference's op-by-op autograd sweep over the attention core
// (src/backprop.rs:52-66 through src/ops.rs:1089-1101, 422-425, 210-214,
// 777-799, 1162-1175, 638-643) by recomputation from (Q, K, V, O, LSE, dO):
//     P  = exp(S*scale + mask - LSE)        dV = P^T dO
//     dP = dO V^T                           dS = P o (dP - delta),  delta = rowsum(dO o O)
//     dQ = scale dS K                       dK = scale dS^T Q
//
// One launch with two roles, no atomics on data, bit-reproducible.  The role bodies are in
// attn_bwd_f16_bp.h (block-pipelined loops over 32-row blocks of the streamed operand):
//   dQ      : a workgroup owns 128 query rows (32 per wave, Q and dO in registers) and walks
//             the key blocks up to the diagonal.  Orientation S^T[kv,q] (one query column per
//             lane, LSE and delta are per-lane scalars); dS^T leaves the accumulators as the B
//             operand of dQ^T += K^T dS^T with K^T fragments read transposed from LDS.  It also
//             publishes, for the rows it owns, negdelta[b,h,t] = -sum_d dO*O and
//             lse2 = -LSE*log2(e) as f32 in a workspace whose rows are padded to a multiple of
//             64 per head (lse2 = -inf and negdelta = 0 in the padding, so padded query rows get
//             probability exactly 0) and its queries scaled by scale*log2(e) as f16 (the
//             values it and the forward form their scores from), then sets the block's flag.
//   dK/dV   : a workgroup owns 128 key rows (32 per wave, K^T and V^T held in registers as B
//             operands) and walks the query blocks at or below the diagonal.  Orientation
//             S[q,kv] (one key column per lane) so P and dS leave the accumulators directly as
//             B operands of dV^T += dO^T P and dK^T += Q^T dS; dO^T / Q^T fragments come from
//             the row-major LDS blocks via ds_read_b64_tr_b16.  The queries it streams are the
//             dQ role's scaled ones; it waits for a query block's rows through the block's flag.
// Recomputing S and dP in both roles costs 7 tile GEMMs instead of 5 but keeps every product
// in registers and needs no dQ accumulation buffer.  Head widths 32 and 64 run two workgroups
// per CU; head width 128 needs more than 256 registers (213 + 160 accumulation registers) and runs one.
#include <type_traits>


#include "attn_bwd_f16_bp.h"
#include "common.h"

namespace deers {

constexpr int kBwdBlk = 128;  // rows owned by a workgroup (keys in dK/dV, queries in dQ)

// One launch for the whole backward: the first half of the grid runs the dQ role, the
// second half the dK/dV role.  Each half is cut into groups of 8 * heads_per_xcd workgroups,
// one block length over all heads per group, and block ids inside a group map to heads the
// same way in both halves (a half is a multiple of 8 long), so the dK/dV workgroups of a
// head share an XCD, and its L2, with the dQ workgroups that publish the head's row
// statistics; they are dispatched after them and poll a per-block flag before they first
// touch a query block's statistics.  Against two launches this saves a dispatch and lets
// the heavy dK/dV blocks start while dQ blocks are still running.
//
// The dK/dV groups run longest first, so the launch ends on its shortest blocks.  The dQ
// groups run longest first too unless `dq_short_first`: then the shortest come first, publish
// their rows' statistics within microseconds and leave, and dK/dV work starts early instead
// of after the longest dQ blocks, which otherwise fill the device alone, have drained.  The
// host asks for that when a group is a sizeable part of what the device holds at once (see
// launch_bwd_f16_d).  Either way every dQ workgroup precedes every dK/dV workgroup in
// dispatch order, and dQ workgroups wait for nothing.
//
// `first_id` is added to blockIdx.x: 0 with a grid of both halves is the single launch;
// a grid of one half with first_id = 0, then one with first_id = the half's length, runs
// the two roles as two launches in stream order (the flags are then already set when the
// second launch starts).  The hand-over inside one launch stores the statistics, drains
// the stores (vmcnt 0) and sets the flag with relaxed atomics and no cache write-back,
// which is only enough when producer and consumer share one L2, i.e. one XCD: the host
// takes the single launch only on a device where workgroup id % 8 is known to be the XCD.
//
// The flags hold epochs (one per backward call, passed by the host) and are never cleared.
// Epoch 0 means that the flags are not used: the dK/dV role does not wait.  The host passes it
// with the two-launch form while the stream is being captured into a graph, whose replays
// could not be given a fresh epoch each.
template <int D>
__global__ __launch_bounds__(256, D == 128 ? 1 : 2) void attn_bwd_f16_bp_kernel(BwdParams p, int BH, int n_blocks,
                                                                                 int heads_per_xcd, int first_id,
                                                                                 int dq_short_first) {
  const int group_wgs = 8 * heads_per_xcd;
  const int per_role = n_blocks * group_wgs;
  const int id = (int)blockIdx.x + first_id;
  int bh, rank;
  if (id < per_role) {
    const int group = id / group_wgs;
    const int r = dq_short_first ? n_blocks - 1 - group : group;
    if (map_block(r * group_wgs + id % group_wgs, n_blocks, heads_per_xcd, BH, &bh, &rank))
      bwd_dq_f16_bp_body<D>(p, __builtin_amdgcn_readfirstlane(bh), n_blocks - 1 - __builtin_amdgcn_readfirstlane(rank),
                            n_blocks, blockIdx.x);
  } else {
    if (map_block(id - per_role, n_blocks, heads_per_xcd, BH, &bh, &rank))
      bwd_dkdv_f16_bp_body<D>(p, __builtin_amdgcn_readfirstlane(bh), __builtin_amdgcn_readfirstlane(rank), n_blocks,
                              blockIdx.x);
  }
}

template <int D>
static void launch_bwd_f16_d(const BwdParams& p, int B, int mode, hipStream_t stream) {
  const int BH = B * p.H;
  const int n_blocks = (p.T + kBwdBlk - 1) / kBwdBlk;
  const int heads_per_xcd = (BH + 7) / 8;
  const int per_role = 8 * n_blocks * heads_per_xcd;
  typedef void (*Kernel)(BwdParams, int, int, int, int, int);
  const Kernel kernel = attn_bwd_f16_bp_kernel<D>;
  const size_t lds = BwdBpCfg<D>::kLds;
  static bool attr_set = false;  // launches are serialised by the caller
  if (!attr_set) {
    if (lds > 64 * 1024)
      (void)hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    attr_set = true;
  }
  if (mode == 2) {  // test hook: consumers only, so that their bounded wait runs out
    LaunchScope scope("attn_bwd_f16_dkdv", stream);
    hipLaunchKernelGGL(kernel, dim3(per_role), dim3(256), lds, stream, p, BH, n_blocks, heads_per_xcd, per_role, 0);
    return;
  }
  if (mode == 1) {
    // Device capacity in workgroups of this kernel, found once (launches are serialised by
    // the caller).  The shortest-first dQ order pays when the longest dQ groups would
    // otherwise hold the device to themselves.
    static int capacity = 0;
    if (capacity == 0) {
      int dev = 0, per_cu = 0;
      hipDeviceProp_t prop;
      if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess &&
          hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, lds) == hipSuccess && per_cu > 0)
        capacity = per_cu * prop.multiProcessorCount;
      else
        capacity = -1;
    }
    const int dq_short_first = capacity > 0 && bwd_dq_short_first(8 * heads_per_xcd, capacity);
    LaunchScope scope("attn_bwd_f16", stream);
    hipLaunchKernelGGL(kernel, dim3(2 * per_role), dim3(256), lds, stream, p, BH, n_blocks, heads_per_xcd, 0,
                       dq_short_first);
    return;
  }
  {
    LaunchScope scope("attn_bwd_f16_dq", stream);
    hipLaunchKernelGGL(kernel, dim3(per_role), dim3(256), lds, stream, p, BH, n_blocks, heads_per_xcd, 0, 0);
  }
  {
    LaunchScope scope("attn_bwd_f16_dkdv", stream);
    hipLaunchKernelGGL(kernel, dim3(per_role), dim3(256), lds, stream, p, BH, n_blocks, heads_per_xcd, per_role, 0);
  }
}

// mode 1: both roles in one grid with the flag hand-over (needs workgroup id % 8 == XCD);
// mode 0: two launches in stream order; mode 2: only the dK/dV half of the single launch
// (host-side test of the bounded wait: nobody publishes, every wait runs out).
void launch_attn_bwd_f16(const BwdParams& p, int B, int D, int mode, hipStream_t stream) {
  switch (D) {
    case 32: launch_bwd_f16_d<32>(p, B, mode, stream); break;
    case 64: launch_bwd_f16_d<64>(p, B, mode, stream); break;
    case 128: launch_bwd_f16_d<128>(p, B, mode, stream); break;
  }
}

}  // namespace deers
