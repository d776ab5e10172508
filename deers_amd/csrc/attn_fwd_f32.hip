// Fused causal attention forward, f32 storage and arithmetic, gfx950.
//
// Same decomposition as the f16 kernel (one query column per lane, S^T = K Q^T,
// O^T += V^T P^T, online softmax in the log2 domain) on v_mfma_f32_32x32x2_f32.
// With one contraction element per lane per MFMA there is no transposed-operand
// problem: V^T fragments are plain 4-byte LDS reads of the row-major V tile, and
// P^T accumulator registers are used as B operands without conversion.
// Contraction over D assigns lane group g the contiguous half [g*D/2, (g+1)*D/2)
// so K fragments are 16-byte LDS reads.
#include <algorithm>
#include <map>
#include <tuple>
#include <vector>

#include "common.h"

namespace deers {

constexpr int kFwd32BM = 128;

// Work lists of the f32 forward.  These kernels are bound by the matrix pipe: with two
// workgroups on a CU the pipe is busy throughout, with one it idles during that workgroup's
// softmax, and a tile lives for up to 16 iterations of 4-8 us, so how the tiles of a
// causal launch are spread over the CUs decides the launch time.  Handed out longest first
// by the dispatcher, the last CU finished 28 % after the first at 8x12x1024x64.  Instead the
// grid has exactly as many workgroups as the device holds and each walks a list built on the
// host: tiles are dealt longest first to the CU with the smallest total, then a CU's tiles to
// its slots the same way.  Workgroup w of an XCD (blockIdx.x / 8) is assumed to land on CU
// w % cus_per_xcd, as the dispatcher does on an empty device; only the balance depends on it.
// lists[w * max_len + k] = (head index within the XCD) << 16 | query tile, -1 ends a list.
struct Fwd32Lists {
  const int* codes = nullptr;  // device memory, owned by the launch code below
  int max_len = 0;
  int wgs_per_xcd = 0;
};

template <int D, int BN>
__global__ __launch_bounds__(256, (D == 32 ? 3 : 2)) void attn_fwd_f32_kernel(FwdParams p, int BH, int n_qtiles,
                                                           int heads_per_xcd, const int* lists,
                                                           int max_len) {
  constexpr int LD = D + 4;   // LDS row stride in floats
  constexpr int KH = D / 2;   // contraction steps (2 elements of D per MFMA)
  constexpr int DB = D / 32;
  constexpr int MB = BN / 32;
  constexpr int CH = D / 4;   // 16-byte chunks per row
  constexpr int NLOAD = BN * CH / 256;

  __shared__ __attribute__((aligned(16))) float Ks[BN * LD];
  __shared__ __attribute__((aligned(16))) float Vs[BN * LD];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5;
  const int T = p.T;

  // (head, query tile) of list position `item`, or bh = -1 past the end of the list.  Without
  // lists a workgroup has the one tile its id names (every tile of a head on one XCD, each
  // XCD's tiles longest first).  List entries of heads past the last one are skipped.
  auto tile_at = [&](int& item, int* bh, int* qtile) {
    *bh = -1;
    if (!lists) {
      int rank;
      if (item == 0 && map_block(blockIdx.x, n_qtiles, heads_per_xcd, BH, bh, &rank))
        *qtile = n_qtiles - 1 - rank;
      else
        *bh = -1;
      return;
    }
    for (; item < max_len; ++item) {
      // the same in every lane: a scalar, so that the trip counts and causal tests that
      // derive from it are scalar too
      const int code = __builtin_amdgcn_readfirstlane(lists[(blockIdx.x >> 3) * max_len + item]);
      if (code < 0) return;
      const int head = (code >> 16) * 8 + (blockIdx.x & 7);
      if (head < BH) {
        *bh = head;
        *qtile = code & 0xffff;
        return;
      }
    }
  };

  floatx4 kreg[NLOAD], vreg[NLOAD];
  auto prefetch = [&](const float* K, const float* V, int tile) {  // K/V rows of one key tile
    const int kv0 = tile * BN;
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
      const int idx = tid + 256 * i;
      const int row = idx / CH, ch = idx % CH;
      const int kv = kv0 + row;
      if (kv < T) {
        kreg[i] = *(const floatx4*)(K + (int64_t)kv * p.sk.t + 4 * ch);
        vreg[i] = *(const floatx4*)(V + (int64_t)kv * p.sv.t + 4 * ch);
      } else {
        kreg[i] = floatx4{0, 0, 0, 0};
        vreg[i] = floatx4{0, 0, 0, 0};
      }
    }
  };
  auto commit = [&]() {
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
      const int idx = tid + 256 * i;
      const int row = idx / CH, ch = idx % CH;
      *(floatx4*)(Ks + row * LD + 4 * ch) = kreg[i];
      *(floatx4*)(Vs + row * LD + 4 * ch) = vreg[i];
    }
  };
  float qf[KH];
  // this lane's half of its query row, times scale * log2(e): the scores then come out of the
  // MFMAs in the exponent's base-2 domain (head width 128 scales the scores instead: with
  // 64 query registers scaled in place its 256 registers no longer suffice)
  constexpr bool kScaledQ = D != 128;
  auto load_q = [&](const float* Q, int qrow) {
#pragma unroll
    for (int c = 0; c < KH / 4; ++c) {
      floatx4 t = floatx4{0, 0, 0, 0};
      if (qrow < T) t = *(const floatx4*)(Q + (int64_t)qrow * p.sq.t + g * KH + 4 * c);
#pragma unroll
      for (int e = 0; e < 4; ++e) qf[4 * c + e] = kScaledQ ? t[e] * p.scale_log2 : t[e];
    }
  };

  int item = 0, bh, qtile;
  tile_at(item, &bh, &qtile);
  if (bh < 0) return;
  {
    const int b = bh / p.H, h = bh % p.H;
    load_q((const float*)p.q + b * p.sq.b + h * p.sq.h, qtile * kFwd32BM + 32 * wave + (lane & 31));
    prefetch((const float*)p.k + b * p.sk.b + h * p.sk.h, (const float*)p.v + b * p.sv.b + h * p.sv.h, 0);
  }

  // One pass of this loop per tile.  The first loads of a tile (its query rows, its first
  // K/V tile) are issued during the last iteration of the tile before it, so a workgroup
  // goes from one tile of its list to the next without waiting for memory.
  for (;;) {
    const int b = bh / p.H, h = bh % p.H;
    const float* K = (const float*)p.k + b * p.sk.b + h * p.sk.h;
    const float* V = (const float*)p.v + b * p.sv.b + h * p.sv.h;
    float* O = (float*)p.o + b * p.so.b + h * p.so.h;
    const int q0 = qtile * kFwd32BM;
    const int qw0 = q0 + 32 * wave;
    const int qrow = qw0 + (lane & 31);
    int last_q = q0 + kFwd32BM - 1;
    if (last_q > T - 1) last_q = T - 1;
    const int n_tiles = last_q / BN + 1;

    int next_item = item + 1, next_bh, next_qtile = 0;
    tile_at(next_item, &next_bh, &next_qtile);
    const int nb = next_bh < 0 ? 0 : next_bh / p.H, nh = next_bh < 0 ? 0 : next_bh % p.H;

    floatx16 oacc[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i) oacc[i] = floatx16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    float m = -INFINITY, lsum = 0.f;

    for (int j = 0; j < n_tiles; ++j) {
      __syncthreads();
      commit();
      __syncthreads();
      const bool last = j + 1 == n_tiles;
      if (!last)
        prefetch(K, V, j + 1);
      else if (next_bh >= 0)
        prefetch((const float*)p.k + nb * p.sk.b + nh * p.sk.h,
                 (const float*)p.v + nb * p.sv.b + nh * p.sv.h, 0);

      const int kv0 = j * BN;
      const bool active = kv0 <= qw0 + 31;  // else the tile lies entirely in this wave's future

      floatx16 s[MB];
      if (active) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          s[mb] = floatx16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
          const float* krow = Ks + (32 * mb + (lane & 31)) * LD + g * KH;
#pragma unroll
          for (int c = 0; c < KH / 4; ++c) {
            const floatx4 a = *(const floatx4*)(krow + 4 * c);
#pragma unroll
            for (int e = 0; e < 4; ++e) s[mb] = mfma_f32(a[e], qf[4 * c + e], s[mb]);
          }
        }
      }
      // the query fragments are dead after the tile's last S: fetch the next tile's
      if (last && next_bh >= 0)
        load_q((const float*)p.q + nb * p.sq.b + nh * p.sq.h,
               next_qtile * kFwd32BM + 32 * wave + (lane & 31));
      if (!active) continue;

      // At head width 64 only the tiles on the diagonal pay for the mask: a branch of its own
      // (the empty asm keeps the compiler from turning it into sixty-four selects on every
      // tile).  The other widths have no registers to spare for it and keep the selects.
      constexpr bool kMaskBranch = D == 64;
      const bool need_mask = kv0 + BN - 1 > qw0;
      if (kMaskBranch && need_mask) {
        asm volatile("" ::: "memory");
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int kv = kv0 + 32 * mb + 8 * (r >> 2) + 4 * g + (r & 3);
            if (kv > qrow) s[mb][r] = -INFINITY;
          }
      }
      float mloc = -INFINITY;
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          if (!kMaskBranch && need_mask) {
            const int kv = kv0 + 32 * mb + 8 * (r >> 2) + 4 * g + (r & 3);
            if (kv > qrow) s[mb][r] = -INFINITY;
          }
          if (!kScaledQ) s[mb][r] *= p.scale_log2;
          mloc = fmaxf(mloc, s[mb][r]);
        }
      mloc = fmaxf(mloc, swap32(mloc));
      const float m_new = fmaxf(m, mloc);
      const float alpha = fast_exp2(m - m_new);
      float rsum = 0.f;
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float e = fast_exp2(s[mb][r] - m_new);
          s[mb][r] = e;
          rsum += e;
        }
      rsum += swap32(rsum);
      lsum = lsum * alpha + rsum;
      m = m_new;
#pragma unroll
      for (int db = 0; db < DB; ++db) oacc[db] *= alpha;

#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = 32 * mb + 8 * (r >> 2) + 4 * g + (r & 3);
#pragma unroll
          for (int db = 0; db < DB; ++db) {
            const float a = Vs[row * LD + 32 * db + (lane & 31)];
            oacc[db] = mfma_f32(a, s[mb][r], oacc[db]);
          }
        }
    }

    if (qrow < T) {
      const float inv = 1.f / lsum;
      float* orow = O + (int64_t)qrow * p.so.t;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          floatx4 out;
#pragma unroll
          for (int e = 0; e < 4; ++e) out[e] = oacc[db][4 * rq + e] * inv;
          *(floatx4*)(orow + 32 * db + 8 * rq + 4 * g) = out;
        }
      if (g == 0) p.lse[(int64_t)bh * T + qrow] = (m + fast_log2(lsum)) * kLn2;
    }
    if (next_bh < 0) break;
    item = next_item;
    bh = next_bh;
    qtile = next_qtile;
  }
}

// Builds (once per geometry, kept for the life of the process) the work lists of a launch
// and uploads them.  Returns lists with codes == nullptr when the kernel's resources cannot
// be queried; the caller then launches one workgroup per tile.
template <int D, int BN>
static Fwd32Lists fwd32_lists(int n_qtiles, int heads_per_xcd, int T, hipStream_t stream) {
  static int slots = 0, cus_per_xcd = 0;  // launches are serialised by the caller
  if (slots == 0) {
    int dev = 0, per_cu = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess &&
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, attn_fwd_f32_kernel<D, BN>, 256, 0) ==
            hipSuccess &&
        per_cu > 0 && prop.multiProcessorCount % 8 == 0) {
      slots = per_cu;
      cus_per_xcd = prop.multiProcessorCount / 8;
    } else {
      slots = -1;
      (void)hipGetLastError();  // the plain grid stands in: leave no error behind for the caller's check
    }
  }
  if (slots < 0) return Fwd32Lists{};
  struct Entry {
    int* dev = nullptr;
    int max_len = 0;
  };
  static std::map<std::tuple<int, int, int>, Entry> cache;
  const auto key = std::make_tuple(n_qtiles, heads_per_xcd, T);
  auto it = cache.find(key);
  if (it == cache.end()) {
    struct Tile {
      int code;
      float weight;
    };
    std::vector<Tile> tiles;
    for (int hx = 0; hx < heads_per_xcd; ++hx)
      for (int qt = 0; qt < n_qtiles; ++qt) {
        const int last_q = std::min(qt * kFwd32BM + kFwd32BM - 1, T - 1);
        // iterations of the tile plus its write-out and the two part-empty diagonal ones
        tiles.push_back({(hx << 16) | qt, (float)(last_q / BN + 1) + 0.4f});
      }
    std::stable_sort(tiles.begin(), tiles.end(),
                     [](const Tile& a, const Tile& b) { return a.weight > b.weight; });
    std::vector<std::vector<Tile>> per_cu(cus_per_xcd);
    std::vector<float> cu_load(cus_per_xcd, 0.f);
    for (const Tile& t : tiles) {
      const int c = (int)(std::min_element(cu_load.begin(), cu_load.end()) - cu_load.begin());
      per_cu[c].push_back(t);
      cu_load[c] += t.weight;
    }
    const int wgs = slots * cus_per_xcd;
    std::vector<std::vector<int>> lists(wgs);
    for (int c = 0; c < cus_per_xcd; ++c) {
      std::vector<float> slot_load(slots, 0.f);
      for (const Tile& t : per_cu[c]) {  // already longest first
        const int sl = (int)(std::min_element(slot_load.begin(), slot_load.end()) - slot_load.begin());
        lists[sl * cus_per_xcd + c].push_back(t.code);
        slot_load[sl] += t.weight;
      }
    }
    Entry e;
    for (const auto& l : lists) e.max_len = std::max(e.max_len, (int)l.size());
    if (e.max_len == 0) e.max_len = 1;
    std::vector<int> flat((size_t)wgs * e.max_len, -1);
    for (int w = 0; w < wgs; ++w)
      for (size_t k = 0; k < lists[w].size(); ++k) flat[(size_t)w * e.max_len + k] = lists[w][k];
    if (hipMalloc(&e.dev, flat.size() * sizeof(int)) != hipSuccess) {
      (void)hipGetLastError();  // the plain grid stands in
      return Fwd32Lists{};
    }
    // the table is read by launches on `stream` only; a synchronous copy keeps `flat` alive
    if (hipMemcpy(e.dev, flat.data(), flat.size() * sizeof(int), hipMemcpyHostToDevice) != hipSuccess) {
      (void)hipFree(e.dev);
      (void)hipGetLastError();
      return Fwd32Lists{};
    }
    (void)stream;
    it = cache.emplace(key, e).first;
  }
  Fwd32Lists out;
  out.codes = it->second.dev;
  out.max_len = it->second.max_len;
  out.wgs_per_xcd = slots * cus_per_xcd;
  return out;
}

template <int D, int BN>
static void launch_fwd32_d(const FwdParams& p, int BH, int n_qtiles, int heads_per_xcd,
                           hipStream_t stream) {
  const Fwd32Lists lists = fwd32_lists<D, BN>(n_qtiles, heads_per_xcd, p.T, stream);
  LaunchScope scope("attn_fwd_f32", stream);
  if (lists.codes) {
    hipLaunchKernelGGL((attn_fwd_f32_kernel<D, BN>), dim3(8 * lists.wgs_per_xcd), dim3(256), 0, stream,
                       p, BH, n_qtiles, heads_per_xcd, lists.codes, lists.max_len);
  } else {
    hipLaunchKernelGGL((attn_fwd_f32_kernel<D, BN>), dim3(8 * n_qtiles * heads_per_xcd), dim3(256), 0,
                       stream, p, BH, n_qtiles, heads_per_xcd, (const int*)nullptr, 0);
  }
}

void launch_attn_fwd_f32(const FwdParams& p, int B, int D, hipStream_t stream) {
  const int BH = B * p.H;
  const int n_qtiles = (p.T + kFwd32BM - 1) / kFwd32BM;
  const int heads_per_xcd = (BH + 7) / 8;
  switch (D) {
    case 32: launch_fwd32_d<32, 64>(p, BH, n_qtiles, heads_per_xcd, stream); break;
    case 64: launch_fwd32_d<64, 64>(p, BH, n_qtiles, heads_per_xcd, stream); break;
    case 128: launch_fwd32_d<128, 32>(p, BH, n_qtiles, heads_per_xcd, stream); break;
  }
}

}  // namespace deers
