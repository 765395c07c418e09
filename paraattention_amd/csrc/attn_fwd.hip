// Attention forward (output + fp32 log-sum-exp, optionally causal) for gfx950.
//
// One workgroup = 4 or 8 wavefronts = 128 or 256 query rows; each wavefront owns
// 32 query rows for the whole key sweep.  Keys/values stream through LDS in
// tiles of 64 rows, double buffered.  The kernels that share the scheme:
//   attn_fwd_kernel            any head_dim (64 when K or V spans 4 GiB or more): global -> registers -> LDS
//   attn_fwd_d128_kernel       head_dim 128, LDS-DMA fills, 64-bit addressing
//   attn_fwd_d128_pipe_kernel  head_dim 128, two-tile software pipeline
//   attn_fwd_d128_stream_kernel  the same pipeline, resident workgroups over a list of pieces (the dense default)
//   attn_fwd_d128_short_kernel   the same pipeline for 449..512 keys per head (cross-attention to a text prompt)
//   attn_fwd_d64_pipe_kernel   head_dim 64, the same pipeline (the default)
//
// Both GEMMs run transposed so that the softmax needs no cross-lane traffic and
// P never leaves registers:
//   S^T[n,m] = sum_d K[n,d] Q[m,d]     A = K tile (LDS), B = Q (registers)
//   O^T[d,m] = sum_n V^T[d,n] P^T[n,m] A = V^T tile (LDS, transposed on the way
//                                      in), B = P^T = the S^T accumulators,
//                                      exponentiated and packed to 16 bit
// With v_mfma_f32_32x32x16 the accumulator of lane (m = lane%32, h = lane/32)
// holds rows n = 8a + 4h + b (a,b = 0..3) of column m, so a query row's 32
// scores of a sub-tile sit in two lanes (reduction = 1 swap), and accumulator
// registers 8c..8c+7 are exactly the 8 contraction slots lane (m,h) must supply
// as B operand of the second GEMM, provided V^T is laid out in LDS with the
// matching permutation of n (bits 2 and 3 of n swapped).
//
// Stands in for the aten flash/efficient/cuDNN forward kernels the reference
// dispatches to (src/para_attn/ops/__init__.py:48-157) and, with a list of key
// ranges per query segment, for the run loop of the reference's block-sparse
// mode (src/para_attn/sparse_attn.py:209-240).  Boolean key masks are taken apart
// on the device (key_mask_*_kernel) and served by the same kernels: in place with
// per-batch key counts where they keep prefixes, on dense copies of the kept rows
// (gather_kept_keys_kernel, the reference's attention_forward_sparse_kv,
// src/para_attn/ops/__init__.py:248-299) where they have holes.

#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <type_traits>

#include "pa_common.h"

namespace pa {

constexpr int BM = 128;       // query rows per workgroup
constexpr int BN = 64;        // key rows per LDS tile
constexpr int NTHREADS = 256;
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;
// The running maximum is only raised when a tile exceeds it by more than this
// many powers of two; below that the accumulators keep their scale (P <= 2^8).
constexpr float RESCALE_SLACK = 8.0f;

// Work plan of attn_fwd_d128_stream_kernel.  The launch has G workgroups of 256 query rows that stay resident.
// A piece is one query tile of one (batch, head) with its L key tiles.  Workgroup g first computes the R whole
// pieces g, g + G, ..., all workgroups sweeping the keys in step (so a K/V tile is fetched once per L2 and
// round); what is left (fewer than G pieces, or more where the plan keeps rounds of pieces back for it) is a list
// of (n_pieces - R G) L key-tile steps cut into Gt ranges: one for each of the first Gt workgroups, or, for long
// launches, rounds of ever shorter ranges that the workgroups draw from a counter as they run out of work.  A
// range that does not cover a whole piece leaves a normalised fp32 partial result and its LSE in the workspace
// (at most two per range: row 2n for a share that begins inside a piece, 2n + 1 for one that begins a piece but
// does not finish it), which attn_stream_merge_kernel folds.  Gt = G cuts the tail evenly; Gt = (pieces left) x s
// cuts every piece left into s shares that begin at the same keys.
// The keys of a piece may come in nseg segments of seg_len keys each (the blocks of a ring sweep), each with
// its own base pointer and the strides of AttnParams.
constexpr int MAX_KEY_SEGS = 16;
constexpr int MAX_TAIL_ROUNDS = 6;
struct StreamPlan {
  int G, R, Gt, L, n_pieces;
  int xcd_order;  // 1: workgroup numbers are dealt so that each of 8 XCDs holds a contiguous eighth of them
  int nseg, seg_len, tps;  // key segments, keys and key tiles per segment
  // The tail's key-tile steps come in n_rounds rounds (steps round_at[r] .. round_at[r + 1] of the tail), each cut
  // into Gt / n_rounds ranges of equal length.  next_range null: one round, range g belongs to workgroup g.
  // Otherwise the ranges (rounds of G, ever shorter) are taken in turn from that counter, 0 before the launch.
  int n_rounds;
  int64_t round_at[MAX_TAIL_ROUNDS + 1];
  int* next_range;
  int solo;  // test aid, with next_range and R = 0 only: workgroup 0 draws and computes every range, the others leave
  int has_kvlen;  // AttnParams.kv_len is set: a piece ends at its batch element's key count (one key segment only)
  const void* kseg[MAX_KEY_SEGS];
  const void* vseg[MAX_KEY_SEGS];
};

struct AttnParams {
  const void* q;
  const void* k;
  const void* v;
  void* out;
  float* lse;
  int B, H, Sq, Skv;
  int64_t qs_b, qs_h, qs_s;
  int64_t ks_b, ks_h, ks_s;
  int64_t vs_b, vs_h, vs_s;
  int64_t os_b, os_h, os_s;
  float scale_log2;  // scale * log2(e), > 0
  int n_qtiles;      // workgroups per (batch, head)
  int bm;            // query rows per workgroup (32 per wavefront)
  int pipe;          // head_dim 128: 1 = pipelined kernel, 0 = the one without 32-bit offset limits
  const int32_t* kv_len;  // dense: optional per-batch key count
  int causal;             // dense: query row i sees keys 0..i only (torch's is_causal, top-left aligned)
  // block-sparse only
  const int32_t* runs;  // count[Hm*nSeg] then range[Hm*nSeg][cap][2]
  const int32_t* order;  // optional [Hm][nQ]: the query blocks of a head by falling number of key tiles (launch order)
  int Hm, nQ, cap;
  int q_lo, q_block;
  int pair;  // block-sparse: each 256-row workgroup holds two 128-row query blocks and walks the union of their ranges
  int tiles_left, tiles_per_block;
  // dense pipelined kernel only: key-split tail.  Workgroups below split_main own a whole query
  // tile; the last split_tiles query tiles are computed by split_s workgroups each, over
  // consecutive shares of the key tiles, which leave normalised fp32 partial outputs and their
  // LSE in the workspace (piece-major) for attn_split_merge_kernel.  split_s <= 1: no split.
  int xcd_chunk;  // block-sparse pipelined kernel: ceil(workgroups / 8), 0 = plain order
  // 256-row dense kernel: *bound_flag != 0 says that no score can leave [-60, 60] in the log2 domain (see
  // score_bound_*_kernel), so the running maximum is not needed; null = not known, keep the maximum
  const int* bound_flag;
  int split_main, split_tiles, split_s;
  float* ws_out;  // [split_s * split_tiles][bm][128]
  float* ws_lse;  // [split_s * split_tiles][bm]
  // dense pipelined kernel only: ring accumulation.  With acc_out set, the result of this launch is
  // folded into the running pair (acc_out fp32 [B,H,Sq,128] contiguous, acc_lse [B,H,Sq]) by the
  // log-sum-exp merge instead of being stored on its own.  acc_first: the pair holds nothing yet
  // and is not read.  With `out` also set (last step) the folded output goes to `out` in the
  // activation type and acc_out is left alone; acc_lse is updated either way; `lse` is unused.
  float* acc_out;
  float* acc_lse;
  int acc_first;
  // attn_fwd_kernel only: an attention mask, one element per (batch, head, query, key) reached through four
  // strides in elements (0 on broadcast dimensions).  MASK_BOOL: bytes, 0 = the key is dropped for that query;
  // MASK_F32 / MASK_ACT: a bias added to the scaled score (fp32, or the activation type).
  const void* mask;
  int64_t ms_b, ms_h, ms_q, ms_k;
  // dense kernels: with `gate` set the launch leaves at once unless bit *gate of gate_mask is set (a decision taken on
  // the device by an earlier launch of the same stream, e.g. whether a key mask is a prefix)
  const int* gate;
  uint32_t gate_mask;
  StreamPlan st;  // attn_fwd_d128_stream_kernel only
};

// Whether the value that an earlier launch left in *gate (0 .. 31) is one of those a launch runs for.
__device__ __forceinline__ bool gate_open(const int* gate, uint32_t mask) { return ((mask >> (*gate & 31)) & 1u) != 0; }

constexpr int MASK_NONE = 0, MASK_BOOL = 1, MASK_F32 = 2, MASK_ACT = 3;


template <int D>
struct Smem {
  static constexpr int KSTRIDE = D + 8;    // elements; +16 B keeps b128 reads conflict free
  static constexpr int VSTRIDE = BN + 8;   // V^T row: 64 keys + 16 B pad
  static constexpr int K_ELEMS = BN * KSTRIDE;
  static constexpr int V_ELEMS = D * VSTRIDE;
  static constexpr int BYTES = 2 * (K_ELEMS + V_ELEMS) * 2;
};

// Key tiles of one workgroup: walks a list of [begin,end) ranges in steps of BN.
struct TileIter {
  const int32_t* ranges;  // pairs
  int nranges;
  int ri;
  int pos, end;
  int limit;      // keys there are: a listed range is cut there (a list built for a longer key sequence must not
                  // lead the walk past the tensors' end; the ranges ascend, so the first one beyond it ends the walk)
  int flag_mask;  // ~3 where a range's first key carries two flag bits (paired query blocks), else ~0
  int one[2];  // storage for the single dense range
  __device__ __forceinline__ void init_dense(int len) {
    one[0] = 0;
    one[1] = len;
    ranges = nullptr;
    nranges = len > 0 ? 1 : 0;
    ri = 0;
    pos = 0;
    end = len;
    limit = len;
    flag_mask = ~0;
  }
  __device__ __forceinline__ void init_range(int b, int e) {
    ranges = nullptr;
    nranges = e > b ? 1 : 0;
    ri = 0;
    pos = b;
    end = e;
    limit = e;
    flag_mask = ~0;
  }
  __device__ __forceinline__ void clip() {
    if (end > limit) end = limit;
    if ((pos & flag_mask) >= end) ri = nranges;
  }
  __device__ __forceinline__ void init_list(const int32_t* r, int n, int key_limit, bool flagged) {
    ranges = r;
    nranges = n;
    ri = 0;
    limit = key_limit;
    flag_mask = flagged ? ~3 : ~0;
    if (n > 0) {
      pos = r[0];
      end = r[1];
      clip();
    } else {
      pos = end = 0;
    }
  }
  __device__ __forceinline__ bool valid() const { return ri < nranges; }
  // current tile: rows [n0, n0 + nvalid), clamp row index to last
  __device__ __forceinline__ void get(int& n0, int& nvalid) const {
    n0 = pos;
    int left = end - pos;
    nvalid = left < BN ? left : BN;
  }
  __device__ __forceinline__ void next() {
    pos += BN;
    if (pos >= end) {
      ++ri;
      if (ri < nranges) {
        pos = ranges[2 * ri];
        end = ranges[2 * ri + 1];
        clip();
      }
    }
  }
};

// Which query rows a workgroup owns and which key ranges it walks.
template <bool SPARSE>
__device__ __forceinline__ void decode_block(const AttnParams& p, int qt, int head, int batch,
                                             int& row_begin, int& row_end, TileIter& it) {
  if constexpr (SPARSE) {
    int seg, tin;
    if (qt < p.tiles_left) {
      seg = 0;
      tin = qt;
      row_begin = tin * p.bm;
      row_end = p.q_lo;
    } else {
      int r = qt - p.tiles_left;
      int blk = r / p.tiles_per_block;
      if (blk < p.nQ) {
        tin = r - blk * p.tiles_per_block;
        // workgroups are started in the order of their numbers: the longest lists of a head first, so that the
        // launch does not end on a few long ones
        if (p.order != nullptr) blk = p.order[(p.Hm == 1 ? 0 : head) * p.nQ + blk];
        seg = 1 + blk;
        row_begin = p.q_lo + blk * p.q_block + tin * p.bm;
        row_end = p.q_lo + (blk + 1) * p.q_block;
      } else {
        seg = p.nQ + 1;
        tin = r - p.nQ * p.tiles_per_block;
        row_begin = p.q_lo + p.nQ * p.q_block + tin * p.bm;
        row_end = p.Sq;
      }
    }
    if (row_end > row_begin + p.bm) row_end = row_begin + p.bm;
    const int nseg = p.nQ + 2;
    const int hm = p.Hm == 1 ? 0 : head;
    const int sidx = hm * nseg + seg;
    const int cnt = p.runs[sidx];
    it.init_list(p.runs + (size_t)p.Hm * nseg + (size_t)sidx * p.cap * 2, cnt, p.Skv, p.pair != 0);
  } else {
    // causal: a workgroup's work grows with its row index, so the longest ones are started first
    if (p.causal) qt = p.n_qtiles - 1 - qt;
    row_begin = qt * p.bm;
    row_end = row_begin + p.bm < p.Sq ? row_begin + p.bm : p.Sq;
    int len = p.Skv;
    if (p.kv_len) {
      int kl = p.kv_len[batch];
      len = kl < len ? (kl < 0 ? 0 : kl) : len;
    }
    if (p.causal && len > row_end) len = row_end;  // no row of this workgroup sees a key past its last row
    it.init_dense(len);
  }

}

template <typename T, int D, bool SPARSE, int MASK = MASK_NONE>
__global__ __launch_bounds__(NTHREADS, 2) void attn_fwd_kernel(const AttnParams p) {
  typedef typename T::vec8 vec8;
  typedef Smem<D> SM;
  if constexpr (!SPARSE) {
    if (p.gate != nullptr && !gate_open(p.gate, p.gate_mask)) return;
  }
  constexpr int DC = D / 16;   // contraction chunks of the first GEMM
  constexpr int DB = D / 32;   // 32-row blocks of O^T
  constexpr int CH = D / 8;    // 16-byte chunks per K/V row
  constexpr int KROWS_PER_PASS = NTHREADS / CH;
  constexpr int KPASSES = BN / KROWS_PER_PASS;
  constexpr int VGROUPS = BN / 4;  // groups of 4 key rows
  static_assert(64 % VGROUPS == 0 && (NTHREADS / 64) * (64 / VGROUPS) >= CH, "V loader mapping");

  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  uint16_t* sK = smem;                        // [2][BN][KSTRIDE]
  uint16_t* sV = smem + 2 * SM::K_ELEMS;      // [2][D][VSTRIDE]  (V^T, keys permuted)

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int hh = lane >> 5;

  // ---- which query rows ------------------------------------------------------
  const int qt = blockIdx.x % p.n_qtiles;
  const int bh = blockIdx.x / p.n_qtiles;
  const int head = bh % p.H;
  const int batch = bh / p.H;

  int row_begin, row_end;  // query rows [row_begin, row_end) of this workgroup
  TileIter it;
  decode_block<SPARSE>(p, qt, head, batch, row_begin, row_end, it);

  const uint16_t* qbase = (const uint16_t*)p.q + batch * p.qs_b + head * p.qs_h;
  const uint16_t* kbase = (const uint16_t*)p.k + batch * p.ks_b + head * p.ks_h;
  const uint16_t* vbase = (const uint16_t*)p.v + batch * p.vs_b + head * p.vs_h;

  // ---- Q fragment: B operand of the first GEMM, kept for the whole sweep -----
  const int my_row = row_begin + wave * 32 + l32;
  const bool row_ok = my_row < row_end;
  vec8 qf[DC];
  {
    int r = row_ok ? my_row : (row_end - 1);
    const uint16_t* qp = qbase + (int64_t)r * p.qs_s + 8 * hh;
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) qf[dc] = *(const vec8*)(qp + 16 * dc);
    // Wait for Q here (vmcnt(0)).  Left pending, the compiler guards every first-GEMM MFMA
    // in the loop with a vmcnt wait that, in steady state, drains the K/V prefetch instead.
    __builtin_amdgcn_s_waitcnt(0x0F70);
  }

  // ---- global -> register staging of one K/V tile ----------------------------
  u32x4 kreg[KPASSES];
  u32x4 vreg[4];
  const int k_chunk = tid % CH;
  const int k_row0 = tid / CH;
  // V loader: a wavefront covers VGROUPS(=16) row groups x 4 column chunks, so that its
  // transposed 8-byte LDS writes (one V^T row per chunk element) spread over all banks
  constexpr int V_CH_PER_WAVE = 64 / VGROUPS;
  const int v_dcol = wave * V_CH_PER_WAVE + (lane % V_CH_PER_WAVE);
  const int v_grp = lane / V_CH_PER_WAVE;  // group of 4 key rows
  const bool v_active = v_dcol < CH;
  // position of the group inside V^T rows: swap the two low bits of the group
  const int v_grp_perm = (v_grp & ~3) | ((v_grp & 1) << 1) | ((v_grp >> 1) & 1);

  // Per-thread byte offsets inside a tile (32 bit); the tile's base address is wave-uniform,
  // so a full tile is fetched with scalar-base + vector-offset loads and no address math.
  const int64_t ks_bytes = p.ks_s * 2, vs_bytes = p.vs_s * 2;
  const uint32_t k_off0 = (uint32_t)(k_row0 * ks_bytes + 16 * k_chunk);
  const uint32_t v_off0 = (uint32_t)(4 * v_grp * vs_bytes + 16 * v_dcol);
  const char* kbytes = (const char*)kbase;
  const char* vbytes = (const char*)vbase;

  auto load_tile = [&](int n0, int nvalid) {
    if (nvalid == BN) {
      const char* kt = kbytes + (int64_t)n0 * ks_bytes;
      const char* vt = vbytes + (int64_t)n0 * vs_bytes;
#pragma unroll
      for (int i = 0; i < KPASSES; ++i)
        kreg[i] = *(const u32x4*)(kt + (int64_t)i * KROWS_PER_PASS * ks_bytes + k_off0);
      if (v_active) {
#pragma unroll
        for (int i = 0; i < 4; ++i) vreg[i] = *(const u32x4*)(vt + (int64_t)i * vs_bytes + v_off0);
      }
    } else {
      // ragged end of a range: rows past the end repeat the last valid row (masked later)
      const int last = n0 + nvalid - 1;
#pragma unroll
      for (int i = 0; i < KPASSES; ++i) {
        int r = n0 + k_row0 + i * KROWS_PER_PASS;
        r = r < last ? r : last;
        kreg[i] = *(const u32x4*)(kbytes + (int64_t)r * ks_bytes + 16 * k_chunk);
      }
      if (v_active) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          int r = n0 + 4 * v_grp + i;
          r = r < last ? r : last;
          vreg[i] = *(const u32x4*)(vbytes + (int64_t)r * vs_bytes + 16 * v_dcol);
        }
      }
    }
  };

  auto store_tile = [&](int buf) {
    uint16_t* dK = sK + buf * SM::K_ELEMS;
    uint16_t* dV = sV + buf * SM::V_ELEMS;
#pragma unroll
    for (int i = 0; i < KPASSES; ++i) {
      int r = k_row0 + i * KROWS_PER_PASS;
      *(u32x4*)(dK + r * SM::KSTRIDE + 8 * k_chunk) = kreg[i];
    }
    if (v_active) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int w = j >> 1;
        const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
        u32x2 t;
        t[0] = __builtin_amdgcn_perm(vreg[1][w], vreg[0][w], sel);
        t[1] = __builtin_amdgcn_perm(vreg[3][w], vreg[2][w], sel);
        *(u32x2*)(dV + (8 * v_dcol + j) * SM::VSTRIDE + 4 * v_grp_perm) = t;
      }
    }
  };

  // ---- accumulators -----------------------------------------------------------
  floatx16 o[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[i][r] = 0.f;
  float m_run = -INFINITY;  // running maximum, in units of log2 (scaled scores)
  float l_run = 0.f;        // this lane's share of the running sum
  const float c = p.scale_log2;

  // ---- pipeline prologue ------------------------------------------------------
  int n0 = 0, nvalid = 0;
  bool have = it.valid();
  if (have) {
    it.get(n0, nvalid);
    load_tile(n0, nvalid);
    it.next();
    store_tile(0);
  }
  int cur_valid = nvalid;
  int cur_n0 = 0;  // first key of the current tile (dense ranges start at key 0 and are contiguous)
  const int wave_row0 = row_begin + 32 * (threadIdx.x >> 6);
  bool have_next = it.valid();
  int next_valid = 0;
  if (have_next) {
    it.get(n0, nvalid);
    next_valid = nvalid;
    load_tile(n0, nvalid);
    it.next();
  }
  __syncthreads();

  int buf = 0;
  while (have) {
    // registers hold tile j+1: park it in the other buffer, then fetch tile j+2
    bool have_next2 = false;
    int next2_valid = 0;
    if (have_next) {
      store_tile(buf ^ 1);
      have_next2 = it.valid();
      if (have_next2) {
        it.get(n0, nvalid);
        next2_valid = nvalid;
        load_tile(n0, nvalid);
        it.next();
      }
    }

    const uint16_t* tK = sK + buf * SM::K_ELEMS;
    const uint16_t* tV = sV + buf * SM::V_ELEMS;

    // ---- S^T = K Q^T -----------------------------------------------------------
    floatx16 s[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int r = 0; r < 16; ++r) s[t][r] = 0.f;
#pragma unroll
      for (int dc = 0; dc < DC; ++dc) {
        vec8 a = *(const vec8*)(tK + (32 * t + l32) * SM::KSTRIDE + 16 * dc + 8 * hh);
        s[t] = T::mfma32(a, qf[dc], s[t]);
      }
    }

    // ---- attention mask: this lane's query row against the tile's keys ------------
    if constexpr (MASK != MASK_NONE) {
      const int64_t mrow = (int64_t)batch * p.ms_b + (int64_t)head * p.ms_h + (int64_t)(row_ok ? my_row : row_end - 1) * p.ms_q;
      const float per_scale = 1.0f / (c * LN2);  // bias / scale, so that (s + that) * c = s * c + bias * log2(e)
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int n = 32 * t + 8 * (r >> 2) + 4 * hh + (r & 3);
          if (n < cur_valid) {  // keys past the end are dealt with below and must not be read
            const int64_t mi = mrow + (int64_t)(cur_n0 + n) * p.ms_k;
            if constexpr (MASK == MASK_BOOL) {
              if (((const uint8_t*)p.mask)[mi] == 0) s[t][r] = -INFINITY;
            } else if constexpr (MASK == MASK_F32) {
              s[t][r] += ((const float*)p.mask)[mi] * per_scale;
            } else {
              const uint32_t w = ((const uint16_t*)p.mask)[mi];
              s[t][r] += T::lo(w) * per_scale;
            }
          }
        }
    }

    // ---- mask the ragged end of a range ---------------------------------------
    if (cur_valid < BN || (!SPARSE && p.causal && cur_n0 + BN - 1 > wave_row0)) {
      int lim = cur_valid;
      if (!SPARSE && p.causal) lim = min(lim, my_row - cur_n0 + 1);  // keys up to the row's own index
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          int n = 32 * t + 8 * (r >> 2) + 4 * hh + (r & 3);
          if (n >= lim) s[t][r] = -INFINITY;
        }
    }

    // ---- online softmax (row = lane%32, spread over the two half-waves) -------
    float mx = s[0][0];
#pragma unroll
    for (int r = 1; r < 16; ++r) mx = fmaxf(mx, s[0][r]);
#pragma unroll
    for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[1][r]);
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float mx_s = mx * c;
    if (__any(mx_s > m_run + RESCALE_SLACK)) {
      const float m_new = fmaxf(m_run, mx_s);
      float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      // the branch is taken by the whole wavefront: a row that has seen no kept key yet (possible under a mask
      // only) still has no maximum, and -inf - -inf must not turn its zeros into NaN
      if (MASK != MASK_NONE && m_new == -INFINITY) alpha = 1.f;
      l_run *= alpha;
#pragma unroll
      for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[i][r] *= alpha;
      m_run = m_new;
    }
    uint32_t pk[2][8];
    float lsum = 0.f;
    // a row whose keys so far were all masked away has no maximum yet: exponentiate against 0 (every term is 0)
    const float m_use = (MASK != MASK_NONE && m_run == -INFINITY) ? 0.f : m_run;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][r], c, -m_use));
        float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][r + 1], c, -m_use));
        lsum += p0 + p1;
        pk[t][r >> 1] = T::pack2(p0, p1);
      }
    l_run += lsum;

    // ---- O^T += V^T P^T ---------------------------------------------------------
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int cc = 0; cc < 2; ++cc) {
        u32x4 bw = {pk[t][4 * cc], pk[t][4 * cc + 1], pk[t][4 * cc + 2], pk[t][4 * cc + 3]};
        vec8 bfrag = __builtin_bit_cast(vec8, bw);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          vec8 a = *(const vec8*)(tV + (32 * db + l32) * SM::VSTRIDE + 32 * t + 16 * cc + 8 * hh);
          o[db] = T::mfma32(a, bfrag, o[db]);
        }
      }

    __syncthreads();
    buf ^= 1;
    have = have_next;
    cur_valid = next_valid;
    cur_n0 += BN;
    have_next = have_next2;
    next_valid = next2_valid;
  }

  // ---- epilogue -----------------------------------------------------------------
  const float l_tot = l_run + __shfl_xor(l_run, 32);
  const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
  if (row_ok) {
    uint16_t* op = (uint16_t*)p.out + batch * p.os_b + head * p.os_h + (int64_t)my_row * p.os_s;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        u32x2 w;
        w[0] = T::pack2(o[db][4 * a] * inv, o[db][4 * a + 1] * inv);
        w[1] = T::pack2(o[db][4 * a + 2] * inv, o[db][4 * a + 3] * inv);
        *(u32x2*)(op + 32 * db + 8 * a + 4 * hh) = w;
      }
    if (p.lse != nullptr && hh == 0) {
      float lse = l_tot > 0.f ? (m_run + __builtin_amdgcn_logf(l_tot)) * LN2 : -INFINITY;
      p.lse[((int64_t)batch * p.H + head) * p.Sq + my_row] = lse;
    }
  }
}


// ---------------------------------------------------------------------------------------------
// head_dim 128: the tuned kernel.
//
// K and V tiles (64 keys x 256 B) go from global memory straight into LDS
// (global_load_lds_dwordx4, no register staging), row-major and unpadded, with the 16-byte
// chunks of every row XOR-swizzled so that both the DMA writes and the fragment reads are free
// of bank conflicts:
//   K row r: logical chunk c is stored at chunk c ^ (r & 15)      (b128 reads down 16 rows)
//   V row r: logical chunk c is stored at chunk c ^ (4 * (r & 3)) (transpose reads of 8x64 B)
// The V^T operand of the second GEMM is read with ds_read_b64_tr_b16, which hands lane j of a
// 16-lane group column j of a 4x16 block: 4 consecutive keys for one head_dim index.
// K is fetched two tiles ahead and V one tile ahead; one workgroup barrier per tile sits between
// the two GEMMs.  Fragment reads run one phase ahead of the MFMAs that use them, in two
// alternating sets of 32 registers (fa / fb).
// ---------------------------------------------------------------------------------------------
constexpr int TILE_BYTES = BN * 256;  // one K or V tile at head_dim 128
// Buffer offset that is out of range for every tensor the pipelined kernel accepts (its host side
// refuses K or V extents of this size or more and takes the kernel above instead).
constexpr uint32_t PIPE_OOB = 0xfffff000u;

typedef __attribute__((address_space(3))) char lds_char;
typedef const __attribute__((address_space(1))) char glb_char;

template <typename T, bool SPARSE>
__global__ __launch_bounds__(NTHREADS, 2) void attn_fwd_d128_kernel(const AttnParams p) {
  typedef typename T::vec8 vec8;
  constexpr int D = 128, DC = 8, DB = 4;
  if constexpr (!SPARSE) {
    if (p.gate != nullptr && !gate_open(p.gate, p.gate_mask)) return;
  }
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  char* const sK = (char*)smem;                    // [2][64][256 B]
  char* const sV = (char*)smem + 2 * TILE_BYTES;   // [2][64][256 B]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int hh = lane >> 5;

  const int qt = blockIdx.x % p.n_qtiles;
  const int bh = blockIdx.x / p.n_qtiles;
  const int head = bh % p.H;
  const int batch = bh / p.H;
  int row_begin, row_end;
  TileIter itK;  // next tile whose K has to be fetched
  decode_block<SPARSE>(p, qt, head, batch, row_begin, row_end, itK);
  TileIter itV = itK;  // next tile whose V has to be fetched

  const uint16_t* qbase = (const uint16_t*)p.q + batch * p.qs_b + head * p.qs_h;
  const char* kbytes = (const char*)((const uint16_t*)p.k + batch * p.ks_b + head * p.ks_h);
  const char* vbytes = (const char*)((const uint16_t*)p.v + batch * p.vs_b + head * p.vs_h);
  const int64_t ks_bytes = p.ks_s * 2, vs_bytes = p.vs_s * 2;

  // ---- Q fragment (B operand of the first GEMM) --------------------------------------------
  const int my_row = row_begin + wave * 32 + l32;
  const bool row_ok = my_row < row_end;
  vec8 qf[DC];
  {
    int r = row_ok ? my_row : (row_end - 1);
    const uint16_t* qp = qbase + (int64_t)r * p.qs_s + 8 * hh;
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) qf[dc] = *(const vec8*)(qp + 16 * dc);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): keep Q out of the loop's wait accounting
  }

  // ---- global -> LDS copies -----------------------------------------------------------------
  // One wave instruction moves 64 x 16 B = 4 tile rows; wave w, step i covers rows 16i+4w..+3.
  const int dma_row = 4 * wave + (lane >> 4);  // row inside a 16-row group
  const int dma_pc = lane & 15;                // chunk position the lane's 16 B land on
  const uint32_t k_off0 = (uint32_t)(dma_row * ks_bytes + 16 * (dma_pc ^ (dma_row & 15)));
  const uint32_t v_off0 = (uint32_t)(dma_row * vs_bytes + 16 * (dma_pc ^ (4 * (dma_row & 3))));

  // Issued as inline assembly on purpose: the compiler then keeps no account of these copies
  // and does not make the LDS reads that follow wait for them; completion is awaited by hand
  // (s_waitcnt vmcnt(0)) in front of the one barrier per tile.  M0 carries the LDS address of
  // the wave's 1 KB destination; lane i's 16 bytes land at M0 + 16 i.
  auto dma_tile = [&](const char* gbase, int64_t row_bytes, uint32_t off0, int swz_is_k, char* dst,
                      int n0, int nvalid) {
    const uint32_t l0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_char*)dst + wave * 1024);
    if (nvalid == BN) {
      const char* g = gbase + (int64_t)n0 * row_bytes;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const char* gi = g + (int64_t)i * 16 * row_bytes;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :: "s"(l0 + i * 4096), "v"(off0), "s"(gi) : "memory");
      }
    } else {
      // ragged end of a range: rows past the end repeat the last valid row (masked later)
      const int last = n0 + nvalid - 1;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        int r = n0 + 16 * i + dma_row;
        r = r < last ? r : last;
        const int swz = swz_is_k ? (dma_row & 15) : 4 * (dma_row & 3);
        const char* ga = gbase + (int64_t)r * row_bytes + 16 * (dma_pc ^ swz);
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                     :: "s"(l0 + i * 4096), "v"(ga) : "memory");
      }
    }
  };
  auto dma_k = [&](int buf) {
    int n0, nv;
    itK.get(n0, nv);
    dma_tile(kbytes, ks_bytes, k_off0, 1, sK + buf * TILE_BYTES, n0, nv);
    itK.next();
  };
  auto dma_v = [&](int buf) {
    int n0, nv;
    itV.get(n0, nv);
    dma_tile(vbytes, vs_bytes, v_off0, 0, sV + buf * TILE_BYTES, n0, nv);
    itV.next();
  };

  // ---- fragment read addresses ---------------------------------------------------------------
  // K (A operand of S^T = K Q^T): lane (l32, hh) reads row 32t + l32, logical chunk 2dc + hh.
  uint32_t ka[DC];
#pragma unroll
  for (int dc = 0; dc < DC; ++dc) ka[dc] = l32 * 256 + 16 * ((2 * dc + hh) ^ (l32 & 15));
  // V (A operand of O^T = V^T P^T) through the transpose read: lane = (group g16, r, cq)
  // supplies the 8 bytes at key row 4*hh + r (+ 32t + 16c + 8a), head_dim 32db + 16*dhalf + 4cq.
  uint32_t va[DB];
  {
    const int g16 = lane >> 4, lg = lane & 15, r = lg >> 2, cq = lg & 3, dhalf = g16 & 1;
#pragma unroll
    for (int db = 0; db < DB; ++db)
      va[db] = (4 * hh + r) * 256 + 16 * ((4 * db + 2 * dhalf + (cq >> 1)) ^ (4 * r)) + 8 * (cq & 1);
  }
  auto read_k = [&](const char* tile, int t, int dc) -> vec8 {
    return *(const vec8*)(tile + t * 32 * 256 + ka[dc]);
  };
  typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4;
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  auto read_vt = [&](const char* tile, int t, int c, int db) -> vec8 {
    const char* a = tile + (32 * t + 16 * c) * 256 + va[db];
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(a));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(a + 8 * 256));
    typedef __attribute__((__vector_size__(8 * sizeof(short)))) short s16x8;
    s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(vec8, v);
  };

  // ---- accumulators ---------------------------------------------------------------------------
  floatx16 o[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[i][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const float c = p.scale_log2;

  // ---- prologue: K0, V0, K1 in flight; first K fragments in registers --------------------------
  int n0 = 0, cur_valid = 0, next_valid = 0;
  int cur_n0 = 0;  // first key of the current tile (dense ranges start at key 0 and are contiguous)
  const int wave_row0 = row_begin + 32 * wave;
  bool have = itK.valid();
  bool have_next = false;
  vec8 fa[8], fb[8];
  if (have) {
    itK.get(n0, cur_valid);
    dma_k(0);
    dma_v(0);
    have_next = itK.valid();
    if (have_next) {
      itK.get(n0, next_valid);
      dma_k(1);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) fa[dc] = read_k(sK, 0, dc);
  }

  // One tile; PAR = which K/V buffer it lives in.
  auto tile_step = [&](auto PAR) {
    constexpr int par = decltype(PAR)::value;
    const char* tK = sK + par * TILE_BYTES;
    const char* tV = sV + par * TILE_BYTES;
    const char* tKn = sK + (par ^ 1) * TILE_BYTES;

    // ---- phase 1: S0 = K[0:32] Q^T, while the fragments of K[32:64] arrive -----------------------
    floatx16 s0, s1;
#pragma unroll
    for (int r = 0; r < 16; ++r) s0[r] = s1[r] = 0.f;
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) fb[dc] = read_k(tK, 1, dc);
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) s0 = T::mfma32(fa[dc], qf[dc], s0);
    __builtin_amdgcn_sched_barrier(0);
    // ---- phase 2: S1 = K[32:64] Q^T ------------------------------------------------------------
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) s1 = T::mfma32(fb[dc], qf[dc], s1);
    __builtin_amdgcn_sched_barrier(0);

    // everything fetched so far has landed; after the barrier nobody still reads what comes next
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    const bool more_k = itK.valid();  // tile j+2
    int k2_valid = 0;
    if (more_k) {
      itK.get(n0, k2_valid);
      dma_k(par);
    }
    if (have_next) dma_v(par ^ 1);
    __builtin_amdgcn_sched_barrier(0);

    // ---- phase 3: V fragments of keys 0..31 on their way, softmax meanwhile ----------------------
#pragma unroll
    for (int cc = 0; cc < 2; ++cc)
#pragma unroll
      for (int db = 0; db < DB; ++db) fa[cc * 4 + db] = read_vt(tV, 0, cc, db);

    if (cur_valid < BN || (!SPARSE && p.causal && cur_n0 + BN - 1 > wave_row0)) {
      int lim = cur_valid;
      if (!SPARSE && p.causal) lim = min(lim, my_row - cur_n0 + 1);  // keys up to the row's own index
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        int n = 8 * (r >> 2) + 4 * hh + (r & 3);
        if (n >= lim) s0[r] = -INFINITY;
        if (n + 32 >= lim) s1[r] = -INFINITY;
      }
    }
    float mx = fmaxf(s0[0], s0[1]);
#pragma unroll
    for (int r = 2; r < 16; r += 2) mx = fmaxf(fmaxf(mx, s0[r]), s0[r + 1]);
#pragma unroll
    for (int r = 0; r < 16; r += 2) mx = fmaxf(fmaxf(mx, s1[r]), s1[r + 1]);
    {
      // other half of the row lives in lane ^ 32
      auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
      mx = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
    }
    const float mx_s = mx * c;
    if (__any(mx_s > m_run + RESCALE_SLACK)) {
      const float m_new = fmaxf(m_run, mx_s);
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      l_run *= alpha;
#pragma unroll
      for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[i][r] *= alpha;
      m_run = m_new;
    }
    // exp of keys 0..31 now; keys 32..63 are exponentiated in the shadow of the first PV MFMAs.
    // The row sum adds the fp32 values before rounding (summing the rounded ones costs up to
    // 3e-3 of LSE on peaked rows).
    uint32_t pk0[8], pk1[8];
    float lsum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s0[r], c, -m_run));
      float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s0[r + 1], c, -m_run));
      pk0[r >> 1] = T::pack2(p0, p1);
      lsum += p0 + p1;
    }

    // ---- phase 4: O^T += V^T[:, 0:32] P^T, while the V fragments of keys 32..63 arrive -----------
#pragma unroll
    for (int cc = 0; cc < 2; ++cc)
#pragma unroll
      for (int db = 0; db < DB; ++db) fb[cc * 4 + db] = read_vt(tV, 1, cc, db);
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      u32x4 bw = {pk0[4 * cc], pk0[4 * cc + 1], pk0[4 * cc + 2], pk0[4 * cc + 3]};
      vec8 bfrag = __builtin_bit_cast(vec8, bw);
#pragma unroll
      for (int db = 0; db < DB; ++db) o[db] = T::mfma32(fa[cc * 4 + db], bfrag, o[db]);
    }
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s1[r], c, -m_run));
      float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s1[r + 1], c, -m_run));
      pk1[r >> 1] = T::pack2(p0, p1);
      lsum += p0 + p1;
    }
    l_run += lsum;
    __builtin_amdgcn_sched_barrier(0);

    // ---- phase 5: O^T += V^T[:, 32:64] P^T, while the next tile's first K fragments arrive --------
    if (have_next) {
#pragma unroll
      for (int dc = 0; dc < DC; ++dc) fa[dc] = read_k(tKn, 0, dc);
    }
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      u32x4 bw = {pk1[4 * cc], pk1[4 * cc + 1], pk1[4 * cc + 2], pk1[4 * cc + 3]};
      vec8 bfrag = __builtin_bit_cast(vec8, bw);
#pragma unroll
      for (int db = 0; db < DB; ++db) o[db] = T::mfma32(fb[cc * 4 + db], bfrag, o[db]);
    }
    __builtin_amdgcn_sched_barrier(0);

    have = have_next;
    cur_valid = next_valid;
    cur_n0 += BN;
    have_next = more_k;
    next_valid = k2_valid;
  };

  while (have) {
    tile_step(std::integral_constant<int, 0>{});
    if (!have) break;
    tile_step(std::integral_constant<int, 1>{});
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // no tile copy may still be on its way to LDS when the wavefront ends

  // ---- epilogue -----------------------------------------------------------------------------------
  float l_tot;
  {
    auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(l_run), __float_as_uint(l_run), false, false);
    l_tot = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
  }
  const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
  if (row_ok) {
    uint16_t* op = (uint16_t*)p.out + batch * p.os_b + head * p.os_h + (int64_t)my_row * p.os_s;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        u32x2 w;
        w[0] = T::pack2(o[db][4 * a] * inv, o[db][4 * a + 1] * inv);
        w[1] = T::pack2(o[db][4 * a + 2] * inv, o[db][4 * a + 3] * inv);
        *(u32x2*)(op + 32 * db + 8 * a + 4 * hh) = w;
      }
    if (p.lse != nullptr && hh == 0) {
      float lse = l_tot > 0.f ? (m_run + __builtin_amdgcn_logf(l_tot)) * LN2 : -INFINITY;
      p.lse[((int64_t)batch * p.H + head) * p.Sq + my_row] = lse;
    }
  }
}


// ---------------------------------------------------------------------------------------------
// head_dim 128, two-tile software pipeline (the kernel used unless K or V spans 4 GiB or more).
//
// Same tile layout in LDS as the kernel above (row-major, XOR-swizzled chunks, LDS-DMA fills,
// transpose reads for V).  What differs is the order of work inside a wavefront.  Iteration j
// holds two score tiles, S(j) being exponentiated and S(j+1) being produced:
//
//   barrier            K(j+1) and V(j) have landed; everybody is done with iteration j-1
//   rare rescale of O  from the row maximum of S(j), taken one iteration earlier
//   stage A  16 x { MFMA of S(j+1) = K(j+1) Q^T, its two key halves alternating ; one LDS-DMA issue
//                   for K(j+2) / V(j+1) (first groups) ; refill of the consumed fragment slot }
//   six slots of the softmax of S(j) (a slot: scale of one score pair, exp2 of the pair before, row sum +
//                   pack of the pair before that), which give the first PV MFMA its operand
//   stage B  16 x { MFMA of O^T += V(j)^T P(j)^T ; refill ; one softmax slot under each of the first
//                   twelve ; the row maximum of S(j+1) }
//
// sched_barrier holds the MFMAs, the LDS reads and the tile copies to that order, but not the softmax
// arithmetic, which is pure; what holds it is the empty asm statement on the row sum in every slot.  Measured
// against this arrangement: softmax slots under the MFMAs of stage A -2..-3.5 % (VALU work between the MFMAs of
// the first GEMM costs more than it hides), the compiler's own placement (22 exponentials in front of stage B,
// the row-sum additions behind the last MFMA) -0.7..-3 %, all of the softmax between the stages -0.5..-1.2 %,
// its first slots right behind the barrier -1.5..-2.5 %.
// Every iteration runs the same code: a tile that does not exist is fetched out of bounds (the
// buffer descriptor returns zeros) and its scores are never used.
// NW = 4 wavefronts (128 query rows, two workgroups per CU) or 8 (256 rows, one per CU: half the
// tile copies per flop).  Dense launches may compute the query tiles of the last round of
// workgroups in several key shares (AttnParams::split_*), fold the result into a running
// (out, lse) pair (acc_*), or apply torch's causal mask (causal).
// ---------------------------------------------------------------------------------------------
template <typename T, bool SPARSE, int NW, bool BOUNDED = false, bool PAIR = false>
__global__ __launch_bounds__(64 * NW, NW == 4 ? 2 : 1) void attn_fwd_d128_pipe_kernel(const AttnParams p) {
  typedef typename T::vec8 vec8;
  constexpr int DC = 8, DB = 4;
  constexpr int IPW = 16 / NW;  // copy instructions per wavefront and K (V) tile
  // With a score bound on record the launch comes twice, once per variant, and the one the flag (computed on
  // the device just before) does not select leaves at once.  BOUNDED: exp2(score) cannot overflow or vanish, so
  // the reference point of the softmax stays 0 and row maxima, rescale checks and rescales are compiled out.
  if constexpr (!SPARSE && NW == 8) {
    if (p.bound_flag != nullptr && (*p.bound_flag != 0) != BOUNDED) return;
  }
  if constexpr (!SPARSE) {
    if (p.gate != nullptr && !gate_open(p.gate, p.gate_mask)) return;
  }
  constexpr int RS = 4 * NW;    // tile rows between two of them
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  char* const sK = (char*)smem;                    // [2][64][256 B]
  char* const sV = (char*)smem + 2 * TILE_BYTES;   // [2][64][256 B]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int hh = lane >> 5;

  int tile = blockIdx.x;
  int piece_slot = -1;  // >= 0: this workgroup computes one key share of a split query tile
  if constexpr (SPARSE) {
    // Workgroups go to the 8 XCDs in turn.  Give each XCD a contiguous eighth of the (head, query
    // tile) list, so that the workgroups sharing an L2 work on neighbouring query blocks of one
    // head, whose kept key blocks overlap, instead of every eighth block of several heads.
    if (p.xcd_chunk > 0) {
      tile = (tile & 7) * p.xcd_chunk + (tile >> 3);
      if (tile >= p.B * p.H * p.n_qtiles) return;
    }
  }
  if constexpr (!SPARSE) {
    if (p.split_s > 1 && tile >= p.split_main) {
      piece_slot = tile - p.split_main;
      tile = p.split_main + piece_slot % p.split_tiles;
    }
  }
  const int qt = tile % p.n_qtiles;
  const int bh = tile / p.n_qtiles;
  const int head = bh % p.H;
  const int batch = bh / p.H;
  int row_begin, row_end;
  TileIter it;
  decode_block<SPARSE>(p, qt, head, batch, row_begin, row_end, it);
  // Keys in segments (the blocks of a ring sweep, StreamPlan::kseg / vseg): the sweep below runs once per
  // segment, with the softmax state carried over in registers.  A key share of a split piece is then a run of
  // whole segments; with one segment it is a range of key tiles.
  int seg_lo = 0, seg_hi = 1;
  if constexpr (!SPARSE) {
    const int nseg = p.st.nseg > 1 ? p.st.nseg : 1;
    seg_hi = nseg;
    if (piece_slot >= 0) {
      const int piece = piece_slot / p.split_tiles;
      if (nseg > 1) {
        seg_lo = piece * nseg / p.split_s;
        seg_hi = (piece + 1) * nseg / p.split_s;
      } else {
        const int len = it.end;
        const int nkt = (len + BN - 1) / BN;
        const int t0 = (int)((int64_t)piece * nkt / p.split_s), t1 = (int)((int64_t)(piece + 1) * nkt / p.split_s);
        it.init_range(t0 * BN, t1 * BN < len ? t1 * BN : len);
      }
    }
  }

  const uint16_t* qbase = (const uint16_t*)p.q + batch * p.qs_b + head * p.qs_h;
  const char* kbytes = (const char*)((const uint16_t*)p.k + batch * p.ks_b + head * p.ks_h);
  const char* vbytes = (const char*)((const uint16_t*)p.v + batch * p.vs_b + head * p.vs_h);
  const uint32_t ks_bytes = (uint32_t)(p.ks_s * 2), vs_bytes = (uint32_t)(p.vs_s * 2);

  // ---- Q fragment (B operand of the first GEMM) --------------------------------------------
  const int my_row = row_begin + wave * 32 + l32;
  const bool row_ok = my_row < row_end;
  vec8 qf[DC];
  {
    int r = row_ok ? my_row : (row_end - 1);
    const uint16_t* qp = qbase + (int64_t)r * p.qs_s + 8 * hh;
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) qf[dc] = *(const vec8*)(qp + 16 * dc);
    // no wait here: the loads overlap the first tile copies, whose wait in front of the first barrier covers them
  }

  // ---- global -> LDS copies: raw buffer loads with the LDS bit ---------------------------------
  // The descriptor bounds the whole K (V) of this batch and head, so rows past the last key come
  // back as zeros instead of needing an address clamp.  One wave instruction moves 4 tile rows;
  // wave w, step i covers rows RS*i+4w..+3; lane l lands on chunk l%16 of row l/16 and fetches
  // the logical chunk that the swizzle maps there.  Inline assembly on purpose: the compiler
  // keeps no account of these copies, so LDS reads that follow do not wait for them; completion
  // is awaited by hand (vmcnt(0)) in front of the barrier.
  auto make_rsrc = [&](const char* base, uint32_t row_bytes, int n_keys) {
    u32x4 r;
    const uint64_t a = (uint64_t)base;
    const uint64_t nbytes = (uint64_t)(n_keys - 1) * row_bytes + 256;  // start of the last row + one row
    r[0] = __builtin_amdgcn_readfirstlane((uint32_t)a);
    r[1] = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32) & 0xffffu);
    r[2] = __builtin_amdgcn_readfirstlane((uint32_t)nbytes);
    r[3] = 0x00020000u;
    return r;
  };
  u32x4 krs = make_rsrc(kbytes, ks_bytes, p.Skv);
  u32x4 vrs = make_rsrc(vbytes, vs_bytes, p.Skv);
  const int dma_row = 4 * wave + (lane >> 4);
  const int dma_pc = lane & 15;
  const uint32_t k_off0 = dma_row * ks_bytes + 16 * (dma_pc ^ (dma_row & 15));
  const uint32_t v_off0 = dma_row * vs_bytes + 16 * (dma_pc ^ (4 * (dma_row & 3)));
  const uint32_t lds_k = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_char*)sK + wave * 1024);
  const uint32_t lds_v = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_char*)sV + wave * 1024);
  constexpr uint32_t OOB = PIPE_OOB;  // first key of a tile that does not exist; also its soffset
  // i-th of the four copy instructions of the K (V) tile starting at key n0, into buffer `buf`
  auto dma_k1 = [&](int buf, uint32_t n0, int i) {
    const uint32_t soff = __builtin_amdgcn_readfirstlane(n0 == OOB ? OOB : (n0 + RS * i) * ks_bytes);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_k + buf * TILE_BYTES + i * (RS * 256)), "v"(k_off0), "s"(krs), "s"(soff) : "memory");
  };
  auto dma_v1 = [&](int buf, uint32_t n0, int i) {
    const uint32_t soff = __builtin_amdgcn_readfirstlane(n0 == OOB ? OOB : (n0 + RS * i) * vs_bytes);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_v + buf * TILE_BYTES + i * (RS * 256)), "v"(v_off0), "s"(vrs), "s"(soff) : "memory");
  };

  // ---- fragment read addresses (as in the kernel above) -------------------------------------------
  uint32_t ka[DC];
#pragma unroll
  for (int dc = 0; dc < DC; ++dc) ka[dc] = l32 * 256 + 16 * ((2 * dc + hh) ^ (l32 & 15));
  uint32_t va[DB];
  {
    const int g16 = lane >> 4, lg = lane & 15, r = lg >> 2, cq = lg & 3, dhalf = g16 & 1;
#pragma unroll
    for (int db = 0; db < DB; ++db)
      va[db] = (4 * hh + r) * 256 + 16 * ((4 * db + 2 * dhalf + (cq >> 1)) ^ (4 * r)) + 8 * (cq & 1);
  }
  auto read_k = [&](const char* tile, int t, int dc) -> vec8 {
    return *(const vec8*)(tile + t * 32 * 256 + ka[dc]);
  };
  typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4;
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  auto read_vt = [&](const char* tile, int t, int c, int db) -> vec8 {
    const char* a = tile + (32 * t + 16 * c) * 256 + va[db];
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(a));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(a + 8 * 256));
    typedef __attribute__((__vector_size__(8 * sizeof(short)))) short s16x8;
    s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(vec8, v);
  };

  // ---- accumulators ---------------------------------------------------------------------------
  floatx16 o[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[i][r] = 0.f;
  float m_run = BOUNDED ? 0.f : -INFINITY, l_run = 0.f;
  const float c = p.scale_log2;

  // window of tiles j (being consumed), j+1 and j+2: (first key or OOB, valid keys)
  uint32_t n_cur, n_nxt, n_nx2;
  int v_cur, v_nxt, v_nx2;
  // PAIR (block-sparse, two adjacent 128-row query blocks per workgroup walking the union of their key ranges):
  // which of the two blocks keeps tiles j, j+1, j+2 (bit 0: the lower block = wavefronts 0..3, bit 1: the
  // upper); a range's first key carries the bits in its two low bits (ranges begin at multiples of 4 there).
  int m_cur = 3, m_nxt = 3, m_nx2 = 3;
  const int my_bit = wave < NW / 2 ? 1 : 2;
  auto pull = [&](uint32_t& n0, int& nv) {
    if constexpr (PAIR) {
      m_cur = m_nxt;
      m_nxt = m_nx2;
    }
    if (it.valid()) {
      int a, b;
      it.get(a, b);
      if constexpr (PAIR) {
        m_nx2 = a & 3;
        a &= ~3;
        const int left = it.end - a;
        b = left < BN ? left : BN;
      }
      it.next();
      n0 = (uint32_t)a;
      nv = b;
    } else {
      n0 = OOB;
      nv = 0;
      if constexpr (PAIR) m_nx2 = 0;
    }
  };
  bool have = false;

  // -inf on the keys past the end of a ragged tile: register r of this lane is key
  // 8*(r/4) + r%4 + 4*hh of the first half (+32 for the second); constants against one per-lane
  // limit, so nothing per register stays live across the loop
  const int wave_row0 = row_begin + 32 * wave;
  // causal: the tile starting at key n0 needs masking for this wavefront if it reaches past its first row
  auto on_diagonal = [&](uint32_t n0) {
    if constexpr (SPARSE) return false;
    else return p.causal != 0 && n0 != OOB && (int)n0 + BN - 1 > wave_row0;
  };
  auto mask_tail = [&](floatx16& a0, floatx16& a1, int nvalid, uint32_t n0) {
    int lim = nvalid;
    if constexpr (!SPARSE) {
      if (p.causal) lim = min(lim, my_row - (int)n0 + 1);  // keys up to the row's own index
    }
    lim -= 4 * hh;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      if (8 * (r >> 2) + (r & 3) >= lim) a0[r] = -INFINITY;
      if (8 * (r >> 2) + (r & 3) + 32 >= lim) a1[r] = -INFINITY;
    }
  };
  // other half of a query row lives in lane ^ 32
  auto across = [&](float x) {
    auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
  };

  vec8 f[8];          // ring of 8 operand fragments: a slot is refilled as soon as its MFMA has issued
  floatx16 sn0, sn1;  // S(j+1) (keys 0..31, 32..63); it is S(j) at the top of the next iteration
  float mx = 0.f;     // row maximum of S(j), masked, unscaled
#pragma unroll
  for (int r = 0; r < 16; ++r) sn0[r] = sn1[r] = 0.f;

  // One iteration; PAR = buffer of tile j (K(j+1) sits in the other K buffer).
  // ACUR / ANXT (PAIR only, else both true): whether this wavefront's query block keeps tile j / tile j+1; what
  // belongs to a tile it does not keep (scores, softmax, second GEMM) is compiled out of that variant, the copies
  // and the barrier stay.
  auto tile_step = [&](auto PAR, auto ACUR, auto ANXT) {
    constexpr int par = decltype(PAR)::value;
    const bool ac = ACUR, an = ANXT;  // constants unless PAIR
    const char* tV = sV + par * TILE_BYTES;
    const char* tKn = sK + (par ^ 1) * TILE_BYTES;
    floatx16 c0 = sn0, c1 = sn1;  // S(j)

    // everything fetched so far has landed; after the barrier nobody still reads what comes next
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();

    // first fragments of K(j+1) on their way while the maximum is settled
    if (an) {
#pragma unroll
      for (int dc = 0; dc < DC; ++dc) f[dc] = read_k(tKn, dc & 1, dc >> 1);
    }

    if (!BOUNDED && ac) {
      const float mx_s = mx * c;
      if (__any(mx_s > m_run + RESCALE_SLACK)) {
        const float m_new = fmaxf(m_run, mx_s);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        l_run *= alpha;
#pragma unroll
        for (int i = 0; i < DB; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[i][r] *= alpha;
        m_run = m_new;
      }
    }
    // Two 128-row workgroups share a CU unsynchronised: the wavefront that is in its second GEMM, where the
    // exponentials sit, gets the issue priority over the one that is in its first (+1.2 % measured; with one
    // 256-row workgroup per CU, whose wavefronts run in step, the same costs 1.5 %).
    if constexpr (NW == 4) __builtin_amdgcn_s_setprio(0);
    __builtin_amdgcn_sched_barrier(0);

    // ---- stage A ---------------------------------------------------------------------------------
    // The 32 scores of S(j) per lane are exponentiated over the 16 groups of stage A and the first
    // 6 of stage B (P of keys 32..63 is only needed by the last 8 MFMAs), which keeps the VALU work
    // per MFMA below the MFMA's own 32 cycles.  The row sum adds the fp32 values before rounding
    // (summing the rounded ones costs up to 3e-3 of LSE on peaked rows).
    uint32_t pk0[8], pk1[8];
    float lsum = 0.f;
    // Pair n of the 16 score pairs (0..7: keys 0..31, 8..15: keys 32..63) goes through three
    // steps in three consecutive slots, so that no instruction of a slot waits for another of
    // the same slot: scale and shift, exponential, sum and pack.
    float tf[2][2], te[2][2];
    auto expo_slot = [&](int n) {
      if (n >= 2 && n < 18) {
        const int j = n - 2;
        lsum += te[j & 1][0] + te[j & 1][1];
        asm volatile("" : "+v"(lsum));  // the addition stays in its slot (left alone it sinks behind the last MFMA)
        (j < 8 ? pk0 : pk1)[j & 7] = T::pack2(te[j & 1][0], te[j & 1][1]);
      }
      if (n >= 1 && n < 17) {
        const int j = n - 1;
        te[j & 1][0] = __builtin_amdgcn_exp2f(tf[j & 1][0]);
        te[j & 1][1] = __builtin_amdgcn_exp2f(tf[j & 1][1]);
      }
      if (n < 16) {
        const floatx16& cs = n < 8 ? c0 : c1;
        tf[n & 1][0] = __builtin_fmaf(cs[2 * (n & 7)], c, -m_run);
        tf[n & 1][1] = __builtin_fmaf(cs[2 * (n & 7) + 1], c, -m_run);
      }
    };
#pragma unroll
    for (int r = 0; r < 16; ++r) sn0[r] = sn1[r] = 0.f;
#pragma unroll
    for (int g = 0; g < 8; ++g) {
      // the two halves of S(j+1) alternate, so that no MFMA waits for the one just issued
      if (an) {
        if (g & 1) sn1 = T::mfma32(f[g], qf[g >> 1], sn1);
        else sn0 = T::mfma32(f[g], qf[g >> 1], sn0);
      }
      if (g < IPW) dma_k1(par, n_nx2, g);                      // K(j+2) takes the buffer K(j) has left
      else if (g < 2 * IPW) dma_v1(par ^ 1, n_nxt, g - IPW);  // V(j+1) takes the buffer V(j-1) has left
      if (an) f[g] = read_k(tKn, g & 1, 4 + (g >> 1));
      __builtin_amdgcn_sched_barrier(0);  // keep the groups in this order
    }
#pragma unroll
    for (int g = 0; g < 8; ++g) {
      if (an) {
        if (g & 1) sn1 = T::mfma32(f[g], qf[4 + (g >> 1)], sn1);
        else sn0 = T::mfma32(f[g], qf[4 + (g >> 1)], sn0);
      }
      if (ac) {
        f[g] = read_vt(tV, 0, g >> 2, g & 3);  // V(j), keys 0..31, takes the slot over
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (an) {
      if (v_nxt < BN || on_diagonal(n_nxt)) mask_tail(sn0, sn1, v_nxt, n_nxt);  // ragged, absent or diagonal tile j+1
    }
    __builtin_amdgcn_sched_barrier(0);

    // The softmax of S(j) begins here, not under the MFMAs of stage A (VALU work between the MFMAs of the first GEMM
    // costs more than it hides): the six slots that the first PV MFMA needs, then one slot under each of the next
    // twelve PV MFMAs, each row-sum addition held in its slot.
    if (ac) {
#pragma unroll
      for (int n = 0; n < 6; ++n) expo_slot(n);
    }
    __builtin_amdgcn_sched_barrier(0);
    // ---- stage B ---------------------------------------------------------------------------------
    if constexpr (NW == 4) __builtin_amdgcn_s_setprio(1);
    __builtin_amdgcn_sched_barrier(0);
    float mxa = fmaxf(sn0[0], sn0[1]), mxb = fmaxf(sn1[0], sn1[1]);
    if (!ac) {
      if (!BOUNDED && an) {  // no second GEMM to spread the row maximum of S(j+1) under
#pragma unroll
        for (int r = 2; r < 16; ++r) {
          mxa = fmaxf(mxa, sn0[r]);
          mxb = fmaxf(mxb, sn1[r]);
        }
      }
    }
    if (ac)
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      u32x4 bw = {pk0[4 * cc], pk0[4 * cc + 1], pk0[4 * cc + 2], pk0[4 * cc + 3]};
      vec8 bfrag = __builtin_bit_cast(vec8, bw);
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const int g = cc * 4 + db;
        o[db] = T::mfma32(f[g], bfrag, o[db]);
        f[g] = read_vt(tV, 1, cc, db);  // keys 32..63
        expo_slot(6 + g);
        if (!BOUNDED && an) {
          if (g < 4) {
          } else if (g < 7) mxa = fmaxf(fmaxf(fmaxf(fmaxf(mxa, sn0[4 * g - 14]), sn0[4 * g - 13]), sn0[4 * g - 12]), sn0[4 * g - 11]);
          else mxa = fmaxf(fmaxf(mxa, sn0[14]), sn0[15]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (ac)
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      u32x4 bw = {pk1[4 * cc], pk1[4 * cc + 1], pk1[4 * cc + 2], pk1[4 * cc + 3]};
      vec8 bfrag = __builtin_bit_cast(vec8, bw);
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const int g = cc * 4 + db;
        o[db] = T::mfma32(f[g], bfrag, o[db]);
        if (g < 4) expo_slot(14 + g);
        if (!BOUNDED && an) {
          if (g > 0) mxb = fmaxf(fmaxf(mxb, sn1[2 * g]), sn1[2 * g + 1]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (ac) l_run += lsum;
    if (!BOUNDED && an) mx = across(fmaxf(mxa, mxb));

    // slide the tile window
    n_cur = n_nxt;
    v_cur = v_nxt;
    n_nxt = n_nx2;
    v_nxt = v_nx2;
    pull(n_nx2, v_nx2);
    have = n_cur != OOB;
  };

  // The keys' segments are swept one after the other, the pipeline drained in between (carrying it across, with
  // the copies' descriptors following their tile's segment, was measured: the bookkeeping that adds to every
  // iteration costs 4.5 % of the sweep, the drains it saves 2 %).
  for (int seg = seg_lo; seg < seg_hi; ++seg) {
    if constexpr (!SPARSE) {
      if (p.st.nseg > 1) {  // this segment's keys and values, all of them
        const int64_t koff = (batch * p.ks_b + head * p.ks_h) * 2, voff = (batch * p.vs_b + head * p.vs_h) * 2;
        krs = make_rsrc((const char*)p.st.kseg[seg] + koff, ks_bytes, p.st.seg_len);
        vrs = make_rsrc((const char*)p.st.vseg[seg] + voff, vs_bytes, p.st.seg_len);
        it.init_dense(p.st.seg_len);
        if (seg > seg_lo) __syncthreads();  // everybody has left the previous segment's last tiles
      }
    }
    pull(n_cur, v_cur);
    pull(n_nxt, v_nxt);
    pull(n_nx2, v_nx2);
    have = n_cur != OOB;
    if (seg > seg_lo) {  // the scores left over from the previous segment's last, absent tile
#pragma unroll
      for (int r = 0; r < 16; ++r) sn0[r] = sn1[r] = 0.f;
    }
    // ---- prologue: K0, V0, K1 copies; S(0) and its row maximum ---------------------------------
    if (have) {
#pragma unroll
      for (int i = 0; i < IPW; ++i) dma_k1(0, n_cur, i);
#pragma unroll
      for (int i = 0; i < IPW; ++i) dma_v1(0, n_cur, i);
#pragma unroll
      for (int i = 0; i < IPW; ++i) dma_k1(1, n_nxt, i);
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();
#pragma unroll
      for (int dc = 0; dc < DC; ++dc) f[dc] = read_k(sK, 0, dc);
#pragma unroll
      for (int dc = 0; dc < DC; ++dc) {
        sn0 = T::mfma32(f[dc], qf[dc], sn0);
        f[dc] = read_k(sK, 1, dc);
      }
#pragma unroll
      for (int dc = 0; dc < DC; ++dc) sn1 = T::mfma32(f[dc], qf[dc], sn1);
      if (v_cur < BN || on_diagonal(n_cur)) mask_tail(sn0, sn1, v_cur, n_cur);
      if constexpr (!BOUNDED) {
        float m2 = fmaxf(sn0[0], sn1[0]);
#pragma unroll
        for (int r = 1; r < 16; ++r) m2 = fmaxf(fmaxf(m2, sn0[r]), sn1[r]);
        mx = across(m2);
      }
    }
    auto step = [&](auto PAR) {
      constexpr std::true_type yes{};
      if constexpr (!PAIR) {
        tile_step(PAR, yes, yes);
      } else {  // wave-uniform: what this wavefront's query block keeps of tiles j and j+1
        tile_step(PAR, (m_cur & my_bit) != 0, (m_nxt & my_bit) != 0);
      }
    };
    while (have) {
      step(std::integral_constant<int, 0>{});
      if (!have) break;
      step(std::integral_constant<int, 1>{});
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // no tile copy may still be on its way to LDS when the segment, or the wavefront, ends
  }

  // ---- epilogue -----------------------------------------------------------------------------------
  float l_tot;
  {
    auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(l_run), __float_as_uint(l_run), false, false);
    l_tot = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
  }
  const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
  if constexpr (!SPARSE) {
    if (piece_slot >= 0) {  // partial result of one key share: fp32, into the workspace
      if (row_ok) {
        const int64_t wrow = (int64_t)piece_slot * p.bm + (my_row - row_begin);
        float* wp = p.ws_out + wrow * 128;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int a = 0; a < 4; ++a) {
            float4 w = {o[db][4 * a] * inv, o[db][4 * a + 1] * inv, o[db][4 * a + 2] * inv, o[db][4 * a + 3] * inv};
            *(float4*)(wp + 32 * db + 8 * a + 4 * hh) = w;
          }
        if (hh == 0) p.ws_lse[wrow] = l_tot > 0.f ? (m_run + __builtin_amdgcn_logf(l_tot)) * LN2 : -INFINITY;
      }
      return;
    }
    if (p.acc_out != nullptr) {  // fold into the running (out, lse) pair
      if (row_ok) {
        const int64_t ridx = ((int64_t)batch * p.H + head) * p.Sq + my_row;
        const float blk = l_tot > 0.f ? (m_run + __builtin_amdgcn_logf(l_tot)) * LN2 : -INFINITY;
        const float old = p.acc_first ? -INFINITY : p.acc_lse[ridx];
        const float mx = fmaxf(old, blk);
        float w_old = 0.f, w_blk = 0.f, lse_new = -INFINITY;
        if (mx > -INFINITY) {
          const float e_old = __expf(old - mx), e_blk = __expf(blk - mx);
          const float den = e_old + e_blk;
          w_old = e_old / den;
          w_blk = e_blk / den * inv;
          lse_new = mx + __logf(den);
        }
        float* ap = p.acc_out + ridx * 128;
        uint16_t* op = p.out ? (uint16_t*)p.out + batch * p.os_b + head * p.os_h + (int64_t)my_row * p.os_s : nullptr;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int a = 0; a < 4; ++a) {
            const int d0 = 32 * db + 8 * a + 4 * hh;
            float4 r = {0.f, 0.f, 0.f, 0.f};
            if (!p.acc_first && w_old > 0.f) r = *(const float4*)(ap + d0);
            r.x = r.x * w_old + o[db][4 * a] * w_blk;
            r.y = r.y * w_old + o[db][4 * a + 1] * w_blk;
            r.z = r.z * w_old + o[db][4 * a + 2] * w_blk;
            r.w = r.w * w_old + o[db][4 * a + 3] * w_blk;
            if (op) {
              u32x2 w;
              w[0] = T::pack2(r.x, r.y);
              w[1] = T::pack2(r.z, r.w);
              *(u32x2*)(op + d0) = w;
            } else {
              *(float4*)(ap + d0) = r;
            }
          }
        if (hh == 0) p.acc_lse[ridx] = lse_new;
      }
      return;
    }
  }
  if (row_ok) {
    uint16_t* op = (uint16_t*)p.out + batch * p.os_b + head * p.os_h + (int64_t)my_row * p.os_s;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        u32x2 w;
        w[0] = T::pack2(o[db][4 * a] * inv, o[db][4 * a + 1] * inv);
        w[1] = T::pack2(o[db][4 * a + 2] * inv, o[db][4 * a + 3] * inv);
        *(u32x2*)(op + 32 * db + 8 * a + 4 * hh) = w;
      }
    if (p.lse != nullptr && hh == 0) {
      float lse = l_tot > 0.f ? (m_run + __builtin_amdgcn_logf(l_tot)) * LN2 : -INFINITY;
      p.lse[((int64_t)batch * p.H + head) * p.Sq + my_row] = lse;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// head_dim 64 (the reference's own op-test shape, tests/ops/test_ops.py:21-24): the two-tile
// pipeline above with half the contraction and half the output width.  A K or V tile is 64 rows of
// 128 bytes; one copy instruction moves 8 rows.  Swizzles for 128-byte rows (two rows share the 64
// banks): K chunk c of row r sits at c ^ ((r >> 1) & 7), so the 16 rows a b128 read touches hit 16
// different 16-byte slots; V chunk c at c ^ (4 * ((r >> 1) & 1)), so the two even (odd) rows of a
// transpose read keep apart.  Per tile and wavefront: 8 MFMAs of S(j+1) (stage A), 8 of
// O^T += V(j)^T P(j)^T (stage B), against the same 32 exponentials per lane as at head_dim 128, so
// this kernel is bound by the VALU, not by the matrix cores.  The 8 fragments of K(j+1) fill the
// ring at the top of an iteration; each stage-A MFMA frees a slot for one of the 8 fragments of
// V(j); of the 18 softmax slots six sit between the stages (what the first PV MFMA needs) and three under
// each of the first four PV MFMAs, held there by an empty asm statement on the row sum.
// ---------------------------------------------------------------------------------------------
constexpr int TILE64_BYTES = BN * 128;

template <typename T, bool SPARSE, int NW, bool BOUNDED = false>
__global__ __launch_bounds__(64 * NW, NW == 4 ? 2 : 1) void attn_fwd_d64_pipe_kernel(const AttnParams p) {
  // BOUNDED and the flag: as in attn_fwd_d128_pipe_kernel
  if constexpr (!SPARSE) {
    if (p.bound_flag != nullptr && (*p.bound_flag != 0) != BOUNDED) return;
    if (p.gate != nullptr && !gate_open(p.gate, p.gate_mask)) return;
  }
  typedef typename T::vec8 vec8;
  constexpr int DC = 4, DB = 2;
  constexpr int IPW = 8 / NW;  // copy instructions per wavefront and K (V) tile
  constexpr int RS = 8 * NW;   // tile rows between two of them
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  char* const sK = (char*)smem;                      // [2][64][128 B]
  char* const sV = (char*)smem + 2 * TILE64_BYTES;   // [2][64][128 B]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int hh = lane >> 5;

  int tile = blockIdx.x;
  if constexpr (SPARSE) {
    if (p.xcd_chunk > 0) {  // one contiguous eighth of the (head, query tile) list per XCD
      tile = (tile & 7) * p.xcd_chunk + (tile >> 3);
      if (tile >= p.B * p.H * p.n_qtiles) return;
    }
  }
  const int qt = tile % p.n_qtiles;
  const int bh = tile / p.n_qtiles;
  const int head = bh % p.H;
  const int batch = bh / p.H;
  int row_begin, row_end;
  TileIter it;
  decode_block<SPARSE>(p, qt, head, batch, row_begin, row_end, it);

  const uint16_t* qbase = (const uint16_t*)p.q + batch * p.qs_b + head * p.qs_h;
  const char* kbytes = (const char*)((const uint16_t*)p.k + batch * p.ks_b + head * p.ks_h);
  const char* vbytes = (const char*)((const uint16_t*)p.v + batch * p.vs_b + head * p.vs_h);
  const uint32_t ks_bytes = (uint32_t)(p.ks_s * 2), vs_bytes = (uint32_t)(p.vs_s * 2);

  const int my_row = row_begin + wave * 32 + l32;
  const bool row_ok = my_row < row_end;
  vec8 qf[DC];
  {
    int r = row_ok ? my_row : (row_end - 1);
    const uint16_t* qp = qbase + (int64_t)r * p.qs_s + 8 * hh;
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) qf[dc] = *(const vec8*)(qp + 16 * dc);
    // no wait here: the loads overlap the first tile copies, whose wait in front of the first barrier covers them
  }

  // global -> LDS copies as in the head_dim-128 pipeline: wave w, step i covers tile rows
  // RS*i + 8w .. +7; lane l lands on chunk l%8 of row l/8
  auto make_rsrc = [&](const char* base, uint32_t row_bytes) {
    u32x4 r;
    const uint64_t a = (uint64_t)base;
    const uint64_t nbytes = (uint64_t)(p.Skv - 1) * row_bytes + 128;  // start of the last row + one row
    r[0] = __builtin_amdgcn_readfirstlane((uint32_t)a);
    r[1] = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32) & 0xffffu);
    r[2] = __builtin_amdgcn_readfirstlane((uint32_t)nbytes);
    r[3] = 0x00020000u;
    return r;
  };
  const u32x4 krs = make_rsrc(kbytes, ks_bytes);
  const u32x4 vrs = make_rsrc(vbytes, vs_bytes);
  const int dma_row = 8 * wave + (lane >> 3);
  const int dma_pc = lane & 7;
  const uint32_t k_off0 = dma_row * ks_bytes + 16 * (dma_pc ^ ((dma_row >> 1) & 7));
  const uint32_t v_off0 = dma_row * vs_bytes + 16 * (dma_pc ^ (4 * ((dma_row >> 1) & 1)));
  const uint32_t lds_k = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_char*)sK + wave * 1024);
  const uint32_t lds_v = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_char*)sV + wave * 1024);
  constexpr uint32_t OOB = PIPE_OOB;
  auto dma_k1 = [&](int buf, uint32_t n0, int i) {
    const uint32_t soff = __builtin_amdgcn_readfirstlane(n0 == OOB ? OOB : (n0 + RS * i) * ks_bytes);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_k + buf * TILE64_BYTES + i * (RS * 128)), "v"(k_off0), "s"(krs), "s"(soff) : "memory");
  };
  auto dma_v1 = [&](int buf, uint32_t n0, int i) {
    const uint32_t soff = __builtin_amdgcn_readfirstlane(n0 == OOB ? OOB : (n0 + RS * i) * vs_bytes);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_v + buf * TILE64_BYTES + i * (RS * 128)), "v"(v_off0), "s"(vrs), "s"(soff) : "memory");
  };

  // fragment read addresses
  uint32_t ka[DC];
#pragma unroll
  for (int dc = 0; dc < DC; ++dc) ka[dc] = l32 * 128 + 16 * ((2 * dc + hh) ^ ((l32 >> 1) & 7));
  uint32_t va[DB];
  {
    const int g16 = lane >> 4, lg = lane & 15, r = lg >> 2, cq = lg & 3, dhalf = g16 & 1;
#pragma unroll
    for (int db = 0; db < DB; ++db)
      va[db] = (4 * hh + r) * 128 + 16 * ((4 * db + 2 * dhalf + (cq >> 1)) ^ (4 * ((r >> 1) & 1))) + 8 * (cq & 1);
  }
  auto read_k = [&](const char* tl, int t, int dc) -> vec8 { return *(const vec8*)(tl + t * 32 * 128 + ka[dc]); };
  typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4;
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  auto read_vt = [&](const char* tl, int t, int c, int db) -> vec8 {
    const char* a = tl + (32 * t + 16 * c) * 128 + va[db];
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(a));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(a + 8 * 128));
    typedef __attribute__((__vector_size__(8 * sizeof(short)))) short s16x8;
    s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(vec8, v);
  };

  floatx16 o[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[i][r] = 0.f;
  float m_run = BOUNDED ? 0.f : -INFINITY, l_run = 0.f;
  const float c = p.scale_log2;

  uint32_t n_cur, n_nxt, n_nx2;
  int v_cur, v_nxt, v_nx2;
  auto pull = [&](uint32_t& n0, int& nv) {
    if (it.valid()) {
      int a, b;
      it.get(a, b);
      it.next();
      n0 = (uint32_t)a;
      nv = b;
    } else {
      n0 = OOB;
      nv = 0;
    }
  };
  pull(n_cur, v_cur);
  pull(n_nxt, v_nxt);
  pull(n_nx2, v_nx2);
  bool have = n_cur != OOB;

  const int wave_row0 = row_begin + 32 * wave;
  auto on_diagonal = [&](uint32_t n0) {
    if constexpr (SPARSE) return false;
    else return p.causal != 0 && n0 != OOB && (int)n0 + BN - 1 > wave_row0;
  };
  auto mask_tail = [&](floatx16& a0, floatx16& a1, int nvalid, uint32_t n0) {
    int lim = nvalid;
    if constexpr (!SPARSE) {
      if (p.causal) lim = min(lim, my_row - (int)n0 + 1);
    }
    lim -= 4 * hh;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      if (8 * (r >> 2) + (r & 3) >= lim) a0[r] = -INFINITY;
      if (8 * (r >> 2) + (r & 3) + 32 >= lim) a1[r] = -INFINITY;
    }
  };
  auto across = [&](float x) {
    auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
  };

  vec8 f[8];
  floatx16 sn0, sn1;
  float mx = 0.f;
#pragma unroll
  for (int r = 0; r < 16; ++r) sn0[r] = sn1[r] = 0.f;

  if (have) {
#pragma unroll
    for (int i = 0; i < IPW; ++i) dma_k1(0, n_cur, i);
#pragma unroll
    for (int i = 0; i < IPW; ++i) dma_v1(0, n_cur, i);
#pragma unroll
    for (int i = 0; i < IPW; ++i) dma_k1(1, n_nxt, i);
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
#pragma unroll
    for (int g = 0; g < 8; ++g) f[g] = read_k(sK, g & 1, g >> 1);
#pragma unroll
    for (int g = 0; g < 8; ++g) {
      if (g & 1) sn1 = T::mfma32(f[g], qf[g >> 1], sn1);
      else sn0 = T::mfma32(f[g], qf[g >> 1], sn0);
    }
    if (v_cur < BN || on_diagonal(n_cur)) mask_tail(sn0, sn1, v_cur, n_cur);
    if constexpr (!BOUNDED) {
      float m2 = fmaxf(sn0[0], sn1[0]);
#pragma unroll
      for (int r = 1; r < 16; ++r) m2 = fmaxf(fmaxf(m2, sn0[r]), sn1[r]);
      mx = across(m2);
    }
  }

  auto tile_step = [&](auto PAR) {
    constexpr int par = decltype(PAR)::value;
    const char* tV = sV + par * TILE64_BYTES;
    const char* tKn = sK + (par ^ 1) * TILE64_BYTES;
    floatx16 c0 = sn0, c1 = sn1;  // S(j)

    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
#pragma unroll
    for (int g = 0; g < 8; ++g) f[g] = read_k(tKn, g & 1, g >> 1);  // all of K(j+1), halves alternating

    const float mx_s = mx * c;
    if (!BOUNDED && __any(mx_s > m_run + RESCALE_SLACK)) {
      const float m_new = fmaxf(m_run, mx_s);
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      l_run *= alpha;
#pragma unroll
      for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[i][r] *= alpha;
      m_run = m_new;
    }
    __builtin_amdgcn_sched_barrier(0);

    uint32_t pk0[8], pk1[8];
    float lsum = 0.f;
    float tf[2][2], te[2][2];
    auto expo_slot = [&](int n) {  // as in the head_dim-128 pipeline: a score pair takes three consecutive slots
      if (n >= 2 && n < 18) {
        const int j = n - 2;
        lsum += te[j & 1][0] + te[j & 1][1];
        asm volatile("" : "+v"(lsum));  // holds the slot's arithmetic where the source puts it
        (j < 8 ? pk0 : pk1)[j & 7] = T::pack2(te[j & 1][0], te[j & 1][1]);
      }
      if (n >= 1 && n < 17) {
        const int j = n - 1;
        te[j & 1][0] = __builtin_amdgcn_exp2f(tf[j & 1][0]);
        te[j & 1][1] = __builtin_amdgcn_exp2f(tf[j & 1][1]);
      }
      if (n < 16) {
        const floatx16& cs = n < 8 ? c0 : c1;
        tf[n & 1][0] = __builtin_fmaf(cs[2 * (n & 7)], c, -m_run);
        tf[n & 1][1] = __builtin_fmaf(cs[2 * (n & 7) + 1], c, -m_run);
      }
    };
#pragma unroll
    for (int r = 0; r < 16; ++r) sn0[r] = sn1[r] = 0.f;
    // ---- stage A: S(j+1) ----------------------------------------------------------------------------
    if constexpr (NW == 4) __builtin_amdgcn_s_setprio(0);  // as in the head_dim 128 kernel
#pragma unroll
    for (int g = 0; g < 8; ++g) {
      if (g & 1) sn1 = T::mfma32(f[g], qf[g >> 1], sn1);
      else sn0 = T::mfma32(f[g], qf[g >> 1], sn0);
      if (g < IPW) dma_k1(par, n_nx2, g);                      // K(j+2) takes the buffer K(j) has left
      else if (g < 2 * IPW) dma_v1(par ^ 1, n_nxt, g - IPW);  // V(j+1) takes the buffer V(j-1) has left
      f[g] = read_vt(tV, g >> 2, (g >> 1) & 1, g & 1);         // V(j) in the order stage B consumes it
      __builtin_amdgcn_sched_barrier(0);
    }
    if (v_nxt < BN || on_diagonal(n_nxt)) mask_tail(sn0, sn1, v_nxt, n_nxt);
    __builtin_amdgcn_sched_barrier(0);

    // the six softmax slots that the first PV MFMA needs (none under the MFMAs of stage A: measured -2 %)
#pragma unroll
    for (int n = 0; n < 6; ++n) expo_slot(n);
    __builtin_amdgcn_sched_barrier(0);
    // ---- stage B: O^T += V(j)^T P(j)^T; slots 6..17, three under each of the first four MFMAs, then the row
    // maximum of S(j+1) ----------------------------------------------------------------------------
    if constexpr (NW == 4) __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      u32x4 bw = {pk0[4 * cc], pk0[4 * cc + 1], pk0[4 * cc + 2], pk0[4 * cc + 3]};
      vec8 bfrag = __builtin_bit_cast(vec8, bw);
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const int g = 2 * cc + db;
        o[db] = T::mfma32(f[g], bfrag, o[db]);
        expo_slot(6 + 3 * g);
        expo_slot(7 + 3 * g);
        expo_slot(8 + 3 * g);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    l_run += lsum;
    float mxa = sn0[0], mxb = sn1[0];
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      u32x4 bw = {pk1[4 * cc], pk1[4 * cc + 1], pk1[4 * cc + 2], pk1[4 * cc + 3]};
      vec8 bfrag = __builtin_bit_cast(vec8, bw);
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const int g = 2 * cc + db;
        o[db] = T::mfma32(f[4 + g], bfrag, o[db]);
        if constexpr (!BOUNDED) {
          mxa = fmaxf(fmaxf(fmaxf(fmaxf(mxa, sn0[4 * g]), sn0[4 * g + 1]), sn0[4 * g + 2]), sn0[4 * g + 3]);
          mxb = fmaxf(fmaxf(fmaxf(fmaxf(mxb, sn1[4 * g]), sn1[4 * g + 1]), sn1[4 * g + 2]), sn1[4 * g + 3]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if constexpr (!BOUNDED) mx = across(fmaxf(mxa, mxb));

    n_cur = n_nxt;
    v_cur = v_nxt;
    n_nxt = n_nx2;
    v_nxt = v_nx2;
    pull(n_nx2, v_nx2);
    have = n_cur != OOB;
  };

  while (have) {
    tile_step(std::integral_constant<int, 0>{});
    if (!have) break;
    tile_step(std::integral_constant<int, 1>{});
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // no tile copy may still be on its way to LDS when the wavefront ends

  float l_tot;
  {
    auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(l_run), __float_as_uint(l_run), false, false);
    l_tot = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
  }
  const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
  if (row_ok) {
    uint16_t* op = (uint16_t*)p.out + batch * p.os_b + head * p.os_h + (int64_t)my_row * p.os_s;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        u32x2 w;
        w[0] = T::pack2(o[db][4 * a] * inv, o[db][4 * a + 1] * inv);
        w[1] = T::pack2(o[db][4 * a + 2] * inv, o[db][4 * a + 3] * inv);
        *(u32x2*)(op + 32 * db + 8 * a + 4 * hh) = w;
      }
    if (p.lse != nullptr && hh == 0) {
      float lse = l_tot > 0.f ? (m_run + __builtin_amdgcn_logf(l_tot)) * LN2 : -INFINITY;
      p.lse[((int64_t)batch * p.H + head) * p.Sq + my_row] = lse;
    }
  }
}

// Where the softmax of a score tile goes in an iteration of attn_fwd_d128_stream_kernel with 64 rows per wavefront
// (see there): 170 small steps, step i in the gap behind MFMA gap[i] of the iteration, -1 for the steps that do
// not exist (the first and last slots hold fewer).
struct Rb2Steps {
  static constexpr int N = 170;
  int gap[N];
  int lo[64], hi[64];  // the steps of gap q are lo[q] .. hi[q] - 1 (their gaps ascend), less those that do not exist
  static constexpr int pair(int i) {
    const int slot = i / 5, kind = i % 5;
    return kind == 0 ? slot - 2 : kind < 3 ? slot - 1 : slot;
  }
  static constexpr int cost(int i) {
    const int n = pair(i), kind = i % 5;
    return n < 0 || n > 31 ? 0 : kind == 0 ? 12 : kind < 3 ? 8 : 12;
  }
  constexpr Rb2Steps() : gap(), lo(), hi() {
    int total = 0;
    for (int i = 0; i < N; ++i) total += cost(i);
    int before = 0;
    for (int i = 0; i < N; ++i) {
      gap[i] = cost(i) == 0 ? -1 : (2 * before + cost(i)) * 30 / total;  // 60 gaps, by the middle of the step's span
      before += cost(i);
    }
    for (int q = 0; q < 64; ++q) {
      lo[q] = N;
      hi[q] = 0;
      for (int i = 0; i < N; ++i)
        if (gap[i] == q) {
          if (i < lo[q]) lo[q] = i;
          hi[q] = i + 1;
        }
    }
  }
};
constexpr Rb2Steps RB2_STEPS{};

// every 16-key chunk of probabilities is packed before the PV MFMAs that take it: row block 0's before MFMA 32 + 8 k,
// row block 1's before MFMA 36 + 8 k (step C of pair n is small step 5 (n + 2))
constexpr bool rb2_steps_meet_deadlines() {
  for (int k = 0; k < 4; ++k)
    if (RB2_STEPS.gap[5 * (8 * k + 3 + 2)] >= 32 + 8 * k || RB2_STEPS.gap[5 * (8 * k + 7 + 2)] >= 36 + 8 * k) return false;
  return true;
}
static_assert(rb2_steps_meet_deadlines(), "softmax steps are dealt too late for the second GEMM");

// ---------------------------------------------------------------------------------------------
// head_dim 128, resident workgroups (StreamPlan above): the two-tile pipeline of
// attn_fwd_d128_pipe_kernel<.., 8> run over a list of pieces per workgroup as ONE stream of key
// tiles.  The copies of K(j+2) and V(j+1) and the scores S(j+1) simply belong to the next piece when
// tile j is the last of its piece, so the next piece's first tiles, its Q fragments (fetched into the
// registers the finished piece's Q has left, one iteration ahead) and its first score tile are all
// under way while the current piece's last tiles are computed; the output of a finished piece is
// stored from inside the loop.  What a launch of one workgroup per piece pays per piece (Q load,
// first copies, S(0), output drain: 5-10 us against 1.7 us per key tile) is hidden behind the
// neighbouring pieces' MFMA work.  Dense, not causal, no per-batch key counts.
//
// RB = query row blocks of 32 per wavefront.  RB = 1: 8 wavefronts of 32 rows, two per SIMD, everything in
// the 256 vector registers a wavefront then has (the form that ships).  RB = 2: 4 wavefronts of 64 rows, one per
// SIMD with 512 registers (the output and score accumulators in accumulation registers); every fragment read
// from LDS feeds two MFMAs, so the workgroup reads half the LDS bytes per flop, but the scores have to be
// read back from the accumulation registers (one more vector instruction per score) and one wavefront has to
// overlap its softmax with its own MFMAs.  Same results bit for bit; measured at the same speed as RB = 1 on
// the long shapes (the kernel sits at the chip's power limit either way: 68 % MFMA occupancy at 1.72 GHz
// against 74 % at 1.60 GHz) and slower on short pieces, so it stays behind the "wave_rows" knob.
// ---------------------------------------------------------------------------------------------
template <typename T, bool BOUNDED, int RB = 1, bool KVLEN = false>
__global__ __launch_bounds__(512 / RB, 1) void attn_fwd_d128_stream_kernel(const AttnParams p) {
  typedef typename T::vec8 vec8;
  static_assert(RB == 1 || RB == 2, "a wavefront owns 32 or 64 query rows");
  constexpr int NW = 8 / RB, DC = 8, DB = 4;
  constexpr int WROWS = 32 * RB;  // query rows of a wavefront: RB blocks of 32
  constexpr int IPW = 16 / NW;  // copy instructions per wavefront and K (V) tile
  constexpr int RS = 4 * NW;    // tile rows between two of them
  if (p.bound_flag != nullptr && (*p.bound_flag != 0) != BOUNDED) return;
  if (p.gate != nullptr && !gate_open(p.gate, p.gate_mask)) return;
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  char* const sK = (char*)smem;                    // [2][64][256 B]
  char* const sV = (char*)smem + 2 * TILE_BYTES;   // [2][64][256 B]
  char* const sStage = (char*)smem + 4 * TILE_BYTES;  // [NW wavefronts][WROWS rows][256 B]: finished outputs on their way out
  int* const sTaken = (int*)((char*)smem + 4 * TILE_BYTES + 8 * 8192);  // the tail range that wavefront 0 drew for the workgroup

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int hh = lane >> 5;
  const StreamPlan& sp = p.st;
  // Workgroups are dealt to the 8 XCDs in turn; with G a multiple of 8 each XCD takes a contiguous eighth of the
  // workgroup numbers, so the pieces its 32 workgroups sweep at one time are neighbours (one or two heads, whose
  // K/V tiles then meet in that XCD's L2), and so are its ranges of the tail.
  const int wg = sp.xcd_order ? (int)(blockIdx.x & 7) * (sp.G >> 3) + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
  if (sp.solo && wg != 0) return;
  constexpr uint32_t OOB = PIPE_OOB;
  // What happens once per piece (a new Q, a new K/V descriptor, a finished piece's output) needs many of the
  // kernel's arguments and little else.  Read through `p` the compiler would load them all once, ahead of the
  // loop, and hold them in scalar registers across it (more than there are: they end up parked in vector
  // lanes and fetched back on every iteration).  Those paths therefore read the argument block where it lies,
  // through a pointer the compiler cannot see through, so the loads stay inside the rare branches.
  typedef const __attribute__((address_space(4))) AttnParams* KArgs;
  auto kargs = [&]() __attribute__((always_inline)) {
    KArgs kp = (KArgs)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(kp));
    return kp;
  };

  // ---- per-piece facts ---------------------------------------------------------------------------
  struct Where {
    int batch, head, row_begin, row_end;
  };
  auto where = [&](KArgs kp, int piece) __attribute__((always_inline)) {
    Where w;
    const int nqt = kp->n_qtiles, H = kp->H, Sq = kp->Sq;
    const int bh = piece / nqt;
    const int qt = piece - bh * nqt;
    w.head = bh % H;
    w.batch = bh / H;
    w.row_begin = qt * 256;
    w.row_end = w.row_begin + 256 < Sq ? w.row_begin + 256 : Sq;
    return w;
  };
  // ---- this workgroup's list of key tiles ------------------------------------------------------
  // R whole pieces, then one range of the tail's key-tile steps, which may run over several pieces.  The
  // generator walks items (piece, first tile, end tile) and inside an item the tiles, keeping (segment, tile
  // in segment).
  // The tail's Gt ranges: without a counter, range wg belongs to this workgroup; with one, a workgroup that has run
  // out of tiles draws the number of its next range from it, so the ranges go to whoever asks first (compute units
  // do not all run at one speed: with equal shares the finish times of the workgroups were measured 7 % apart).
  int tail_left = 0;  // key tiles of the current tail range still to hand out
  int g_range = 0;    // the current range
  struct Desc {
    int piece;    // < 0: no such tile
    int flags;    // LAST: the item's last tile; FULL: the item is a whole piece; MID: the item begins inside a piece
    int seg;      // key segment
    uint32_t n0;  // first key inside the segment, or OOB
  };
  constexpr int LAST = 1, FULL = 2, MID = 4;
  int g_round = -1, g_piece = 0, g_j = 0, g_kind = 0, g_jend = 0, g_seg = 0, g_jj = 0;
  bool g_in_tail = false, g_done = false;
  // A variant of its own: in one kernel the paths it adds cost the plain calls 0.3 %.  Inside the variant the test
  // stays a run-time one on purpose: as a compile-time constant the same code came out with spills in the hot loop
  // (17.3 ms against 16.6 ms for the 119k-token call with a text-padding mask).
  const bool has_kvlen = KVLEN && sp.has_kvlen != 0;
  // keys of a piece: its batch element's count where the call gives per-batch key counts, else all of the segment's
  auto key_limit = [&](int piece) __attribute__((always_inline)) {
    const KArgs kp = kargs();
    const int n = kp->kv_len[where(kp, piece).batch], all = kp->st.seg_len;
    return n < 0 ? 0 : n < all ? n : all;
  };
  // An item is a run of key tiles of one piece.  With per-batch key counts it ends where the piece's keys end and
  // may come out empty (g_j >= g_jend): see write_empty.
  auto start_item = [&](int piece, int j0, int jend) __attribute__((always_inline)) {
    g_piece = piece;
    g_kind = (j0 == 0 && jend == sp.L ? FULL : 0) | (j0 > 0 ? MID : 0) | (g_range << 3);
    if (has_kvlen) {
      const int tiles = (key_limit(piece) + BN - 1) / BN;
      jend = jend < tiles ? jend : tiles;
    }
    g_j = j0;
    g_jend = jend;
    g_seg = j0 / sp.tps;
    g_jj = j0 - g_seg * sp.tps;
  };
  // valid keys of a tile (0 for a tile that does not exist)
  auto valid_keys = [&](const Desc& d) __attribute__((always_inline)) {
    if (d.n0 == OOB) return 0;
    const int left = (has_kvlen ? key_limit(d.piece) : sp.seg_len) - (int)d.n0;
    return left < BN ? left : BN;
  };
  // The result of an item without keys, written where finish_item would write it: zeros and an LSE of -inf, as the
  // output of a whole piece or as a partial result (whose row the fold kernel reads whatever it holds).
  auto write_empty = [&]() __attribute__((always_inline)) {
    const KArgs kp = kargs();
    const Where w = where(kp, g_piece);
    int ln = lane;
    asm volatile("" : "+v"(ln));
    const int l32 = ln & 31, hh = ln >> 5;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int my_row = w.row_begin + wave * WROWS + 32 * rb + l32;
      if (my_row >= w.row_end) continue;
      if (g_kind & FULL) {
        uint16_t* op = (uint16_t*)kp->out + w.batch * kp->os_b + w.head * kp->os_h + (int64_t)my_row * kp->os_s + 64 * hh;
        const u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int i = 0; i < 8; ++i) *(u32x4*)(op + 8 * i) = z;
        float* const lse_out = kp->lse;
        if (lse_out != nullptr && hh == 0) lse_out[((int64_t)w.batch * kp->H + w.head) * kp->Sq + my_row] = -INFINITY;
      } else {
        const int64_t wrow = (int64_t)(2 * (g_kind >> 3) + ((g_kind & MID) ? 0 : 1)) * 256 + (my_row - w.row_begin);
        float* wp = kp->ws_out + wrow * 128 + 64 * hh;
        const float4 z = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 16; ++i) *(float4*)(wp + 4 * i) = z;
        if (hh == 0) kp->ws_lse[wrow] = -INFINITY;
      }
    }
  };
  auto advance_item = [&]() __attribute__((always_inline)) -> bool {
    const KArgs kp = kargs();
    const int R = kp->st.R, G = kp->st.G, L = kp->st.L;
    if (g_round + 1 < R) {
      ++g_round;
      start_item(wg + g_round * G, 0, L);
      return true;
    }
    int piece, j0;
    if (tail_left <= 0) {  // the next range
      const int Gt = kp->st.Gt;
      int* const counter = kp->st.next_range;
      int n;
      if (counter != nullptr) {
        // Every wavefront of the workgroup comes by here in the same iteration.  Wavefront 0 draws the number and
        // leaves it in LDS; the second barrier keeps it from writing the next one (an empty range is followed by
        // another draw at once) before every wavefront has read this one.
        if (wave == 0) {
          int v = 0;
          if (lane == 0) v = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          *(volatile int*)sTaken = __builtin_amdgcn_readfirstlane(v);
        }
        __syncthreads();
        n = __builtin_amdgcn_readfirstlane(*(volatile int*)sTaken);
        __syncthreads();
        if (n < 0) return false;
      } else if (!g_in_tail) {
        n = wg;
      } else {
        return false;
      }
      if (n >= Gt) return false;  // no range left
      g_in_tail = true;
      g_range = n;
      const int per_round = Gt / kp->st.n_rounds;
      const int rd = n / per_round, i = n - rd * per_round;
      const int64_t r0 = kp->st.round_at[rd], Tr = kp->st.round_at[rd + 1] - r0;
      const int64_t ta = r0 + (int64_t)i * Tr / per_round;
      tail_left = (int)(r0 + (int64_t)(i + 1) * Tr / per_round - ta);
      if (tail_left <= 0) return false;
      piece = R * G + (int)(ta / L);
      j0 = (int)(ta % L);
    } else {
      piece = g_piece + 1;
      j0 = 0;
    }
    const int n = tail_left < L - j0 ? tail_left : L - j0;
    start_item(piece, j0, j0 + n);
    tail_left -= n;
    return true;
  };
  auto pull = [&](Desc& d) __attribute__((always_inline)) {
    if (!g_done && g_j >= g_jend) {
      g_done = !advance_item();
      if (has_kvlen)
        while (!g_done && g_j >= g_jend) {  // an item beyond its piece's keys
          write_empty();
          g_done = !advance_item();
        }
    }
    if (g_done) {
      d.piece = -1; d.flags = 0; d.seg = 0; d.n0 = OOB;
      return;
    }
    d.piece = g_piece;
    d.flags = (g_j == g_jend - 1 ? LAST : 0) | g_kind;
    d.seg = g_seg;
    d.n0 = (uint32_t)g_jj * BN;
    ++g_j;
    if (++g_jj == sp.tps) {
      g_jj = 0;
      ++g_seg;
    }
  };
  Desc cur, nxt, nx2;
  pull(cur);
  pull(nxt);
  pull(nx2);
  if (cur.piece < 0) return;  // nothing for this workgroup (before any barrier: the whole workgroup leaves)

  vec8 qf[RB][DC];  // B operand of the first GEMM: the Q rows of the piece whose scores are computed next
  auto load_q = [&](int piece) __attribute__((always_inline)) {
    const KArgs kp = kargs();
    const Where w = where(kp, piece);
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      int r = w.row_begin + wave * WROWS + 32 * rb + l32;
      r = r < w.row_end ? r : w.row_end - 1;
      const uint16_t* qp = (const uint16_t*)kp->q + w.batch * kp->qs_b + w.head * kp->qs_h + (int64_t)r * kp->qs_s + 8 * hh;
#pragma unroll
      for (int dc = 0; dc < DC; ++dc) qf[rb][dc] = *(const vec8*)(qp + 16 * dc);
    }
  };

  // ---- global -> LDS copies (as in attn_fwd_d128_pipe_kernel); the descriptor follows the tile's piece and segment
  const uint32_t ks_bytes = (uint32_t)(p.ks_s * 2), vs_bytes = (uint32_t)(p.vs_s * 2);
  auto make_rsrc = [&](bool is_v, int seg, int piece) __attribute__((always_inline)) {
    const KArgs kp = kargs();
    const Where w = where(kp, piece);
    const void* seg_base = is_v ? kp->st.vseg[seg] : kp->st.kseg[seg];
    const int64_t sb = is_v ? kp->vs_b : kp->ks_b, sh = is_v ? kp->vs_h : kp->ks_h;
    const uint32_t row_bytes = (uint32_t)((is_v ? kp->vs_s : kp->ks_s) * 2);
    const uint64_t a = (uint64_t)((const uint16_t*)seg_base + w.batch * sb + w.head * sh);
    const uint64_t nbytes = (uint64_t)(kp->st.seg_len - 1) * row_bytes + 256;  // start of the last row + one row
    u32x4 r;
    r[0] = __builtin_amdgcn_readfirstlane((uint32_t)a);
    r[1] = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32) & 0xffffu);
    r[2] = __builtin_amdgcn_readfirstlane((uint32_t)nbytes);
    r[3] = 0x00020000u;
    return r;
  };
  u32x4 krs = {0, 0, 0, 0x00020000u}, vrs = {0, 0, 0, 0x00020000u};
  int k_piece = -1, k_seg = -1, v_piece = -1, v_seg = -1;
  auto aim_k = [&](const Desc& d) __attribute__((always_inline)) {  // point the K descriptor at the tile's piece and segment
    if (d.piece >= 0 && (d.piece != k_piece || d.seg != k_seg)) {
      krs = make_rsrc(false, d.seg, d.piece);
      k_piece = d.piece;
      k_seg = d.seg;
    }
  };
  auto aim_v = [&](const Desc& d) __attribute__((always_inline)) {
    if (d.piece >= 0 && (d.piece != v_piece || d.seg != v_seg)) {
      vrs = make_rsrc(true, d.seg, d.piece);
      v_piece = d.piece;
      v_seg = d.seg;
    }
  };
  const int dma_row = 4 * wave + (lane >> 4);
  const int dma_pc = lane & 15;
  const uint32_t k_off0 = dma_row * ks_bytes + 16 * (dma_pc ^ (dma_row & 15));
  const uint32_t v_off0 = dma_row * vs_bytes + 16 * (dma_pc ^ (4 * (dma_row & 3)));
  const uint32_t lds_k = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_char*)sK + wave * 1024);
  const uint32_t lds_v = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_char*)sV + wave * 1024);
  // `there`: the tile is known to exist (no test for OOB)
  auto dma_k1 = [&](int buf, uint32_t n0, int i, bool there = false) __attribute__((always_inline)) {
    const uint32_t soff = __builtin_amdgcn_readfirstlane(!there && n0 == OOB ? OOB : (n0 + RS * i) * ks_bytes);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_k + buf * TILE_BYTES + i * (RS * 256)), "v"(k_off0), "s"(krs), "s"(soff) : "memory");
  };
  auto dma_v1 = [&](int buf, uint32_t n0, int i, bool there = false) __attribute__((always_inline)) {
    const uint32_t soff = __builtin_amdgcn_readfirstlane(!there && n0 == OOB ? OOB : (n0 + RS * i) * vs_bytes);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_v + buf * TILE_BYTES + i * (RS * 256)), "v"(v_off0), "s"(vrs), "s"(soff) : "memory");
  };

  // ---- fragment read addresses (as in attn_fwd_d128_pipe_kernel) ------------------------------------
  uint32_t ka[DC];
#pragma unroll
  for (int dc = 0; dc < DC; ++dc) ka[dc] = l32 * 256 + 16 * ((2 * dc + hh) ^ (l32 & 15));
  uint32_t va[DB];
  {
    const int g16 = lane >> 4, lg = lane & 15, r = lg >> 2, cq = lg & 3, dhalf = g16 & 1;
#pragma unroll
    for (int db = 0; db < DB; ++db)
      va[db] = (4 * hh + r) * 256 + 16 * ((4 * db + 2 * dhalf + (cq >> 1)) ^ (4 * r)) + 8 * (cq & 1);
  }
  auto read_k = [&](const char* tile, int t, int dc) __attribute__((always_inline)) -> vec8 {
    return *(const vec8*)(tile + t * 32 * 256 + ka[dc]);
  };
  typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4;
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  auto read_vt = [&](const char* tile, int t, int c, int db) __attribute__((always_inline)) -> vec8 {
    const char* a = tile + (32 * t + 16 * c) * 256 + va[db];
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(a));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(a + 8 * 256));
    typedef __attribute__((__vector_size__(8 * sizeof(short)))) short s16x8;
    s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(vec8, v);
  };

  // ---- accumulators ---------------------------------------------------------------------------
  floatx16 o[RB][DB];
  float m_run[RB], l_run[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[rb][i][r] = 0.f;
    m_run[rb] = BOUNDED ? 0.f : -INFINITY;
    l_run[rb] = 0.f;
  }
  const float c = p.scale_log2;

  auto mask_tail = [&](floatx16& a0, floatx16& a1, int nvalid) __attribute__((always_inline)) {
    const int lim = nvalid - 4 * hh;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      if (8 * (r >> 2) + (r & 3) >= lim) a0[r] = -INFINITY;
      if (8 * (r >> 2) + (r & 3) + 32 >= lim) a1[r] = -INFINITY;
    }
  };
  auto across = [&](float x) __attribute__((always_inline)) {
    auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
  };

  // ---- output of a finished item ---------------------------------------------------------------
  auto finish_item = [&](const Desc& d) __attribute__((always_inline)) {
    const KArgs kp = kargs();
    const Where w = where(kp, d.piece);
    float* const acc_out = kp->acc_out;
    // The addresses below are worked out here, from a lane number the compiler cannot see through.  Derived from
    // `lane` they are loop invariants: two dozen registers held across the hot loop, spilled, and fetched back one
    // by one between the output stores -- and a fetch from scratch memory waits for every store issued before it.
    int ln = lane;
    asm volatile("" : "+v"(ln));
    const int l32 = ln & 31, hh = ln >> 5, lane = ln;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      float l_tot;
      {
        auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(l_run[rb]), __float_as_uint(l_run[rb]), false, false);
        l_tot = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
      }
      const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
      const float lse_nat = l_tot > 0.f ? (m_run[rb] + __builtin_amdgcn_logf(l_tot)) * LN2 : -INFINITY;
      const int my_row = w.row_begin + wave * WROWS + 32 * rb + l32;
      if ((d.flags & FULL) && acc_out == nullptr) {
        // A whole piece's output.  In the accumulator layout a lane holds 8-byte pieces of its row, 16 bytes apart,
        // and a store instruction would touch 64 of them in 32 rows; staged through this wavefront's own 8 KB of
        // LDS (16-byte chunks XOR-swizzled by the row, as the tiles are) the same data leaves as whole 256-byte rows,
        // four per instruction.  Short pieces (cross-attention) store an output every few key tiles, and every
        // store has to be through before the next barrier (one counter covers tile copies and stores).
        char* const st = sStage + wave * (WROWS * 256) + rb * 8192;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int a = 0; a < 4; ++a) {
            u32x2 x;
            x[0] = T::pack2(o[rb][db][4 * a] * inv, o[rb][db][4 * a + 1] * inv);
            x[1] = T::pack2(o[rb][db][4 * a + 2] * inv, o[rb][db][4 * a + 3] * inv);
            *(u32x2*)(st + l32 * 256 + 16 * ((4 * db + a) ^ (l32 & 15)) + 8 * hh) = x;
          }
        uint16_t* const obase = (uint16_t*)kp->out + w.batch * kp->os_b + w.head * kp->os_h;
        const int64_t os_s = kp->os_s;
        const int row0 = w.row_begin + wave * WROWS + 32 * rb;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int r = 4 * i + (lane >> 4), ch = lane & 15;
          const u32x4 x = *(const u32x4*)(st + r * 256 + 16 * (ch ^ (r & 15)));
          if (row0 + r < w.row_end) __builtin_nontemporal_store(x, (u32x4*)(obase + (int64_t)(row0 + r) * os_s + 8 * ch));
        }
        float* const lse_out = kp->lse;
        if (lse_out != nullptr && hh == 0 && my_row < w.row_end)
          lse_out[((int64_t)w.batch * kp->H + w.head) * kp->Sq + my_row] = lse_nat;
      } else if (my_row < w.row_end) {
        if (!(d.flags & FULL)) {  // a share of a piece: normalised fp32 partial + LSE into the workspace
          const int64_t wrow = (int64_t)(2 * (d.flags >> 3) + ((d.flags & MID) ? 0 : 1)) * 256 + (my_row - w.row_begin);
          float* wp = kp->ws_out + wrow * 128;
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int a = 0; a < 4; ++a) {
              float4 x = {o[rb][db][4 * a] * inv, o[rb][db][4 * a + 1] * inv, o[rb][db][4 * a + 2] * inv, o[rb][db][4 * a + 3] * inv};
              *(float4*)(wp + 32 * db + 8 * a + 4 * hh) = x;
            }
          if (hh == 0) kp->ws_lse[wrow] = lse_nat;
        } else if (acc_out != nullptr) {  // fold into the running (out, lse) pair
          const int64_t ridx = ((int64_t)w.batch * kp->H + w.head) * kp->Sq + my_row;
          const int acc_first = kp->acc_first;
          float* const acc_lse = kp->acc_lse;
          const float old = acc_first ? -INFINITY : acc_lse[ridx];
          const float mx2 = fmaxf(old, lse_nat);
          float w_old = 0.f, w_blk = 0.f, lse_new = -INFINITY;
          if (mx2 > -INFINITY) {
            const float e_old = __expf(old - mx2), e_blk = __expf(lse_nat - mx2);
            const float den = e_old + e_blk;
            w_old = e_old / den;
            w_blk = e_blk / den * inv;
            lse_new = mx2 + __logf(den);
          }
          float* ap = acc_out + ridx * 128;
          uint16_t* op = kp->out ? (uint16_t*)kp->out + w.batch * kp->os_b + w.head * kp->os_h + (int64_t)my_row * kp->os_s : nullptr;
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int a = 0; a < 4; ++a) {
              const int d0 = 32 * db + 8 * a + 4 * hh;
              float4 r = {0.f, 0.f, 0.f, 0.f};
              if (!acc_first && w_old > 0.f) r = *(const float4*)(ap + d0);
              r.x = r.x * w_old + o[rb][db][4 * a] * w_blk;
              r.y = r.y * w_old + o[rb][db][4 * a + 1] * w_blk;
              r.z = r.z * w_old + o[rb][db][4 * a + 2] * w_blk;
              r.w = r.w * w_old + o[rb][db][4 * a + 3] * w_blk;
              if (op) {
                u32x2 x;
                x[0] = T::pack2(r.x, r.y);
                x[1] = T::pack2(r.z, r.w);
                *(u32x2*)(op + d0) = x;
              } else {
                *(float4*)(ap + d0) = r;
              }
            }
          if (hh == 0) acc_lse[ridx] = lse_new;
        }
      }
    }
    // the next item starts from nothing
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
      for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[rb][i][r] = 0.f;
      m_run[rb] = BOUNDED ? 0.f : -INFINITY;
      l_run[rb] = 0.f;
    }
  };

  vec8 f[8];          // ring of 8 operand fragments
  // S(j+1) per row block (keys 0..31, 32..63); with 64 rows per wavefront two sets that alternate by the iteration's parity
  floatx16 sbuf[RB][RB][2];
  floatx16 (&sn)[RB][2] = sbuf[0];
  float mx[RB];        // row maximum of S(j), masked, unscaled
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    mx[rb] = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) sn[rb][0][r] = sn[rb][1][r] = 0.f;
  }

  // ---- prologue: Q of the first piece; K0, V0, K1 copies; S(0) and its row maximum -------------------
  load_q(cur.piece);
  aim_k(cur);
  aim_v(cur);
#pragma unroll
  for (int i = 0; i < IPW; ++i) dma_k1(0, cur.n0, i);
#pragma unroll
  for (int i = 0; i < IPW; ++i) dma_v1(0, cur.n0, i);
  aim_k(nxt);
#pragma unroll
  for (int i = 0; i < IPW; ++i) dma_k1(1, nxt.n0, i);
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
#pragma unroll
  for (int dc = 0; dc < DC; ++dc) f[dc] = read_k(sK, 0, dc);
#pragma unroll
  for (int dc = 0; dc < DC; ++dc) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) sn[rb][0] = T::mfma32(f[dc], qf[rb][dc], sn[rb][0]);
    f[dc] = read_k(sK, 1, dc);
  }
#pragma unroll
  for (int dc = 0; dc < DC; ++dc)
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) sn[rb][1] = T::mfma32(f[dc], qf[rb][dc], sn[rb][1]);
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int nv0 = valid_keys(cur);
    if (nv0 < BN) mask_tail(sn[rb][0], sn[rb][1], nv0);
    if constexpr (!BOUNDED) {
      float m2 = fmaxf(sn[rb][0][0], sn[rb][1][0]);
#pragma unroll
      for (int r = 1; r < 16; ++r) m2 = fmaxf(fmaxf(m2, sn[rb][0][r]), sn[rb][1][r]);
      mx[rb] = across(m2);
    }
  }
  // the scores of the second tile already belong to another piece: its Q replaces the first piece's
  if (nxt.piece >= 0 && nxt.piece != cur.piece) load_q(nxt.piece);

  // One iteration; PAR = buffer of tile j (K(j+1) sits in the other K buffer).  INSIDE: tiles j .. j+3 are
  // whole tiles of one item and one segment, none of them the item's last: nothing but the tile itself happens,
  // and the window moves on by 64 keys.
  auto tile_step = [&](auto PAR, auto INSIDE) __attribute__((always_inline)) {
    constexpr int par = decltype(PAR)::value;
    constexpr bool inside = decltype(INSIDE)::value;
    const char* tV = sV + par * TILE_BYTES;
    const char* tKn = sK + (par ^ 1) * TILE_BYTES;
    if constexpr (RB == 1) {
        floatx16 c0 = sn[0][0], c1 = sn[0][1];  // S(j)

      // everything fetched so far has landed (tile copies, a new piece's Q, a finished piece's stores);
      // after the barrier nobody still reads what comes next
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();

#pragma unroll
      for (int dc = 0; dc < DC; ++dc) f[dc] = read_k(tKn, dc & 1, dc >> 1);

      if constexpr (!BOUNDED) {
        const float mx_s = mx[0] * c;
        if (__any(mx_s > m_run[0] + RESCALE_SLACK)) {
          const float m_new = fmaxf(m_run[0], mx_s);
          const float alpha = __builtin_amdgcn_exp2f(m_run[0] - m_new);
          l_run[0] *= alpha;
#pragma unroll
          for (int i = 0; i < DB; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[0][i][r] *= alpha;
          m_run[0] = m_new;
        }
      }
      __builtin_amdgcn_sched_barrier(0);

      // ---- stage A: S(j+1) = K(j+1) Q^T, the copies of K(j+2) and V(j+1), the softmax of S(j) -------
      uint32_t pk0[8], pk1[8];
      float lsum = 0.f;
      float tf[2][2], te[2][2];
      auto expo_slot = [&](int n) __attribute__((always_inline)) {
        if (n >= 2 && n < 18) {
          const int j = n - 2;
          lsum += te[j & 1][0] + te[j & 1][1];
          asm volatile("" : "+v"(lsum));  // the addition stays in its slot (left alone it sinks behind the last MFMA: -1.6 %)
          (j < 8 ? pk0 : pk1)[j & 7] = T::pack2(te[j & 1][0], te[j & 1][1]);
        }
        if (n >= 1 && n < 17) {
          const int j = n - 1;
          te[j & 1][0] = __builtin_amdgcn_exp2f(tf[j & 1][0]);
          te[j & 1][1] = __builtin_amdgcn_exp2f(tf[j & 1][1]);
        }
        if (n < 16) {
          const floatx16& cs = n < 8 ? c0 : c1;
          tf[n & 1][0] = __builtin_fmaf(cs[2 * (n & 7)], c, -m_run[0]);
          tf[n & 1][1] = __builtin_fmaf(cs[2 * (n & 7) + 1], c, -m_run[0]);
        }
      };
#pragma unroll
      for (int r = 0; r < 16; ++r) sn[0][0][r] = sn[0][1][r] = 0.f;
#pragma unroll
      for (int g = 0; g < 8; ++g) {
        if (g & 1) sn[0][1] = T::mfma32(f[g], qf[0][g >> 1], sn[0][1]);
        else sn[0][0] = T::mfma32(f[g], qf[0][g >> 1], sn[0][0]);
        if (g < IPW) dma_k1(par, nx2.n0, g, inside);
        else if (g < 2 * IPW) dma_v1(par ^ 1, nxt.n0, g - IPW, inside);
        f[g] = read_k(tKn, g & 1, 4 + (g >> 1));
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int g = 0; g < 8; ++g) {
        if (g & 1) sn[0][1] = T::mfma32(f[g], qf[0][4 + (g >> 1)], sn[0][1]);
        else sn[0][0] = T::mfma32(f[g], qf[0][4 + (g >> 1)], sn[0][0]);
        f[g] = read_vt(tV, 0, g >> 2, g & 3);
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (!inside) {
        const int nv1 = valid_keys(nxt);
        if (nv1 < BN) mask_tail(sn[0][0], sn[0][1], nv1);  // ragged or absent tile j+1
        // Q of the piece after next takes over the registers, if tile j+2 opens another piece than tile j+1
        if (nx2.piece >= 0 && nx2.piece != nxt.piece) load_q(nx2.piece);
      }
      __builtin_amdgcn_sched_barrier(0);
      // The softmax of S(j) begins here, not under the MFMAs of stage A: VALU work between the MFMAs of the first
      // GEMM costs more than it hides (measured: -3.5 %): the first six slots, which the first PV MFMA needs, in front
      // of it, then one slot under each of the next twelve PV MFMAs.
#pragma unroll
      for (int n = 0; n < 6; ++n) expo_slot(n);
      __builtin_amdgcn_sched_barrier(0);

      // ---- stage B: O^T += V(j)^T P(j)^T, the rest of the softmax, the row maximum of S(j+1) ----------
      float mxa = fmaxf(sn[0][0][0], sn[0][0][1]), mxb = fmaxf(sn[0][1][0], sn[0][1][1]);
#pragma unroll
      for (int cc = 0; cc < 2; ++cc) {
        u32x4 bw = {pk0[4 * cc], pk0[4 * cc + 1], pk0[4 * cc + 2], pk0[4 * cc + 3]};
        vec8 bfrag = __builtin_bit_cast(vec8, bw);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const int g = cc * 4 + db;
          o[0][db] = T::mfma32(f[g], bfrag, o[0][db]);
          f[g] = read_vt(tV, 1, cc, db);
          expo_slot(6 + g);
          if constexpr (!BOUNDED) {
            if (g < 4) {
            } else if (g < 7) mxa = fmaxf(fmaxf(fmaxf(fmaxf(mxa, sn[0][0][4 * g - 14]), sn[0][0][4 * g - 13]), sn[0][0][4 * g - 12]), sn[0][0][4 * g - 11]);
            else mxa = fmaxf(fmaxf(mxa, sn[0][0][14]), sn[0][0][15]);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
#pragma unroll
      for (int cc = 0; cc < 2; ++cc) {
        u32x4 bw = {pk1[4 * cc], pk1[4 * cc + 1], pk1[4 * cc + 2], pk1[4 * cc + 3]};
        vec8 bfrag = __builtin_bit_cast(vec8, bw);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const int g = cc * 4 + db;
          o[0][db] = T::mfma32(f[g], bfrag, o[0][db]);
          if (g < 4) expo_slot(14 + g);
          if constexpr (!BOUNDED) {
            if (g > 0) mxb = fmaxf(fmaxf(mxb, sn[0][1][2 * g]), sn[0][1][2 * g + 1]);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      l_run[0] += lsum;
      if constexpr (!BOUNDED) mx[0] = across(fmaxf(mxa, mxb));

    } else {
      // ---- 64 query rows per wavefront, one wavefront per SIMD ------------------------------------------
      // Every K and V^T fragment read from LDS feeds two MFMAs (one per row block), so the workgroup reads half
      // the LDS bytes per flop of the 32-row form.  No second wavefront shares the SIMD: the softmax of S(j) has
      // to run under this wavefront's own MFMAs, a few instructions behind each of them (an MFMA leaves about 20
      // of its 32 clocks to other vector instructions of the same wavefront), spread evenly over both GEMMs, each
      // group of 16 probabilities finished just before the PV MFMAs that take it.  The score tiles live in
      // accumulation registers; two sets alternate by the iteration's parity, S(j) is read from one pair by pair
      // where the softmax takes it while S(j+1) gathers in the other, and no copy of a whole tile is made.
      floatx16 (&cs)[RB][2] = sbuf[par];      // S(j)
      floatx16 (&sn)[RB][2] = sbuf[par ^ 1];  // S(j+1)

      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();

#pragma unroll
      for (int dc = 0; dc < DC; ++dc) f[dc] = read_k(tKn, dc & 1, dc >> 1);

      if constexpr (!BOUNDED) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          const float mx_s = mx[rb] * c;
          if (__any(mx_s > m_run[rb] + RESCALE_SLACK)) {
            const float m_new = fmaxf(m_run[rb], mx_s);
            const float alpha = __builtin_amdgcn_exp2f(m_run[rb] - m_new);
            l_run[rb] *= alpha;
#pragma unroll
            for (int i = 0; i < DB; ++i)
#pragma unroll
              for (int r = 0; r < 16; ++r) o[rb][i][r] *= alpha;
            m_run[rb] = m_new;
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);

      // Softmax of S(j) in 32 pairs of scores, in the order the second GEMM takes them: pair n belongs to the
      // 16-key chunk n / 8 (key half t = n / 16, chunk cc of it), row block (n / 4) % 2, registers 8 cc + 2 (n % 4).
      // A pair passes three steps -- scale (A), exponentials (B), sum + pack (C), the first two one score at a time
      // -- and the steps of consecutive pairs interleave as C(n-2), B(n-1), A(n); that sequence of 160 small steps
      // is dealt out to the gaps behind the iteration's MFMAs by its running cost in clocks, so every gap holds
      // about the same amount of it.
      uint32_t pk[RB][2][8];
      float lsum[RB];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) lsum[rb] = 0.f;
      float tf[2][2], te[2][2];
      auto step_a = [&](int n, int x) __attribute__((always_inline)) {
        const int rb = (n >> 2) & 1, k = n >> 3;
        const floatx16& src = cs[rb][k >> 1];
        const int r0 = 8 * (k & 1) + 2 * (n & 3);
        tf[n & 1][x] = __builtin_fmaf(src[r0 + x], c, -m_run[rb]);
      };
      auto step_b = [&](int n, int x) __attribute__((always_inline)) {
        te[n & 1][x] = __builtin_amdgcn_exp2f(tf[n & 1][x]);
      };
      auto step_c = [&](int n) __attribute__((always_inline)) {
        const int rb = (n >> 2) & 1, k = n >> 3;
        lsum[rb] += te[n & 1][0] + te[n & 1][1];
        asm volatile("" : "+v"(lsum[rb]));
        pk[rb][k >> 1][4 * (k & 1) + (n & 3)] = T::pack2(te[n & 1][0], te[n & 1][1]);
      };
      // small steps i = 0..169: slot i / 5 holds C(slot - 2), B(slot - 1) twice, A(slot) twice; their clocks: 12, 8, 8,
      // 12, 12 (A: a read of an accumulation register and a multiplication) -- 52 per pair, 1664 in all, dealt to
      // gaps 0..59 by the middle of each step's span (Rb2Steps, worked out at compile time)
      auto run_steps = [&](int q) __attribute__((always_inline)) {
#pragma unroll
        for (int i = RB2_STEPS.lo[q]; i < RB2_STEPS.hi[q]; ++i) {
          if (RB2_STEPS.gap[i] == q) {
            const int kind = i % 5, n = Rb2Steps::pair(i);
            if (kind == 0) step_c(n);
            else if (kind < 3) step_b(n, kind - 1);
            else step_a(n, kind - 3);
          }
        }
      };

      // ---- S(j+1) = K(j+1) Q^T: 32 MFMAs; the copies of K(j+2) and V(j+1) behind the first eight -------
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int r = 0; r < 16; ++r) sn[rb][0][r] = sn[rb][1][r] = 0.f;
#pragma unroll
      for (int g = 0; g < 8; ++g) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          const int q = 2 * g + rb;
          sn[rb][g & 1] = T::mfma32(f[g], qf[rb][g >> 1], sn[rb][g & 1]);
          if (q < IPW) dma_k1(par, nx2.n0, q, inside);
          else if (q < 2 * IPW) dma_v1(par ^ 1, nxt.n0, q - IPW, inside);
          if (rb == RB - 1) f[g] = read_k(tKn, g & 1, 4 + (g >> 1));
          run_steps(q);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
#pragma unroll
      for (int g = 0; g < 8; ++g) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          const int q = 16 + 2 * g + rb;
          sn[rb][g & 1] = T::mfma32(f[g], qf[rb][4 + (g >> 1)], sn[rb][g & 1]);
          if (rb == RB - 1) f[g] = read_vt(tV, 0, g >> 2, g & 3);
          run_steps(q);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      if constexpr (!inside) {
        const int nv1 = valid_keys(nxt);
        if (nv1 < BN) {  // ragged or absent tile j+1
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) mask_tail(sn[rb][0], sn[rb][1], nv1);
        }
        // Q of the piece after next takes over the registers, if tile j+2 opens another piece than tile j+1
        if (nx2.piece >= 0 && nx2.piece != nxt.piece) load_q(nx2.piece);
      }
      __builtin_amdgcn_sched_barrier(0);

      // ---- O^T += V(j)^T P(j)^T: 32 MFMAs, chunk by chunk of 16 keys, row block 0 then 1 with the same fragments;
      // the rest of the softmax, and the row maxima of S(j+1) ----------------------------------------
      float mxv[RB];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) mxv[rb] = -INFINITY;
#pragma unroll
      for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) {
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) {
            u32x4 bw = {pk[rb][t][4 * cc], pk[rb][t][4 * cc + 1], pk[rb][t][4 * cc + 2], pk[rb][t][4 * cc + 3]};
            vec8 bfrag = __builtin_bit_cast(vec8, bw);
#pragma unroll
            for (int db = 0; db < DB; ++db) {
              const int u = 8 * (2 * t + cc) + 4 * rb + db;  // MFMA 32 + u of the iteration
              const int g = cc * 4 + db;
              o[rb][db] = T::mfma32(f[g], bfrag, o[rb][db]);
              if (t == 0 && rb == RB - 1) f[g] = read_vt(tV, 1, cc, db);
              run_steps(32 + u);
              if constexpr (!BOUNDED) {
                const floatx16& sx = sn[u >> 4][(u >> 3) & 1];
                const int i = u & 7;
                mxv[u >> 4] = fmaxf(fmaxf(mxv[u >> 4], sx[2 * i]), sx[2 * i + 1]);
              }
              __builtin_amdgcn_sched_barrier(0);
            }
          }
        }
      }
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        l_run[rb] += lsum[rb];
        if constexpr (!BOUNDED) mx[rb] = across(mxv[rb]);
      }
    }

    if constexpr (inside) {
      cur.n0 = nxt.n0;
      nxt.n0 = nx2.n0;
      nx2.n0 += BN;
    } else {
      if (cur.flags & LAST) finish_item(cur);

      // slide the tile window and point the descriptors at what the next iteration copies (this iteration's
      // copies are all issued); done here, under the last MFMAs, and not behind the next barrier, where every
      // wavefront of the workgroup would wait for it
      cur = nxt;
      nxt = nx2;
      pull(nx2);
      aim_k(nx2);
      aim_v(nxt);
    }
  };
  // How many of the coming iterations are INSIDE ones: the window lies in one piece and segment (so tile j is not
  // an item's last, tile j+1 is whole, no Q or descriptor changes), and the tiles the generator hands out next
  // stay in that item and segment without being the last of either (their descriptors differ from tile j+2's in
  // the first key only).
  auto inside_run = [&]() __attribute__((always_inline)) {
    if (nx2.piece < 0 || cur.piece != nx2.piece || cur.seg != nx2.seg || g_jj == 0) return 0;
    // (two items in a row can belong to one piece: a workgroup that draws the range after its own)
    if ((cur.flags | nxt.flags) & LAST) return 0;
    const int a = g_jend - 1 - g_j, b = sp.tps - 1 - g_jj;
    const int n = a < b ? a : b;
    return n > 0 ? n : 0;
  };

  aim_k(nx2);
  aim_v(nxt);
  constexpr std::integral_constant<int, 0> even{};
  constexpr std::integral_constant<int, 1> odd{};
  while (cur.piece >= 0) {
    int pairs = inside_run() >> 1;
    if (pairs > 0) {
      g_j += 2 * pairs;  // the generator hands these tiles out in one go
      g_jj += 2 * pairs;
      do {
        tile_step(even, std::true_type{});
        tile_step(odd, std::true_type{});
      } while (--pairs > 0);
    }
    tile_step(even, std::false_type{});
    if (cur.piece < 0) break;
    tile_step(odd, std::false_type{});
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // no tile copy may still be on its way to LDS when the wavefront ends
}

// ---------------------------------------------------------------------------------------------
// head_dim 128, 449..512 keys per (batch, head): cross-attention of many query rows to a short text.
// A piece (256 query rows of one head) lives for eight key tiles only, so what happens once per piece -- its Q
// rows coming in, its output going out -- decides the speed; attn_fwd_d128_stream_kernel pays for both in every
// wavefront at the same time, in front of a workgroup barrier.  Here the key tiles of a head go round in a
// circle (step s copies tile s mod 8; softmax does not care where in the circle a row begins), and the two
// wavefronts of a SIMD are half a circle apart: wavefronts 0..3 begin their pieces at tile 0, wavefronts 4..7
// at tile 4, so while one of a SIMD's two wavefronts changes pieces the other is in mid-piece and keeps the
// matrix cores busy.  The half that is in mid-piece also issues all the tile copies; the half that changes
// pieces issues none for four steps and therefore never waits at a barrier for its own loads and stores (one
// counter covers tile copies, Q loads and output stores): its next Q rows travel into the wavefront's own 8 KB
// of LDS a step before they are needed, and its output leaves through the same 8 KB in two parts, each behind
// the last MFMA of a step.  The wavefront that changes pieces has priority over the other one of its SIMD.
// Workgroup g takes the pieces [g P / G, (g + 1) P / G); consecutive pieces of one head form a run of
// 8 n + 4 steps (wavefronts 4..7 idle for the first four, 0..3 for the last four).
// Dense, not causal, no per-batch key counts, no accumulation.
// ---------------------------------------------------------------------------------------------
constexpr int SHORT_NT = 8;  // key tiles of a piece
constexpr int SHORT_QI = 5;  // step of a piece (0..7) in which the next piece's Q rows are sent for

template <typename T>
__global__ __launch_bounds__(512, 1) void attn_fwd_d128_short_kernel(const AttnParams p) {
  typedef typename T::vec8 vec8;
  constexpr int DC = 8, DB = 4, NT = SHORT_NT, QI = SHORT_QI;
  if (p.gate != nullptr && !gate_open(p.gate, p.gate_mask)) return;
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  char* const sK = (char*)smem;                   // [2][64][256 B]
  char* const sV = (char*)smem + 2 * TILE_BYTES;  // [2][64][256 B]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  char* const sMine = (char*)smem + 4 * TILE_BYTES + wave * 8192;  // [32 rows][256 B]: Q on its way in, output on its way out
  const int l32 = lane & 31;
  const int hh = lane >> 5;
  const int phase = wave >> 2;  // 0: pieces begin at tile 0; 1: at tile 4
  const int cw = wave & 3;      // this wavefront's share of a tile copy
  const int G = p.st.G, P = p.st.n_pieces;
  const int wg = p.st.xcd_order ? (int)(blockIdx.x & 7) * (G >> 3) + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
  int piece0 = (int)((int64_t)wg * P / G);
  const int piece_end = (int)((int64_t)(wg + 1) * P / G);
  if (piece0 >= piece_end) return;  // before any barrier: the whole workgroup leaves

  auto lds_barrier = [&]() __attribute__((always_inline)) {  // orders LDS traffic only: loads and stores to memory stay in flight
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
  };
  auto wait_vm = [&]() __attribute__((always_inline)) { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };

  // ---- global -> LDS copies: 4 wavefronts move a tile, 4 instructions each -----------------------
  const uint32_t ks_bytes = (uint32_t)(p.ks_s * 2), vs_bytes = (uint32_t)(p.vs_s * 2), qs_bytes = (uint32_t)(p.qs_s * 2);
  auto make_rsrc = [&](const void* base, uint64_t nbytes) __attribute__((always_inline)) {
    const uint64_t a = (uint64_t)base;
    u32x4 r;
    r[0] = __builtin_amdgcn_readfirstlane((uint32_t)a);
    r[1] = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32) & 0xffffu);
    r[2] = __builtin_amdgcn_readfirstlane((uint32_t)nbytes);
    r[3] = 0x00020000u;
    return r;
  };
  u32x4 krs = {0, 0, 0, 0x00020000u}, vrs = krs, qrs = krs, ors = krs;
  const uint32_t os_bytes = (uint32_t)(p.os_s * 2);
  const int dma_row = 4 * cw + (lane >> 4);
  const int dma_pc = lane & 15;
  const uint32_t k_off0 = dma_row * ks_bytes + 16 * (dma_pc ^ (dma_row & 15));
  const uint32_t v_off0 = dma_row * vs_bytes + 16 * (dma_pc ^ (4 * (dma_row & 3)));
  const uint32_t lds_k = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_char*)sK + cw * 1024);
  const uint32_t lds_v = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_char*)sV + cw * 1024);
  const uint32_t lds_mine = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_char*)sMine);
  // instruction i of 4: rows 16 i + 4 cw .. + 3 of tile `tile` of the head
  auto dma_k1 = [&](int buf, int tile, int i) __attribute__((always_inline)) {
    const uint32_t soff = __builtin_amdgcn_readfirstlane((uint32_t)(tile * BN + 16 * i) * ks_bytes);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_k + buf * TILE_BYTES + i * 4096), "v"(k_off0), "s"(krs), "s"(soff) : "memory");
  };
  auto dma_v1 = [&](int buf, int tile, int i) __attribute__((always_inline)) {
    const uint32_t soff = __builtin_amdgcn_readfirstlane((uint32_t)(tile * BN + 16 * i) * vs_bytes);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_v + buf * TILE_BYTES + i * 4096), "v"(v_off0), "s"(vrs), "s"(soff) : "memory");
  };
  // this wavefront's 32 query rows from row0 on -> its own 8 KB, 16-byte chunks XOR-swizzled by the row as in a K tile
  // (rows past the last query row of the head lie outside the descriptor and arrive as zeros)
  auto dma_q = [&](int row0) __attribute__((always_inline)) {
    const uint32_t soff = __builtin_amdgcn_readfirstlane((uint32_t)row0 * qs_bytes);
    int lane = tid & 63;  // the eight offsets are worked out here, not held across the loop
    asm volatile("" : "+v"(lane));
    const int dma_pc = lane & 15;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int rr = 4 * i + (lane >> 4);
      const uint32_t voff = rr * qs_bytes + 16 * (dma_pc ^ (rr & 15));
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                   :: "s"(lds_mine + i * 1024), "v"(voff), "s"(qrs), "s"(soff) : "memory");
    }
  };

  // ---- fragment read addresses (as in attn_fwd_d128_pipe_kernel) ------------------------------------
  uint32_t ka[DC];
#pragma unroll
  for (int dc = 0; dc < DC; ++dc) ka[dc] = l32 * 256 + 16 * ((2 * dc + hh) ^ (l32 & 15));
  uint32_t va[DB];
  {
    const int g16 = lane >> 4, lg = lane & 15, r = lg >> 2, cq = lg & 3, dhalf = g16 & 1;
#pragma unroll
    for (int db = 0; db < DB; ++db)
      va[db] = (4 * hh + r) * 256 + 16 * ((4 * db + 2 * dhalf + (cq >> 1)) ^ (4 * r)) + 8 * (cq & 1);
  }
  auto read_k = [&](const char* tile, int t, int dc) __attribute__((always_inline)) -> vec8 {
    return *(const vec8*)(tile + t * 32 * 256 + ka[dc]);
  };
  typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4;
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  auto read_vt = [&](const char* tile, int t, int c, int db) __attribute__((always_inline)) -> vec8 {
    const char* a = tile + (32 * t + 16 * c) * 256 + va[db];
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(a));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(a + 8 * 256));
    typedef __attribute__((__vector_size__(8 * sizeof(short)))) short s16x8;
    s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(vec8, v);
  };

  vec8 qf[DC];  // B operand of the first GEMM
#pragma unroll
  for (int dc = 0; dc < DC; ++dc) qf[dc] = __builtin_bit_cast(vec8, (u32x4){0u, 0u, 0u, 0u});
  auto read_q = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) qf[dc] = *(const vec8*)(sMine + ka[dc]);
  };

  floatx16 o[DB];
  float m_run = -INFINITY, l_run = 0.f;
  auto reset_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[i][r] = 0.f;
    m_run = -INFINITY;
    l_run = 0.f;
  };
  const float c = p.scale_log2;
  const int nv_last = p.Skv - (NT - 1) * BN;  // keys of tile 7: 1..64
  const bool ragged = nv_last < BN;

  auto mask_tail = [&](floatx16& a0, floatx16& a1, int nvalid) __attribute__((always_inline)) {
    const int lim = nvalid - 4 * hh;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      if (8 * (r >> 2) + (r & 3) >= lim) a0[r] = -INFINITY;
      if (8 * (r >> 2) + (r & 3) + 32 >= lim) a1[r] = -INFINITY;
    }
  };
  auto across = [&](float x) __attribute__((always_inline)) {
    auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
  };

  vec8 f[8];          // ring of 8 operand fragments
  floatx16 sn0, sn1;  // S(s+1): keys 0..31, 32..63 of the tile
  float mx = 0.f;     // row maximum of S(s), masked, unscaled

  while (piece0 < piece_end) {
    // ---- a run of n consecutive pieces of one (batch, head) -----------------------------------------
    const int nqt = p.n_qtiles;
    const int bh = piece0 / nqt, qt0 = piece0 - bh * nqt;
    const int n = piece_end - piece0 < nqt - qt0 ? piece_end - piece0 : nqt - qt0;
    const int batch = bh / p.H, head = bh - batch * p.H;
    const int steps = NT * n + NT / 2;
    krs = make_rsrc((const uint16_t*)p.k + batch * p.ks_b + head * p.ks_h, (uint64_t)(p.Skv - 1) * ks_bytes + 256);
    vrs = make_rsrc((const uint16_t*)p.v + batch * p.vs_b + head * p.vs_h, (uint64_t)(p.Skv - 1) * vs_bytes + 256);
    qrs = make_rsrc((const uint16_t*)p.q + batch * p.qs_b + head * p.qs_h, (uint64_t)(p.Sq - 1) * qs_bytes + 256);
    ors = make_rsrc((const uint16_t*)p.out + batch * p.os_b + head * p.os_h, (uint64_t)(p.Sq - 1) * os_bytes + 256);
    auto row_of = [&](int k) __attribute__((always_inline)) { return (qt0 + k) * 256 + 32 * wave; };  // this wavefront's first row of piece k of the run

    // A finished piece leaves in two parts, each at the end of a step, where the wavefront that changes pieces (it has
    // priority over the other wavefront of its SIMD from step QI of a piece to step 0 of the next) would otherwise
    // wait at the barrier: behind the piece's last step the accumulators are scaled, packed and staged in the
    // wavefront's 8 KB, so that the data can leave as whole 256-byte rows, four per instruction; behind the next
    // piece's first step the rows are stored.  Addresses come from a lane number the compiler cannot see through
    // (see finish_item of attn_fwd_d128_stream_kernel).
    float lse_kept = 0.f;
    auto finish_stage = [&]() __attribute__((always_inline)) {
      int ln = lane;
      asm volatile("" : "+v"(ln));
      const int l32 = ln & 31, hh = ln >> 5;
      float l_tot;
      {
        auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(l_run), __float_as_uint(l_run), false, false);
        l_tot = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
      }
      const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
      lse_kept = l_tot > 0.f ? (m_run + __builtin_amdgcn_logf(l_tot)) * LN2 : -INFINITY;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          u32x2 x;
          x[0] = T::pack2(o[db][4 * a] * inv, o[db][4 * a + 1] * inv);
          x[1] = T::pack2(o[db][4 * a + 2] * inv, o[db][4 * a + 3] * inv);
          *(u32x2*)(sMine + l32 * 256 + 16 * ((4 * db + a) ^ (l32 & 15)) + 8 * hh) = x;
        }
    };
    auto finish_store = [&](int k) __attribute__((always_inline)) {
      int ln = lane;
      asm volatile("" : "+v"(ln));
      const int l32 = ln & 31, hh = ln >> 5;
      const int row0 = row_of(k);
      // eight stores of four rows each through the output's descriptor: a row past the head's last query row lies
      // outside it and is dropped, so the sequence needs no branch.  Non-temporal: nothing here reads the output
      // again, and the launch runs at the chip's power limit, where the hint is worth 2.5 % of the time.
      const int lr = ln >> 4, ch = ln & 15;
      u32x4 x[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] = *(const u32x4*)(sMine + (4 * i + lr) * 256 + 16 * (ch ^ ((4 * i + lr) & 15)));
      const uint32_t voff = lr * os_bytes + 16 * ch;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t soff = __builtin_amdgcn_readfirstlane((uint32_t)(row0 + 4 * i) * os_bytes);
        asm volatile("buffer_store_dwordx4 %0, %1, %2, %3 offen nt" :: "v"(x[i]), "v"(voff), "s"(ors), "s"(soff) : "memory");
      }
      float* const lse_out = p.lse;
      if (lse_out != nullptr && hh == 0 && row0 + l32 < p.Sq)
        lse_out[((int64_t)batch * p.H + head) * p.Sq + row0 + l32] = lse_kept;
    };

    // ---- start of the run: wavefronts 4..7 (idle for four steps) copy K(0), V(0), K(1); 0..3 fetch their Q --------
    wait_vm();
    lds_barrier();  // nobody still reads the tiles of the run before
    if (phase == 1) {
#pragma unroll
      for (int i = 0; i < 4; ++i) dma_k1(0, 0, i);
#pragma unroll
      for (int i = 0; i < 4; ++i) dma_v1(0, 0, i);
#pragma unroll
      for (int i = 0; i < 4; ++i) dma_k1(1, 1, i);
    } else {
      dma_q(row_of(0));
    }
    wait_vm();
    lds_barrier();
    if (phase == 0) read_q();
#pragma unroll
    for (int r = 0; r < 16; ++r) sn0[r] = sn1[r] = 0.f;
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) f[dc] = read_k(sK, 0, dc);
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) {
      sn0 = T::mfma32(f[dc], qf[dc], sn0);
      f[dc] = read_k(sK, 1, dc);
    }
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) sn1 = T::mfma32(f[dc], qf[dc], sn1);
    {
      float m2 = fmaxf(sn0[0], sn1[0]);
#pragma unroll
      for (int r = 1; r < 16; ++r) m2 = fmaxf(fmaxf(m2, sn0[r]), sn1[r]);
      mx = across(m2);
    }
    reset_acc();

    // One step; PAR = s & 1 = buffer of tile s (K(s+1) sits in the other K buffer).
    auto step = [&](auto PAR, int s) __attribute__((always_inline)) {
      constexpr int par = decltype(PAR)::value;
      const char* tV = sV + par * TILE_BYTES;
      const char* tKn = sK + (par ^ 1) * TILE_BYTES;
      const int rel = s - (NT / 2) * phase;
      const int r = rel & (NT - 1);   // step of this wavefront's piece
      const int k = rel >> 3;         // its piece of the run (-1: not yet; n: no more)
      const bool copier = ((r - QI) & 7) >= 4;
      const bool was_copier = ((r - 1 - QI) & 7) >= 4;

      if (was_copier) wait_vm();  // the tile copies this wavefront issued in the step before have landed
      lds_barrier();
      // Of a SIMD's two wavefronts the older one (0..3) wins every arbitration and reaches the next barrier about a
      // thousand clocks before the other.  The one that changes pieces in this step or the next has more to do, so
      // it is given that lead.
      if (r == QI) __builtin_amdgcn_s_setprio(2);
      if (r == 1) __builtin_amdgcn_s_setprio(0);

      const bool copy_k = copier && s + 2 < steps, copy_v = copier && s + 1 < steps;
      const int tile_k = (s + 2) & (NT - 1), tile_v = (s + 1) & (NT - 1);
      if (rel < -1 || rel >= NT * n) {
        // No piece of this wavefront is in reach (the first steps of a run for wavefronts 4..7, the last ones for
        // 0..3): only its share of the tile copies, and what the ends of its first and last piece need.
        if (copy_k) {
#pragma unroll
          for (int i = 0; i < 4; ++i) dma_k1(par, tile_k, i);
        }
        if (copy_v) {
#pragma unroll
          for (int i = 0; i < 4; ++i) dma_v1(par ^ 1, tile_v, i);
        }
        if (r == QI && k + 1 < n) dma_q(row_of(k + 1));
        if (r == NT - 2 && k + 1 < n) {
          wait_vm();
          read_q();
        }
        if (r == 0 && k >= 1 && k <= n) finish_store(k - 1);
        return;
      }

      floatx16 c0 = sn0, c1 = sn1;  // S(s)
#pragma unroll
      for (int dc = 0; dc < DC; ++dc) f[dc] = read_k(tKn, dc & 1, dc >> 1);

      {
        const float mx_s = mx * c;
        if (r == 0) {
          m_run = mx_s;  // a piece's first tile: the accumulators hold nothing yet, so there is nothing to rescale
        } else if (__any(mx_s > m_run + RESCALE_SLACK)) {
          const float m_new = fmaxf(m_run, mx_s);
          const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
          l_run *= alpha;
#pragma unroll
          for (int i = 0; i < DB; ++i)
#pragma unroll
            for (int r2 = 0; r2 < 16; ++r2) o[i][r2] *= alpha;
          m_run = m_new;
        }
      }
      __builtin_amdgcn_sched_barrier(0);

      // ---- stage A: S(s+1) = K(s+1) Q^T, the copies of K(s+2) and V(s+1) --------------------------
      uint32_t pk0[8], pk1[8];
      float lsum = 0.f;
      float tf[2][2], te[2][2];
      auto expo_slot = [&](int nn) __attribute__((always_inline)) {
        if (nn >= 2 && nn < 18) {
          const int j = nn - 2;
          lsum += te[j & 1][0] + te[j & 1][1];
          asm volatile("" : "+v"(lsum));
          (j < 8 ? pk0 : pk1)[j & 7] = T::pack2(te[j & 1][0], te[j & 1][1]);
        }
        if (nn >= 1 && nn < 17) {
          const int j = nn - 1;
          te[j & 1][0] = __builtin_amdgcn_exp2f(tf[j & 1][0]);
          te[j & 1][1] = __builtin_amdgcn_exp2f(tf[j & 1][1]);
        }
        if (nn < 16) {
          const floatx16& cs = nn < 8 ? c0 : c1;
          tf[nn & 1][0] = __builtin_fmaf(cs[2 * (nn & 7)], c, -m_run);
          tf[nn & 1][1] = __builtin_fmaf(cs[2 * (nn & 7) + 1], c, -m_run);
        }
      };
#pragma unroll
      for (int r2 = 0; r2 < 16; ++r2) sn0[r2] = sn1[r2] = 0.f;
#pragma unroll
      for (int g = 0; g < 8; ++g) {
        if (g & 1) sn1 = T::mfma32(f[g], qf[g >> 1], sn1);
        else sn0 = T::mfma32(f[g], qf[g >> 1], sn0);
        if (g < 4) {
          if (copy_k) dma_k1(par, tile_k, g);
        } else {
          if (copy_v) dma_v1(par ^ 1, tile_v, g - 4);
        }
        f[g] = read_k(tKn, g & 1, 4 + (g >> 1));
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int g = 0; g < 8; ++g) {
        if (g & 1) sn1 = T::mfma32(f[g], qf[4 + (g >> 1)], sn1);
        else sn0 = T::mfma32(f[g], qf[4 + (g >> 1)], sn0);
        f[g] = read_vt(tV, 0, g >> 2, g & 3);
        __builtin_amdgcn_sched_barrier(0);
      }
      // the next piece's Q rows are sent for here, between the two GEMMs, and not at the top of the step, where the
      // eight copy instructions would stand in front of the first fragment reads (measured: 2.2 % of the launch)
      if (r == QI && k + 1 < n) dma_q(row_of(k + 1));
      if (ragged && tile_v == NT - 1) mask_tail(sn0, sn1, nv_last);
      // the next piece's Q rows take over the registers (the scores of its first tile are computed in the next step)
      if (r == NT - 2 && k + 1 < n) {
        wait_vm();
        read_q();
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int nn = 0; nn < 6; ++nn) expo_slot(nn);
      __builtin_amdgcn_sched_barrier(0);

      // ---- stage B: O^T += V(s)^T P(s)^T, the rest of the softmax, the row maximum of S(s+1) ----------
      float mxa = fmaxf(sn0[0], sn0[1]), mxb = fmaxf(sn1[0], sn1[1]);
#pragma unroll
      for (int cc = 0; cc < 2; ++cc) {
        u32x4 bw = {pk0[4 * cc], pk0[4 * cc + 1], pk0[4 * cc + 2], pk0[4 * cc + 3]};
        vec8 bfrag = __builtin_bit_cast(vec8, bw);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const int g = cc * 4 + db;
          o[db] = T::mfma32(f[g], bfrag, o[db]);
          f[g] = read_vt(tV, 1, cc, db);
          expo_slot(6 + g);
          if (g < 4) {
          } else if (g < 7) mxa = fmaxf(fmaxf(fmaxf(fmaxf(mxa, sn0[4 * g - 14]), sn0[4 * g - 13]), sn0[4 * g - 12]), sn0[4 * g - 11]);
          else mxa = fmaxf(fmaxf(mxa, sn0[14]), sn0[15]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
#pragma unroll
      for (int cc = 0; cc < 2; ++cc) {
        u32x4 bw = {pk1[4 * cc], pk1[4 * cc + 1], pk1[4 * cc + 2], pk1[4 * cc + 3]};
        vec8 bfrag = __builtin_bit_cast(vec8, bw);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const int g = cc * 4 + db;
          o[db] = T::mfma32(f[g], bfrag, o[db]);
          if (g < 4) expo_slot(14 + g);
          if (g > 0) mxb = fmaxf(fmaxf(mxb, sn1[2 * g]), sn1[2 * g + 1]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      l_run += lsum;
      mx = across(fmaxf(mxa, mxb));

      if (r == NT - 1) {  // the piece's last tile: the next piece starts from nothing
        if (k >= 0 && k < n) finish_stage();
        reset_acc();
      }
      if (r == 0 && k >= 1 && k <= n) finish_store(k - 1);
    };

    constexpr std::integral_constant<int, 0> even{};
    constexpr std::integral_constant<int, 1> odd{};
    for (int s = 0; s < steps; s += 2) {
      step(even, s);
      step(odd, s + 1);
    }
    if (phase == 1) finish_store(n - 1);  // the run ends with the last tile of wavefronts 4..7
    __builtin_amdgcn_s_setprio(0);
    piece0 += n;
  }
  wait_vm();  // no tile copy may still be on its way to LDS when the wavefront ends
}

// Folds the partial results of the pieces that attn_fwd_d128_stream_kernel computed in shares (StreamPlan):
// the log-sum-exp merge of torch's _SDPAMerger over all shares of a piece at once, plus the running pair of a
// ring accumulation.  16 workgroups per tail piece, 16 query rows each; one thread = 8 consecutive output elements.
template <typename T>
__global__ __launch_bounds__(256) void attn_stream_merge_kernel(const AttnParams p) {
  if (p.gate != nullptr && !gate_open(p.gate, p.gate_mask)) return;
  const StreamPlan& sp = p.st;
  const int tp = blockIdx.x >> 4;  // tail piece
  const int local = ((blockIdx.x & 15) << 4) + (threadIdx.x >> 4);
  const int c8 = (threadIdx.x & 15) * 8;
  const int tail0 = sp.R * sp.G;
  // range that holds tail step t: in its round (of Tr steps from r0 on, cut into n ranges) the largest i with i * Tr / n <= t - r0
  auto slot = [&](int64_t t) {
    const int n = sp.Gt / sp.n_rounds;
    int rd = 0;
    while (rd + 1 < sp.n_rounds && t >= sp.round_at[rd + 1]) ++rd;
    const int64_t r0 = sp.round_at[rd], Tr = sp.round_at[rd + 1] - r0;
    return rd * n + (int)(((t - r0 + 1) * n + Tr - 1) / Tr) - 1;
  };
  const int g_first = slot((int64_t)tp * sp.L), g_last = slot((int64_t)(tp + 1) * sp.L - 1);
  if (g_first == g_last) return;  // computed whole by one workgroup, which stored it itself
  const int piece = tail0 + tp;
  const int bh = piece / p.n_qtiles, qt = piece - bh * p.n_qtiles;
  const int head = bh % p.H, batch = bh / p.H;
  const int qrow = qt * 256 + local;
  if (qrow >= p.Sq) return;
  const int64_t ridx = ((int64_t)batch * p.H + head) * p.Sq + qrow;
  auto part_row = [&](int g) { return (int64_t)(2 * g + (g == g_first ? 1 : 0)) * 256 + local; };
  const float old = (p.acc_out != nullptr && !p.acc_first) ? p.acc_lse[ridx] : -INFINITY;
  float m = old;
  for (int g = g_first; g <= g_last; ++g) m = fmaxf(m, p.ws_lse[part_row(g)]);
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float den = 0.f;
  if (old > -INFINITY) {
    const float w = __expf(old - m);
    const float4 a = *(const float4*)(p.acc_out + ridx * 128 + c8);
    const float4 b = *(const float4*)(p.acc_out + ridx * 128 + c8 + 4);
    den = w;
    acc[0] = w * a.x; acc[1] = w * a.y; acc[2] = w * a.z; acc[3] = w * a.w;
    acc[4] = w * b.x; acc[5] = w * b.y; acc[6] = w * b.z; acc[7] = w * b.w;
  }
  if (m > -INFINITY) {
    for (int g = g_first; g <= g_last; ++g) {
      const int64_t wrow = part_row(g);
      const float w = __expf(p.ws_lse[wrow] - m);  // an empty share has LSE -inf: weight 0
      const float4 a = *(const float4*)(p.ws_out + wrow * 128 + c8);
      const float4 b = *(const float4*)(p.ws_out + wrow * 128 + c8 + 4);
      den += w;
      acc[0] += w * a.x; acc[1] += w * a.y; acc[2] += w * a.z; acc[3] += w * a.w;
      acc[4] += w * b.x; acc[5] += w * b.y; acc[6] += w * b.z; acc[7] += w * b.w;
    }
  }
  const float inv = den > 0.f ? 1.0f / den : 0.f;
  if (p.out != nullptr) {
    u32x4 w;
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = T::pack2(acc[2 * i] * inv, acc[2 * i + 1] * inv);
    uint16_t* op = (uint16_t*)p.out + batch * p.os_b + head * p.os_h + (int64_t)qrow * p.os_s + c8;
    *(u32x4*)op = w;
  } else {
    float* ap = p.acc_out + ridx * 128 + c8;
    *(float4*)ap = float4{acc[0] * inv, acc[1] * inv, acc[2] * inv, acc[3] * inv};
    *(float4*)(ap + 4) = float4{acc[4] * inv, acc[5] * inv, acc[6] * inv, acc[7] * inv};
  }
  float* lse_dst = p.acc_out != nullptr ? p.acc_lse : p.lse;
  if (lse_dst != nullptr && c8 == 0) lse_dst[ridx] = den > 0.f ? m + __logf(den) : -INFINITY;
}

// Folds the split_s partial results of each split query tile into out and lse: the log-sum-exp
// merge of torch's _SDPAMerger (used by src/para_attn/sparse_attn.py:174-189) over all pieces at
// once.  One thread = 8 consecutive output elements of one query row; 16 rows per workgroup.
template <typename T>
__global__ __launch_bounds__(256) void attn_split_merge_kernel(const AttnParams p) {
  if (p.gate != nullptr && !gate_open(p.gate, p.gate_mask)) return;
  const int64_t r = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  const int c8 = (threadIdx.x & 15) * 8;
  const int tl = (int)(r / p.bm), local = (int)(r % p.bm);
  if (tl >= p.split_tiles) return;
  const int tile = p.split_main + tl;
  const int qt = tile % p.n_qtiles, bh = tile / p.n_qtiles;
  const int head = bh % p.H, batch = bh / p.H;
  const int qrow = qt * p.bm + local;
  if (qrow >= p.Sq) return;
  const int64_t ridx = ((int64_t)batch * p.H + head) * p.Sq + qrow;
  // ring accumulation: the running pair is one more term of the merge
  const float old = (p.acc_out != nullptr && !p.acc_first) ? p.acc_lse[ridx] : -INFINITY;
  float m = old;
  for (int i = 0; i < p.split_s; ++i) m = fmaxf(m, p.ws_lse[((int64_t)i * p.split_tiles + tl) * p.bm + local]);
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float den = 0.f;
  if (old > -INFINITY) {
    const float w = __expf(old - m);
    const float4 a = *(const float4*)(p.acc_out + ridx * 128 + c8);
    const float4 b = *(const float4*)(p.acc_out + ridx * 128 + c8 + 4);
    den = w;
    acc[0] = w * a.x; acc[1] = w * a.y; acc[2] = w * a.z; acc[3] = w * a.w;
    acc[4] = w * b.x; acc[5] = w * b.y; acc[6] = w * b.z; acc[7] = w * b.w;
  }
  if (m > -INFINITY) {
    for (int i = 0; i < p.split_s; ++i) {
      const int64_t wrow = ((int64_t)i * p.split_tiles + tl) * p.bm + local;
      const float w = __expf(p.ws_lse[wrow] - m);  // an empty share has LSE -inf: weight 0
      const float4 a = *(const float4*)(p.ws_out + wrow * 128 + c8);
      const float4 b = *(const float4*)(p.ws_out + wrow * 128 + c8 + 4);
      den += w;
      acc[0] += w * a.x; acc[1] += w * a.y; acc[2] += w * a.z; acc[3] += w * a.w;
      acc[4] += w * b.x; acc[5] += w * b.y; acc[6] += w * b.z; acc[7] += w * b.w;
    }
  }
  const float inv = den > 0.f ? 1.0f / den : 0.f;
  if (p.out != nullptr) {
    u32x4 w;
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = T::pack2(acc[2 * i] * inv, acc[2 * i + 1] * inv);
    uint16_t* op = (uint16_t*)p.out + batch * p.os_b + head * p.os_h + (int64_t)qrow * p.os_s + c8;
    *(u32x4*)op = w;
  } else {
    float* ap = p.acc_out + ridx * 128 + c8;
    *(float4*)ap = float4{acc[0] * inv, acc[1] * inv, acc[2] * inv, acc[3] * inv};
    *(float4*)(ap + 4) = float4{acc[4] * inv, acc[5] * inv, acc[6] * inv, acc[7] * inv};
  }
  float* lse_dst = p.acc_out != nullptr ? p.acc_lse : p.lse;
  if (lse_dst != nullptr && c8 == 0) lse_dst[ridx] = den > 0.f ? m + __logf(den) : -INFINITY;
}

// Turns a [Hm,nQ,nK] block mask into per-segment lists of key ranges.
// One wavefront per (hm, segment): the lanes look at 64 key blocks at a time, vote where runs of kept
// blocks begin and end, and each beginning / ending lane writes its bound of its range (the runs the
// scan of src/para_attn/sparse_attn.py:215-234 finds), merged with the dense key margins where they touch.
// Segments 0 and nQ+1 are the dense query margins.
__global__ __launch_bounds__(64) void build_runs_kernel(const uint8_t* mask, int Hm, int nQ, int nK,
                                                        int Skv, int kv_lo, int kv_block, int cap,
                                                        int32_t* ws, int32_t* kept_out) {
  const int nseg = nQ + 2;
  const int idx = blockIdx.x;  // grid = Hm * nseg
  const int lane = threadIdx.x;
  const int hm = idx / nseg;
  const int seg = idx % nseg;
  int32_t* cnt = ws + idx;
  int32_t* rg = ws + (size_t)Hm * nseg + (size_t)idx * cap * 2;
  if (seg == 0 || seg == nQ + 1) {
    if (lane == 0) {
      if (Skv > 0) {
        rg[0] = 0;
        rg[1] = Skv;
      }
      *cnt = Skv > 0 ? 1 : 0;
    }
    return;
  }
  const uint8_t* row = mask + ((size_t)hm * nQ + (seg - 1)) * nK;
  const int kv_hi = kv_lo + nK * kv_block;
  // Every lane looks at one key block per pass: a run begins at a kept block whose left neighbour is dropped and
  // ends at a kept block whose right neighbour is dropped; the k-th begin and the k-th end (counted with ballots
  // and a running total) belong to range k.  The dense margins [0, kv_lo) and [kv_hi, Skv) join the first / last
  // run where block 0 / block nK - 1 is kept, and stand as ranges of their own otherwise.
  const bool left = kv_lo > 0, right = Skv > kv_hi;
  const bool first_kept = row[0] != 0, last_kept = row[nK - 1] != 0;
  const int first_idx = left && !first_kept ? 1 : 0;  // range index of the first run
  int begins = 0, ends = 0;                           // runs begun / ended in the passes so far
  int kept = 0;                                       // kept key blocks of this query block
  const uint64_t below = lane == 0 ? 0 : (~0ull >> (64 - lane));
  for (int base = 0; base < nK; base += 64) {
    const int j = base + lane;
    const bool keep = j < nK && row[j] != 0;
    kept += __builtin_popcountll(__ballot(keep));
    const bool begin = keep && (j == 0 || row[j - 1] == 0);
    const bool end = keep && (j == nK - 1 || row[j + 1] == 0);
    const uint64_t bb = __ballot(begin), eb = __ballot(end);
    if (begin) {
      const int k = begins + __builtin_popcountll(bb & below);
      rg[2 * (first_idx + k)] = (j == 0 && left) ? 0 : kv_lo + j * kv_block;
    }
    if (end) {
      const int k = ends + __builtin_popcountll(eb & below);
      rg[2 * (first_idx + k) + 1] = (j == nK - 1 && right) ? Skv : kv_lo + (j + 1) * kv_block;
    }
    begins += __builtin_popcountll(bb);
    ends += __builtin_popcountll(eb);
  }
  if (lane == 0) {
    int n = first_idx + begins;
    if (left && !first_kept) {
      rg[0] = 0;
      rg[1] = kv_lo;
    }
    if (right && !last_kept) {
      rg[2 * n] = kv_hi;
      rg[2 * n + 1] = Skv;
      ++n;
    }
    *cnt = n;
    if (kept_out != nullptr) kept_out[(size_t)hm * nQ + (seg - 1)] = kept;  // what sparse_order_kernel ranks the block by
  }
}

// The same lists for pairs of adjacent query blocks: segment 1 + i covers query blocks 2i and 2i + 1 and walks the
// union of their kept key blocks.  A range is a run of key blocks kept by the same blocks of the pair; its first
// key carries which in its two low bits (1: the lower query block, 2: the upper, 3: both), so kv_lo, kv_block
// and Skv are multiples of 4 here.  Up to nK + 2 ranges per segment.  The dense margins belong to both.
__global__ __launch_bounds__(64) void build_pair_runs_kernel(const uint8_t* mask, int Hm, int nQ, int nK,
                                                             int Skv, int kv_lo, int kv_block, int cap,
                                                             int32_t* ws) {
  const int nseg = nQ / 2 + 2;
  const int idx = blockIdx.x;  // grid = Hm * nseg
  const int lane = threadIdx.x;
  const int hm = idx / nseg;
  const int seg = idx % nseg;
  int32_t* cnt = ws + idx;
  int32_t* rg = ws + (size_t)Hm * nseg + (size_t)idx * cap * 2;
  if (seg == 0 || seg == nseg - 1) {
    if (lane == 0) {
      if (Skv > 0) {
        rg[0] = 0 | 3;
        rg[1] = Skv;
      }
      *cnt = Skv > 0 ? 1 : 0;
    }
    return;
  }
  const uint8_t* row_a = mask + ((size_t)hm * nQ + 2 * (seg - 1)) * nK;
  const uint8_t* row_b = row_a + nK;
  const int kv_hi = kv_lo + nK * kv_block;
  int n = 0;
  int cur_b = -1, cur_e = -1, cur_m = 0;  // open range (lane 0 only)
  auto flush = [&] {
    if (cur_e > cur_b) {
      rg[2 * n] = cur_b | cur_m;
      rg[2 * n + 1] = cur_e;
      ++n;
    }
  };
  auto push = [&](int b, int e, int m) {
    if (e <= b || m == 0) return;
    if (cur_e == b && cur_m == m) {
      cur_e = e;
    } else {
      flush();
      cur_b = b;
      cur_e = e;
      cur_m = m;
    }
  };
  if (lane == 0) push(0, kv_lo, 3);
  for (int base = 0; base < nK; base += 64) {
    const int j = base + lane;
    const uint64_t in_a = __ballot(j < nK && row_a[j] != 0);
    const uint64_t in_b = __ballot(j < nK && row_b[j] != 0);
    if (lane == 0) {
      const int lim = nK - base < 64 ? nK - base : 64;
      for (int i = 0; i < lim; ++i) {
        const int m = (int)((in_a >> i) & 1) | ((int)((in_b >> i) & 1) << 1);
        const int b = kv_lo + (base + i) * kv_block;
        push(b, b + kv_block, m);
      }
    }
  }
  if (lane == 0) {
    push(kv_hi, Skv, 3);
    flush();
    *cnt = n;
  }
}

// ---------------------------------------------------------------------------------------------
// Score bound for the dense pipelined kernels.  |q.k| <= |q| |k|, so with Mq = the largest row
// norm of Q and Mk that of K no score leaves [-Mq Mk scale, Mq Mk scale]; in the log2 domain of the
// kernel that is +-bound.  If bound <= `limit` (60 for bf16 P, whose exponent range is fp32's; 14
// for fp16 P) then exp2(score) can neither overflow nor vanish, sums of up to 2^31 of them stay far
// inside fp32, and the softmax needs no running maximum: a common factor 2^-m cancels in O / l and
// in m + log2(l) whatever m is, so m = 0 gives the same results.  Models that normalise q and k
// (RMS norm per head) sit near bound = 16.  Two launches: per-block maxima of the squared row
// norms (blocks [0, G) over Q, [G, 2G) over K, 8 elements of a row per lane), then one block that
// folds them and writes the flag.  An infinite element makes the bound infinite (flag 0); a NaN element
// is not seen by the maxima, and its scores are NaN in either variant of the kernel.
// ---------------------------------------------------------------------------------------------
constexpr int BOUND_G = 1024;                                   // blocks per tensor
constexpr size_t BOUND_WS_BYTES = (2 * BOUND_G + 64) * 4;       // partial maxima + the flag word (+ padding)
// with the keys in n segments: one set of partial maxima per segment, then the flag word
// The query blocks of every head by falling number of kept key blocks (ties by block number): the launch order of
// the block-sparse kernels.  Workgroups start in the order of their numbers as slots fall free, so a launch that
// hands the lists out as they come ends on whatever long lists happen to come late (4 % of the launch on a mask
// whose lists differ by 9 % rms), and workgroups that run side by side are at different places of the key axis.
// Longest first within a head, the launch ends on the short lists, and neighbours in the order are lists of
// nearly the same length, which start and end together and sweep the keys in step: half the reads from beyond
// the L2 on the same mask.  One workgroup per mask head; `kept` comes from build_runs_kernel.
constexpr int SPARSE_ORDER_MAX_BLOCKS = 2048;  // the ranking below is quadratic in the blocks of a head
__global__ __launch_bounds__(256) void sparse_order_kernel(const int32_t* kept, int nQ, int32_t* order) {
  extern __shared__ int len_of[];
  const int hm = blockIdx.x;
  for (int blk = threadIdx.x; blk < nQ; blk += 256) len_of[blk] = kept[(size_t)hm * nQ + blk];
  __syncthreads();
  for (int blk = threadIdx.x; blk < nQ; blk += 256) {
    const int mine = len_of[blk];
    int rank = 0;
    for (int j = 0; j < nQ; ++j) {
      const int other = len_of[j];
      rank += (other > mine || (other == mine && j < blk)) ? 1 : 0;
    }
    order[(size_t)hm * nQ + rank] = blk;
  }
}

static inline size_t bound_ws_bytes(int nseg) { return ((size_t)2 * BOUND_G * (nseg < 1 ? 1 : nseg) + 64) * 4; }

template <typename T, int D>
__global__ __launch_bounds__(256) void score_bound_partial_kernel(const AttnParams p, float* part, const void* keys, int n_keys, int q_too) {
  constexpr int LPR = D / 8;       // lanes per row: 8 elements each
  constexpr int RPB = 256 / LPR;   // rows per block and step
  // q_too: BOUND_G blocks for Q, then BOUND_G for the keys; otherwise the key blocks alone (a further key segment of
  // a sweep: the Q rows were looked at with the first)
  const bool is_k = !q_too || blockIdx.x >= BOUND_G;
  const int blk = q_too && is_k ? blockIdx.x - BOUND_G : blockIdx.x;
  const uint16_t* base = (const uint16_t*)(is_k ? keys : p.q);  // keys: p.k, or one segment of the keys
  const int64_t sb = is_k ? p.ks_b : p.qs_b, sh = is_k ? p.ks_h : p.qs_h, ss = is_k ? p.ks_s : p.qs_s;
  const int S = is_k ? n_keys : p.Sq;
  const int64_t rows = (int64_t)p.B * p.H * S;
  const int sub = threadIdx.x % LPR;
  float best = 0.f;
  for (int64_t r = (int64_t)blk * RPB + threadIdx.x / LPR; r < rows; r += (int64_t)BOUND_G * RPB) {
    const int s_ = (int)(r % S);
    const int64_t bh = r / S;
    const uint16_t* rp = base + (bh / p.H) * sb + (bh % p.H) * sh + (int64_t)s_ * ss + 8 * sub;
    const u32x4 w = *(const u32x4*)rp;
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float a = T::lo(w[i]), b = T::hi(w[i]);
      acc = __builtin_fmaf(a, a, acc);
      acc = __builtin_fmaf(b, b, acc);
    }
#pragma unroll
    for (int d = 1; d < LPR; d <<= 1) acc += __shfl_xor(acc, d, LPR);
    best = fmaxf(best, acc);
  }
  __shared__ float sm[256];
  sm[threadIdx.x] = best;
  __syncthreads();
  for (int d = 128; d > 0; d >>= 1) {
    if ((int)threadIdx.x < d) {
      sm[threadIdx.x] = fmaxf(sm[threadIdx.x], sm[threadIdx.x + d]);
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) part[is_k ? BOUND_G + blk : blk] = sm[0];
}

__global__ __launch_bounds__(256) void score_bound_flag_kernel(const float* part, int nparts, float scale_log2, float limit, int* flag) {
  __shared__ float sq[256], sk[256];
  float mq = 0.f, mk = 0.f;
  for (int i = threadIdx.x; i < BOUND_G * nparts; i += 256) {  // nparts sets of (BOUND_G for Q, BOUND_G for a key segment)
    const int set = i / BOUND_G, e = i - set * BOUND_G;
    if (set == 0) mq = fmaxf(mq, part[e]);  // the Q rows go with the first key segment only
    mk = fmaxf(mk, part[2 * BOUND_G * set + BOUND_G + e]);
  }
  sq[threadIdx.x] = mq;
  sk[threadIdx.x] = mk;
  __syncthreads();
  for (int d = 128; d > 0; d >>= 1) {
    if ((int)threadIdx.x < d) {
      sq[threadIdx.x] = fmaxf(sq[threadIdx.x], sq[threadIdx.x + d]);
      sk[threadIdx.x] = fmaxf(sk[threadIdx.x], sk[threadIdx.x + d]);
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    const float bound = sqrtf(sq[0]) * sqrtf(sk[0]) * scale_log2;
    *flag = bound <= limit ? 1 : 0;
  }
}

// A key-only boolean mask [B, Skv] (byte strides mb, mk): per batch element the number of kept keys, and
// whether in every batch element the kept keys are exactly the leading ones (then the dense kernels take the
// counts as kv_len and the mask need not be looked at again).  One workgroup; out[0..B) = counts,
// out[B] = 1 if all are prefixes else 0.
// A boolean key mask is taken apart on the device.  Result: out[b] = kept keys of batch element b; out[B] = bit 0:
// every element keeps a prefix of its keys, bit 1: every element keeps at least 7/8 of them.
// Short masks: one workgroup does it all.
__global__ __launch_bounds__(1024) void key_mask_small_kernel(const uint8_t* mask, int64_t mb, int64_t mk, int B,
                                                              int Skv, int32_t* out) {
  __shared__ int s_cnt[1024];
  __shared__ int s_last[1024];
  int all_prefix = 1, fewest = Skv;
  for (int b = 0; b < B; ++b) {
    int cnt = 0, last = -1;
    for (int j = threadIdx.x; j < Skv; j += 1024) {
      if (mask[(int64_t)b * mb + (int64_t)j * mk] != 0) {
        ++cnt;
        last = j;
      }
    }
    s_cnt[threadIdx.x] = cnt;
    s_last[threadIdx.x] = last;
    __syncthreads();
    for (int d = 512; d > 0; d >>= 1) {
      if ((int)threadIdx.x < d) {
        s_cnt[threadIdx.x] += s_cnt[threadIdx.x + d];
        s_last[threadIdx.x] = max(s_last[threadIdx.x], s_last[threadIdx.x + d]);
      }
      __syncthreads();
    }
    if (threadIdx.x == 0) out[b] = s_cnt[0];
    if (s_cnt[0] != s_last[0] + 1) all_prefix = 0;
    fewest = min(fewest, s_cnt[0]);
    __syncthreads();
  }
  if (threadIdx.x == 0) out[B] = all_prefix | ((int64_t)fewest * 8 >= (int64_t)Skv * 7 ? 2 : 0);
}

// Long masks, first step: kept keys and last kept key of every chunk of MASK_CHUNK keys (one workgroup per chunk
// and batch element).
constexpr int MASK_CHUNK = 1024;
__global__ __launch_bounds__(256) void key_mask_chunk_kernel(const uint8_t* mask, int64_t mb, int64_t mk, int Skv, int nchunk,
                                                             int32_t* chunk_cnt, int32_t* chunk_last) {
  __shared__ int s_cnt[256];
  __shared__ int s_last[256];
  const int b = blockIdx.y, c = blockIdx.x, t = threadIdx.x;
  const uint8_t* mrow = mask + (int64_t)b * mb;
  int cnt = 0, last = -1;
  for (int i = 0; i < MASK_CHUNK / 256; ++i) {
    const int j = c * MASK_CHUNK + i * 256 + t;
    if (j < Skv && mrow[(int64_t)j * mk] != 0) {
      ++cnt;
      last = j;
    }
  }
  s_cnt[t] = cnt;
  s_last[t] = last;
  __syncthreads();
  for (int d = 128; d > 0; d >>= 1) {
    if (t < d) {
      s_cnt[t] += s_cnt[t + d];
      s_last[t] = max(s_last[t], s_last[t + d]);
    }
    __syncthreads();
  }
  if (t == 0) {
    chunk_cnt[b * nchunk + c] = s_cnt[0];
    chunk_last[b * nchunk + c] = s_last[0];
  }
}

// Second step (one workgroup): where each chunk's kept keys begin among its batch element's kept keys, and the result.
__global__ __launch_bounds__(256) void key_mask_scan_kernel(int B, int Skv, int nchunk, const int32_t* chunk_cnt, const int32_t* chunk_last,
                                                            int32_t* chunk_off, int32_t* out) {
  __shared__ int s_scan[256];
  __shared__ int s_last[256];
  const int t = threadIdx.x;
  int all_prefix = 1, fewest = Skv;
  for (int b = 0; b < B; ++b) {
    int running = 0, last = -1;
    for (int base = 0; base < nchunk; base += 256) {
      const int c = base + t;
      const int v = c < nchunk ? chunk_cnt[b * nchunk + c] : 0;
      s_scan[t] = v;
      s_last[t] = c < nchunk ? chunk_last[b * nchunk + c] : -1;
      __syncthreads();
      for (int d = 1; d < 256; d <<= 1) {
        const int add = t >= d ? s_scan[t - d] : 0;
        const int other = t >= d ? s_last[t - d] : -1;
        __syncthreads();
        s_scan[t] += add;
        s_last[t] = max(s_last[t], other);
        __syncthreads();
      }
      if (c < nchunk) chunk_off[b * nchunk + c] = running + s_scan[t] - v;
      running += s_scan[255];
      last = max(last, s_last[255]);
      __syncthreads();
    }
    if (t == 0) out[b] = running;
    if (running != last + 1) all_prefix = 0;
    fewest = min(fewest, running);
  }
  if (t == 0) out[B] = all_prefix | ((int64_t)fewest * 8 >= (int64_t)Skv * 7 ? 2 : 0);
}

// Gathers the kept key and value rows of a key mask that is not a prefix into dense copies [B][H][Skv][D] (the
// reference's attention_forward_sparse_kv selects them with index_select, src/para_attn/ops/__init__.py:283-287), in
// their order.  One workgroup per chunk of MASK_CHUNK keys, head and batch element: it ranks the chunk's kept keys
// (wavefront ballots), then copies their rows to where the chunk's keys begin (chunk_off), 16 bytes per thread.  The
// rows from the last kept key to the end of its key tile are cleared: the kernels read whole tiles, and a
// probability of 0 times whatever the workspace held would still be a NaN.
template <int D>
__global__ __launch_bounds__(256) void gather_kept_keys_kernel(const AttnParams p, const uint8_t* mask, int64_t mb, int64_t mk, int nchunk,
                                                               const int32_t* count, const int32_t* chunk_off, uint16_t* kc, uint16_t* vc) {
  if (p.gate != nullptr && !gate_open(p.gate, p.gate_mask)) return;
  constexpr int CPR = D / 8;      // 16-byte chunks per row
  constexpr int RPB = 256 / CPR;  // rows per pass of the workgroup
  __shared__ int s_src[MASK_CHUNK];
  __shared__ int s_wave[4];
  const int b = blockIdx.z, h = blockIdx.y, c = blockIdx.x, t = threadIdx.x;
  const int lane = t & 63, wave = t >> 6;
  const uint8_t* mrow = mask + (int64_t)b * mb;
  int m = 0;
  for (int i = 0; i < MASK_CHUNK / 256; ++i) {
    const int j = c * MASK_CHUNK + i * 256 + t;
    const bool kept = j < p.Skv && mrow[(int64_t)j * mk] != 0;
    const uint64_t votes = __ballot(kept);
    if (lane == 0) s_wave[wave] = __popcll(votes);
    __syncthreads();
    int before = 0, all = 0;
    for (int w = 0; w < 4; ++w) {
      if (w < wave) before += s_wave[w];
      all += s_wave[w];
    }
    if (kept) s_src[m + before + __popcll(votes & ((1ull << lane) - 1ull))] = j;
    m += all;
    __syncthreads();
  }
  const uint16_t* kb = (const uint16_t*)p.k + b * p.ks_b + h * p.ks_h;
  const uint16_t* vb = (const uint16_t*)p.v + b * p.vs_b + h * p.vs_h;
  const int64_t dst0 = ((int64_t)b * p.H + h) * p.Skv;
  const int cc = t % CPR;
  const int first = chunk_off[b * nchunk + c];
  for (int r = t / CPR; r < m; r += RPB) {
    const int64_t s_row = s_src[r];
    const u32x4 kx = *(const u32x4*)(kb + s_row * p.ks_s + 8 * cc);
    const u32x4 vx = *(const u32x4*)(vb + s_row * p.vs_s + 8 * cc);
    *(u32x4*)(kc + (dst0 + first + r) * D + 8 * cc) = kx;
    *(u32x4*)(vc + (dst0 + first + r) * D + 8 * cc) = vx;
  }
  if (c == nchunk - 1) {
    const int n = count[b];
    const int n_end = min(p.Skv, (n + BN - 1) / BN * BN);
    const u32x4 z = {0u, 0u, 0u, 0u};
    for (int i = n + t / CPR; i < n_end; i += RPB) {
      *(u32x4*)(kc + (dst0 + i) * D + 8 * cc) = z;
      *(u32x4*)(vc + (dst0 + i) * D + 8 * cc) = z;
    }
  }
}

}  // namespace pa

using namespace pa;

static int check_common(const void* q, const void* k, const void* v, void* out, int dtype, int B,
                        int H, int Sq, int Skv, int D, const int64_t* qs, const int64_t* ks,
                        const int64_t* vs, const int64_t* os, float scale) {
  if (B < 0 || H < 0 || Sq < 0 || Skv < 0) PA_FAIL(PA_ERR_INVALID, "negative size");
  // an operand without elements may come as a null pointer (torch hands out none for empty tensors)
  const bool any_row = B > 0 && H > 0 && Sq > 0;
  if (!qs || !ks || !vs || !os || (any_row && (!q || !out)) || (any_row && Skv > 0 && (!k || !v)))
    PA_FAIL(PA_ERR_INVALID, "null pointer argument");
  if (dtype != PA_DTYPE_BF16 && dtype != PA_DTYPE_F16)
    PA_FAIL(PA_ERR_UNSUPPORTED, "attention dtype must be bf16 or f16 (got code %d)", dtype);
  if (D != 128 && D != 64) PA_FAIL(PA_ERR_UNSUPPORTED, "head_dim %d not supported (64 or 128)", D);
  if (!(scale > 0.f) || !(scale < INFINITY)) PA_FAIL(PA_ERR_UNSUPPORTED, "scale must be positive and finite");
  const int64_t* st[4] = {qs, ks, vs, os};
  const void* ptr[4] = {q, k, v, out};
  const char* nm[4] = {"query", "key", "value", "out"};
  for (int i = 0; i < 4; ++i) {
    if (((uintptr_t)ptr[i]) % 16) PA_FAIL(PA_ERR_UNSUPPORTED, "%s pointer not 16-byte aligned", nm[i]);
    for (int j = 0; j < 3; ++j) {
      if (st[i][j] < 0) PA_FAIL(PA_ERR_UNSUPPORTED, "%s has a negative stride", nm[i]);
      if (st[i][j] % 8) PA_FAIL(PA_ERR_UNSUPPORTED, "%s stride %lld not a multiple of 8 elements", nm[i], (long long)st[i][j]);
    }
  }
  if ((int64_t)B * H * ((Sq + BM - 1) / BM + 2) > 0x7fffffffLL) PA_FAIL(PA_ERR_UNSUPPORTED, "grid too large");
  return PA_OK;
}

static void fill_params(AttnParams& p, const void* q, const void* k, const void* v, void* out,
                        float* lse, int B, int H, int Sq, int Skv, const int64_t* qs,
                        const int64_t* ks, const int64_t* vs, const int64_t* os, float scale) {
  p.q = q; p.k = k; p.v = v; p.out = out; p.lse = lse;
  p.B = B; p.H = H; p.Sq = Sq; p.Skv = Skv;
  p.qs_b = qs[0]; p.qs_h = qs[1]; p.qs_s = qs[2];
  p.ks_b = ks[0]; p.ks_h = ks[1]; p.ks_s = ks[2];
  p.vs_b = vs[0]; p.vs_h = vs[1]; p.vs_s = vs[2];
  p.os_b = os[0]; p.os_h = os[1]; p.os_s = os[2];
  p.scale_log2 = scale * LOG2E;
  p.kv_len = nullptr;
  p.runs = nullptr;
  p.order = nullptr;
  p.Hm = 0; p.nQ = 0; p.cap = 0; p.q_lo = 0; p.q_block = 0; p.pair = 0; p.tiles_left = 0; p.tiles_per_block = 0;
  p.bm = BM; p.pipe = 0;
  p.xcd_chunk = 0;
  p.causal = 0;
  p.acc_out = nullptr; p.acc_lse = nullptr; p.acc_first = 0;
  p.split_main = 0; p.split_tiles = 0; p.split_s = 0; p.ws_out = nullptr; p.ws_lse = nullptr;
  p.bound_flag = nullptr;
  p.mask = nullptr; p.ms_b = p.ms_h = p.ms_q = p.ms_k = 0;
  p.gate = nullptr; p.gate_mask = 0;
  p.st = StreamPlan{};
}

template <typename T, int D, bool SPARSE>
static int launch_attn(const AttnParams& p, hipStream_t stream) {
  int64_t nblocks = (int64_t)p.B * p.H * p.n_qtiles;
  if (nblocks == 0) return PA_OK;
  // only the head_dim-128 pipelined kernel folds into a running pair or splits keys; the others would
  // store through the (absent) plain output
  if ((p.acc_out != nullptr || p.split_s > 1) && !(D == 128 && p.pipe && !SPARSE))
    PA_FAIL(PA_ERR_UNSUPPORTED, "accumulation / key split reached a kernel that has neither");
  if (p.out == nullptr && p.acc_out == nullptr) PA_FAIL(PA_ERR_INVALID, "null output pointer");
  if (p.split_s > 1) nblocks = (int64_t)p.split_main + (int64_t)p.split_tiles * p.split_s;
  if (p.xcd_chunk > 0) nblocks = 8 * (int64_t)p.xcd_chunk;
  const void* fn;
  size_t smem;
  int slot;
  if constexpr (D == 128) {
    smem = 4 * TILE_BYTES;
    if (p.pipe && p.bm == 256) { fn = (const void*)attn_fwd_d128_pipe_kernel<T, SPARSE, 8>; slot = 2; }
    else if (p.pipe) { fn = (const void*)attn_fwd_d128_pipe_kernel<T, SPARSE, 4>; slot = 1; }
    else { fn = (const void*)attn_fwd_d128_kernel<T, SPARSE>; slot = 0; }
  } else {
    if (p.pipe && p.bm == 256) { fn = (const void*)attn_fwd_d64_pipe_kernel<T, SPARSE, 8>; slot = 2; smem = 4 * TILE64_BYTES; }
    else if (p.pipe) { fn = (const void*)attn_fwd_d64_pipe_kernel<T, SPARSE, 4>; slot = 1; smem = 4 * TILE64_BYTES; }
    else { fn = (const void*)attn_fwd_kernel<T, D, SPARSE>; slot = 0; smem = Smem<D>::BYTES; }
  }
  // the attribute belongs to the function on one device: remembered per device and kernel variant
  if (p.bound_flag != nullptr && (SPARSE || !(D == 128 ? slot == 2 : slot >= 1)))
    PA_FAIL(PA_ERR_UNSUPPORTED, "score bound reached a kernel that does not read it");
  static bool attr_done[PA_MAX_DEVICES][6] = {};  // benign race: the call is idempotent
  const int dev = current_device();
  if (dev < 0 || !attr_done[dev][slot]) {
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) PA_FAIL(PA_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    if (dev >= 0) attr_done[dev][slot] = true;
  }
  if constexpr (!SPARSE) {
    if (p.bound_flag != nullptr) {  // the variant without a running maximum first; one of the two returns at once
      const void* fb;
      if constexpr (D == 128) fb = (const void*)attn_fwd_d128_pipe_kernel<T, false, 8, true>;
      else fb = slot == 2 ? (const void*)attn_fwd_d64_pipe_kernel<T, false, 8, true> : (const void*)attn_fwd_d64_pipe_kernel<T, false, 4, true>;
      const int bslot = 3 + (D == 64 && slot == 1 ? 1 : 0);
      if (dev < 0 || !attr_done[dev][bslot]) {
        hipError_t e = hipFuncSetAttribute(fb, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) PA_FAIL(PA_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
        if (dev >= 0) attr_done[dev][bslot] = true;
      }
      if constexpr (D == 128)
        hipLaunchKernelGGL((attn_fwd_d128_pipe_kernel<T, false, 8, true>), dim3((unsigned)nblocks), dim3(512), smem, stream, p);
      else if (slot == 2)
        hipLaunchKernelGGL((attn_fwd_d64_pipe_kernel<T, false, 8, true>), dim3((unsigned)nblocks), dim3(512), smem, stream, p);
      else
        hipLaunchKernelGGL((attn_fwd_d64_pipe_kernel<T, false, 4, true>), dim3((unsigned)nblocks), dim3(256), smem, stream, p);
      PA_CHECK_LAUNCH("attention kernel (bounded scores)");
    }
  }
  if constexpr (D == 128 && SPARSE) {
    if (p.pair) {
      const void* fp = (const void*)attn_fwd_d128_pipe_kernel<T, true, 8, false, true>;
      if (dev < 0 || !attr_done[dev][5]) {
        hipError_t e = hipFuncSetAttribute(fp, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) PA_FAIL(PA_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
        if (dev >= 0) attr_done[dev][5] = true;
      }
      hipLaunchKernelGGL((attn_fwd_d128_pipe_kernel<T, true, 8, false, true>), dim3((unsigned)nblocks), dim3(512), smem, stream, p);
      PA_CHECK_LAUNCH("attention kernel (paired query blocks)");
      return PA_OK;
    }
  }
  if constexpr (D == 128) {
    if (slot == 2)
      hipLaunchKernelGGL((attn_fwd_d128_pipe_kernel<T, SPARSE, 8>), dim3((unsigned)nblocks), dim3(512), smem, stream, p);
    else if (slot == 1)
      hipLaunchKernelGGL((attn_fwd_d128_pipe_kernel<T, SPARSE, 4>), dim3((unsigned)nblocks), dim3(256), smem, stream, p);
    else
      hipLaunchKernelGGL((attn_fwd_d128_kernel<T, SPARSE>), dim3((unsigned)nblocks), dim3(NTHREADS), smem, stream, p);
  } else {
    if (slot == 2)
      hipLaunchKernelGGL((attn_fwd_d64_pipe_kernel<T, SPARSE, 8>), dim3((unsigned)nblocks), dim3(512), smem, stream, p);
    else if (slot == 1)
      hipLaunchKernelGGL((attn_fwd_d64_pipe_kernel<T, SPARSE, 4>), dim3((unsigned)nblocks), dim3(256), smem, stream, p);
    else
      hipLaunchKernelGGL((attn_fwd_kernel<T, D, SPARSE>), dim3((unsigned)nblocks), dim3(NTHREADS), smem, stream, p);
  }
  PA_CHECK_LAUNCH("attention kernel");
  if constexpr (D == 128 && !SPARSE) {
    if (p.split_s > 1) {
      const int64_t rows = (int64_t)p.split_tiles * p.bm;
      hipLaunchKernelGGL((attn_split_merge_kernel<T>), dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, stream, p);
      PA_CHECK_LAUNCH("attention split merge kernel");
    }
  }
  return PA_OK;
}

// Key-split tail.  All workgroups of the dense kernel cost the same, so a grid of n_tiles
// workgroups on `slots` resident places takes ceil(n_tiles / slots) rounds however empty the last
// round is.  Computing the last T query tiles in s key shares each (T*s workgroups of 1/s the
// length, plus a small merge) turns that into (n_tiles - T) / slots + ceil(T*s / slots) / s.
// T is the remainder of n_tiles modulo slots, or that plus one more round; s <= 8 and every share
// keeps at least 16 key tiles.  A workgroup's fixed cost (Q load, first tile copies, output) is
// priced at 4 key tiles, so a share of a tile with n key tiles costs (n/s + 4) / (n + 4) of a
// whole one.  Returns s = 1 unless the estimate improves by 3 %.
struct SplitPlan {
  int tiles, s;
  double rounds;
};
// The planners' measured constants (microseconds per key tile, what 256-row workgroups gain over 128-row ones, the
// dealing of workgroups to 8 XCDs) are MI355X's: 256 compute units in 8 XCDs.  On a device that reports another
// compute-unit count the launches fall back to plain plans: no key split priced by those constants, no XCD order.
static bool mi355x_layout() { return device_cus() == 256; }
static SplitPlan plan_split(int64_t n_tiles, int slots, int kv_tiles, int bm, bool allow) {
  if (slots <= 0) return {0, 1, 1.0};  // no device to ask: no estimate, no split
  SplitPlan best = {0, 1, (double)((n_tiles + slots - 1) / slots)};
  if (!allow || n_tiles % slots == 0) return best;
  SplitPlan found = best;
  double best_found = best.rounds;
  // one round in microseconds (a key tile takes a workgroup about 1.75 us), to price the merge launch in
  // rounds: about 8 us of launch gap plus its partials at 3 TB/s (measured: 17.7 us for 46 MB; at 4608 keys
  // that is 0.13 of a round and the split loses, at 119k keys 0.03 and it wins)
  const double round_us = ((double)kv_tiles + 4.0) * 1.75;
  for (int extra = 0; extra < 2; ++extra) {
    const int64_t T = n_tiles % slots + (int64_t)extra * slots;
    if (T > n_tiles || T * 8 > 0x7fffffffLL) break;
    for (int s = 2; s <= 8 && kv_tiles / s >= 16; ++s) {
      const double share = ((double)kv_tiles / s + 4.0) / ((double)kv_tiles + 4.0);
      const double merge_us = 8.0 + (double)T * s * bm * 129.0 * 4.0 / 3.0e6;
      const double r = (double)((n_tiles - T) / slots) + (double)((T * s + slots - 1) / slots) * share + merge_us / round_us;
      if (r < best.rounds * 0.97 && r < best_found) { best_found = r; found = {(int)T, s, r}; }
    }
  }
  return found;
}

// Tuning and test aids.  The environment gives the initial values and is read once per process
// (at the first launch); pa_set_tuning() changes them afterwards.
//   PARAATTN_NO_PIPE=1       "no_pipe"       the kernels without 32-bit offset limits
//   PARAATTN_BM=128|256      "bm"            query rows per workgroup (0 = choose)
//   PARAATTN_NO_SPLIT=1      "no_split"      no key-split tail
//   PARAATTN_NO_XCD_ORDER=1  "no_xcd_order"  block-sparse workgroups in plain order
//   PARAATTN_BOUND=0|1       "bound"         never / always compute the score bound (-1 = by size)
//   PARAATTN_STREAM=0|1      "stream"        never / wherever possible the resident-workgroup kernel (-1 = by shape)
//   PARAATTN_STREAM_EVEN=0|1 "stream_even"   its tail cut into shares that begin at the same keys / into equal ranges (-1 = by size)
//   PARAATTN_STREAM_DYN=0|2..6 "stream_dyn"  its tail in equal ranges, one per workgroup / in that many rounds of ranges drawn by the workgroups, wherever two rounds fit (-1 = 4 rounds, by size)
//   PARAATTN_STREAM_SOLO=1   "stream_solo"   test aid: where every piece is cut into drawn ranges, one workgroup draws and computes them all, one after the other
//   PARAATTN_SPARSE_PAIR=1   "sparse_pair"   block-sparse with 128-row query blocks: two adjacent blocks per 256-row workgroup
//   PARAATTN_WAVE_ROWS=64    "wave_rows"     the resident-workgroup kernel as 4 wavefronts of 64 query rows instead of 8 of 32
//   PARAATTN_SPARSE_ORDER=0  "sparse_order"  block-sparse: 0 = the query blocks of a head in their own order instead of longest list first
//   PARAATTN_SHORT_KEYS=0|1  "short_keys"    never / wherever it applies the kernel for 449..512 keys (-1 = by the number of pieces)
struct Tuning {
  std::atomic<int> no_pipe, no_split, no_xcd_order, forced_bm, bound, stream, stream_even, stream_dyn, stream_solo, sparse_pair, wave_rows, short_keys, sparse_order;
};
static Tuning& tuning() {
  static Tuning t;
  static const bool init = [] {
    auto num = [](const char* name, int dflt) {
      const char* e = getenv(name);
      return e && *e ? atoi(e) : dflt;
    };
    t.no_pipe = num("PARAATTN_NO_PIPE", 0) == 1;
    t.no_split = num("PARAATTN_NO_SPLIT", 0) == 1;
    t.no_xcd_order = num("PARAATTN_NO_XCD_ORDER", 0) == 1;
    t.forced_bm = num("PARAATTN_BM", 0);
    const int b = num("PARAATTN_BOUND", -1);
    t.bound = b == 0 || b == 1 ? b : -1;
    const int st = num("PARAATTN_STREAM", -1);
    t.stream = st == 0 || st == 1 ? st : -1;
    const int se = num("PARAATTN_STREAM_EVEN", -1);
    t.stream_even = se == 0 || se == 1 ? se : -1;
    const int sd = num("PARAATTN_STREAM_DYN", -1);
    t.stream_dyn = sd == 0 || (sd > 1 && sd <= MAX_TAIL_ROUNDS) ? sd : -1;
    t.stream_solo = num("PARAATTN_STREAM_SOLO", 0) == 1;
    t.sparse_pair = num("PARAATTN_SPARSE_PAIR", 0) == 1;
    t.wave_rows = num("PARAATTN_WAVE_ROWS", 0) == 64 ? 64 : 0;
    const int sk = num("PARAATTN_SHORT_KEYS", -1);
    t.short_keys = sk == 0 || sk == 1 ? sk : -1;
    t.sparse_order = num("PARAATTN_SPARSE_ORDER", 1) != 0;
    return true;
  }();
  (void)init;
  return t;
}

extern "C" int pa_set_tuning(const char* name, int value) {
  if (!name) PA_FAIL(PA_ERR_INVALID, "pa_set_tuning: null name");
  Tuning& t = tuning();
  if (!strcmp(name, "no_pipe")) t.no_pipe = value == 1;
  else if (!strcmp(name, "no_split")) t.no_split = value == 1;
  else if (!strcmp(name, "no_xcd_order")) t.no_xcd_order = value == 1;
  else if (!strcmp(name, "bm")) {
    if (value != 0 && value != 128 && value != 256) PA_FAIL(PA_ERR_INVALID, "pa_set_tuning: bm must be 0, 128 or 256");
    t.forced_bm = value;
  } else if (!strcmp(name, "bound")) t.bound = value == 0 || value == 1 ? value : -1;
  else if (!strcmp(name, "stream")) t.stream = value == 0 || value == 1 ? value : -1;
  else if (!strcmp(name, "stream_even")) t.stream_even = value == 0 || value == 1 ? value : -1;
  else if (!strcmp(name, "stream_dyn")) t.stream_dyn = value == 0 || (value > 1 && value <= MAX_TAIL_ROUNDS) ? value : -1;
  else if (!strcmp(name, "stream_solo")) t.stream_solo = value == 1;
  else if (!strcmp(name, "sparse_pair")) t.sparse_pair = value == 1;
  else if (!strcmp(name, "wave_rows")) t.wave_rows = value == 64 ? 64 : 0;
  else if (!strcmp(name, "short_keys")) t.short_keys = value == 0 || value == 1 ? value : -1;
  else if (!strcmp(name, "sparse_order")) t.sparse_order = value != 0;
  else PA_FAIL(PA_ERR_INVALID, "pa_set_tuning: unknown knob '%s'", name);
  return PA_OK;
}

// Bytes of workspace the key-split tail of the plan for bm rows per workgroup needs.
static size_t split_ws_bytes(const SplitPlan& pl, int bm) {
  return pl.s > 1 ? (size_t)pl.tiles * pl.s * bm * (128 + 1) * sizeof(float) : 0;
}

// Picks the kernel, the query rows per workgroup and the key-split tail.  The pipelined
// head_dim-128 kernel needs K and V to span less than 4 GiB (32-bit buffer offsets).  128 rows = 4
// wavefronts, two workgroups per CU; 256 rows = 8 wavefronts sharing one K/V stream (half the tile
// copies per flop: measured 5.5 % more throughput per full round at the 119k-token shape, but one
// workgroup per CU makes a partly filled last round dearer).  The choice is the smaller estimate
// of rounds / throughput; PARAATTN_BM=128|256 forces it, PARAATTN_NO_SPLIT=1 forbids the split.
// `ws_bytes` is what the caller can lend (0: none); q_block limits 256 for block-sparse launches.
static void choose_kernel(AttnParams& p, int D, int q_block, bool dense, size_t ws_bytes, size_t* ws_needed) {
  if (ws_needed) *ws_needed = 0;
  p.pipe = 0;
  p.bm = 128;
  p.split_s = 0;
  auto finish = [&] { p.n_qtiles = (p.Sq + p.bm - 1) / p.bm; };
  if (D != 128 && D != 64) return finish();
  if (p.Skv <= 0 || (uint64_t)(p.Skv - 1) * (uint64_t)p.ks_s * 2 + 256 >= PIPE_OOB ||
      (uint64_t)(p.Skv - 1) * (uint64_t)p.vs_s * 2 + 256 >= PIPE_OOB)
    return finish();
  if (tuning().no_pipe) return finish();  // test aid: the kernels without offset limits
  p.pipe = 1;
  const int forced = tuning().forced_bm;  // tuning aid
  if (D == 64) {  // no key split at head_dim 64; 128 rows unless asked otherwise
    if (forced == 256 && (dense || q_block % 256 == 0)) p.bm = 256;
    return finish();
  }
  if (!dense) {  // block-sparse: workgroups differ in length, no split
    // query blocks that are multiples of 256 rows take 256-row workgroups where there are two or more of them per
    // compute unit (measured on a 30 % mask of 256 x 256 blocks, B1 H24 S32768: 3.46 against 3.54 ms)
    const int cus = device_cus();
    const bool enough = cus > 0 && (int64_t)p.B * p.H * ((p.Sq + 255) / 256) >= (int64_t)2 * cus;
    if (q_block % 256 == 0 && (forced == 256 || (forced == 0 && enough))) p.bm = 256;
    return finish();
  }
  const int cus = device_cus();
  // (causal workgroups differ in length: the rounds estimate does not apply, no split)
  const bool allow = cus > 0 && mi355x_layout() && !p.causal && !tuning().no_split && (ws_needed != nullptr || ws_bytes > 0);
  const int kv_tiles = (p.Skv + BN - 1) / BN;
  const int64_t bh = (int64_t)p.B * p.H;
  const int64_t n128 = bh * ((p.Sq + 127) / 128), n256 = bh * ((p.Sq + 255) / 256);
  SplitPlan p128 = plan_split(n128, 2 * cus, kv_tiles, 128, allow), p256 = plan_split(n256, cus, kv_tiles, 256, allow);
  if (!ws_needed) {  // the plan must fit what was lent
    if (split_ws_bytes(p128, 128) > ws_bytes) p128 = plan_split(n128, 2 * cus, kv_tiles, 128, false);
    if (split_ws_bytes(p256, 256) > ws_bytes) p256 = plan_split(n256, cus, kv_tiles, 256, false);
  }
  // an unsplit last round of 128-row workgroups that leaves every CU at most one of them runs
  // about 1.5 times faster per workgroup
  double r128 = p128.rounds, r256 = p256.rounds;
  if (cus > 0 && p128.s == 1 && n128 % (2 * cus) != 0 && n128 % (2 * cus) <= cus) r128 -= 0.33;
  // measured throughput of a full round of 256-row workgroups against one of 128-row workgroups:
  // +4..10 % from 4608 keys up, -4 % at 512 keys
  const double gain256 = !mi355x_layout() ? 1.0 : kv_tiles >= 32 ? 1.055 : 0.95;
  bool use256 = cus > 0 && n256 >= cus && r256 / gain256 < r128;
  // is_causal: workgroups differ in length and are started longest first, so whole rounds mean nothing; measured
  // (B1, 24..40 heads): 128 rows are 3..12 % faster from 2048 to 32768 keys (the finer grain fills the chip's
  // tail), 256 rows 8 % faster at 119056 (half the tile copies per flop, a third of the reads from beyond the L2)
  if (p.causal) use256 = cus > 0 && n256 >= cus && kv_tiles >= 1024;
  if (forced == 128) use256 = false;
  if (forced == 256) use256 = true;
  const SplitPlan& pl = use256 ? p256 : p128;
  p.bm = use256 ? 256 : 128;
  finish();
  if (ws_needed) *ws_needed = split_ws_bytes(pl, p.bm);
  if (pl.s > 1 && !ws_needed) {
    p.split_s = pl.s;
    p.split_tiles = pl.tiles;
    p.split_main = (int)(bh * p.n_qtiles - pl.tiles);
  }
}

template <bool SPARSE>
static int dispatch_attn(const AttnParams& p, int dtype, int D, hipStream_t stream) {
  if (dtype == PA_DTYPE_BF16) {
    if (D == 128) return launch_attn<BF16, 128, SPARSE>(p, stream);
    return launch_attn<BF16, 64, SPARSE>(p, stream);
  }
  if (D == 128) return launch_attn<F16, 128, SPARSE>(p, stream);
  return launch_attn<F16, 64, SPARSE>(p, stream);
}

// Whether a dense launch of this size is worth the two small launches that bound its scores.  They read Q and K
// once, the attention kernel gains 4 % (head_dim 128, 256 rows) to 6 % (head_dim 64): measured, the reads cost
// 225..300 / S of the kernel's time at Sq = Skv = S (35 us against 17.6 ms at 119k tokens), so the sequences
// must be long (Sq Skv / (Sq + Skv) >= 6144: 12k tokens) and the launch long enough to carry three more launch
// gaps (1e12 flop).  PARAATTN_BOUND=1 asks for the bound at any size, =0 never (tuning and test aid).
static bool bound_wanted(int B, int H, int Sq, int Skv, int D) {
  if ((D != 128 && D != 64) || B <= 0 || H <= 0 || Sq <= 0 || Skv <= 0) return false;
  if (tuning().bound >= 0) return tuning().bound == 1;
  return (double)Sq * Skv >= 6144.0 * ((double)Sq + Skv) && 4.0 * B * H * (double)Sq * (double)Skv * D >= 1.0e12;
}

// The keys and values of a dense launch in several segments of equal length (the blocks of a ring sweep).
struct KeySegs {
  int n, len;
  const void* const* k;
  const void* const* v;
};

// Plan for attn_fwd_d128_stream_kernel (see StreamPlan).  Returns false where that kernel does not apply or is
// not expected to pay; otherwise fills p.st, p.bm, p.n_qtiles, and *ws_need with the bytes of workspace its
// partial results take (0: no piece is cut).  `sizing`: report the plan that a sufficient workspace would get.
static bool plan_stream(AttnParams& p, int D, const KeySegs* segs, size_t ws_avail, bool sizing, size_t* ws_need, bool allow_drawn = true,
                        bool allow_kvlen = false) {
  *ws_need = 0;
  const bool multi = segs != nullptr;
  const int want = tuning().stream;
  if (want == 0 || (want < 0 && tuning().forced_bm != 0)) return false;  // switched off, or a workgroup size of the other kernels asked for
  // per-batch key counts: only for a caller who knows that they leave nearly all keys (the plan is made for all of
  // them, and pieces that end early leave their workgroups idle), one key segment
  if (p.kv_len != nullptr && (!allow_kvlen || multi)) return false;
  if (D != 128 || p.causal || tuning().no_pipe) return false;
  const int cus = device_cus();
  if (cus <= 0) return false;
  const int seg_len = multi ? segs->len : p.Skv, nseg = multi ? segs->n : 1;
  if (seg_len <= 0 || nseg <= 0 || nseg > MAX_KEY_SEGS || p.Sq <= 0) return false;
  if ((uint64_t)(seg_len - 1) * (uint64_t)p.ks_s * 2 + 256 >= PIPE_OOB || (uint64_t)(seg_len - 1) * (uint64_t)p.vs_s * 2 + 256 >= PIPE_OOB)
    return false;
  const int tps = (seg_len + BN - 1) / BN;
  const int64_t L64 = (int64_t)nseg * tps;
  const int nqt = (p.Sq + 255) / 256;
  const int64_t P64 = (int64_t)p.B * p.H * nqt;
  if (L64 > 0x3fffffff || P64 > 0x3fffffff) return false;
  const int L = (int)L64, P = (int)P64;
  // Small problems -- fewer pieces than compute units and no more than 6144 key-tile steps in all -- are left to the
  // kernels with one workgroup per query tile: this kernel would cut every piece into ranges and pay a second
  // launch to fold them, which at 30..80 us per call is 8..40 % (measured over 2..64 heads and 576..4608 tokens).
  if (want < 0 && !multi && P < cus && (int64_t)P * L <= 6144) return false;
  // Taken wherever it applies (measured against attn_fwd_d128_pipe_kernel + key-split tail on one box: 119056 keys
  // +0.6 %, Wan self-attention +0.9 %, a ring sweep's block +3.5 %, the sweep in one launch +1.3 %, 16k / 8k / 6k /
  // 3k tokens +1.5 / +2.4 / +7 / +7 %, FLUX +10..17 %, cross-attention to 512 keys +6 %): the hot loop is the same,
  // and resident workgroups hide what a workgroup per piece pays per piece and cut a ragged last round finely.
  StreamPlan& st = p.st;
  st.G = cus;
  st.xcd_order = mi355x_layout() && (cus & 7) == 0;
  st.R = P / st.G;
  st.L = L;
  st.n_pieces = P;
  st.nseg = nseg;
  st.seg_len = seg_len;
  st.tps = tps;
  st.next_range = nullptr;
  st.solo = 0;
  st.has_kvlen = p.kv_len != nullptr;
  st.n_rounds = 1;
  st.round_at[0] = st.round_at[1] = 0;
  for (int i = 0; i < nseg; ++i) {
    st.kseg[i] = multi ? segs->k[i] : p.k;
    st.vseg[i] = multi ? segs->v[i] : p.v;
  }
  // equal ranges by default: shares of whole pieces that begin at the same keys keep the tail's workgroups in step
  // on the keys, but leave workgroups idle; measured slower or equal at every shape from 3000 to 119056 keys
  const int ev = tuning().stream_even;
  const bool even = ev != 0;
  // Rounds of ever shorter ranges that go to whoever asks first (StreamPlan::next_range), from 2048 key-tile steps per
  // workgroup on.  Workgroups given equal shares finish up to 7 % apart (some XCDs are slower than others, by box);
  // drawn ranges bring that below 1 % and take 1.7 .. 2.9 % off the time of launches of 4 ms and more (119056 keys,
  // Wan self-attention, a ring sweep, 16k tokens x 40 heads) on boxes with such a spread, 0 .. 1 % on boxes whose XCDs
  // run alike.  Their 4 G partial results cost about 35 us to write and fold, which shorter launches do not earn
  // back (+1 .. +8 % from 0.4 to 1.2 ms on any box; between 1024 and 2048 steps -0.6 .. -1 % on a box with the spread,
  // +0.6 .. +1.2 % on one without).
  int dyn = 0;
  if (allow_drawn && even && !tuning().no_split && (sizing || ws_avail > 0)) {
    const int want_dyn = tuning().stream_dyn;
    if (want_dyn > 1) dyn = want_dyn;
    else if (want_dyn < 0 && (int64_t)P * L >= (int64_t)2048 * st.G) dyn = 4;
  }
  int p_tail = P - st.R * st.G;
  if (dyn > 1) {
    // they need a tail worth handing out, a twelfth of the work or more, and long enough for two rounds
    int r = st.R, pt = p_tail;
    while (r > 0 && (int64_t)pt * 12 < P) {
      --r;
      pt += st.G;
    }
    if ((int64_t)pt * L / 4 >= (int64_t)16 * st.G) {
      st.R = r;
      p_tail = pt;
    } else {
      dyn = 0;
    }
  }
  st.Gt = 0;
  if (p_tail > 0) {
    const int64_t t_tail = (int64_t)p_tail * L;
    int gt;
    if (even) {
      const int64_t by_size = t_tail / 8;  // at least 8 key tiles per workgroup
      gt = (int)(by_size < st.G ? (by_size < 1 ? 1 : by_size) : st.G);
    } else {
      int sh = st.G / p_tail;
      if (sh > 8) sh = 8;
      if (sh > L / 16) sh = L / 16;
      if (sh < 1) sh = 1;
      gt = p_tail * sh;
    }
    // rounds of G ranges, each round half of what is left (the last one all of it), none with ranges below 16 steps
    int rounds = 1;
    int64_t at[MAX_TAIL_ROUNDS + 1] = {0};
    if (even && gt == st.G && dyn > 1) {
      int64_t left = t_tail;
      rounds = 0;
      while (rounds + 1 < dyn && rounds + 1 < MAX_TAIL_ROUNDS && left / 4 >= (int64_t)16 * st.G) {
        at[rounds + 1] = at[rounds] + left / 2;
        left -= left / 2;
        ++rounds;
      }
      ++rounds;  // the last round takes what is left
      gt = rounds * st.G;
    }
    if (tuning().no_split) gt = p_tail;
    const size_t per_range = (size_t)2 * 256 * (128 + 1) * sizeof(float);  // two partial results per range
    size_t need = gt != p_tail ? gt * per_range + (rounds > 1 ? 256 : 0) : 0;
    if (need > ws_avail && !sizing && dyn > 1) return plan_stream(p, D, segs, ws_avail, sizing, ws_need, false, allow_kvlen);
    if (need > ws_avail && !sizing) {  // as many ranges as the workspace holds, if that still beats whole pieces
      const int64_t fit = (int64_t)(ws_avail / per_range);
      if (even && fit > p_tail) {
        gt = (int)(fit < st.G ? fit : st.G);
        need = gt * per_range;
      } else {
        gt = p_tail;
        need = 0;
      }
    }
    if (gt <= st.G) rounds = 1;
    st.n_rounds = rounds;
    for (int r = 1; r < rounds; ++r) st.round_at[r] = at[r];
    st.round_at[0] = 0;
    st.round_at[rounds] = t_tail;
    st.Gt = gt;
    *ws_need = need;
  }
  p.pipe = 1;
  p.bm = 256;
  p.n_qtiles = nqt;
  p.split_s = 0;
  return true;
}

// Plan for attn_fwd_d128_short_kernel: 449..512 keys per head, head_dim 128, dense.  By default from 2 pieces per
// compute unit on (measured against the resident-workgroup kernel at 40 heads: level at 1 piece per compute unit,
// 3 % faster from 2 to 10, 5 % at 20); knob short_keys = 1: wherever it applies.
static bool plan_short(AttnParams& p, int D) {
  const int want = tuning().short_keys;
  if (want == 0 || tuning().forced_bm != 0 || tuning().no_pipe) return false;
  if (want < 0 && tuning().stream == 1) return false;  // the resident-workgroup kernel was asked for by name
  if (D != 128 || p.causal || p.kv_len != nullptr || p.Sq <= 0) return false;
  if (p.Skv <= (SHORT_NT - 1) * BN || p.Skv > SHORT_NT * BN) return false;
  const int cus = device_cus();
  if (cus <= 0) return false;
  if ((uint64_t)(p.Skv - 1) * (uint64_t)p.ks_s * 2 + 256 >= PIPE_OOB || (uint64_t)(p.Skv - 1) * (uint64_t)p.vs_s * 2 + 256 >= PIPE_OOB ||
      (uint64_t)(p.Sq + 255) * (uint64_t)p.qs_s * 2 + 256 >= PIPE_OOB || (uint64_t)(p.Sq + 255) * (uint64_t)p.os_s * 2 + 256 >= PIPE_OOB)
    return false;
  const int nqt = (p.Sq + 255) / 256;
  const int64_t P64 = (int64_t)p.B * p.H * nqt;
  if (P64 > 0x3fffffff) return false;
  if (want < 0 && P64 < (int64_t)2 * cus) return false;
  p.st.G = cus;
  p.st.xcd_order = mi355x_layout() && (cus & 7) == 0;
  p.st.n_pieces = (int)P64;
  p.n_qtiles = nqt;
  p.bm = 256;
  p.pipe = 1;
  p.split_s = 0;
  return true;
}

template <typename T>
static int launch_short(const AttnParams& p, hipStream_t stream) {
  if (p.out == nullptr) PA_FAIL(PA_ERR_INVALID, "null output pointer");
  const size_t smem = 4 * TILE_BYTES + 8 * 8192;  // two K and two V tiles, and 8 KB per wavefront for Q rows and outputs
  static bool attr_done[PA_MAX_DEVICES] = {};  // benign race: the call is idempotent
  const int dev = current_device();
  if (dev < 0 || !attr_done[dev]) {
    hipError_t e = hipFuncSetAttribute((const void*)attn_fwd_d128_short_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) PA_FAIL(PA_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    if (dev >= 0) attr_done[dev] = true;
  }
  hipLaunchKernelGGL((attn_fwd_d128_short_kernel<T>), dim3((unsigned)p.st.G), dim3(512), smem, stream, p);
  PA_CHECK_LAUNCH("attention kernel (short keys)");
  return PA_OK;
}

template <typename T, int RB, bool KVLEN>
static int launch_stream_rb(const AttnParams& p, hipStream_t stream) {
  const size_t smem = 4 * TILE_BYTES + 8 * 8192 + 16;  // two K and two V tiles, a staging area for outputs, two words
  static bool attr_done[PA_MAX_DEVICES][2] = {};  // benign race: the call is idempotent
  const int dev = current_device();
  for (int b = 0; b < 2; ++b) {
    if (b == 1 && p.bound_flag == nullptr) break;
    if (dev >= 0 && attr_done[dev][b]) continue;
    const void* fn = b ? (const void*)attn_fwd_d128_stream_kernel<T, true, RB, KVLEN> : (const void*)attn_fwd_d128_stream_kernel<T, false, RB, KVLEN>;
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) PA_FAIL(PA_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    if (dev >= 0) attr_done[dev][b] = true;
  }
  if (p.bound_flag != nullptr) {  // one of the two variants leaves at once
    hipLaunchKernelGGL((attn_fwd_d128_stream_kernel<T, true, RB, KVLEN>), dim3((unsigned)p.st.G), dim3(512 / RB), smem, stream, p);
    PA_CHECK_LAUNCH("attention kernel (resident workgroups, bounded scores)");
  }
  hipLaunchKernelGGL((attn_fwd_d128_stream_kernel<T, false, RB, KVLEN>), dim3((unsigned)p.st.G), dim3(512 / RB), smem, stream, p);
  PA_CHECK_LAUNCH("attention kernel (resident workgroups)");
  return PA_OK;
}

__global__ void clear_word_kernel(int* w, const int* gate, uint32_t gate_mask) {
  if (gate != nullptr && !gate_open(gate, gate_mask)) return;
  *w = 0;
}

template <typename T>
static int launch_stream(const AttnParams& p, hipStream_t stream) {
  if (p.out == nullptr && p.acc_out == nullptr) PA_FAIL(PA_ERR_INVALID, "null output pointer");
  if (p.st.next_range != nullptr) {  // a kernel, not a memset: the call may be under graph capture
    hipLaunchKernelGGL(clear_word_kernel, dim3(1), dim3(1), 0, stream, p.st.next_range, p.gate, p.gate_mask);
    PA_CHECK_LAUNCH("range counter");
  }
  // (per-batch key counts: the form with 32 rows per wavefront only)
  const int rc = p.st.has_kvlen ? launch_stream_rb<T, 1, true>(p, stream)
                 : tuning().wave_rows == 64 ? launch_stream_rb<T, 2, false>(p, stream) : launch_stream_rb<T, 1, false>(p, stream);
  if (rc != PA_OK) return rc;
  const int p_tail = p.st.n_pieces - p.st.R * p.st.G;
  if (p_tail > 0 && p.st.Gt != p_tail) {
    hipLaunchKernelGGL((attn_stream_merge_kernel<T>), dim3((unsigned)p_tail * 16), dim3(256), 0, stream, p);
    PA_CHECK_LAUNCH("attention share merge kernel");
  }
  return PA_OK;
}

// Where launch_bound leaves its flag in `ws`.
static const int* bound_flag_address(const void* ws, int nseg) { return (const int*)((const float*)ws + (size_t)2 * BOUND_G * nseg); }

// Launches the two small kernels that bound the scores (see score_bound_partial_kernel) into `ws` and returns the flag's address.
static int launch_bound(const AttnParams& p, int dtype, int D, const KeySegs* segs, void* ws, hipStream_t st, const int** flag_out) {
  float* part = (float*)ws;
  const int nseg = segs ? segs->n : 1;
  int* flag = (int*)(part + (size_t)2 * BOUND_G * nseg);
  const float limit = dtype == PA_DTYPE_BF16 ? 60.f : 14.f;
  for (int i = 0; i < nseg; ++i) {
    const void* keys = segs ? segs->k[i] : p.k;
    const int n_keys = segs ? segs->len : p.Skv;
    float* dst = part + (size_t)2 * BOUND_G * i;
    if (dtype == PA_DTYPE_BF16 && D == 128)
      hipLaunchKernelGGL((score_bound_partial_kernel<BF16, 128>), dim3(i == 0 ? 2 * BOUND_G : BOUND_G), dim3(256), 0, st, p, dst, keys, n_keys, i == 0 ? 1 : 0);
    else if (dtype == PA_DTYPE_BF16)
      hipLaunchKernelGGL((score_bound_partial_kernel<BF16, 64>), dim3(i == 0 ? 2 * BOUND_G : BOUND_G), dim3(256), 0, st, p, dst, keys, n_keys, i == 0 ? 1 : 0);
    else if (D == 128)
      hipLaunchKernelGGL((score_bound_partial_kernel<F16, 128>), dim3(i == 0 ? 2 * BOUND_G : BOUND_G), dim3(256), 0, st, p, dst, keys, n_keys, i == 0 ? 1 : 0);
    else
      hipLaunchKernelGGL((score_bound_partial_kernel<F16, 64>), dim3(i == 0 ? 2 * BOUND_G : BOUND_G), dim3(256), 0, st, p, dst, keys, n_keys, i == 0 ? 1 : 0);
    PA_CHECK_LAUNCH("score bound kernel");
  }
  hipLaunchKernelGGL(score_bound_flag_kernel, dim3(1), dim3(256), 0, st, (const float*)part, nseg, p.scale_log2, limit, flag);
  PA_CHECK_LAUNCH("score bound flag kernel");
  *flag_out = flag;
  return PA_OK;
}

// Extras of a dense call that pa_attn_fwd_masked makes twice over one workspace, under a gate that lets one run.
struct DenseOpts {
  bool stream_kvlen = false;  // the per-batch key counts leave nearly all keys wherever the gate lets this call run: they may go
                              // to the resident-workgroup kernel, and the call fails if that kernel does not take the shape
  int* bound_done = nullptr;  // in/out: the score bound's words at the front of the workspace are (now) computed
};

static int attn_fwd_dense(const void* q, const void* k, const void* v, void* out, float* lse,
                          int dtype, int B, int H, int Sq, int Skv, int D,
                          const int64_t q_strides[3], const int64_t k_strides[3],
                          const int64_t v_strides[3], const int64_t out_strides[3], float scale,
                          const int32_t* kv_len, int is_causal, void* workspace, size_t workspace_bytes,
                          void* stream, float* acc_out = nullptr, float* acc_lse = nullptr, int acc_first = 0,
                          const int* gate = nullptr, uint32_t gate_mask = 0, const KeySegs* segs = nullptr,
                          const DenseOpts* opts = nullptr) {
  const int64_t zero3[3] = {0, 0, 0};
  const bool accumulate = acc_out != nullptr;
  if (accumulate) {
    if (!acc_lse) PA_FAIL(PA_ERR_INVALID, "null pointer argument");
    if (((uintptr_t)acc_out) % 16) PA_FAIL(PA_ERR_UNSUPPORTED, "accumulator not 16-byte aligned");
    if (!out) out_strides = zero3;
  }
  int rc = check_common(q, k, v, accumulate && !out ? (void*)acc_out : out, dtype, B, H, Sq, Skv, D, q_strides,
                        k_strides, v_strides, out_strides, scale);
  if (rc) return rc;
  if (workspace && ((uintptr_t)workspace) % 16) PA_FAIL(PA_ERR_WORKSPACE, "attention workspace not 16-byte aligned");
  AttnParams p;
  fill_params(p, q, k, v, out, lse, B, H, Sq, Skv, q_strides, k_strides, v_strides, out_strides, scale);
  p.kv_len = kv_len;
  p.causal = is_causal != 0;
  p.gate = gate;
  p.gate_mask = gate_mask;
  if (!accumulate && !segs && plan_short(p, D))
    return dtype == PA_DTYPE_BF16 ? launch_short<BF16>(p, (hipStream_t)stream) : launch_short<F16>(p, (hipStream_t)stream);
  const size_t ws_avail = workspace ? workspace_bytes : 0;
  char* ws_base = (char*)workspace;
  const int nseg = segs ? segs->n : 1;
  // the workspace starts with the score bound's words where there is room for them beside the partial results
  const size_t bound_bytes = bound_ws_bytes(nseg);
  const bool want_bound = bound_wanted(B, H, Sq, Skv, D);
  size_t stream_bytes = 0;
  const bool stream_kvlen = opts != nullptr && opts->stream_kvlen && !accumulate;
  bool streamed = plan_stream(p, D, segs, ws_avail > bound_bytes && want_bound ? ws_avail - bound_bytes : ws_avail, false, &stream_bytes,
                              true, stream_kvlen);
  if (stream_kvlen && !streamed) PA_FAIL(PA_ERR_LAUNCH, "the resident-workgroup kernel does not take this shape (launch plans disagree)");
  if (!streamed) choose_kernel(p, D, 256, true, ws_avail, nullptr);
  if (segs && !streamed) {
    if (D != 128 || !p.pipe || p.causal || kv_len != nullptr || segs->n > MAX_KEY_SEGS ||
        (uint64_t)(segs->len - 1) * (uint64_t)p.ks_s * 2 + 256 >= PIPE_OOB || (uint64_t)(segs->len - 1) * (uint64_t)p.vs_s * 2 + 256 >= PIPE_OOB)
      PA_FAIL(PA_ERR_UNSUPPORTED, "a sweep over key segments needs head_dim 128, at most %d segments, all keys together below 4 GiB per head, no causal mask", MAX_KEY_SEGS);
    if (p.split_s > segs->n) p.split_s = 0;  // a key share is a run of whole segments
    p.st.nseg = segs->n;
    p.st.seg_len = segs->len;
    for (int i = 0; i < segs->n; ++i) {
      p.st.kseg[i] = segs->k[i];
      p.st.vseg[i] = segs->v[i];
    }
  }
  const size_t split_bytes = streamed ? stream_bytes
                             : p.split_s > 1 ? (size_t)p.split_tiles * p.split_s * p.bm * (128 + 1) * sizeof(float) : 0;
  if (want_bound && p.pipe && (D == 64 || p.bm == 256) && ws_avail >= split_bytes + bound_bytes) {
    ws_base += bound_bytes;
    if (opts != nullptr && opts->bound_done != nullptr && *opts->bound_done) {
      p.bound_flag = bound_flag_address(workspace, nseg);
    } else {
      rc = launch_bound(p, dtype, D, segs, workspace, (hipStream_t)stream, &p.bound_flag);
      if (rc) return rc;
      if (opts != nullptr && opts->bound_done != nullptr) *opts->bound_done = 1;
    }
  }
  if (accumulate) {
    if (p.causal) PA_FAIL(PA_ERR_UNSUPPORTED, "ring accumulation is not causal");
    if (!p.pipe || D != 128)  // only the head_dim-128 pipelined kernels have the folding epilogue
      PA_FAIL(PA_ERR_UNSUPPORTED, "ring accumulation needs head_dim 128 and K/V below 4 GiB per head; run pa_attn_fwd_lse and pa_merge_lse");
    p.acc_out = acc_out; p.acc_lse = acc_lse; p.acc_first = acc_first != 0;
    p.lse = nullptr;
  }
  if (streamed) {
    if (stream_bytes > 0) {
      p.ws_out = (float*)ws_base;
      p.ws_lse = p.ws_out + (size_t)2 * p.st.Gt * 256 * 128;
      if (p.st.n_rounds > 1) {
        p.st.next_range = (int*)(ws_base + stream_bytes - 256);
        p.st.solo = tuning().stream_solo && p.st.R == 0;
      }
    }
    if (B == 0 || H == 0 || Sq == 0) return PA_OK;
    return dtype == PA_DTYPE_BF16 ? launch_stream<BF16>(p, (hipStream_t)stream) : launch_stream<F16>(p, (hipStream_t)stream);
  }
  if (p.split_s > 1) {
    p.ws_out = (float*)ws_base;
    p.ws_lse = p.ws_out + (size_t)p.split_tiles * p.split_s * p.bm * 128;
  }
  return dispatch_attn<false>(p, dtype, D, (hipStream_t)stream);
}

extern "C" int pa_attn_fwd_lse(const void* q, const void* k, const void* v, void* out, float* lse,
                               int dtype, int B, int H, int Sq, int Skv, int D,
                               const int64_t q_strides[3], const int64_t k_strides[3],
                               const int64_t v_strides[3], const int64_t out_strides[3],
                               float scale, const int32_t* kv_len, int is_causal, void* stream) {
  return attn_fwd_dense(q, k, v, out, lse, dtype, B, H, Sq, Skv, D, q_strides, k_strides, v_strides,
                        out_strides, scale, kv_len, is_causal, nullptr, 0, stream);
}

extern "C" int pa_attn_fwd_lse_ws(const void* q, const void* k, const void* v, void* out, float* lse,
                                  int dtype, int B, int H, int Sq, int Skv, int D,
                                  const int64_t q_strides[3], const int64_t k_strides[3],
                                  const int64_t v_strides[3], const int64_t out_strides[3],
                                  float scale, const int32_t* kv_len, int is_causal, void* workspace,
                                  size_t workspace_bytes, void* stream) {
  return attn_fwd_dense(q, k, v, out, lse, dtype, B, H, Sq, Skv, D, q_strides, k_strides, v_strides,
                        out_strides, scale, kv_len, is_causal, workspace, workspace_bytes, stream);
}

extern "C" int pa_attn_fwd_accumulate(const void* q, const void* k, const void* v, float* acc_out,
                                      float* acc_lse, void* out, int dtype, int B, int H, int Sq,
                                      int Skv, int D, const int64_t q_strides[3],
                                      const int64_t k_strides[3], const int64_t v_strides[3],
                                      const int64_t out_strides[3], float scale,
                                      const int32_t* kv_len, int first, void* workspace,
                                      size_t workspace_bytes, void* stream) {
  if (!acc_out || !acc_lse) PA_FAIL(PA_ERR_INVALID, "null pointer argument");
  if (out && !out_strides) PA_FAIL(PA_ERR_INVALID, "null pointer argument");
  return attn_fwd_dense(q, k, v, out, nullptr, dtype, B, H, Sq, Skv, D, q_strides, k_strides, v_strides,
                        out_strides, scale, kv_len, 0, workspace, workspace_bytes, stream, acc_out, acc_lse, first);
}

extern "C" int pa_attn_fwd_sweep(const void* q, const void* const* k_blocks, const void* const* v_blocks, int n_blocks,
                                 int block_len, void* out, float* lse, int dtype, int B, int H, int Sq, int D,
                                 const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                                 const int64_t out_strides[3], float scale, void* workspace, size_t workspace_bytes,
                                 void* stream) {
  if (!k_blocks || !v_blocks) PA_FAIL(PA_ERR_INVALID, "null pointer argument");
  if (n_blocks <= 0 || n_blocks > MAX_KEY_SEGS) PA_FAIL(PA_ERR_UNSUPPORTED, "a sweep takes 1 to %d key/value blocks (got %d)", MAX_KEY_SEGS, n_blocks);
  if (block_len <= 0) PA_FAIL(PA_ERR_INVALID, "key/value blocks must not be empty");
  if ((int64_t)n_blocks * block_len > 0x7fffffffLL) PA_FAIL(PA_ERR_UNSUPPORTED, "too many keys");
  for (int i = 0; i < n_blocks; ++i) {
    if (!k_blocks[i] || !v_blocks[i]) PA_FAIL(PA_ERR_INVALID, "null pointer argument");
    if (((uintptr_t)k_blocks[i]) % 16 || ((uintptr_t)v_blocks[i]) % 16) PA_FAIL(PA_ERR_UNSUPPORTED, "key/value block pointer not 16-byte aligned");
  }
  if (D != 128) PA_FAIL(PA_ERR_UNSUPPORTED, "a sweep over key/value blocks needs head_dim 128 (got %d)", D);
  const KeySegs segs = {n_blocks, block_len, k_blocks, v_blocks};
  return attn_fwd_dense(q, k_blocks[0], v_blocks[0], out, lse, dtype, B, H, Sq, n_blocks * block_len, D, q_strides,
                        k_strides, v_strides, out_strides, scale, nullptr, 0, workspace, workspace_bytes, stream,
                        nullptr, nullptr, 0, nullptr, 0, &segs);
}

extern "C" size_t pa_attn_fwd_sweep_workspace_bytes(int B, int H, int Sq, int n_blocks, int block_len, int D,
                                                    const int64_t k_strides[3], const int64_t v_strides[3]) {
  if (B <= 0 || H <= 0 || Sq <= 0 || n_blocks <= 0 || n_blocks > MAX_KEY_SEGS || block_len <= 0 || D != 128 || !k_strides || !v_strides) return 0;
  AttnParams p;
  const int64_t zero[3] = {0, 0, 0};
  fill_params(p, nullptr, nullptr, nullptr, nullptr, nullptr, B, H, Sq, n_blocks * block_len, zero, k_strides, v_strides, zero, 1.f);
  const void* none[MAX_KEY_SEGS] = {};
  const KeySegs segs = {n_blocks, block_len, none, none};
  size_t need = 0;
  if (!plan_stream(p, D, &segs, 0, true, &need)) {
    choose_kernel(p, D, 256, true, 0, &need);
    if (!p.pipe) return 0;
  }
  if (bound_wanted(B, H, Sq, n_blocks * block_len, D) && p.bm == 256) need += bound_ws_bytes(n_blocks);
  return need;
}

// Workspace of a dense call: partial results of the plan plus the score bound's words.  which = 0: the plan of a
// call without per-batch key counts and is_causal (resident workgroups where they apply); 1: the plan of a call
// with per-batch key counts (one workgroup per query tile, key-split tail); 2: the plan of an is_causal call
// (never split: only the score bound's words); WS_ANY: the largest of them.
constexpr int WS_ANY = 3;
static size_t dense_ws_need(int B, int H, int Sq, int Skv, int D, const int64_t k_strides[3], const int64_t v_strides[3], int which,
                            bool allow_drawn = true) {
  const int64_t zero[3] = {0, 0, 0};
  size_t best = 0;
  for (int plan = 0; plan < 3; ++plan) {
    if (which != WS_ANY && which != plan) continue;
    AttnParams p;
    fill_params(p, nullptr, nullptr, nullptr, nullptr, nullptr, B, H, Sq, Skv, zero, k_strides, v_strides, zero, 1.f);
    p.causal = plan == 2;
    size_t need = 0;
    if (plan != 0 || !plan_stream(p, D, nullptr, 0, true, &need, allow_drawn)) {
      need = 0;
      choose_kernel(p, D, 256, true, 0, &need);
    }
    if (bound_wanted(B, H, Sq, Skv, D) && p.pipe && (D == 64 || p.bm == 256)) need += BOUND_WS_BYTES;
    if (need > best) best = need;
  }
  return best;
}

extern "C" size_t pa_attn_fwd_workspace_bytes(int B, int H, int Sq, int Skv, int D,
                                              const int64_t k_strides[3], const int64_t v_strides[3]) {
  if (B <= 0 || H <= 0 || Sq <= 0 || Skv <= 0 || (D != 128 && D != 64) || !k_strides || !v_strides) return 0;
  // the larger of what the two plans ask for: which of them a call gets depends on arguments this function does not
  // see (per-batch key counts and is_causal go to attn_fwd_d128_pipe_kernel)
  return dense_ws_need(B, H, Sq, Skv, D, k_strides, v_strides, WS_ANY);
}

extern "C" size_t pa_attn_fwd_call_workspace_bytes(int B, int H, int Sq, int Skv, int D, const int64_t k_strides[3],
                                                   const int64_t v_strides[3], int has_kv_len, int is_causal) {
  if (B <= 0 || H <= 0 || Sq <= 0 || Skv <= 0 || (D != 128 && D != 64) || !k_strides || !v_strides) return 0;
  return dense_ws_need(B, H, Sq, Skv, D, k_strides, v_strides, is_causal ? 2 : has_kv_len ? 1 : 0);
}

// The generic kernel with an attention mask (any head_dim it is built for, any strides).
template <typename T, int D>
static int launch_masked(const AttnParams& p, int mask_kind, hipStream_t stream) {
  const int64_t nblocks = (int64_t)p.B * p.H * p.n_qtiles;
  if (nblocks == 0) return PA_OK;
  const void* fn = mask_kind == MASK_BOOL ? (const void*)attn_fwd_kernel<T, D, false, MASK_BOOL>
                   : mask_kind == MASK_F32 ? (const void*)attn_fwd_kernel<T, D, false, MASK_F32>
                                           : (const void*)attn_fwd_kernel<T, D, false, MASK_ACT>;
  const size_t smem = Smem<D>::BYTES;
  static bool attr_done[PA_MAX_DEVICES][4] = {};  // benign race: the call is idempotent
  const int dev = current_device();
  if (dev < 0 || !attr_done[dev][mask_kind]) {
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) PA_FAIL(PA_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    if (dev >= 0) attr_done[dev][mask_kind] = true;
  }
  if (mask_kind == MASK_BOOL)
    hipLaunchKernelGGL((attn_fwd_kernel<T, D, false, MASK_BOOL>), dim3((unsigned)nblocks), dim3(NTHREADS), smem, stream, p);
  else if (mask_kind == MASK_F32)
    hipLaunchKernelGGL((attn_fwd_kernel<T, D, false, MASK_F32>), dim3((unsigned)nblocks), dim3(NTHREADS), smem, stream, p);
  else
    hipLaunchKernelGGL((attn_fwd_kernel<T, D, false, MASK_ACT>), dim3((unsigned)nblocks), dim3(NTHREADS), smem, stream, p);
  PA_CHECK_LAUNCH("masked attention kernel");
  return PA_OK;
}

// Whether a dense call with per-batch key counts that leave nearly all keys would go to the resident-workgroup
// kernel: where that kernel takes the shape with `ws_avail` bytes of workspace and the launch is long enough for its
// advantage over the kernel with one workgroup per query tile to outweigh a third, empty launch: from 512 key-tile
// steps per workgroup on (measured with 100 keys masked: +5 / +1 % at 121 / 216 steps, level at 384, -0.7 .. -1 % at
// 576 .. 640, -2 .. -3 % from 1536 on, -5 % at the 119k-token shape).
static bool stream_takes_key_counts(int B, int H, int Sq, int Skv, int D, const int64_t k_strides[3], const int64_t v_strides[3], size_t ws_avail) {
  if (B <= 0 || H <= 0 || Sq <= 0 || Skv <= 0 || D != 128) return false;
  const int64_t zero[3] = {0, 0, 0};
  static const int32_t some_count = 0;
  AttnParams p;
  fill_params(p, nullptr, nullptr, nullptr, nullptr, nullptr, B, H, Sq, Skv, zero, k_strides, v_strides, zero, 1.f);
  p.kv_len = &some_count;  // never read: only its presence counts for the plan
  const size_t bound_bytes = bound_ws_bytes(1);
  const bool want_bound = bound_wanted(B, H, Sq, Skv, D);
  size_t need = 0;
  if (!plan_stream(p, D, nullptr, ws_avail > bound_bytes && want_bound ? ws_avail - bound_bytes : ws_avail, false, &need, true, true)) return false;
  return (int64_t)p.st.n_pieces * p.st.L >= (int64_t)512 * p.st.G;
}

// Words at the front of pa_attn_fwd_masked's workspace: kept-key counts per batch element and the flag, then three
// words per batch element and chunk of MASK_CHUNK keys (kept keys, last kept key, first position among the kept).
static int mask_chunks(int Skv) { return (Skv + MASK_CHUNK - 1) / MASK_CHUNK; }
static size_t mask_scan_bytes(int B, int Skv) {
  return (((size_t)B + 1 + (size_t)3 * B * mask_chunks(Skv)) * sizeof(int32_t) + 255) & ~(size_t)255;
}

// pa_attn_fwd_masked's workspace when it gathers the kept keys of a mask with holes: the scan's words, dense copies
// of K and V [B][H][Skv][D], then the workspace of the dense launches.
struct MaskedLayout {
  size_t kc, vc, dense;
};
static MaskedLayout masked_layout(int B, int H, int Skv, int D) {
  auto up = [](size_t n) { return (n + 255) & ~(size_t)255; };
  MaskedLayout l;
  l.kc = mask_scan_bytes(B, Skv);
  l.vc = l.kc + up((size_t)B * H * Skv * D * 2);
  l.dense = l.vc + up((size_t)B * H * Skv * D * 2);
  return l;
}

extern "C" size_t pa_attn_fwd_masked_workspace_bytes(int B, int H, int Sq, int Skv, int D,
                                                     const int64_t k_strides[3], const int64_t v_strides[3]) {
  if (B <= 0) return 0;
  const size_t dense = pa_attn_fwd_workspace_bytes(B, H, Sq, Skv, D, k_strides, v_strides);
  if (H <= 0 || Sq <= 0 || Skv <= 0 || (D != 128 && D != 64)) return mask_scan_bytes(B, Skv > 0 ? Skv : 1) + dense;
  // room to gather the kept keys of a mask with holes (from 3e11 flop on; see pa_attn_fwd_masked), and for the dense
  // launches over the gathered copies, whose strides are those of contiguous tensors
  if (4.0 * B * H * (double)Sq * (double)Skv * D < 3.0e11) return mask_scan_bytes(B, Skv > 0 ? Skv : 1) + dense;
  const int64_t cs[3] = {(int64_t)H * Skv * D, (int64_t)Skv * D, D};
  const size_t dense_c = pa_attn_fwd_workspace_bytes(B, H, Sq, Skv, D, cs, cs);
  return masked_layout(B, H, Skv, D).dense + (dense > dense_c ? dense : dense_c);
}

extern "C" int pa_attn_fwd_masked(const void* q, const void* k, const void* v, void* out, float* lse,
                                  int dtype, int B, int H, int Sq, int Skv, int D,
                                  const int64_t q_strides[3], const int64_t k_strides[3],
                                  const int64_t v_strides[3], const int64_t out_strides[3], float scale,
                                  const void* mask, int mask_kind, const int64_t mask_strides[4],
                                  void* workspace, size_t workspace_bytes, void* stream) {
  int rc = check_common(q, k, v, out, dtype, B, H, Sq, Skv, D, q_strides, k_strides, v_strides, out_strides, scale);
  if (rc) return rc;
  if (mask_kind != MASK_BOOL && mask_kind != MASK_F32 && mask_kind != MASK_ACT)
    PA_FAIL(PA_ERR_INVALID, "mask kind %d is none of PA_MASK_BOOL, PA_MASK_F32, PA_MASK_ACT", mask_kind);
  if (!mask_strides) PA_FAIL(PA_ERR_INVALID, "null pointer argument");
  const bool any = B > 0 && H > 0 && Sq > 0 && Skv > 0;
  if (any && !mask) PA_FAIL(PA_ERR_INVALID, "null pointer argument");
  for (int i = 0; i < 4; ++i)
    if (mask_strides[i] < 0) PA_FAIL(PA_ERR_UNSUPPORTED, "mask has a negative stride");
  if (workspace && ((uintptr_t)workspace) % 16) PA_FAIL(PA_ERR_WORKSPACE, "attention workspace not 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  AttnParams p;
  fill_params(p, q, k, v, out, lse, B, H, Sq, Skv, q_strides, k_strides, v_strides, out_strides, scale);
  p.bm = BM;
  p.n_qtiles = (Sq + BM - 1) / BM;
  p.mask = mask;
  p.ms_b = mask_strides[0]; p.ms_h = mask_strides[1]; p.ms_q = mask_strides[2]; p.ms_k = mask_strides[3];
  // A boolean mask that only selects keys (the same for every head and query row; what the text padding of
  // video DiTs looks like) is usually a prefix per batch element.  Whether it is, is found out on the device: a
  // small scan writes the kept-key counts and a flag, then both the dense launch (counts as kv_len) and the
  // masked launch are enqueued, and the one the flag does not select leaves at once.  Nothing is read back.
  const bool key_only = mask_kind == MASK_BOOL && (H == 1 || p.ms_h == 0) && (Sq == 1 || p.ms_q == 0);
  const size_t scan = mask_scan_bytes(B, Skv > 0 ? Skv : 1);
  if (key_only && any && workspace && workspace_bytes >= scan) {
    int32_t* words = (int32_t*)workspace;
    const int* flag = words + B;  // bit 0: prefixes; bit 1: at least 7/8 of the keys kept everywhere
    constexpr uint32_t PREFIX_FEWER = 1u << 1, PREFIX_MOST = 1u << 3, HOLES_FEWER = 1u << 0, HOLES_MOST = 1u << 2;
    // A mask with holes (what the reference's sequence-parallel HunyuanVideo adapter builds: every rank's text
    // padding ends up inside the gathered sequence, context_parallel/diffusers_adapters/hunyuan_video.py:86-100) is
    // served as the reference's attention_forward_sparse_kv serves it (ops/__init__.py:276-296): the kept K and V
    // rows are gathered into dense copies, on which the fast kernels run with the counts as kv_len.  From 3e11 flop
    // on (0.3 ms), where a handful of launches that return at once no longer count, and where the workspace has room.
    const MaskedLayout lay = masked_layout(B, H, Skv, D);
    const double flops = 4.0 * B * H * (double)Sq * (double)Skv * D;
    const bool gather = flops >= 3.0e11 && workspace_bytes >= lay.dense;
    const size_t dense_off = gather ? lay.dense : scan;
    char* const dense_ws = (char*)workspace + dense_off;
    const size_t dense_bytes = workspace_bytes - dense_off;
    const int nchunk = mask_chunks(Skv);
    int32_t* const chunk_cnt = words + B + 1;
    int32_t* const chunk_last = chunk_cnt + (size_t)B * nchunk;
    int32_t* const chunk_off = chunk_last + (size_t)B * nchunk;
    if (gather || Skv > 8192) {
      hipLaunchKernelGGL(key_mask_chunk_kernel, dim3(nchunk, B), dim3(256), 0, st, (const uint8_t*)mask, p.ms_b, p.ms_k, Skv, nchunk, chunk_cnt, chunk_last);
      PA_CHECK_LAUNCH("key mask chunk kernel");
      hipLaunchKernelGGL(key_mask_scan_kernel, dim3(1), dim3(256), 0, st, B, Skv, nchunk, (const int32_t*)chunk_cnt, (const int32_t*)chunk_last, chunk_off, words);
      PA_CHECK_LAUNCH("key mask scan kernel");
    } else {
      hipLaunchKernelGGL(key_mask_small_kernel, dim3(1), dim3(1024), 0, st, (const uint8_t*)mask, p.ms_b, p.ms_k, B, Skv, words);
      PA_CHECK_LAUNCH("key mask kernel");
    }
    int bound_done = 0;
    DenseOpts most, fewer;
    most.stream_kvlen = true;
    most.bound_done = fewer.bound_done = &bound_done;
    // Longer launches whose counts leave nearly all keys (a text prompt's padding in 119k tokens) go to the
    // resident-workgroup kernel, whose plan is made for all keys: one more launch, of which again only one runs.
    // All dense launches of the call share one workspace and one score bound (computed over all keys).
    bool dual = stream_takes_key_counts(B, H, Sq, Skv, D, k_strides, v_strides, dense_bytes);
    if (dual) {
      rc = attn_fwd_dense(q, k, v, out, lse, dtype, B, H, Sq, Skv, D, q_strides, k_strides, v_strides, out_strides,
                          scale, words, 0, dense_ws, dense_bytes, stream, nullptr, nullptr, 0, flag, PREFIX_MOST, nullptr, &most);
      if (rc) return rc;
    }
    rc = attn_fwd_dense(q, k, v, out, lse, dtype, B, H, Sq, Skv, D, q_strides, k_strides, v_strides, out_strides,
                        scale, words, 0, dense_ws, dense_bytes, stream, nullptr, nullptr, 0, flag,
                        dual ? PREFIX_FEWER : PREFIX_FEWER | PREFIX_MOST, nullptr, &fewer);
    if (rc) return rc;
    if (gather) {
      uint16_t* const kc = (uint16_t*)((char*)workspace + lay.kc);
      uint16_t* const vc = (uint16_t*)((char*)workspace + lay.vc);
      AttnParams g = p;
      g.gate = flag;
      g.gate_mask = HOLES_FEWER | HOLES_MOST;
      if (D == 128)
        hipLaunchKernelGGL((gather_kept_keys_kernel<128>), dim3(nchunk, H, B), dim3(256), 0, st, g, (const uint8_t*)mask, p.ms_b, p.ms_k, nchunk,
                           (const int32_t*)words, (const int32_t*)chunk_off, kc, vc);
      else
        hipLaunchKernelGGL((gather_kept_keys_kernel<64>), dim3(nchunk, H, B), dim3(256), 0, st, g, (const uint8_t*)mask, p.ms_b, p.ms_k, nchunk,
                           (const int32_t*)words, (const int32_t*)chunk_off, kc, vc);
      PA_CHECK_LAUNCH("key gather kernel");
      const int64_t cs[3] = {(int64_t)H * Skv * D, (int64_t)Skv * D, D};
      dual = stream_takes_key_counts(B, H, Sq, Skv, D, cs, cs, dense_bytes);
      if (dual) {
        rc = attn_fwd_dense(q, kc, vc, out, lse, dtype, B, H, Sq, Skv, D, q_strides, cs, cs, out_strides,
                            scale, words, 0, dense_ws, dense_bytes, stream, nullptr, nullptr, 0, flag, HOLES_MOST, nullptr, &most);
        if (rc) return rc;
      }
      return attn_fwd_dense(q, kc, vc, out, lse, dtype, B, H, Sq, Skv, D, q_strides, cs, cs, out_strides,
                            scale, words, 0, dense_ws, dense_bytes, stream, nullptr, nullptr, 0, flag,
                            dual ? HOLES_FEWER : HOLES_FEWER | HOLES_MOST, nullptr, &fewer);
    }
    p.gate = flag;
    p.gate_mask = HOLES_FEWER | HOLES_MOST;
  }
  if (!any) {  // no rows, or no keys: the dense path writes what an empty softmax gives
    return attn_fwd_dense(q, k, v, out, lse, dtype, B, H, Sq, Skv, D, q_strides, k_strides, v_strides, out_strides,
                          scale, nullptr, 0, nullptr, 0, stream);
  }
  if (dtype == PA_DTYPE_BF16) return D == 128 ? launch_masked<BF16, 128>(p, mask_kind, st) : launch_masked<BF16, 64>(p, mask_kind, st);
  return D == 128 ? launch_masked<F16, 128>(p, mask_kind, st) : launch_masked<F16, 64>(p, mask_kind, st);
}

// ---------------------------------------------------------------------------------------------
// The dense op for callers that cannot allocate (code under HIP graph capture, tight serving loops):
// the workspace of pa_attn_fwd_lse_ws lives in a file-scope device array instead of coming from the
// caller.  Every device the library runs on holds its own copy of the array, at its own address,
// until the process ends; host code must not pass the array's name to a kernel (on the host it is
// only a stand-in for the symbol), so the device address is looked up once per device with
// hipGetSymbolAddress and that pointer is what the kernels receive.
// ---------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[PA_NOALLOC_SCRATCH_BYTES];

// Device address of `scratch` on the current device, looked up at the first call on that device.
static int scratch_address(void** out) {
  static std::atomic<void*> addr[PA_MAX_DEVICES];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) PA_FAIL(PA_ERR_LAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= PA_MAX_DEVICES) PA_FAIL(PA_ERR_UNSUPPORTED, "device index %d beyond the %d this library keeps state for", dev, PA_MAX_DEVICES);
  void* p = addr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) PA_FAIL(PA_ERR_LAUNCH, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    addr[dev].store(p, std::memory_order_release);  // benign race: every thread stores the same address
  }
  *out = p;
  return PA_OK;
}

extern "C" int pa_attn_fwd_lse_noalloc(const void* q, const void* k, const void* v, void* out, float* lse,
                                       int dtype, int B, int H, int Sq, int Skv, int D,
                                       const int64_t q_strides[3], const int64_t k_strides[3],
                                       const int64_t v_strides[3], const int64_t out_strides[3],
                                       float scale, const int32_t* kv_len, int is_causal, void* stream) {
  // what the same problem would ask of a caller's workspace (0 for sizes that use none)
  const bool shaped = B > 0 && H > 0 && Sq > 0 && Skv > 0 && (D == 128 || D == 64) && k_strides && v_strides;
  // (the plan with one tail range per workgroup: the one a call falls back to when the workspace cannot hold the
  // partial results of drawn ranges, which take four times as many)
  const size_t need = shaped ? dense_ws_need(B, H, Sq, Skv, D, k_strides, v_strides, is_causal ? 2 : kv_len != nullptr ? 1 : 0, false) : 0;
  if (need > (size_t)PA_NOALLOC_SCRATCH_BYTES)
    PA_FAIL(PA_ERR_WORKSPACE, "this problem's launch plan needs %zu bytes of scratch, the static buffer holds %zu: "
            "call pa_attn_fwd_lse_ws with a workspace of your own", need, (size_t)PA_NOALLOC_SCRATCH_BYTES);
  void* ws = nullptr;
  if (need > 0) {
    const int rc = scratch_address(&ws);
    if (rc) return rc;
  }
  return attn_fwd_dense(q, k, v, out, lse, dtype, B, H, Sq, Skv, D, q_strides, k_strides, v_strides,
                        out_strides, scale, kv_len, is_causal, ws, ws ? (size_t)PA_NOALLOC_SCRATCH_BYTES : 0, stream);
}

// The lists of paired query blocks (build_pair_runs_kernel): half the segments, up to nK + 2 ranges each.
static size_t pair_runs_bytes(int Hm, int nQ, int nK) {
  const size_t nseg = (size_t)nQ / 2 + 2;
  const size_t cap = (size_t)nK + 3;
  return sizeof(int32_t) * ((size_t)Hm * nseg + (size_t)Hm * nseg * cap * 2);
}

// Room for either form of the lists (per query block: up to nK / 2 + 2 ranges each; per pair of query blocks).
extern "C" size_t pa_blocksparse_workspace_bytes(int Hm, int nQ, int nK) {
  if (Hm <= 0 || nQ <= 0 || nK <= 0) return 0;
  const size_t nseg = (size_t)nQ + 2;
  const size_t cap = (size_t)nK / 2 + 3;
  const size_t single = sizeof(int32_t) * ((size_t)Hm * nseg + (size_t)Hm * nseg * cap * 2 + (size_t)2 * Hm * nQ);  // the lists, the launch order, the kept blocks per list
  const size_t pairs = pair_runs_bytes(Hm, nQ, nK);
  return single > pairs ? single : pairs;
}

// Where the launch order of the query blocks lies in a buffer of single-block lists (words from its start).
static size_t order_offset_words(int Hm, int nQ, int nK) {
  const size_t nseg = (size_t)nQ + 2;
  const size_t cap = (size_t)nK / 2 + 3;
  return (size_t)Hm * nseg + (size_t)Hm * nseg * cap * 2;
}

extern "C" int pa_blocksparse_build_runs(const uint8_t* block_mask, int Hm, int nQ, int nK, int Skv,
                                         int kv_lo, int kv_block, int32_t* runs_ws,
                                         size_t runs_ws_bytes, void* stream) {
  if (!block_mask || !runs_ws) PA_FAIL(PA_ERR_INVALID, "null pointer argument");
  if (Hm <= 0 || nQ <= 0 || nK <= 0 || kv_block <= 0 || kv_lo < 0 || Skv < 0)
    PA_FAIL(PA_ERR_INVALID, "bad block mask geometry");
  if ((int64_t)kv_lo + (int64_t)nK * kv_block > Skv)
    PA_FAIL(PA_ERR_INVALID, "key blocks [%d + %d*%d) exceed Skv=%d", kv_lo, nK, kv_block, Skv);
  if (runs_ws_bytes < pa_blocksparse_workspace_bytes(Hm, nQ, nK))
    PA_FAIL(PA_ERR_WORKSPACE, "runs workspace too small");
  const int total = Hm * (nQ + 2);
  const int cap = nK / 2 + 3;
  int32_t* const order = runs_ws + order_offset_words(Hm, nQ, nK);
  int32_t* const kept = order + (size_t)Hm * nQ;
  const bool ranked = nQ <= SPARSE_ORDER_MAX_BLOCKS;
  hipLaunchKernelGGL(build_runs_kernel, dim3(total), dim3(64), 0, (hipStream_t)stream,
                     block_mask, Hm, nQ, nK, Skv, kv_lo, kv_block, cap, runs_ws, ranked ? kept : nullptr);
  PA_CHECK_LAUNCH("build_runs_kernel");
  if (ranked) {
    hipLaunchKernelGGL(sparse_order_kernel, dim3(Hm), dim3(256), (size_t)nQ * sizeof(int), (hipStream_t)stream,
                       (const int32_t*)kept, nQ, order);
    PA_CHECK_LAUNCH("sparse_order_kernel");
  }
  return PA_OK;
}

// Shared tail of the two block-sparse entry points: `runs` already holds the key ranges.
static int blocksparse_launch(const void* q, const void* k, const void* v, void* out, float* lse, int dtype,
                              int B, int H, int Sq, int Skv, int D, const int64_t q_strides[3],
                              const int64_t k_strides[3], const int64_t v_strides[3],
                              const int64_t out_strides[3], float scale, int Hm, int nQ, int nK, int q_lo,
                              int q_block, const int32_t* runs, void* stream, bool pair = false) {
  AttnParams p;
  fill_params(p, q, k, v, out, lse, B, H, Sq, Skv, q_strides, k_strides, v_strides, out_strides, scale);
  p.runs = runs;
  p.Hm = Hm; p.nQ = nQ; p.cap = nK / 2 + 3;
  p.q_lo = q_lo; p.q_block = q_block;
  if (!pair && nQ <= SPARSE_ORDER_MAX_BLOCKS && tuning().sparse_order) p.order = runs + order_offset_words(Hm, nQ, nK);
  choose_kernel(p, D, (q_block % 256 == 0 && q_lo % 256 == 0) ? 256 : 128, false, 0, nullptr);
  if (pair) {  // `runs` holds the lists of pairs: 256-row workgroups over nQ / 2 double blocks
    if (!p.pipe || D != 128 || q_block != 128 || nQ % 2 != 0 || q_lo % 256 != 0)
      PA_FAIL(PA_ERR_UNSUPPORTED, "paired query blocks need the pipelined head_dim-128 kernel, 128-row blocks in even number from a multiple of 256");
    p.pair = 1;
    p.bm = 256;
    p.nQ = nQ / 2;
    p.q_block = 256;
    p.cap = nK + 3;
    nQ = p.nQ;
    q_block = 256;
  }
  p.tiles_left = (q_lo + p.bm - 1) / p.bm;
  p.tiles_per_block = (q_block + p.bm - 1) / p.bm;
  const int q_hi = q_lo + nQ * q_block;
  const int tiles_right = (Sq - q_hi + p.bm - 1) / p.bm;
  p.n_qtiles = p.tiles_left + nQ * p.tiles_per_block + tiles_right;
  if (D == 128 && p.pipe && !tuning().no_xcd_order && mi355x_layout())
    p.xcd_chunk = (int)(((int64_t)B * H * p.n_qtiles + 7) / 8);
  return dispatch_attn<true>(p, dtype, D, (hipStream_t)stream);
}

static int blocksparse_check(const void* q, const void* k, const void* v, void* out, int dtype, int B, int H,
                             int Sq, int Skv, int D, const int64_t* qs, const int64_t* ks, const int64_t* vs,
                             const int64_t* os, float scale, int Hm, int nQ, int nK, int q_lo, int q_block) {
  int rc = check_common(q, k, v, out, dtype, B, H, Sq, Skv, D, qs, ks, vs, os, scale);
  if (rc) return rc;
  if (Hm != 1 && Hm != H) PA_FAIL(PA_ERR_INVALID, "block mask heads must be 1 or H=%d (got %d)", H, Hm);
  if (nQ <= 0 || nK <= 0) PA_FAIL(PA_ERR_INVALID, "bad block mask geometry");
  if (q_block <= 0 || q_lo < 0 || (int64_t)q_lo + (int64_t)nQ * q_block > Sq)
    PA_FAIL(PA_ERR_INVALID, "query blocks [%d + %d*%d) exceed Sq=%d", q_lo, nQ, q_block, Sq);
  return PA_OK;
}

extern "C" int pa_attn_fwd_blocksparse(const void* q, const void* k, const void* v, void* out,
                                       float* lse, int dtype, int B, int H, int Sq, int Skv, int D,
                                       const int64_t q_strides[3], const int64_t k_strides[3],
                                       const int64_t v_strides[3], const int64_t out_strides[3],
                                       float scale, const uint8_t* block_mask, int Hm, int nQ, int nK,
                                       int q_lo, int q_block, int kv_lo, int kv_block,
                                       int32_t* runs_ws, size_t runs_ws_bytes, void* stream) {
  int rc = blocksparse_check(q, k, v, out, dtype, B, H, Sq, Skv, D, q_strides, k_strides, v_strides, out_strides,
                             scale, Hm, nQ, nK, q_lo, q_block);
  if (rc) return rc;
  // two 128-row query blocks per workgroup (tuning knob, off by default): their own lists in the same workspace
  const uint64_t kv_span = Skv > 0 ? (uint64_t)(Skv - 1) * 2 : 0;
  if (tuning().sparse_pair && !tuning().no_pipe && D == 128 && q_block == 128 && nQ % 2 == 0 && q_lo % 256 == 0 &&
      kv_lo % 4 == 0 && kv_block % 4 == 0 && Skv % 4 == 0 && Skv > 0 && block_mask && runs_ws && kv_block > 0 &&
      kv_lo >= 0 && (int64_t)kv_lo + (int64_t)nK * kv_block <= Skv &&
      kv_span * (uint64_t)k_strides[2] + 256 < PIPE_OOB && kv_span * (uint64_t)v_strides[2] + 256 < PIPE_OOB &&
      runs_ws_bytes >= pair_runs_bytes(Hm, nQ, nK)) {
    hipLaunchKernelGGL(build_pair_runs_kernel, dim3(Hm * (nQ / 2 + 2)), dim3(64), 0, (hipStream_t)stream,
                       block_mask, Hm, nQ, nK, Skv, kv_lo, kv_block, nK + 3, runs_ws);
    PA_CHECK_LAUNCH("build_pair_runs_kernel");
    return blocksparse_launch(q, k, v, out, lse, dtype, B, H, Sq, Skv, D, q_strides, k_strides, v_strides,
                              out_strides, scale, Hm, nQ, nK, q_lo, q_block, runs_ws, stream, true);
  }
  rc = pa_blocksparse_build_runs(block_mask, Hm, nQ, nK, Skv, kv_lo, kv_block, runs_ws, runs_ws_bytes, stream);
  if (rc) return rc;
  return blocksparse_launch(q, k, v, out, lse, dtype, B, H, Sq, Skv, D, q_strides, k_strides, v_strides,
                            out_strides, scale, Hm, nQ, nK, q_lo, q_block, runs_ws, stream);
}

extern "C" int pa_attn_fwd_blocksparse_runs(const void* q, const void* k, const void* v, void* out,
                                            float* lse, int dtype, int B, int H, int Sq, int Skv, int D,
                                            const int64_t q_strides[3], const int64_t k_strides[3],
                                            const int64_t v_strides[3], const int64_t out_strides[3],
                                            float scale, int Hm, int nQ, int nK, int q_lo, int q_block,
                                            const int32_t* runs, size_t runs_bytes, void* stream) {
  int rc = blocksparse_check(q, k, v, out, dtype, B, H, Sq, Skv, D, q_strides, k_strides, v_strides, out_strides,
                             scale, Hm, nQ, nK, q_lo, q_block);
  if (rc) return rc;
  if (!runs) PA_FAIL(PA_ERR_INVALID, "null pointer argument");
  if (runs_bytes < pa_blocksparse_workspace_bytes(Hm, nQ, nK)) PA_FAIL(PA_ERR_WORKSPACE, "runs buffer too small for this mask geometry");
  return blocksparse_launch(q, k, v, out, lse, dtype, B, H, Sq, Skv, D, q_strides, k_strides, v_strides,
                            out_strides, scale, Hm, nQ, nK, q_lo, q_block, runs, stream);
}
