// Latent attention on the matrix cores (gfx950, bf16): prefill tiles and decode rows in one kernel.
//
// In latent space every head of a token attends over the SAME entries (latent | rotated key part,
// RANK + ROT values per token), so a work item is a tile of up to 64 query slots = (token, head) pairs
// of one sequence, token-major: consecutive tokens x all heads for prefill chunks (heads <= 64), one
// token's heads (in runs of 64) for decode rows.  The tile walks its sequence's pages; a page is
// exactly one key tile (64 entries, contiguous in the pool).
//
// Workgroup = 4 waves; wave w owns slots 16 w .. 16 w + 15 end to end (its queries stay in registers
// as MFMA B operands, its output accumulators [16 slots x RANK] too), so the waves share nothing but
// the staged page:
//   K image  [64 keys][RANK + ROT]  (+16 B row padding): A operand of  S^T = K Q^T
//   V^T image [RANK][64 keys]       (+16 B row padding): A operand of  O^T = V^T P^T
// The V^T image is made while staging: a thread loads a 4-key x 8-channel block (coalesced 16-byte
// loads), stores its rows into the K image and the 4 x 8 transpose into the V^T image.  The keys of
// the V^T image are permuted so that the 8 keys a lane owns in the S^T accumulators (v_mfma 16x16x32:
// lane = query l % 16, keys 4 (l / 16) + e of four 16-key tiles) are 16 contiguous bytes: P goes from
// the S accumulators into the second product without leaving the lane.  (The 16-byte chunks of a V^T row
// are XOR-swizzled with (row / 8) % 8: the transposing stores of neighbouring lanes lie 8 rows apart.)
// The next page's global loads are issued before the current page is multiplied.
//
// Softmax state (running max, sum) is fp32 per slot; an optional per-head sink logit starts the state
// (max = sink, sum = 1).  With key-range splits every split writes unnormalised partial outputs and
// (max, sum) to a workspace and a merge kernel adds the sink and normalises.
#include "common.h"

namespace {

struct LatTile {
  int seq, row0, n_tok, pos0, head0, hcount;
};

__device__ __forceinline__ u32x4 ld16(const uint16_t* p) { return *reinterpret_cast<const u32x4*>(p); }

template <int RANK, int ROT>
__global__ __launch_bounds__(256) void latent_mfma_kernel(
    const uint16_t* __restrict__ q_lat, long ql_row, long ql_head, const uint16_t* __restrict__ q_rot, long qr_row,
    long qr_head, const uint16_t* __restrict__ cache, long page_stride, const int* __restrict__ block_tables,
    int bt_stride, const int* __restrict__ tiles, const int* __restrict__ positions, int heads,
    const float* __restrict__ sink, uint16_t* __restrict__ out, long o_row, long o_head, float scale, int splits,
    float* __restrict__ ws_o, float* __restrict__ ws_ml) {
  constexpr int ENTRY = RANK + ROT;
  constexpr int KS = ENTRY / 32;
  constexpr int DT = RANK / 16;
  constexpr int PK = ENTRY * 2 + 16;
  constexpr int PV = 64 * 2 + 16;
  constexpr int NBLK = 2 * RANK;              // 4-key x 8-channel blocks of the latent part: 16 key quads x RANK / 8
  constexpr int RB = (NBLK + 255) / 256;      // of which a thread takes this many
  constexpr int CB = ROT / 32;    // 16-byte chunks of the rotated part per thread
  extern __shared__ __attribute__((aligned(16))) char lds[];
  char* kimg = lds;
  char* vimg = lds + 64 * PK;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c16 = lane & 15, g = lane >> 4;
  LatTile t;
  if (tiles) {
    const int* e = tiles + 6 * blockIdx.x;
    t = {e[0], e[1], e[2], e[3], e[4], e[5]};
  } else {  // decode rows: row r is sequence r, one token, its heads in runs of 64
    const int runs = (heads + 63) >> 6;
    const int row = blockIdx.x / runs, h0 = (blockIdx.x % runs) << 6;
    t = {row, row, 1, positions[row], h0, min(64, heads - h0)};
  }
  if (t.seq < 0) return;
  const int slot = wave * 16 + c16;
  const bool valid = slot < t.n_tok * t.hcount;
  const bool wave_active = wave * 16 < t.n_tok * t.hcount;  // wave-uniform
  const int tok = valid ? slot / t.hcount : 0;
  const int head = t.head0 + (valid ? slot % t.hcount : 0);
  const long row = t.row0 + tok;
  const int my_pos = valid ? t.pos0 + tok : -1;
  const int n_pages = (t.pos0 + t.n_tok + PAGE - 1) / PAGE;
  const int per = (n_pages + splits - 1) / splits;
  const int p_begin = blockIdx.y * per, p_end = min(n_pages, p_begin + per);
  const int* bt = block_tables + (long)t.seq * bt_stride;

  bf16x8 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d = 32 * ks + 8 * g;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (valid)
      v = d < RANK ? ld16(q_lat + row * ql_row + head * ql_head + d) : ld16(q_rot + row * qr_row + head * qr_head + (d - RANK));
    qf[ks] = __builtin_bit_cast(bf16x8, v);
  }
  const bool seeded = splits == 1 && sink != nullptr && valid;
  float m = seeded ? sink[head] : -INFINITY;
  float l = seeded ? 1.f : 0.f;
  f32x4 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = (f32x4){0.f, 0.f, 0.f, 0.f};

  // staging registers: the page's latent part in 4-key x 8-channel blocks, its rotated part in chunks
  u32x4 rb[RB][4];
  u32x4 cb[CB > 0 ? CB : 1];
  auto fetch = [&](int p) {
    const uint16_t* src = cache + (long)bt[p] * page_stride;
#pragma unroll
    for (int b = 0; b < RB; ++b) {
      const int id = tid + 256 * b, dc = id % (RANK / 8), kq = id / (RANK / 8);
      if (id < NBLK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) rb[b][i] = ld16(src + (long)(4 * kq + i) * ENTRY + 8 * dc);
      }
    }
#pragma unroll
    for (int b = 0; b < CB; ++b) {
      const int id = tid + 256 * b, dc = id % (ROT / 8), key = id / (ROT / 8);
      cb[b] = ld16(src + (long)key * ENTRY + RANK + 8 * dc);
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int b = 0; b < RB; ++b) {
      const int id = tid + 256 * b, dc = id % (RANK / 8), kq = id / (RANK / 8);
      if (id >= NBLK) continue;
#pragma unroll
      for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(kimg + (4 * kq + i) * PK + 16 * dc) = rb[b][i];
      // keys 4 kq .. 4 kq + 3 = 16 n + 4 gg + e  ->  image position (n / 2) * 32 + gg * 8 + (n % 2) * 4 + e
      // = 16-byte chunk (n / 2) * 4 + gg, half n % 2.  Rows 8 dc .. 8 dc + 7 are written by one lane and
      // consecutive lanes hold consecutive dc, 8 rows = 1152 B apart: the chunk index is XORed with dc % 8
      // (= (row / 8) % 8, which the reader undoes) so that those lanes spread over the banks.
      const int n = kq >> 2, gg = kq & 3;
      const int koff = ((((n >> 1) * 4 + gg) ^ (dc & 7)) << 4) + ((n & 1) << 3);
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const uint32_t a0 = rb[b][0][w], a1 = rb[b][1][w], a2 = rb[b][2][w], a3 = rb[b][3][w];
        u32x2 even = {(a0 & 0xffffu) | (a1 << 16), (a2 & 0xffffu) | (a3 << 16)};
        u32x2 odd = {(a0 >> 16) | (a1 & 0xffff0000u), (a2 >> 16) | (a3 & 0xffff0000u)};
        *reinterpret_cast<u32x2*>(vimg + (8 * dc + 2 * w) * PV + koff) = even;
        *reinterpret_cast<u32x2*>(vimg + (8 * dc + 2 * w + 1) * PV + koff) = odd;
      }
    }
#pragma unroll
    for (int b = 0; b < CB; ++b) {
      const int id = tid + 256 * b, dc = id % (ROT / 8), key = id / (ROT / 8);
      *reinterpret_cast<u32x4*>(kimg + key * PK + 2 * RANK + 16 * dc) = cb[b];
    }
  };

  // V^T fragment of (d tile dt, key half kk): row 16 dt + c16, chunk (4 kk + g) ^ ((row / 8) % 8); the row's
  // share of the swizzle is (2 dt) % 8 | c16 / 8, so eight lane offsets cover every dt
  int voff[2][4];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk)
#pragma unroll
    for (int j = 0; j < 4; ++j) voff[kk][j] = c16 * PV + (((kk * 4 + g) ^ (c16 >> 3) ^ (2 * j)) << 4);

  if (p_begin < p_end) fetch(p_begin);
  for (int p = p_begin; p < p_end; ++p) {
    __syncthreads();  // the previous page's fragment reads are done
    stash();
    __syncthreads();
    if (p + 1 < p_end) fetch(p + 1);  // in flight while this page is multiplied
    if (!wave_active) continue;       // a wave without slots (decode rows of few heads) only helps staging

    f32x4 s[4];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) s[nt] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(kimg + (16 * nt + c16) * PK + (32 * ks + 8 * g) * 2);
        s[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qf[ks], s[nt], 0, 0, 0);
      }
    float mx = -INFINITY;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int key = p * PAGE + 16 * nt + 4 * g + e;
        const float v = key <= my_pos ? s[nt][e] * scale : -INFINITY;
        s[nt][e] = v;
        mx = fmaxf(mx, v);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float mn = fmaxf(m, mx);
    const bool dead = mn == -INFINITY;  // nothing seen so far and nothing visible here
    const float corr = (dead || m == -INFINITY) ? (dead ? 1.f : 0.f) : __expf(m - mn);
    float ps = 0.f;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float pv = dead ? 0.f : __expf(s[nt][e] - mn);
        s[nt][e] = pv;
        ps += pv;
      }
    ps += __shfl_xor(ps, 16, 64);
    ps += __shfl_xor(ps, 32, 64);
    l = l * corr + ps;
    m = mn;
    bf16x8 pf[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      u32x4 w = {pack_bf16x2(s[2 * kk][0], s[2 * kk][1]), pack_bf16x2(s[2 * kk][2], s[2 * kk][3]),
                 pack_bf16x2(s[2 * kk + 1][0], s[2 * kk + 1][1]), pack_bf16x2(s[2 * kk + 1][2], s[2 * kk + 1][3])};
      pf[kk] = __builtin_bit_cast(bf16x8, w);
    }
    if (!__all(corr == 1.f)) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) o[dt] *= corr;
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(vimg + voff[kk][dt & 3] + dt * 16 * PV);
        o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pf[kk], o[dt], 0, 0, 0);
      }
    }
  }

  if (!valid) return;
  if (splits == 1) {
    const float inv = l > 0.f ? 1.f / l : 0.f;
    uint16_t* dst = out + row * o_row + head * o_head + 4 * g;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      u32x2 w = {pack_bf16x2(o[dt][0] * inv, o[dt][1] * inv), pack_bf16x2(o[dt][2] * inv, o[dt][3] * inv)};
      *reinterpret_cast<u32x2*>(dst + 16 * dt) = w;
    }
  } else {
    const long rec = ((long)blockIdx.x * splits + blockIdx.y) * 64 + slot;
    float* dst = ws_o + rec * RANK + 4 * g;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<f32x4*>(dst + 16 * dt) = o[dt];
    if (g == 0) {
      ws_ml[2 * rec] = m;
      ws_ml[2 * rec + 1] = l;
    }
  }
}

// One workgroup per (tile, slot): out = sum_s o_s exp(m_s - M) / (sum_s l_s exp(m_s - M) + exp(sink - M))
__global__ __launch_bounds__(128) void latent_merge_kernel(const float* __restrict__ ws_o, const float* __restrict__ ws_ml,
                                                           const int* __restrict__ tiles, int heads,
                                                           const float* __restrict__ sink, uint16_t* __restrict__ out,
                                                           long o_row, long o_head, int splits, int rank) {
  const int tile = blockIdx.x, slot = blockIdx.y;
  int row0, n_tok, head0, hcount;
  if (tiles) {
    const int* e = tiles + 6 * tile;
    if (e[0] < 0) return;
    row0 = e[1], n_tok = e[2], head0 = e[4], hcount = e[5];
  } else {
    const int runs = (heads + 63) >> 6;
    row0 = tile / runs, n_tok = 1, head0 = (tile % runs) << 6, hcount = min(64, heads - head0);
  }
  if (slot >= n_tok * hcount) return;
  const long row = row0 + slot / hcount;
  const int head = head0 + slot % hcount;
  float big = sink ? sink[head] : -INFINITY;
  for (int s = 0; s < splits; ++s) big = fmaxf(big, ws_ml[2 * (((long)tile * splits + s) * 64 + slot)]);
  float den = sink ? __expf(sink[head] - big) : 0.f;
  for (int s = 0; s < splits; ++s) {
    const long rec = ((long)tile * splits + s) * 64 + slot;
    const float ms = ws_ml[2 * rec];
    if (ms != -INFINITY) den += ws_ml[2 * rec + 1] * __expf(ms - big);
  }
  const float inv = den > 0.f ? 1.f / den : 0.f;
  for (int d = threadIdx.x; d < rank; d += 128) {
    float a = 0.f;
    for (int s = 0; s < splits; ++s) {
      const long rec = ((long)tile * splits + s) * 64 + slot;
      const float ms = ws_ml[2 * rec];
      if (ms != -INFINITY) a += ws_o[rec * rank + d] * __expf(ms - big);
    }
    const bf16_t v = (bf16_t)(a * inv);
    out[row * o_row + head * o_head + d] = __builtin_bit_cast(uint16_t, v);
  }
}

template <int RANK, int ROT>
int launch(const void* q_lat, long ql_row, long ql_head, const void* q_rot, long qr_row, long qr_head,
           const void* cache, long page_stride, const int* block_tables, int bt_stride, const int* tiles,
           const int* positions, int n_tiles, int heads, const float* sink, void* out, long o_row, long o_head,
           float scale, int splits, float* ws_o, float* ws_ml, hipStream_t st) {
  constexpr int LDS = 64 * ((RANK + ROT) * 2 + 16) + RANK * (64 * 2 + 16);
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)latent_mfma_kernel<RANK, ROT>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            LDS) != hipSuccess)
      return -2;
    attr_set = true;
  }
  latent_mfma_kernel<RANK, ROT><<<dim3(n_tiles, splits), dim3(256), LDS, st>>>(
      (const uint16_t*)q_lat, ql_row, ql_head, (const uint16_t*)q_rot, qr_row, qr_head, (const uint16_t*)cache,
      page_stride, block_tables, bt_stride, tiles, positions, heads, sink, (uint16_t*)out, o_row, o_head, scale,
      splits, ws_o, ws_ml);
  if (splits > 1)
    latent_merge_kernel<<<dim3(n_tiles, 64), dim3(128), 0, st>>>(ws_o, ws_ml, tiles, heads, sink, (uint16_t*)out,
                                                                 o_row, o_head, splits, RANK);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

}  // namespace

// 1 when the matrix-core kernel tiles entries of this shape
// (latent entries: rank + rot; expanded per-head entries of a prefill: value | unrotated key | rotated key part,
// rank = value channels, rot = the key's channels)
#define LAT_SHAPES(X) \
  X(64, 32) X(64, 64) X(128, 32) X(128, 64) X(256, 32) X(256, 64) X(512, 32) X(512, 64) \
  X(32, 64) X(64, 96) X(64, 128) X(128, 128) X(128, 192)

VPSA_EXPORT int vpsa_latent_mfma_supported(int rank, int rot) {
#define LAT_IS(R, C) if (rank == R && rot == C) return 1;
  LAT_SHAPES(LAT_IS)
#undef LAT_IS
  return 0;
}

// tiles: int32 [n_tiles, 6] = (sequence, first query row, tokens, position of the first token, first head,
// heads per token) with tokens * heads <= 64 and sequence < 0 for an unused entry; null = decode rows
// (n_tiles = rows * ceil(heads / 64), positions [rows]).  Row and head strides in elements; every query
// and output vector 16-byte / 8-byte aligned.  splits > 1 needs ws_o [n_tiles * splits * 64 * rank] and
// ws_ml [n_tiles * splits * 64 * 2] floats.
VPSA_EXPORT int vpsa_latent_attention_mfma(const void* q_lat, long ql_row, long ql_head, const void* q_rot,
                                           long qr_row, long qr_head, const void* cache, long page_stride,
                                           const int* block_tables, int bt_stride, const int* tiles,
                                           const int* positions, int n_tiles, int heads, const float* sink, void* out,
                                           long o_row, long o_head, int rank, int rot, float scale, int splits,
                                           float* ws_o, float* ws_ml, hipStream_t st) {
  if (n_tiles <= 0) return 0;
  if (splits < 1 || splits > 65535 || (splits > 1 && (!ws_o || !ws_ml)) || (!tiles && !positions)) return -1;
  if (((ql_row | ql_head | qr_row | qr_head) & 7) || ((o_row | o_head) & 3) || (page_stride & 7)) return -1;
#define LAT_CASE(R, C)                                                                                              \
  if (rank == R && rot == C)                                                                                        \
    return launch<R, C>(q_lat, ql_row, ql_head, q_rot, qr_row, qr_head, cache, page_stride, block_tables, bt_stride, \
                        tiles, positions, n_tiles, heads, sink, out, o_row, o_head, scale, splits, ws_o, ws_ml, st);
  LAT_SHAPES(LAT_CASE)
#undef LAT_CASE
  return -1;
}
