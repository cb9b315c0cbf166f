// MFMA kernel for windowed latent attention with sinks (bf16 storage).
//
// All heads of a token score the SAME cached row [rank + rot] and sum the same
// latent, so the natural matrix shape is: rows = (token, head) pairs, columns =
// keys.  One workgroup (4 waves) owns 64 such rows — 64/H consecutive tokens of
// one sequence times its H heads (or one token and 64 heads of it when H > 64)
// — and walks the keys its tokens can see in tiles of 32.  A single decoding
// token is the case "one token per workgroup".
//
// Per tile:
//   stage   the 32 rows are copied once into LDS (K image, padded rows) and
//           their latent part once more transposed (V^T image) — every wave
//           and every head reuses both
//   scores  swapped operands, S^T = K . Q^T on v_mfma_f32_16x16x32_bf16: a lane
//           then holds 8 scores of ONE query row, so max and sum need two
//           xor-shuffles, and the bf16 probabilities are already laid out as
//           the B operand of the next product (the key order inside the
//           contraction is permuted to match; the V^T image is stored in that
//           same slot order so its A fragments are single 16-byte reads)
//   values  O^T += V^T . P^T, rank/16 accumulator tiles per wave, rescaled by
//           the per-row online-softmax factor
// The next tile's global loads are issued one tile ahead into registers, the
// workgroup's slice of the block table sits in LDS, and single-query steps let
// the waves that share a row tile split the latent dims (and, for small
// batches, slice the keys over workgroups with a merge kernel).
// Scores, softmax statistics and accumulators are f32; the sink enters the
// denominator at the end.  Window and causality are applied per element from
// the row's position.  Shapes are compile-time (rank/16, (rank+rot)/32) for a
// fixed list; other shapes use the general kernel.

#include "common.h"

typedef __attribute__((ext_vector_type(8))) short bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __hip_bfloat16 bf16;

#define LM_THREADS 256
#define LM_ROWS 64
#define LM_KT 32
#define LM_KPAD 8
#define LM_VROW 40
#define LM_BT_MAX 512    // block-table entries kept in LDS per workgroup

DEVINLINE short f32_to_bf16_bits(float x) {
  return __builtin_bit_cast(short, __float2bfloat16(x));
}

// DS = 1: the four waves own four 16-row tiles (64 rows).  DS = 4 / 2: at most
// 16 / 32 rows (a single query of <= 16 / 32 heads): the waves that share a row
// tile all score it and each owns a quarter / half of the latent dims for the
// value product — fewer accumulators per wave, so two workgroups fit a CU.
template <int NT, int KS, int DS>
__global__ __launch_bounds__(LM_THREADS) void latent_attn_mfma_kernel(
    bf16* __restrict__ out, long o_st, long o_sh,
    const bf16* __restrict__ q_lat, long ql_st, long ql_sh,
    const bf16* __restrict__ q_rot, long qr_st, long qr_sh,
    const bf16* __restrict__ cache, const int* __restrict__ block_tables,
    int bt_stride, const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    const float* __restrict__ sinks, float scale, int window, int heads, int tq,
    int hpb, int block_size, int nsplit, int two_term,
    float* __restrict__ part_acc, float* __restrict__ part_ml) {
  constexpr int RANK = NT * 16;
  constexpr int D = KS * 32;
  constexpr int KROW = D + LM_KPAD;
  constexpr int NTW = NT / DS;     // accumulator tiles per wave
  // Double-buffered images (stage tile i+1 under tile i's products, two
  // barriers per tile) measured SLOWER than single buffers: the doubled LDS
  // halves the workgroups per CU, and residency is what hides the latencies.
  constexpr bool DB = false;
  constexpr int IMG = LM_KT * KROW + RANK * LM_VROW;   // one K image + one V^T image
  extern __shared__ char lds_raw[];
  bf16* k_img = reinterpret_cast<bf16*>(lds_raw);   // [32][KROW]
  bf16* v_img = k_img + LM_KT * KROW;               // [RANK][LM_VROW]
  int* bt_s = reinterpret_cast<int*>(k_img + (DB ? 2 : 1) * IMG);   // [LM_BT_MAX]

  const int seq = blockIdx.y;
  int q0, nq;
  if (qsl != nullptr) {
    q0 = qsl[seq];
    nq = qsl[seq + 1] - q0;
  } else {
    q0 = seq;
    nq = 1;
  }
  const int slen = seq_lens[seq];
  // nsplit > 1 (single-query steps only): blockIdx.x is a slice of the keys
  const int split = (nsplit > 1) ? blockIdx.x : 0;
  const int t0 = (nsplit > 1) ? 0 : blockIdx.x * tq;
  if (t0 >= nq) return;
  const int nt = min(tq, nq - t0);
  const int h0 = blockIdx.z * hpb;
  const int nh = min(hpb, heads - h0);
  const int nrows = nt * nh;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 15, g = lane >> 4;
  constexpr int RT = 4 / DS;
  const int rt = wave % RT;              // row tile of this wave
  const int dp = wave / RT;              // dim part of this wave
  const int r = rt * 16 + n;
  const bool row_ok = r < nrows;
  const int tl = row_ok ? r / nh : 0;
  const int head = h0 + (row_ok ? r % nh : 0);
  const long qrow = q0 + t0 + tl;
  bf16* orow = out + qrow * o_st + head * o_sh;

  if (slen <= 0) {   // padding row of a captured bucket
    if (row_ok && split == 0 && dp == 0)
      for (int k = g; k < RANK; k += 4) orow[k] = __float2bfloat16(0.f);
    if (nsplit > 1 && row_ok && g == 0 && dp == 0) {
      float* ml = part_ml + (((long)seq * nsplit + split) * heads + head) * 2;
      ml[0] = -INFINITY;
      ml[1] = -1.f;     // tells the merge: nothing to do, the row is zero already
    }
    return;
  }

  const int pos0 = slen - nq + t0;
  int kend = pos0 + nt;
  int kstart = (window > 0) ? max(0, pos0 - window + 1) : 0;
  if (nsplit > 1) {
    const int per = ((kend - kstart + nsplit - 1) / nsplit + LM_KT - 1) / LM_KT * LM_KT;
    kstart = kstart + split * per;
    kend = min(kend, kstart + per);
  }
  const int qpos = pos0 + tl;
  const int klo = (window > 0) ? qpos - window + 1 : 0;
  const int* bt = block_tables + (long)seq * bt_stride;
  const bool wave_active = rt * 16 < nrows;

  // The block-table entries of this workgroup's key range go to LDS once: a
  // tile's row addresses then depend on no global load (a table read in the
  // loop would put two memory latencies in series per tile).
  const int bs_shift = ((block_size & (block_size - 1)) == 0) ? __ffs(block_size) - 1 : -1;
  const int blk0 = (kstart < kend ? kstart : 0) / block_size;
  const int nblk = (kstart < kend) ? (kend - 1) / block_size - blk0 + 1 : 0;
  const bool bt_in_lds = nblk <= LM_BT_MAX;
  if (bt_in_lds)
    for (int i = tid; i < nblk; i += LM_THREADS) bt_s[i] = bt[blk0 + i];
  __syncthreads();
  auto row_offset = [&](int kk) -> long {
    const int b = (bs_shift >= 0) ? (kk >> bs_shift) : (kk / block_size);
    const int in = kk - b * block_size;
    const int phys = bt_in_lds ? bt_s[b - blk0] : bt[b];
    return ((long)phys * block_size + in) * D;
  };

  bf16x8_t qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int dim = ks * 32 + g * 8;
    bf16x8_t v = {};
    if (row_ok) {
      const bf16* src = (dim < RANK)
          ? q_lat + qrow * ql_st + head * ql_sh + dim
          : q_rot + qrow * qr_st + head * qr_sh + (dim - RANK);
      v = *reinterpret_cast<const bf16x8_t*>(src);
    }
    qf[ks] = v;
  }

  f32x4_t acc[NTW];
#pragma unroll
  for (int i = 0; i < NTW; ++i) acc[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_part = 0.f;

  // global loads of a tile are issued one tile ahead and parked in registers:
  // their latency hides under the previous tile's products
  constexpr int CPR = D / 8;                                     // 16-byte chunks per row
  constexpr int CPT = (LM_KT * CPR + LM_THREADS - 1) / LM_THREADS;  // chunks per thread
  bf16x8_t pre[CPT];
  auto fetch = [&](int base) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * LM_THREADS;
      if (c < LM_KT * CPR) {
        const int key = c / CPR, ch = c - key * CPR;
        const int kk = min(base + key, kend - 1);
        pre[i] = *reinterpret_cast<const bf16x8_t*>(cache + row_offset(kk) + ch * 8);
      }
    }
  };
  // pieces of one tile's work; `kb` / `vb` pick the image buffers
  auto write_k = [&](bf16* kb) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + i * LM_THREADS;
      if (c < LM_KT * CPR) {
        const int key = c / CPR, ch = c - key * CPR;
        *reinterpret_cast<bf16x8_t*>(kb + key * KROW + ch * 8) = pre[i];
      }
    }
  };
  // latent part once more, transposed, keys in contraction-slot order
  auto transpose = [&](const bf16* kb, bf16* vb) {
    for (int c = tid; c < LM_KT * (RANK / 8); c += LM_THREADS) {
      const int key = c & 31, ch = c >> 5;
      const bf16x8_t v = *reinterpret_cast<const bf16x8_t*>(kb + key * KROW + ch * 8);
      const int slot = ((key & 15) >> 2) * 8 + (key >> 4) * 4 + (key & 3);
      short* dst = reinterpret_cast<short*>(vb) + (ch * 8) * LM_VROW + slot;
#pragma unroll
      for (int u = 0; u < 8; ++u) dst[u * LM_VROW] = v[u];
    }
  };
  bf16x8_t pb;   // this tile's probabilities, B operand of the value product
  // two_term: what rounding to bf16 left of them, a second B operand, so that
  // the weights reach the value product with 16 mantissa bits
  bf16x8_t pb_rest = {};
  auto scores = [&](const bf16* kb, int base) {
    f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
    if (wave_active) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const bf16x8_t a0 = *reinterpret_cast<const bf16x8_t*>(
            kb + n * KROW + ks * 32 + g * 8);
        const bf16x8_t a1 = *reinterpret_cast<const bf16x8_t*>(
            kb + (16 + n) * KROW + ks * 32 + g * 8);
        s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, qf[ks], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, qf[ks], s1, 0, 0, 0);
      }
    }
    float sv[8];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int kk = base + (i >> 2) * 16 + 4 * g + (i & 3);
      const bool ok = row_ok && kk <= qpos && kk >= klo;
      const float s = (i < 4 ? s0[i & 3] : s1[i & 3]) * scale;
      sv[i] = ok ? s : -INFINITY;
      mx = fmaxf(mx, sv[i]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE_SIZE));
    mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE_SIZE));
    const float m_new = fmaxf(m_run, mx);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = (m_run == -INFINITY) ? 0.f : __expf(m_run - m_safe);
    float ps = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float p = (sv[i] == -INFINITY) ? 0.f : __expf(sv[i] - m_safe);
      ps += p;
      pb[i] = f32_to_bf16_bits(p);
      if (two_term)
        pb_rest[i] = f32_to_bf16_bits(
            p - __uint_as_float(((unsigned)(unsigned short)pb[i]) << 16));
    }
    l_part = l_part * alpha + ps;
    m_run = m_new;
#pragma unroll
    for (int i = 0; i < NTW; ++i) {
      acc[i][0] *= alpha; acc[i][1] *= alpha; acc[i][2] *= alpha; acc[i][3] *= alpha;
    }
  };
  auto values = [&](const bf16* vb) {
    if (wave_active) {
#pragma unroll
      for (int dt = 0; dt < NTW; ++dt) {
        const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(
            vb + ((dp * NTW + dt) * 16 + n) * LM_VROW + g * 8);
        acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb, acc[dt], 0, 0, 0);
        if (two_term)
          acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb_rest, acc[dt], 0, 0, 0);
      }
    }
  };

  if (DB) {
    // Two image buffers: tile i+1 is staged (K image written, latent part
    // transposed) while tile i is scored and summed — two barriers per tile,
    // and the staging LDS traffic fills the gaps between dependent MFMAs.
    bf16* kbuf[2] = {k_img, k_img + IMG};
    bf16* vbuf[2] = {v_img, v_img + IMG};
    if (kstart < kend) {
      fetch(kstart);
      write_k(kbuf[0]);
      if (kstart + LM_KT < kend) fetch(kstart + LM_KT);
      __syncthreads();
      transpose(kbuf[0], vbuf[0]);
    }
    int cur = 0;
    for (int base = kstart; base < kend; base += LM_KT, cur ^= 1) {
      const bool has_next = base + LM_KT < kend;
      __syncthreads();   // images of `cur` complete; nobody reads the other pair
      if (has_next) {
        write_k(kbuf[cur ^ 1]);
        if (base + 2 * LM_KT < kend) fetch(base + 2 * LM_KT);
      }
      scores(kbuf[cur], base);
      __syncthreads();   // next K image complete
      if (has_next) transpose(kbuf[cur ^ 1], vbuf[cur ^ 1]);
      values(vbuf[cur]);
    }
  } else {
    if (kstart < kend) fetch(kstart);
    for (int base = kstart; base < kend; base += LM_KT) {
      __syncthreads();   // readers of the previous tile's images are done
      write_k(k_img);
      if (base + LM_KT < kend) fetch(base + LM_KT);
      __syncthreads();
      transpose(k_img, v_img);
      scores(k_img, base);
      __syncthreads();   // V^T image complete
      values(v_img);
    }
  }

  float l = l_part;
  l += __shfl_xor(l, 16, WAVE_SIZE);
  l += __shfl_xor(l, 32, WAVE_SIZE);
  if (nsplit > 1) {
    // unnormalised slice result; the merge kernel adds the sink and divides
    if (row_ok) {
      const long pr = ((long)seq * nsplit + split) * heads + head;
      if (g == 0 && dp == 0) {
        part_ml[pr * 2] = m_run;
        part_ml[pr * 2 + 1] = l;
      }
#pragma unroll
      for (int dt = 0; dt < NTW; ++dt)
        *reinterpret_cast<f32x4_t*>(part_acc + pr * RANK + (dp * NTW + dt) * 16 + 4 * g) = acc[dt];
    }
    return;
  }
  float rescale = 1.f;
  if (sinks != nullptr) {
    const float sk = sinks[head];
    const float m_fin = fmaxf(m_run, sk);
    rescale = (m_run == -INFINITY) ? 0.f : __expf(m_run - m_fin);
    l = l * rescale + __expf(sk - m_fin);
  }
  const float inv = (l > 0.f) ? rescale / l : 0.f;
  if (row_ok) {
#pragma unroll
    for (int dt = 0; dt < NTW; ++dt) {
      union { short s[4]; uint2 v; } o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o.s[i] = f32_to_bf16_bits(acc[dt][i] * inv);
      *reinterpret_cast<uint2*>(orow + (dp * NTW + dt) * 16 + 4 * g) = o.v;
    }
  }
}

// Sum of the key slices of a single-query step: out = sum_s acc_s e^(m_s - m)
// / (sum_s l_s e^(m_s - m) + e^(sink - m)), m the max over slices and sink.
__global__ void latent_attn_merge_kernel(bf16* __restrict__ out, long o_st, long o_sh,
                                         const float* __restrict__ part_acc,
                                         const float* __restrict__ part_ml,
                                         const float* __restrict__ sinks,
                                         int nsplit, int heads, int rank) {
  const int seq = blockIdx.x, head = blockIdx.y;
  const long p0 = ((long)seq * nsplit) * heads + head;
  if (part_ml[p0 * 2 + 1] < 0.f) return;   // padding row, zeroed by the slices
  float m = (sinks != nullptr) ? sinks[head] : -INFINITY;
  for (int s = 0; s < nsplit; ++s) m = fmaxf(m, part_ml[(p0 + (long)s * heads) * 2]);
  float l = (sinks != nullptr) ? __expf(sinks[head] - m) : 0.f;
  for (int s = 0; s < nsplit; ++s) {
    const float ms = part_ml[(p0 + (long)s * heads) * 2];
    if (ms != -INFINITY) l += part_ml[(p0 + (long)s * heads) * 2 + 1] * __expf(ms - m);
  }
  const float inv = (l > 0.f) ? 1.f / l : 0.f;
  bf16* orow = out + seq * o_st + head * o_sh;
  for (int k = threadIdx.x; k < rank; k += blockDim.x) {
    float a = 0.f;
    for (int s = 0; s < nsplit; ++s) {
      const long pr = p0 + (long)s * heads;
      const float ms = part_ml[pr * 2];
      if (ms != -INFINITY) a += part_acc[pr * rank + k] * __expf(ms - m);
    }
    orow[k] = __float2bfloat16(a * inv);
  }
}

// Key slices per sequence for single-query steps: a pure function of shapes
// (captured graphs replay the same grid).  Slices cost an f32 partial row per
// (slice, head) written and read again, so they are only used to give every CU
// a workgroup when the batch alone does not.
int latent_decode_num_splits(int nseq, int heads, int max_keys) {
  const int cap = heads <= 16 ? 16 : (heads <= 32 ? 32 : LM_ROWS);
  const int groups = (heads + cap - 1) / cap;
  const int tiles = (max_keys + LM_KT - 1) / LM_KT;
  // the dim-split variants (<= 32 heads) fit two workgroups per CU
  const int target = heads <= 32 ? 512 : 256;
  int want = (target + nseq * groups - 1) / (nseq * groups);
  if (want > tiles / 2) want = tiles / 2;   // at least two tiles per slice
  if (want > 32) want = 32;
  return want < 1 ? 1 : want;
}

#define LM_SHAPES(X) \
  X(2, 2) X(2, 3) X(4, 3) X(4, 4) X(6, 4) X(6, 5) X(8, 5) X(8, 6) X(16, 9) \
  X(16, 10) X(32, 17) X(32, 18)                                             \
  /* no rotated part */ X(2, 1) X(4, 2) X(8, 4) X(16, 8) X(32, 16)

bool latent_prefill_mfma_usable(int rank, int rot, int block_size) {
  (void)block_size;
  if (rank % 16 != 0 || (rank + rot) % 32 != 0 || rot % 8 != 0) return false;
  const int nt = rank / 16, ks = (rank + rot) / 32;
#define X(A, B) if (nt == A && ks == B) return true;
  LM_SHAPES(X)
#undef X
  return false;
}

template <int NT, int KS, int DS>
static void launch_one(bf16* out, long o_st, long o_sh, const bf16* q_lat,
                       long ql_st, long ql_sh, const bf16* q_rot, long qr_st,
                       long qr_sh, const bf16* cache, const int* block_tables,
                       int bt_stride, const int* qsl, const int* seq_lens,
                       int nseq, const float* sinks, float scale, int window,
                       int max_q, int heads, int block_size, int nsplit,
                       int two_term, float* part_acc, float* part_ml,
                       hipStream_t stream) {
  constexpr int RANK = NT * 16, D = KS * 32;
  const size_t smem = sizeof(bf16) * (LM_KT * (D + LM_KPAD) + RANK * LM_VROW) *
                          1 +
                      sizeof(int) * LM_BT_MAX;
  static bool configured = false;
  if (!configured) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&latent_attn_mfma_kernel<NT, KS, DS>),
                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    configured = true;
  }
  const int rows_cap = LM_ROWS / DS;   // DS waves share a row tile
  const int hpb = heads < rows_cap ? heads : rows_cap;
  const int tq = rows_cap / hpb;
  dim3 grid(nsplit > 1 ? nsplit : (max_q + tq - 1) / tq, nseq, (heads + hpb - 1) / hpb);
  latent_attn_mfma_kernel<NT, KS, DS><<<grid, LM_THREADS, smem, stream>>>(
      out, o_st, o_sh, q_lat, ql_st, ql_sh, q_rot, qr_st, qr_sh, cache,
      block_tables, bt_stride, qsl, seq_lens, sinks, scale, window, heads, tq,
      hpb, block_size, nsplit, two_term, part_acc, part_ml);
  if (nsplit > 1) {
    dim3 mg(nseq, heads);
    latent_attn_merge_kernel<<<mg, 128, 0, stream>>>(out, o_st, o_sh, part_acc, part_ml,
                                                    sinks, nsplit, heads, RANK);
  }
}

void launch_latent_attn_mfma(bf16* out, long o_st, long o_sh, const bf16* q_lat,
                             long ql_st, long ql_sh, const bf16* q_rot,
                             long qr_st, long qr_sh, const bf16* cache,
                             const int* block_tables, int bt_stride,
                             const int* qsl, const int* seq_lens, int nseq,
                             const float* sinks, float scale, int window,
                             int max_q, int heads, int rank, int rot,
                             int block_size, int nsplit, int two_term,
                             float* part_acc, float* part_ml,
                             hipStream_t stream) {
  const int nt = rank / 16, ks = (rank + rot) / 32;
  // one query per sequence and at most one 16-row tile of heads
  // single queries: as many waves per row tile as the head count leaves free.
  // (Prompt portions keep four row tiles: splitting dims there — 32 rows per
  // workgroup, two workgroups per CU at rank 512 — measured 25% slower, the
  // doubled staging and score work outweighs the residency.)
  const int dim_split = (qsl != nullptr || heads > 32) ? 1 : (heads <= 16 ? 4 : 2);
#define X(A, B)                                                               \
  if (nt == A && ks == B) {                                                   \
    if (dim_split == 4 && A % 4 == 0)                                         \
      launch_one<A, B, (A % 4 == 0 ? 4 : 1)>(                                 \
          out, o_st, o_sh, q_lat, ql_st, ql_sh, q_rot, qr_st, qr_sh, cache,  \
          block_tables, bt_stride, qsl, seq_lens, nseq, sinks, scale, window, \
          max_q, heads, block_size, nsplit, two_term, part_acc, part_ml,      \
          stream);                                                            \
    else if (dim_split >= 2)                                                  \
      launch_one<A, B, 2>(                                                    \
          out, o_st, o_sh, q_lat, ql_st, ql_sh, q_rot, qr_st, qr_sh, cache,  \
          block_tables, bt_stride, qsl, seq_lens, nseq, sinks, scale, window, \
          max_q, heads, block_size, nsplit, two_term, part_acc, part_ml,      \
          stream);                                                            \
    else                                                                      \
      launch_one<A, B, 1>(                                                    \
          out, o_st, o_sh, q_lat, ql_st, ql_sh, q_rot, qr_st, qr_sh, cache,  \
          block_tables, bt_stride, qsl, seq_lens, nseq, sinks, scale, window, \
          max_q, heads, block_size, nsplit, two_term, part_acc, part_ml,      \
          stream);                                                            \
    return;                                                                   \
  }
  LM_SHAPES(X)
#undef X
}
