// Split-key paged attention on the matrix cores for tokens that each bring one query (decoding),
// bfloat16. A workgroup takes one (token, key/value head, chunk of keys) and serves all query heads
// of that key/value head's group; its waves (up to 8; 4 for heads wider than 64 where a wave has more than one step) take the chunk's
// 32-key steps in turn:
//     S^T[key, head] = K[key, :] · Q[head, :]      v_mfma_f32_16x16x32_bf16, keys as rows
//     online softmax per head (32-bit), P = 2^(S - m)
//     O[head, :]    += P[head, key] · V[key, :]
// The result layout of the first product is the operand layout of the second, so P never leaves
// its registers. Keys are read as 16-byte pieces of their rows; values are read from pages that
// hold them transposed ([head_dim, page_size] per head), so that the eight consecutive keys an
// operand needs lie side by side in memory. The waves' partial results meet in LDS. With one chunk
// per token (few tokens, contexts short enough for one workgroup to stream) the workgroup
// normalises and writes the output itself. Otherwise a chunk's unnormalised output with its running
// max and sum goes to a 32-bit workspace, and a second kernel combines the chunks of a token in
// ascending order. Chunk boundaries are multiples of the chunk size counted from position 0.
#include "attention_mfma.h"

#define DEC_MAX_WAVES 8
// heads wider than 64 keep two steps of wide rows in registers in the general loop: its workgroups
// have up to 4 waves then (with 8, a lane's 256 registers are overrun by 22, and 64 tokens over
// 2,560 keys take 137 µs instead of 122); the instance with a single step per wave has room for 8
#define DEC_WAVES_FOR(HD, ONE) ((HD) > 64 && !(ONE) ? 4 : DEC_MAX_WAVES)

// ONE: a wave has a single 32-key step (chunk = 32 waves); without the second buffer of the
// general loop the kernel needs fewer registers and more workgroups share a compute unit
template <int HD, bool ONE>
__global__ void __launch_bounds__(DEC_WAVES_FOR(HD, ONE) * TS_WAVE)
attn_decode_mfma_kernel(bf16_t* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml,
                        const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
                        const int32_t* __restrict__ block_tables, const int32_t* __restrict__ seq_of_token,
                        const int32_t* __restrict__ positions, int nh, int G, int page_size, int page_shift, int page_run,
                        int64_t kp, int64_t ks, int64_t kh, int64_t vp, int64_t vh, int64_t vd, int max_blocks,
                        int num_splits, int chunk, float scale2, int window) {
  constexpr int NC = HD / 32;    // 32-dimension pieces of a key row (one 16-byte load per lane each)
  constexpr int NDB = HD / 16;   // 16-dimension blocks of the output
  ts_fetch_arguments<164>();     // (nine pointers, five numbers, six strides, four more numbers and the scale)
  extern __shared__ __align__(16) float smem[];
  const int nw = blockDim.x / TS_WAVE;
  float* wm = smem;                       // [waves][16]
  float* wl = wm + nw * 16;               // [waves][16]
  float* wo = wl + nw * 16;               // [waves][G][HD]

  const int tid = threadIdx.x, wave = wave_index(), lane = tid & (TS_WAVE - 1);
  const int r = lane & 15, g = lane >> 4;
  const int split = blockIdx.x, kvh = blockIdx.y, t = blockIdx.z;
  int pos = positions[t];
  int seq = seq_of_token[t];                    // (asked for with the position: one trip to memory, not one after the other;
  asm volatile("" : "+s"(pos), "+s"(seq));      //  left to itself the compiler fetches it when it has seen that the chunk is visible)
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int k0 = split * chunk;
  if (k0 > pos || k0 + chunk <= lo) return;     // nothing of this chunk is visible
  const int32_t* table = block_tables + (int64_t)seq * max_blocks;
  const PageMath pm{page_size, page_shift, page_run};

  uint4 qreg[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) qreg[c] = make_uint4(0, 0, 0, 0);
  if (r < G) {
    const bf16_t* qrow = q + ((int64_t)t * nh + (int64_t)kvh * G + r) * HD + 8 * g;
#pragma unroll
    for (int c = 0; c < NC; ++c) qreg[c] = *(const uint4*)(qrow + 32 * c);
  }
  float m = -INFINITY, l = 0.f;
  float4_t o[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db) o[db] = (float4_t){0.f, 0.f, 0.f, 0.f};

  // the chunk's visible keys, 32 at a time, dealt to the waves in turn (however few keys a request
  // has in the chunk, every wave gets its share of them, and the workgroup reads the chunk front to
  // back); the next step's loads are issued before this step's products
  const int stride = 32 * nw;
  int kend = k0 + chunk;
  if (kend > pos + 1) kend = pos + 1;
  int kb = (k0 > (lo & ~31) ? k0 : (lo & ~31)) + 32 * wave;
#define TS_LOAD(T, KB) load_tile<HD>(T, KB, r, g, lo, pos, kvh, table, pm, k_cache, v_cache, kp, ks, kh, vp, vh, vd)
#define TS_USE(T, KB) use_tile_auto<HD>(T, KB, r, g, lo, pos, pos, lo, qreg, scale2, m, l, o)
  if (ONE) {
    if (kb < kend) {
      KVTile<HD> A;
      TS_LOAD(A, kb);
      TS_USE(A, kb);
    }
  } else if (kb < kend) {
    // (the next step is asked for on every path, this step again where there is none: with a load that
    // may or may not have been issued the compiler waits for all of them before it uses any)
    KVTile<HD> A, B;
    TS_LOAD(A, kb);
    while (true) {
      const bool more_b = kb + stride < kend;
      TS_LOAD(B, more_b ? kb + stride : kb);
      TS_USE(A, kb);
      if (!more_b) break;
      kb += stride;
      const bool more_a = kb + stride < kend;
      TS_LOAD(A, more_a ? kb + stride : kb);
      TS_USE(B, kb);
      if (!more_a) break;
      kb += stride;
    }
  }
#undef TS_LOAD
#undef TS_USE
  // ---- the waves meet
  l = row_sum(l);
  if (g == 0) { wm[wave * 16 + r] = m; wl[wave * 16 + r] = l; }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int head = 4 * g + j;
    if (head < G) {
#pragma unroll
      for (int db = 0; db < NDB; ++db) wo[((int64_t)wave * G + head) * HD + 16 * db + r] = o[db][j];
    }
  }
  __syncthreads();
  for (int i = tid; i < G * HD; i += blockDim.x) {
    const int head = i / HD, d = i - head * HD;
    float M = -INFINITY;
    for (int w = 0; w < nw; ++w) M = fmaxf(M, wm[w * 16 + head]);
    float acc = 0.f, L = 0.f;
    for (int w = 0; w < nw; ++w) {
      const float wgt = fast_exp2(wm[w * 16 + head] - M);   // a wave without keys: 2^-inf = 0
      acc = fmaf(wo[((int64_t)w * G + head) * HD + d], wgt, acc);
      L = fmaf(wl[w * 16 + head], wgt, L);
    }
    if (num_splits == 1) {                  // the whole context was this workgroup's: position `pos` is always visible
      out[((int64_t)t * nh + (int64_t)kvh * G + head) * HD + d] = f2bf(acc / L);
    } else {
      const int64_t row = ((int64_t)t * nh + (int64_t)kvh * G + head) * num_splits + split;
      part_o[row * HD + d] = acc;
      if (d == 0) { part_ml[row * 2] = M; part_ml[row * 2 + 1] = L; }
    }
  }
}

// out[t, h, :] = sum_s o_s 2^{m_s - M} / sum_s l_s 2^{m_s - M} over the chunks s that hold visible keys
// (the running maxima are in units of log2).
// One 64-thread workgroup per (token, head): the lanes fetch the chunks' (m, l) side by side, then
// every lane sums its output dimensions over the chunks in ascending order.
#define COMBINE_MAX_SPLITS 1024
__global__ void __launch_bounds__(TS_WAVE)
attn_decode_combine_kernel(bf16_t* __restrict__ out, const float* __restrict__ part_o,
                           const float* __restrict__ part_ml, const int32_t* __restrict__ positions, int nh, int hd,
                           int num_splits, int chunk, int window) {
  __shared__ float wgt[COMBINE_MAX_SPLITS];
  const int t = blockIdx.x / nh, lane = threadIdx.x;
  const int64_t th = blockIdx.x;
  const int pos = positions[t];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int s0 = min(lo / chunk, num_splits - 1), s1 = min(pos / chunk, num_splits - 1);  // the last chunk is open-ended
  const float* ml = part_ml + th * num_splits * 2;
  float M = -INFINITY;
  for (int s = s0 + lane; s <= s1; s += TS_WAVE) M = fmaxf(M, ml[2 * s]);
  M = wave_max(M);
  float L = 0.f;
  for (int s = s0 + lane; s <= s1; s += TS_WAVE) {
    const float w = fast_exp2(ml[2 * s] - M);
    wgt[s - s0] = w;
    L += ml[2 * s + 1] * w;
  }
  L = wave_sum(L);
  wave_sync();
  const float inv = 1.0f / L;
  const float* po = part_o + (th * num_splits + s0) * hd;
  for (int d = lane; d < hd; d += TS_WAVE) {
    float acc = 0.f;
#pragma unroll 4
    for (int s = 0; s <= s1 - s0; ++s) acc = fmaf(po[(int64_t)s * hd + d], wgt[s], acc);
    out[th * hd + d] = f2bf(acc * inv);
  }
}

// The combining kernel alone: out [tokens, nh, hd] bfloat16 from the parts that ts_paged_attention_decode leaves
// with combine 0.
extern "C" int ts_attention_combine(void* out, const float* part_o, const float* part_ml, const int32_t* positions,
                                    int num_tokens, int nh, int hd, int num_splits, int chunk, int window, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (!out || !part_o || !part_ml || !positions || nh <= 0 || hd <= 0 || num_splits < 1 || chunk <= 0) return TS_BAD_SHAPE;
  return ts_launch_attention_combine(out, part_o, part_ml, positions, num_tokens, nh, hd, num_splits, chunk, window, stream);
}

// The combining kernel alone, for the prefill kernel's split walks (declared in attention_mfma.h).
int ts_launch_attention_combine(void* out, const float* part_o, const float* part_ml, const int32_t* positions,
                                int num_tokens, int nh, int hd, int num_splits, int chunk, int window,
                                hipStream_t stream) {
  if (num_splits > COMBINE_MAX_SPLITS) return TS_BAD_SHAPE;
  attn_decode_combine_kernel<<<num_tokens * nh, TS_WAVE, 0, stream>>>((bf16_t*)out, part_o, part_ml, positions, nh, hd,
                                                                      num_splits, chunk, window);
  return ts_check_launch();
}

// part_o [tokens, nh, num_splits, hd] and part_ml [tokens, nh, num_splits, 2] are float workspaces
// (unused and may be null when num_splits is 1). num_splits * chunk must cover every position that
// `positions` holds; a workgroup has `waves` waves that take the chunk's 32-key steps in turn (chunk is a multiple of 32 waves). (Letting the last workgroup
// of a token combine its chunks inside the first kernel was tried and is slower: on a GPU of several
// dies the device-scope fences it needs write back and invalidate each die's L2.) Keys: rows dense in
// head_dim, strides kp/ks/kh (page, slot, head). Values: transposed pages, slot stride 1, strides
// vp/vh/vd (page, head, dimension). An entry of block_tables names 2^page_run consecutive pages of page_size
// keys (entry e: the pages e 2^page_run + j); max_blocks is the tables' width in entries.
extern "C" int ts_paged_attention_decode(void* out, float* part_o, float* part_ml, const void* q, const void* k_cache,
                                         const void* v_cache, const int32_t* block_tables,
                                         const int32_t* seq_of_token, const int32_t* positions, int num_tokens, int nh,
                                         int nkv, int hd, int page_size, int64_t kp, int64_t ks, int64_t kh,
                                         int64_t vp, int64_t vh, int64_t vd, int max_blocks, int num_splits, int chunk,
                                         int waves, float scale, int window, int page_run, int combine, hipStream_t stream) {
  if (num_tokens <= 0) return TS_OK;
  if (nkv <= 0 || nh % nkv || page_size <= 0 || page_size % 8 || max_blocks <= 0 || num_splits <= 0 || page_run < 0 || page_run > 16)
    return TS_BAD_SHAPE;
  if (waves < 1 || waves > DEC_WAVES_FOR(hd, chunk == 32 * waves) || chunk <= 0 || chunk % (32 * waves) || num_splits > COMBINE_MAX_SPLITS)
    return TS_BAD_SHAPE;
  if (num_splits > 1 && (!part_o || !part_ml)) return TS_BAD_SHAPE;
  if (num_tokens > 65535 || nkv > 65535) return TS_BAD_SHAPE;
  const int G = nh / nkv;
  if (G > 16 || G * hd > 2048) return TS_BAD_SHAPE;
  // 16-byte loads: key rows and the 8-key pieces of value rows must be 16-byte aligned
  if ((kp % 8) || (ks % 8) || (kh % 8) || (vp % 8) || (vh % 8) || (vd % 8)) return TS_BAD_SHAPE;
  if ((((uintptr_t)q) | ((uintptr_t)k_cache) | ((uintptr_t)v_cache)) & 15) return TS_BAD_SHAPE;
  const size_t smem = sizeof(float) * (2 * waves * 16 + (size_t)waves * G * hd);
  if (smem > 65536) return TS_BAD_SHAPE;
  int page_shift = -1;
  if ((page_size & (page_size - 1)) == 0) {
    page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
  }
  dim3 grid(num_splits, nkv, num_tokens);
#define TS_DEC1(HH, ON)                                                                                         \
  attn_decode_mfma_kernel<HH, ON><<<grid, waves * TS_WAVE, smem, stream>>>(                                 \
      (bf16_t*)out, part_o, part_ml, (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache,          \
      block_tables, seq_of_token, positions, nh, G, page_size, page_shift, page_run, kp, ks, kh, vp, vh, vd, max_blocks,  \
      num_splits, chunk, scale * 1.44269504088896340736f, window)
#define TS_DEC(HH) if (chunk == 32 * waves) TS_DEC1(HH, true); else TS_DEC1(HH, false)
  switch (hd) {
    case 32: TS_DEC(32); break;
    case 64: TS_DEC(64); break;
    case 96: TS_DEC(96); break;
    case 128: TS_DEC(128); break;
    default: return TS_BAD_SHAPE;
  }
#undef TS_DEC
#undef TS_DEC1
  int rc = ts_check_launch();
  if (rc || num_splits == 1 || !combine) return rc;     // (combine 0: the caller's next kernel reads the parts itself)
  attn_decode_combine_kernel<<<num_tokens * nh, TS_WAVE, 0, stream>>>((bf16_t*)out, part_o, part_ml, positions, nh, hd,
                                                                      num_splits, chunk, window);
  return ts_check_launch();
}
