// Latent attention: every token keeps one vector of R + dr numbers that all heads share (the RMS-normed latent c
// [R] and one rotated key part kr [dr]); a head's unrotated key is Wuk_h c and its value Wuv_h c. The products
// with Wuk and Wuv are moved to the query side (the "absorbed" form), so the kernels here never expand a key:
//
//   qa_h = [ Wuk_h^T qn_h | rot(qr_h) ]          (R + dr numbers a head, made before these kernels run)
//   s_j  = scale * < qa_h , [c_j | kr_j] >       j <= p  (and j > p - window, where a window is given)
//   ol_h = sum_j softmax(s)_j c_j                (R numbers a head; the caller multiplies by Wuv_h)
//
// which is attention with one shared key/value head whose keys are R + dr wide and whose values are the first R
// numbers of the same row. Cache pages: [blocks][page][R + dr], one row a token.
//
//   latent_post    from the step's projections: RMS norm of the latent (float), rotation of the shared key part and
//                  of every head's rotated query part (pairs (2i, 2i+1), float angles from a table), the latent row
//                  written to its cache slot, the rotated query part written beside the absorbed part
//   latent_attn_ref  one wave per (token, head), keys in ascending tiles of 64, float arithmetic, any sizes: the
//                  kernel of the 32-bit path and the reference beside the MFMA kernel
//   latent_attn_mfma bf16: a workgroup takes 16 (token, head) rows of one request (heads fastest) and walks the keys in
//                  blocks of 32 through LDS; each of its waves takes every fourth block and keeps its own
//                  (max, sum, output); they meet in LDS at the end. With `splits` > 1 the keys of a request are cut
//                  into that many parts on the device (single rows: decode) and a merge kernel joins them.
#include "common.cuh"

using namespace dinfer;

namespace {

constexpr int MAX_DK = 1280;  // R + dr
constexpr int MAX_R = 1024;
constexpr int WAVES = 4;

// ---- projections -> absorbed-query buffer and cache -------------------------------------------------------------
template <class S>
__global__ void __launch_bounds__(256) latent_post_kernel(
    const S* __restrict__ proj, int64_t ld, int q_off, int c_off, int H, int dn, int dr, int R,
    const void* __restrict__ gain, int wf32, float eps, const int32_t* __restrict__ positions,
    const float* __restrict__ cos_sin, int rot, S* __restrict__ qa, int64_t ld_qa, S* __restrict__ cache,
    const int64_t* __restrict__ slots) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const S* row = proj + t * ld;
  const int pos = positions[t];
  const float* cs = cos_sin ? cos_sin + (int64_t)pos * rot : nullptr;
  const int half = rot / 2;
  // every head's rotated query part
  const int pairs = dr / 2;
  for (int i = threadIdx.x; i < H * pairs; i += blockDim.x) {
    const int h = i / pairs, j = i - h * pairs;
    const S* src = row + q_off + (int64_t)h * (dn + dr) + dn + 2 * j;
    float u = to_f32(src[0]), v = to_f32(src[1]);
    if (cs && j < half) {
      const float c = cs[j], s = cs[half + j];
      const float a = rotated_first(u, v, c, s), b = rotated_second(u, v, c, s);
      u = a; v = b;
    }
    S* dst = qa + t * ld_qa + (int64_t)h * (R + dr) + R + 2 * j;
    dst[0] = from_f32<S>(u);
    dst[1] = from_f32<S>(v);
  }
  if (dr & 1) {   // an odd last entry passes unchanged
    for (int h = threadIdx.x; h < H; h += blockDim.x)
      qa[t * ld_qa + (int64_t)h * (R + dr) + R + dr - 1] = row[q_off + (int64_t)h * (dn + dr) + dn + dr - 1];
  }
  if (c_off < 0 || !slots) return;
  const int64_t slot = slots[t];
  if (slot < 0) return;   // (uniform over the workgroup)
  const S* c = row + c_off;
  float ss = 0.f;
  for (int i = threadIdx.x; i < R; i += blockDim.x) ss = add_square(ss, to_f32(c[i]));
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)R + eps);
  S* dst = cache + slot * (int64_t)(R + dr);
  for (int i = threadIdx.x; i < R; i += blockDim.x) dst[i] = from_f32<S>(to_f32(c[i]) * inv * ld_param<S>(gain, i, wf32));
  for (int j = threadIdx.x; j < pairs; j += blockDim.x) {
    float u = to_f32(c[R + 2 * j]), v = to_f32(c[R + 2 * j + 1]);
    if (cs && j < half) {
      const float co = cs[j], si = cs[half + j];
      const float a = rotated_first(u, v, co, si), b = rotated_second(u, v, co, si);
      u = a; v = b;
    }
    dst[R + 2 * j] = from_f32<S>(u);
    dst[R + 2 * j + 1] = from_f32<S>(v);
  }
  if ((dr & 1) && threadIdx.x == 0) dst[R + dr - 1] = c[R + dr - 1];
}

// ---- plain attention over the latent pages ----------------------------------------------------------------------
template <class S>
__global__ void __launch_bounds__(WAVES * 64) latent_attn_ref_kernel(
    const S* __restrict__ qa, int64_t ld_qa, S* __restrict__ out, int64_t ld_out, const S* __restrict__ cache,
    const int32_t* __restrict__ block_table, int64_t max_blocks, const int32_t* __restrict__ cu_seqlens,
    const int32_t* __restrict__ seq_lens, int num_reqs, float scale, int window, int H, int R, int dr, int page) {
  extern __shared__ float lds[];
  const int DK = R + dr;
  float* qs = lds;                   // [WAVES][DK]
  float* ps = lds + WAVES * DK;      // [WAVES][64]
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int h = blockIdx.y * WAVES + wave;
  const bool live = h < H;
  int lo_b = 0, hi_b = num_reqs - 1;
  while (lo_b < hi_b) {
    const int mid = (lo_b + hi_b + 1) >> 1;
    if (cu_seqlens[mid] <= t) lo_b = mid; else hi_b = mid - 1;
  }
  const int b = lo_b;
  const int q_len = cu_seqlens[b + 1] - cu_seqlens[b];
  const int p = seq_lens[b] - q_len + (t - cu_seqlens[b]);
  const int first_key = window > 0 ? (p - window + 1 > 0 ? p - window + 1 : 0) : 0;
  const int32_t* bt = block_table + (int64_t)b * max_blocks;
  if (live) {
    const S* qr = qa + (int64_t)t * ld_qa + (int64_t)h * DK;
    for (int d = lane; d < DK; d += 64) qs[wave * DK + d] = to_f32(qr[d]);
  }
  __syncthreads();
  constexpr int NC = MAX_R / 64;
  float o[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) o[c] = 0.f;
  float m = -INFINITY, l = 0.f;
  for (int j0 = first_key; j0 <= p; j0 += 64) {
    const int j = j0 + lane;
    float s = -INFINITY;
    if (live && j <= p) {
      const S* kr = cache + ((int64_t)bt[j / page] * page + (j % page)) * DK;
      float acc = 0.f;
      for (int d = 0; d < DK; ++d) acc = fmaf(qs[wave * DK + d], to_f32(kr[d]), acc);
      s = acc * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float pj = (live && j <= p) ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);
    l = l * alpha + wave_sum(pj);
    m = m_new;
    __syncthreads();
    ps[wave * 64 + lane] = pj;
    __syncthreads();
    if (live) {
      const int n = p - j0 + 1 < 64 ? p - j0 + 1 : 64;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int d = lane + 64 * c;
        if (d < R) {
          float acc = o[c] * alpha;
          for (int jj = 0; jj < n; ++jj) {
            const int key = j0 + jj;
            acc = fmaf(ps[wave * 64 + jj], to_f32(cache[((int64_t)bt[key / page] * page + (key % page)) * DK + d]), acc);
          }
          o[c] = acc;
        }
      }
    }
  }
  if (live) {
    S* orow = out + (int64_t)t * ld_out + (int64_t)h * R;
    const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int d = lane + 64 * c;
      if (d < R) orow[d] = from_f32<S>(o[c] * inv);
    }
  }
}

}  // namespace

// proj [T, ld]: the queries at column q_off (head h at h*(dn+dr): dn unrotated, then dr rotated), the down projection
// at c_off (R latent, then dr shared key part; c_off < 0: this layer has none and nothing is written to the cache).
// cos_sin [positions, rot] = [cos | sin] of rot/2 angles (null: no rotation); the first `rot` entries of a rotated part
// turn. qa [T, ld_qa]: head h at h*(R+dr); its last dr entries are written here. cache [blocks*page, R+dr].
extern "C" int dinfer_latent_post(int dtype, const void* proj, int64_t tokens, int64_t ld, int q_off, int c_off, int heads,
                                  int dn, int dr, int R, const void* gain, int w_f32, float eps,
                                  const int32_t* positions, const float* cos_sin, int rot, void* qa, int64_t ld_qa,
                                  void* cache, const int64_t* slots, hipStream_t stream) {
  if (tokens <= 0) return OK;
  if (heads <= 0 || dn < 0 || dr < 0 || R <= 0 || rot < 0 || rot > dr || (rot & 1) || tokens > 0x7fffffff ||
      ld_qa < (int64_t)heads * (R + dr))
    return ERR_BAD_SHAPE;
  DINFER_DISPATCH_DTYPE(dtype, {
    latent_post_kernel<S><<<(unsigned)tokens, 256, 0, stream>>>((const S*)proj, ld, q_off, c_off, heads, dn, dr, R, gain,
                                                               w_f32, eps, positions, cos_sin, rot, (S*)qa, ld_qa,
                                                               (S*)cache, slots);
  });
  return launch_status();
}

extern "C" int dinfer_latent_attn_ref(int dtype, const void* qa, int64_t ld_qa, void* out, int64_t ld_out,
                                      const void* cache, const int32_t* block_table, int64_t max_blocks,
                                      const int32_t* cu_seqlens, const int32_t* seq_lens, int num_reqs, int64_t tokens,
                                      float scale, int window, int heads, int R, int dr, int page_size,
                                      hipStream_t stream) {
  if (tokens <= 0 || num_reqs <= 0) return OK;
  if (heads <= 0 || R <= 0 || dr < 0 || page_size <= 0 || max_blocks <= 0 || window < 0 || tokens > 0x7fffffff)
    return ERR_BAD_SHAPE;
  if (R > MAX_R || R + dr > MAX_DK) return ERR_UNSUPPORTED;
  const dim3 grid((unsigned)tokens, (unsigned)((heads + WAVES - 1) / WAVES));
  const size_t lds = (size_t)WAVES * (R + dr + 64) * sizeof(float);
  DINFER_DISPATCH_DTYPE(dtype, {
    latent_attn_ref_kernel<S><<<grid, WAVES * 64, lds, stream>>>((const S*)qa, ld_qa, (S*)out, ld_out, (const S*)cache,
                                                                 block_table, max_blocks, cu_seqlens, seq_lens,
                                                                 num_reqs, scale, window, heads, R, dr, page_size);
  });
  return launch_status();
}
