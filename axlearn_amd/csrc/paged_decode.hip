// Single-token decode attention for gfx950: paged KV pool and contiguous KV cache.
//
// Replaces axlearn/common/flash_attention/gpu_paged_attention.py:38-152 (`_paged_attention_kernel`)
// with its launcher and XLA combine (:164-296), and axlearn/common/flash_attention/
// gpu_decoding.py:71-283 (`_attn_forward_kernel`, `_decode_attn_unbatched`).
//
// The operation is bound by HBM: every K and V byte of the live context is read exactly once.
//   * split-K over the context: a workgroup (4 wavefronts) owns `chunk_pages` consecutive logical
//     pages (16 tokens each) of one (sequence, kv head); chunks past the sequence length exit at
//     once, so long and short sequences load the chip evenly;
//   * a wavefront streams one page at a time.  K is read straight into the B-operand layout of
//     v_mfma_f32_16x16x32_bf16 (lane = token, 64-byte segments per row) and all query heads of the
//     kv head (padded to 16 rows) are scored with D/32 MFMAs; V is read fully coalesced (16 lanes
//     cover one 256-byte token row) and accumulated with fp32 FMAs, each 16-lane group keeping its
//     own partial output for the tokens it owns; register sets are re-issued as soon as they are
//     consumed so loads for the next page are in flight during the arithmetic of this one;
//   * probabilities travel from the MFMA layout to the V layout through 1 KB of LDS per wavefront;
//   * partial (o, m, l) per chunk go to an fp32 workspace (the reference stores partial o in the
//     query dtype, gpu_paged_attention.py:272) and a second small kernel merges them.
// Keys at index >= length are masked (gpu_paged_attention.py:100, gpu_decoding.py:109); the query
// position is length-1, so a sliding window w also masks keys with (length-1) - j > w.  A page
// index outside the pool reads as zeros and a negative one counts from the end of the pool, as the
// reference's gather does (kv_cache/paged_kv_cache.py:32).
#include "common.h"

namespace axl {

struct DecArgs {
  const __bf16* q;        // [B, Hq, D]
  const __bf16* k;        // paged: [Hkv, P, 16, D]; contiguous: [B, S, Hkv, D] (strided)
  const __bf16* v;
  const int32_t* page_tables;  // [B, pps] (paged only)
  const int32_t* lengths;      // [B]
  __bf16* out;                 // [B, Hq, D]
  float* ws_o;                 // [B, Hkv, NCH, GP, D]
  float* ws_m;                 // [B, Hkv, NCH, GP]
  float* ws_l;                 // [B, Hkv, NCH, GP]
  Strides3 ks, vs;             // contiguous only
  int B, Hq, Hkv, G;
  int num_pages, pps;          // pool pages; logical pages per sequence (ceil(S/16) if contiguous)
  int kv_len;                  // contiguous only
  int chunk_pages, nch;
  int window;
  float scale;
};

constexpr int kPage = 16;

__device__ __forceinline__ float row16_max(float x) {
  x = fmaxf(x, __shfl_xor(x, 1, 64));
  x = fmaxf(x, __shfl_xor(x, 2, 64));
  x = fmaxf(x, __shfl_xor(x, 4, 64));
  x = fmaxf(x, __shfl_xor(x, 8, 64));
  return x;
}
__device__ __forceinline__ float row16_sum(float x) {
  x += __shfl_xor(x, 1, 64);
  x += __shfl_xor(x, 2, 64);
  x += __shfl_xor(x, 4, 64);
  x += __shfl_xor(x, 8, 64);
  return x;
}

template <int D, int GP, bool PAGED>
__global__ __launch_bounds__(256) void decode_split_kernel(const DecArgs a) {
  constexpr int KSTEPS = D / 32;        // MFMA k-steps over head_dim
  constexpr int SL = D / 8;             // 16-byte slices per token row
  constexpr int TPL = 64 / SL;          // token rows covered by one wave-wide V load
  constexpr int NLOAD = kPage / TPL;    // V loads per page
  constexpr int HG = GP / 4;            // 4-head groups in use (MFMA row groups)
  __shared__ __attribute__((aligned(16))) float p_lds[4][kPage + 1][16];   // [wave][token | corr][head]
  __shared__ __attribute__((aligned(16))) float red_o[4 * TPL][GP * D / 4 + 4]; // epilogue partials, see below
  __shared__ float red_m[4][16], red_l[4][16];

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int chunk = blockIdx.x, hk = blockIdx.y, b = blockIdx.z;
  const int len = a.lengths[b];
  int npages = (len + kPage - 1) / kPage;
  npages = min(npages, a.pps);
  int first_page = 0;
  if (a.window >= 0) first_page = max(0, (len - 1 - a.window)) / kPage;
  const int c_begin = max(chunk * a.chunk_pages, first_page);
  const int c_end = min((chunk + 1) * a.chunk_pages, npages);
  if (c_begin >= c_end) return;  // nothing live in this chunk (uniform for the whole workgroup)

  // Q as MFMA A operand: lane (head row = lane%16, k-group = lane/16) holds d = 32s + 8kg .. +7.
  const int qrow = lane & 15, kg = lane >> 4;
  bf16x8 qf[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; s++) {
    if (qrow < a.G) {
      qf[s] = *(const bf16x8*)(a.q + ((int64_t)b * a.Hq + hk * a.G + qrow) * D + 32 * s + 8 * kg);
    } else {
#pragma unroll
      for (int e = 0; e < 8; e++) qf[s][e] = (__bf16)0.f;
    }
  }
  const int tok = lane & 15;          // K layout / MFMA C layout: token column
  const int hg = lane >> 4;           // MFMA C layout: heads 4hg..4hg+3
  const int vslice = lane % SL;       // V layout: 16-byte slice of the row
  const int vtok = lane / SL;         // V layout: token row within a load
  const float c = a.scale * kLog2e;

  float m_run[4], l_run[4];
#pragma unroll
  for (int r = 0; r < 4; r++) { m_run[r] = kNegInf; l_run[r] = 0.f; }
  float o[GP][8];
#pragma unroll
  for (int gq = 0; gq < GP; gq++)
#pragma unroll
    for (int e = 0; e < 8; e++) o[gq][e] = 0.f;

  auto page_base = [&](int j, const __bf16* base, const Strides3& st, bool& valid) -> const __bf16* {
    if (PAGED) {
      int pg = __builtin_amdgcn_readfirstlane(a.page_tables[(int64_t)b * a.pps + j]);
      if (pg < 0) pg += a.num_pages;  // negative indices count from the end, as in the reference's gather
      valid = (unsigned)pg < (unsigned)a.num_pages;
      return base + ((int64_t)hk * a.num_pages + (valid ? pg : 0)) * (kPage * D);
    } else {
      valid = true;
      return base + b * st.b + (int64_t)j * kPage * st.s + hk * st.h;
    }
  };
  const int64_t k_row_stride = PAGED ? D : a.ks.s;
  const int64_t v_row_stride = PAGED ? D : a.vs.s;

  uint4 kreg[KSTEPS], vreg[NLOAD];
  auto load_k = [&](int j) {
    bool valid;
    const __bf16* base = page_base(j, a.k, a.ks, valid);
#pragma unroll
    for (int s = 0; s < KSTEPS; s++) {
      const bool ok = valid && (PAGED || j * kPage + tok < a.kv_len);
      kreg[s] = ok ? *(const uint4*)(base + tok * k_row_stride + 32 * s + 8 * kg) : uint4{0, 0, 0, 0};
    }
  };
  auto load_v = [&](int j) {
    bool valid;
    const __bf16* base = page_base(j, a.v, a.vs, valid);
#pragma unroll
    for (int i = 0; i < NLOAD; i++) {
      const int t = TPL * i + vtok;
      const bool ok = valid && (PAGED || j * kPage + t < a.kv_len);
      vreg[i] = ok ? *(const uint4*)(base + t * v_row_stride + 8 * vslice) : uint4{0, 0, 0, 0};
    }
  };

  int j = c_begin + wave;
  if (j < c_end) {
    load_k(j);
    load_v(j);
  }
  for (; j < c_end; j += 4) {
    // ---- scores for this page: S[head][token] = Q K^T
    floatx4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int st = 0; st < KSTEPS; st++) {
      union { uint4 u; bf16x8 v; } kf;
      kf.u = kreg[st];
      s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[st], kf.v, s, 0, 0, 0);
    }
    const int jn = j + 4;
    if (jn < c_end) load_k(jn);  // K registers are free again: next page's K goes in flight now
    const int tpos = j * kPage + tok;
    bool keep = tpos < len;
    if (a.window >= 0) keep = keep && (len - 1 - tpos <= a.window);
    float pm[4], corr[4];
    bool changed = false;
#pragma unroll
    for (int r = 0; r < 4; r++) {
      s[r] = keep ? s[r] : kMasked;
      pm[r] = row16_max(s[r]);
      const float mn = fmaxf(m_run[r], pm[r]);
      changed = changed || (mn != m_run[r]);
      corr[r] = fast_exp2((m_run[r] - mn) * c);
      m_run[r] = mn;
      s[r] = fast_exp2((s[r] - mn) * c);
      l_run[r] = l_run[r] * corr[r] + s[r];
    }
    const bool any_changed = __builtin_amdgcn_ballot_w64(changed && hg < HG) != 0;
    if (hg < HG) {
      *(float4*)&p_lds[wave][tok][4 * hg] = float4{s[0], s[1], s[2], s[3]};
      if (any_changed && tok == 0)
        *(float4*)&p_lds[wave][kPage][4 * hg] = float4{corr[0], corr[1], corr[2], corr[3]};
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // ---- O += P V on the coalesced V layout
    // A page that straddles the length (or the window start) holds tokens whose probability is
    // exactly 0; their V rows may be uninitialised pool memory, and 0 * NaN would poison the sum,
    // so those rows are replaced by zeros.  Only boundary pages pay for this.
    const bool boundary = (j * kPage + kPage > len) || (a.window >= 0 && len - 1 - j * kPage > a.window);
    if (boundary) {
#pragma unroll
      for (int i = 0; i < NLOAD; i++) {
        const int vpos = j * kPage + TPL * i + vtok;
        bool vkeep = vpos < len;
        if (a.window >= 0) vkeep = vkeep && (len - 1 - vpos <= a.window);
        if (!vkeep) vreg[i] = uint4{0, 0, 0, 0};
      }
    }
    if (any_changed) {
#pragma unroll
      for (int gq = 0; gq < GP; gq++) {
        const float cg = p_lds[wave][kPage][gq];
#pragma unroll
        for (int e = 0; e < 8; e++) o[gq][e] *= cg;
      }
    }
#pragma unroll
    for (int i = 0; i < NLOAD; i++) {
      float pv[GP];
#pragma unroll
      for (int g4 = 0; g4 < GP / 4; g4++) {
        const float4 x = *(const float4*)&p_lds[wave][TPL * i + vtok][4 * g4];
        pv[4 * g4 + 0] = x.x; pv[4 * g4 + 1] = x.y; pv[4 * g4 + 2] = x.z; pv[4 * g4 + 3] = x.w;
      }
      const uint32_t w[4] = {vreg[i].x, vreg[i].y, vreg[i].z, vreg[i].w};
      float ve[8];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        ve[2 * e] = __uint_as_float(w[e] << 16);
        ve[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
      }
#pragma unroll
      for (int gq = 0; gq < GP; gq++)
#pragma unroll
        for (int e = 0; e < 8; e++) o[gq][e] = __builtin_fmaf(pv[gq], ve[e], o[gq][e]);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (jn < c_end) load_v(jn);
  }

  // ---- merge the 4 wavefronts x (64/SL) lane groups of this workgroup.
#pragma unroll
  for (int r = 0; r < 4; r++) l_run[r] = row16_sum(l_run[r]);
  if (tok == 0 && hg < HG) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
      red_m[wave][4 * hg + r] = m_run[r];
      red_l[wave][4 * hg + r] = l_run[r];
    }
  }
  __syncthreads();
  float f_wave[GP];
#pragma unroll
  for (int gq = 0; gq < GP; gq++) {
    const float mw = fmaxf(fmaxf(red_m[0][gq], red_m[1][gq]), fmaxf(red_m[2][gq], red_m[3][gq]));
    f_wave[gq] = fast_exp2((red_m[wave][gq] - mw) * c);
  }
  // red_o rows: one per partial (wave * TPL + vtok); columns: head-in-quarter * D + d.  The heads
  // are reduced a quarter at a time to keep the staging buffer small.
  constexpr int NPART = 4 * TPL;  // partial outputs per element
  float* out_ws = a.ws_o + (((int64_t)b * a.Hkv + hk) * a.nch + chunk) * (GP * D);
#pragma unroll
  for (int q4 = 0; q4 < 4; q4++) {  // heads q4*GP/4 .. (q4+1)*GP/4 - 1
    __syncthreads();
#pragma unroll
    for (int gi = 0; gi < GP / 4; gi++) {
      const int gq = q4 * (GP / 4) + gi;
      float* dst = &red_o[wave * TPL + vtok][gi * D + 8 * vslice];
      *(float4*)dst = float4{o[gq][0] * f_wave[gq], o[gq][1] * f_wave[gq], o[gq][2] * f_wave[gq], o[gq][3] * f_wave[gq]};
      *(float4*)(dst + 4) = float4{o[gq][4] * f_wave[gq], o[gq][5] * f_wave[gq], o[gq][6] * f_wave[gq], o[gq][7] * f_wave[gq]};
    }
    __syncthreads();
    for (int idx = tid; idx < GP / 4 * D; idx += 256) {
      float acc = 0.f;
#pragma unroll
      for (int pidx = 0; pidx < NPART; pidx++) acc += red_o[pidx][idx];
      out_ws[q4 * (GP / 4) * D + idx] = acc;
    }
  }
  if (tid < GP) {
    const float mw = fmaxf(fmaxf(red_m[0][tid], red_m[1][tid]), fmaxf(red_m[2][tid], red_m[3][tid]));
    float lw = 0.f;
#pragma unroll
    for (int w = 0; w < 4; w++) lw += red_l[w][tid] * fast_exp2((red_m[w][tid] - mw) * c);
    const int64_t sidx = (((int64_t)b * a.Hkv + hk) * a.nch + chunk) * GP + tid;
    a.ws_m[sidx] = mw;
    a.ws_l[sidx] = lw;
  }
}

// Merges the per-chunk partials of one (sequence, kv head): the "final round of flash"
// (gpu_paged_attention.py:287-296, gpu_decoding.py:277-283).
template <int D, int GP>
__global__ __launch_bounds__(256) void decode_combine_kernel(const DecArgs a) {
  const int hk = blockIdx.x, b = blockIdx.y;
  const int tid = threadIdx.x;
  const int len = a.lengths[b];
  int npages = min((len + kPage - 1) / kPage, a.pps);
  int first_page = 0;
  if (a.window >= 0) first_page = max(0, (len - 1 - a.window)) / kPage;
  const int ch0 = first_page / a.chunk_pages;
  const int ch1 = (npages + a.chunk_pages - 1) / a.chunk_pages;  // exclusive
  const float c = a.scale * kLog2e;
  const int64_t base = ((int64_t)b * a.Hkv + hk) * a.nch;
  for (int idx = tid; idx < a.G * D; idx += 256) {
    const int gq = idx / D, d = idx % D;
    float mw = kNegInf;
    for (int ch = ch0; ch < ch1; ch++) mw = fmaxf(mw, a.ws_m[(base + ch) * GP + gq]);
    float l = 0.f, acc = 0.f;
    for (int ch = ch0; ch < ch1; ch++) {
      const float f = fast_exp2((a.ws_m[(base + ch) * GP + gq] - mw) * c);
      l += a.ws_l[(base + ch) * GP + gq] * f;
      acc += a.ws_o[(base + ch) * (GP * D) + gq * D + d] * f;
    }
    a.out[((int64_t)b * a.Hq + hk * a.G + gq) * D + d] = (__bf16)(acc / l);
  }
}

static int pick_chunk_pages(int pps) {
  // 32 pages = 512 tokens = 256 KB of K+V per workgroup at head_dim 128.
  int cp = 32;
  if (pps < cp) cp = ((pps + 3) / 4) * 4;
  return cp < 4 ? 4 : cp;
}

static size_t ws_bytes(int B, int Hkv, int nch, int gp, int D) {
  return (size_t)B * Hkv * nch * ((size_t)gp * D + 2 * gp) * sizeof(float);
}

static int gp_of(int G) { return G <= 4 ? 4 : 8; }

size_t paged_decode_workspace_bytes(const AxlPagedDecodeParams& p) {
  if (p.pages_per_seq <= 0 || p.num_kv_heads <= 0) return 0;
  const int cp = pick_chunk_pages(p.pages_per_seq);
  const int nch = (p.pages_per_seq + cp - 1) / cp;
  return ws_bytes(p.batch, p.num_kv_heads, nch, gp_of(p.num_q_heads / p.num_kv_heads), p.head_dim);
}

size_t decode_workspace_bytes(const AxlDecodeParams& p) {
  if (p.kv_len <= 0 || p.num_kv_heads <= 0) return 0;
  const int pps = (p.kv_len + kPage - 1) / kPage;
  const int cp = pick_chunk_pages(pps);
  const int nch = (pps + cp - 1) / cp;
  return ws_bytes(p.batch, p.num_kv_heads, nch, gp_of(p.num_q_heads / p.num_kv_heads), p.head_dim);
}

template <bool PAGED>
static int launch_common(DecArgs a, int D, hipStream_t stream, const char* who) {
  const int gp = gp_of(a.G);
  if (a.G > 8) return set_error(AXL_ERR_UNSUPPORTED, "%s: more than 8 query heads per kv head", who);
  a.chunk_pages = pick_chunk_pages(a.pps);
  a.nch = (a.pps + a.chunk_pages - 1) / a.chunk_pages;
  float* ws = a.ws_o;
  const size_t n_o = (size_t)a.B * a.Hkv * a.nch * gp * D;
  const size_t n_s = (size_t)a.B * a.Hkv * a.nch * gp;
  a.ws_m = ws + n_o;
  a.ws_l = ws + n_o + n_s;
  const dim3 grid(a.nch, a.Hkv, a.B), cgrid(a.Hkv, a.B);
#define AXL_DEC(DD, GG)                                                                   \
  do {                                                                                    \
    hipLaunchKernelGGL((decode_split_kernel<DD, GG, PAGED>), grid, dim3(256), 0, stream, a); \
    hipLaunchKernelGGL((decode_combine_kernel<DD, GG>), cgrid, dim3(256), 0, stream, a);  \
  } while (0)
  if (D == 128 && gp == 4) AXL_DEC(128, 4);
  else if (D == 128) AXL_DEC(128, 8);
  else if (gp == 4) AXL_DEC(64, 4);
  else AXL_DEC(64, 8);
#undef AXL_DEC
  hipError_t err = hipGetLastError();
  if (err != hipSuccess)
    return set_error(AXL_ERR_LAUNCH, "%s: launch failed: %s", who, hipGetErrorString(err));
  return AXL_OK;
}

int launch_paged_decode(const AxlPagedDecodeParams& p, hipStream_t stream) {
  DecArgs a{};
  a.q = (const __bf16*)p.q; a.k = (const __bf16*)p.k_pages; a.v = (const __bf16*)p.v_pages;
  a.page_tables = p.page_tables; a.lengths = p.lengths; a.out = (__bf16*)p.out;
  a.ws_o = (float*)p.workspace;
  a.B = p.batch; a.Hq = p.num_q_heads; a.Hkv = p.num_kv_heads; a.G = p.num_q_heads / p.num_kv_heads;
  a.num_pages = p.num_pages; a.pps = p.pages_per_seq; a.kv_len = p.pages_per_seq * kPage;
  a.window = p.sliding_window < 0 ? -1 : p.sliding_window;
  a.scale = p.softmax_scale;
  return launch_common<true>(a, p.head_dim, stream, "axl_paged_decode");
}

int launch_decode(const AxlDecodeParams& p, hipStream_t stream) {
  DecArgs a{};
  a.q = (const __bf16*)p.q; a.k = (const __bf16*)p.k; a.v = (const __bf16*)p.v;
  a.page_tables = nullptr; a.lengths = p.lengths; a.out = (__bf16*)p.out;
  a.ws_o = (float*)p.workspace;
  a.ks = Strides3{p.k_strides.batch, p.k_strides.seq, p.k_strides.head};
  a.vs = Strides3{p.v_strides.batch, p.v_strides.seq, p.v_strides.head};
  a.B = p.batch; a.Hq = p.num_q_heads; a.Hkv = p.num_kv_heads; a.G = p.num_q_heads / p.num_kv_heads;
  a.num_pages = 0; a.pps = (p.kv_len + kPage - 1) / kPage; a.kv_len = p.kv_len;
  a.window = p.sliding_window < 0 ? -1 : p.sliding_window;
  a.scale = p.softmax_scale;
  return launch_common<false>(a, p.head_dim, stream, "axl_decode");
}

}  // namespace axl
