// A chain of dependent decode matmuls (one activation row, Q4 weights) in ONE launch.
//
// The reference submits a whole step as one command buffer (src/runtime.rs:2843-2959) and a decode
// step is a chain of small dependent matmuls (src/models/smollm2.rs:392-405: norm -> q, k, v;
// o + residual; norm -> gate | up; SwiGLU -> down + residual).  Launched one by one, every such
// matmul pays what a dependent launch costs on this GPU (about 2.5 us, more than the matmul
// itself at these sizes).  Here the whole chain is one resident launch: one workgroup per CU walks
// the list of stages, taking its share of each stage's column quads, and the data dependencies
// are carried by the data itself.  Every stage output that a later stage reads goes (besides the
// caller's buffer) into a slot of the chain's own workspace, whose words all hold kHandoverEmpty
// before the launch; a reading thread polls the words it needs until none is empty any more.  No
// counters, no grid-wide barrier: a stage starts on a CU as soon as that CU is done with the
// previous one and its inputs have arrived, and the first weight blocks of a stage are requested
// before the wait for its activations.  The workspace has two sets of slots that launches use
// alternately; a launch empties the other set for the launch after it (by then the launch that
// used it has ended).  Waits are bounded (spin_limit polls, then the context's fault word is set,
// the thread goes on with what it has and the next synchronising call reports it).
// Stages that read nothing from each other (q, k, v and the o-projection of a layer) share the
// workgroups between them, so the length of a chain in hand-overs is its number of such phases;
// a hand-over costs about 3.3 us (eight SmolLM2 decode layers, 48 stages in 24 phases: 79 us, against
// 127 us as 32 separate launches).  Measured and not kept: running the chain on the workgroups of
// one XCD, so that hand-overs meet in that XCD's L2 (13.0 against 10.2 us per layer: an eighth of
// the CUs streams the weights), requesting the norm weights and the residual ahead of the polling
// (+0.1 .. +0.3 us per layer) and the next stage's table entry ahead of its stage (+1.1 us).
//
// A stage is the one-row Q4 decode matmul of kernels_gemv_mfma.hip.h in loop form: the
// activations go through the optional prologue (rms_norm, SwiGLU), are scaled per 32-element block
// by a power of two, cut into three base-128 digits and laid out in LDS as the A operands of
// v_mfma_i32_4x4x4_16B_i8; lane (b, i) multiplies its own quant block (K block 16 s + b of column
// 4 q + i) as plain nibble bytes, three blocks in flight ahead of the one in use; the K splits of
// a quad meet in LDS in a fixed order.
#include <algorithm>

#include "kernels_gemv_prep.hip.h"

namespace mgn {
namespace {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef int intx4 __attribute__((ext_vector_type(4)));
constexpr int kDeviceScope = 16;  // the sc1 bit of a buffer instruction's cache policy

// Eight consecutive floats at p + elem.  `poll`: they are made by another workgroup of this launch;
// read past the caches (device scope) until none of the words is empty any more, at most
// spin_limit times.
__device__ __forceinline__ void load8(const float* p, uint32_t elem, bool poll, uint32_t spin_limit, float (&v)[8], bool* gave_up) {
  if (!poll) {
    const float4* src = (const float4*)(p + elem);
    const float4 a = src[0], b = src[1];
    v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
    return;
  }
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)p, 0, 0x7FFFFFFF, 0x00020000);
  uint32_t w[8];
#pragma unroll
  for (int e = 0; e < 8; e++) w[e] = kHandoverEmpty;
  for (uint32_t polls = 0;; polls++) {
    if (polls >= spin_limit) {  // (a limit of 0 looks at nothing: the give-up path, for tests)
      *gave_up = true;
      break;
    }
    const u32x4_t a = __builtin_amdgcn_raw_buffer_load_b128(rsrc, elem * 4, 0, kDeviceScope);
    const u32x4_t b = __builtin_amdgcn_raw_buffer_load_b128(rsrc, elem * 4 + 16, 0, kDeviceScope);
    w[0] = a.x, w[1] = a.y, w[2] = a.z, w[3] = a.w, w[4] = b.x, w[5] = b.y, w[6] = b.z, w[7] = b.w;
    bool missing = false;
#pragma unroll
    for (int e = 0; e < 8; e++) missing |= w[e] == kHandoverEmpty;
    if (!missing) break;
    __builtin_amdgcn_s_sleep(1);
    asm volatile("" ::: "memory");  // the loads are issued anew on every round
  }
#pragma unroll
  for (int e = 0; e < 8; e++) v[e] = __builtin_bit_cast(float, w[e]);
}

__device__ __forceinline__ float load1_polled(const float* p, uint32_t spin_limit, bool* gave_up) {
  float x = __builtin_bit_cast(float, kHandoverEmpty);
  for (uint32_t polls = 0;; polls++) {
    if (polls >= spin_limit) {
      *gave_up = true;
      break;
    }
    x = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (__builtin_bit_cast(uint32_t, x) != kHandoverEmpty) break;
    __builtin_amdgcn_s_sleep(2);
  }
  return x;
}

// Weight blocks in flight per lane ahead of the one in use.  Only requests for items the wave really
// has: the stages of a decode layer leave a wave one or two items, and a request past the last one
// (the last block again, to keep the code free of branches) was a third of its memory
// instructions.  Measured, us per decode layer / FFN pair as one chain: 3 with the surplus
// requests 9.36 / 29.0; without them 3: 8.75 / 26.2, 2: 8.68 / 25.6, 1: 8.78 / 27.3.
constexpr int kRing = 2;

// grid = one workgroup per CU (or fewer), 1024 threads.  Every workgroup walks all stages in order.
__global__ __launch_bounds__(1024) void chain_kernel_q4(const ChainStageDev* __restrict__ stages, uint32_t nstages,
                                                        uint32_t* __restrict__ clear_ptr, uint32_t clear_words, uint32_t spin_limit,
                                                        uint32_t* __restrict__ fault_flag) {
  extern __shared__ uint4 lds4[];
  const uint32_t wg = blockIdx.x, nwg = gridDim.x;
  const uint32_t tid = threadIdx.x, lane = tid & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t b = lane >> 2, i = lane & 3;
  // the other set of slots: empty again for the launch after this one
  for (uint32_t w = wg * 1024 + tid; w < clear_words; w += nwg * 1024)
    __hip_atomic_store(clear_ptr + w, kHandoverEmpty, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  bool gave_up = false;
  for (uint32_t s = 0; s < nstages; s++) {
    // (the table is read-only for the whole launch: scalar loads through the constant address space)
    typedef const uint32_t __attribute__((address_space(4))) * ConstWords;
    ChainStageDev st;
    {
      static_assert(sizeof(ChainStageDev) % 4 == 0, "copied word by word");
      const ConstWords src = (ConstWords)(uintptr_t)(stages + s);
      uint32_t words[sizeof(ChainStageDev) / 4];
#pragma unroll
      for (uint32_t j = 0; j < sizeof(ChainStageDev) / 4; j++) words[j] = src[j];
      __builtin_memcpy(&st, words, sizeof(st));
    }
    // (the whole workgroup: no barrier is skipped by part of it)
    if (wg < st.wg_first || wg >= st.wg_first + st.wgs) continue;
    const uint32_t wgl = wg - st.wg_first;  // this workgroup's index among those that serve the stage
    const uint32_t k = st.k, n = st.n, bpc = k / 32, bpc_pad = (bpc + 15) & ~15u;
    const uint32_t ksc = 1u << st.ksc_log2, nslots = st.nslots;
    const uint32_t slot = wave >> st.ksc_log2, ks = wave & (ksc - 1);
    const uint32_t nquads = (n + 3) / 4;
    const uint32_t quad0 = wgl * st.qpw_wg;
    const uint32_t quads_here = min(st.qpw_wg, nquads - quad0);
    const uint32_t my_quads = slot < nslots && slot < quads_here ? (quads_here - slot + nslots - 1) / nslots : 0;
    const uint32_t steps_total = bpc_pad / 16, step_begin = ks * st.steps;
    const uint32_t my_steps = step_begin < steps_total ? min(st.steps, steps_total - step_begin) : 0;
    const uint32_t total = my_quads * my_steps;  // this wave's (quad, step) items, quad-major
    uint4* const xa = lds4;                                          // [bpc_pad] x 128 bytes: digit planes
    float2* const cinit = (float2*)(lds4 + (size_t)bpc_pad * 8);     // [bpc_pad]
    float* const red = (float*)(cinit + bpc_pad);                    // [qpw_wg][ksc][4]
    float* const nrm = red + st.qpw_wg * ksc * 4;                    // [16] sums of squares (kProRmsNorm)

    // ---- the wave's first weight blocks: requested before anything is waited for ----
    u32x4_t rq[kRing];
    uint32_t rm[kRing];
    uint32_t fq = 0, fs = 0;  // the item the next request is for: (quad index, step) of this wave
    auto fetch = [&](int u) {
      const uint32_t quad = quad0 + slot + fq * nslots;
      const uint32_t col = min(quad * 4 + i, n - 1);
      const size_t at = (size_t)col * bpc + (step_begin + fs) * 16 + b;
      rq[u] = __builtin_nontemporal_load((const u32x4_t*)((const char*)st.quants + at * 16));
      rm[u] = __builtin_nontemporal_load((const uint32_t*)((const char*)st.meta + at * 4));
      if (fq * my_steps + fs + 1 < total) {
        fs++;
        if (fs == my_steps) fs = 0, fq++;
      }
    };
    if (total != 0) {
#pragma unroll
      for (int u = 0; u < kRing; u++)
        if ((uint32_t)u < total) fetch(u);
    }
    for (uint32_t t = tid; t < st.qpw_wg * ksc * 4; t += 1024) red[t] = 0.0f;

    // ---- activations -> prologue -> integer digits in LDS (once per workgroup and stage) ----
    const bool swi = st.pro == kProSwiglu, rms = st.pro == kProRmsNorm;
    float x[kMaxTasks][8];
    float ss = 0.0f;
#pragma unroll
    for (int tt = 0; tt < kMaxTasks; tt++) {
      const uint32_t t = tid + tt * 1024, kb = t >> 2, ch = t & 3;
      const bool live = kb < bpc;
#pragma unroll
      for (int e = 0; e < 8; e++) x[tt][e] = 0.0f;
      if (live) {
        load8(st.a, kb * 32 + ch * 8, st.a_poll != 0, spin_limit, x[tt], &gave_up);
        if (swi) {
          float up[8];
          load8(st.a, k + kb * 32 + ch * 8, st.a_poll != 0, spin_limit, up, &gave_up);
#pragma unroll
          for (int e = 0; e < 8; e++) x[tt][e] = swiglu_act(x[tt][e], up[e]);
        }
        if (rms) {
#pragma unroll
          for (int e = 0; e < 8; e++) ss = __fmaf_rn(x[tt][e], x[tt][e], ss);
        }
      }
    }
    if (rms) {
      // src/shaders/rms_norm.wgsl:1-57: x * rsqrt(mean(x^2) + eps) * weight.  The activations are
      // staged as x * weight; the row's one factor is applied to the finished sums below, so the
      // staging does not wait for the sum of squares (the barrier behind the staging publishes it)
      ss = group_sum<64>(ss);
      if (lane == 0) nrm[wave] = ss;
#pragma unroll
      for (int tt = 0; tt < kMaxTasks; tt++) {
        const uint32_t t = tid + tt * 1024, kb = t >> 2, ch = t & 3;
        if (kb < bpc) {
          const float4* gp = (const float4*)(st.norm_w + kb * 32 + ch * 8);
          const float4 g0 = gp[0], g1 = gp[1];
          const float g[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
#pragma unroll
          for (int e = 0; e < 8; e++) x[tt][e] = x[tt][e] * g[e];
        }
      }
    }
#pragma unroll
    for (int tt = 0; tt < kMaxTasks; tt++) {
      const uint32_t t = tid + tt * 1024, kb = t >> 2, ch = t & 3;
      if (t < bpc_pad * 4) {  // whole waves take this branch together (bpc_pad * 4 is a multiple of 64)
        const float(&v)[8] = x[tt];
        // block maximum over the quad's 32 values; NaN never wins fmaxf.  Integers cannot carry a
        // NaN along: a block that holds one (or an infinity, or values beyond 2^100, which are not
        // rescaled) is given a NaN factor, so its column sums come out non-finite
        float am = fmaxf(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))),
                         fmaxf(fmaxf(fabsf(v[4]), fabsf(v[5])), fmaxf(fabsf(v[6]), fabsf(v[7]))));
        const bool has_nan = __builtin_isunordered(v[0], v[1]) || __builtin_isunordered(v[2], v[3]) ||
                             __builtin_isunordered(v[4], v[5]) || __builtin_isunordered(v[6], v[7]);
        am = has_nan ? __builtin_inff() : am;
        am = fmaxf(am, dpp_move<kDppQuadXor1>(am));
        am = fmaxf(am, dpp_move<kDppQuadXor2>(am));
        float inv;
        float scale = block_scale(am, &inv);
        // |x| * scale < 2^20 (block_scale leaves 2^12), so the top digit stays within int8
        scale *= 256.0f, inv *= 0.00390625f;
        if (!(am < 1.0e30f)) inv = __builtin_nanf("");
        const float xs[8] = {v[0] * scale, v[1] * scale, v[2] * scale, v[3] * scale, v[4] * scale, v[5] * scale, v[6] * scale, v[7] * scale};
        uint32_t dlo[3], dhi[3];
        int isum;
        const int order[8] = {0, 2, 4, 6, 1, 3, 5, 7};
        make_digits(xs, order, dlo, dhi, &isum);
        uint32_t* const xw = (uint32_t*)xa;
#pragma unroll
        for (int pl = 0; pl < 3; pl++) *(uint2*)(xw + kb * 32 + pl * 8 + 2 * ch) = make_uint2(dlo[pl], dhi[pl]);
        isum += __builtin_amdgcn_update_dpp(0, isum, kDppQuadXor1, 0xF, 0xF, true);
        isum += __builtin_amdgcn_update_dpp(0, isum, kDppQuadXor2, 0xF, 0xF, true);
        if (ch == 0) cinit[kb] = make_float2(-8.0f * (float)isum, inv);
      }
    }
    lds_barrier();

    // ---- the walk: this wave's items, kRing requests ahead ----
    if (total != 0) {
      float acc = 0.0f;
      uint32_t cq = 0, cs = 0;
      for (uint32_t t0 = 0; t0 < total; t0 += kRing) {
#pragma unroll
        for (int u = 0; u < kRing; u++) {
          if (t0 + u < total) {  // uniform
            const u32x4_t q = rq[u];
            const uint32_t kb = (step_begin + cs) * 16 + b;
            const uint32_t meta = kb < bpc ? rm[u] : 0u;  // a block past the end of K counts for nothing
            __builtin_amdgcn_sched_barrier(0);
            if (t0 + u + kRing < total) fetch(u);
            __builtin_amdgcn_sched_barrier(0);
            const char* const xa_step = (const char*)xa + (size_t)kb * 128 + i * 32;
            const uint4 a0 = *(const uint4*)xa_step, a1 = *(const uint4*)(xa_step + 16);
            const float2 ci0 = cinit[kb];
            const uint32_t aw[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
            const uint32_t words[4] = {q.x, q.y, q.z, q.w};
            intx4 dsum = {0, 0, 0, 0};
#pragma unroll
            for (int ch = 0; ch < 4; ch++) {
              const uint32_t wd = words[ch];
              const uint32_t even = wd & 0x0F0F0F0Fu, odd = (wd >> 4) & 0x0F0F0F0Fu;  // (n0,n2,n4,n6), (n1,n3,n5,n7)
              dsum = __builtin_amdgcn_mfma_i32_4x4x4i8((int)aw[2 * ch], (int)even, dsum, 0, 0, 0);
              dsum = __builtin_amdgcn_mfma_i32_4x4x4i8((int)aw[2 * ch + 1], (int)odd, dsum, 0, 0, 0);
            }
            const int tot = (((dsum[2] << 7) + dsum[1]) << 7) + dsum[0];  // digits back together: sum n * x
            const float dscale = half_bits_to_float(meta & 0xFFFFu);
            const float mneg = __fmaf_rn(-0.125f, half_bits_to_float(meta >> 16), -dscale);  // (m + 8 d) S = mneg * (-8 S)
            float v = dscale * ((float)tot + ci0.x);
            v = __fmaf_rn(mneg, ci0.x, v);
            acc = __fmaf_rn(v, ci0.y, acc);
            cs++;
            if (cs == my_steps) {  // the quad is done: its 16 lanes per column meet, lanes 0..3 hold the four columns
              const float one[1] = {acc};
              uint32_t row;
              bool writer;
              const float sum = sum_rows_over_blocks<1>(one, lane, &row, &writer);
              if (writer) red[((slot + cq * nslots) * ksc + ks) * 4 + lane] = sum;
              acc = 0.0f, cs = 0, cq++;
            }
          }
        }
      }
    }
    lds_barrier();

    // ---- the K splits meet (fixed order), residual, unary operations, store ----
    const float rstd = rms ? 1.0f / sqrtf(group_sum<16>(nrm[lane & 15u]) / (float)k + st.eps) : 1.0f;
    for (uint32_t t = tid; t < quads_here * 4; t += 1024) {
      const uint32_t ql = t >> 2, col = t & 3, nidx = (quad0 + ql) * 4 + col;
      if (nidx < n) {
        float v = 0.0f;
        for (uint32_t sp = 0; sp < ksc; sp++) v += red[(ql * ksc + sp) * 4 + col];
        v *= rstd;
        if (st.d) v += st.d_poll ? load1_polled(st.d + nidx, spin_limit, &gave_up) : st.d[nidx];
        v = apply_epilogue(v, st.epilogue);
        st.c[nidx] = v;
        if (st.c_slot) {
          const uint32_t bits = __builtin_bit_cast(uint32_t, v);
          __hip_atomic_store(st.c_slot + nidx, __builtin_bit_cast(float, bits == kHandoverEmpty ? 0x7FC00000u : bits),
                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
    lds_barrier();  // the next stage lays out LDS anew
  }
  if (gave_up && fault_flag) *fault_flag = 1u;
}

}  // namespace

// Fills the plan fields of a stage (K, N and the format must be set); false if the chain kernel
// does not serve it.  *lds gets the dynamic LDS the stage needs.
bool plan_chain_stage(int fmt, int num_cus, ChainStageDev* st, size_t* lds) {
  if (fmt != MGN_FMT_Q4 || st->k == 0 || st->k % 32 != 0 || st->n == 0 || num_cus <= 0) return false;
  const uint32_t bpc = st->k / 32, bpc_pad = (bpc + 15) & ~15u;
  if (bpc_pad * 4 > kMaxTasks * 1024) return false;  // two activation chunks per thread at most: K <= 16384
  const uint32_t steps_total = bpc_pad / 16, nquads = (st->n + 3) / 4;
  // K splits across waves: at most 8 steps per wave; more when the quads alone would leave most waves idle
  uint32_t log2 = 0;
  while ((steps_total + (1u << log2) - 1) / (1u << log2) > 8) log2++;
  while (log2 < 4 && (uint64_t)nquads << (log2 + 1) <= (uint64_t)num_cus * 16 && (steps_total >> (log2 + 1)) >= 1) log2++;
  if (log2 > 4) return false;
  const uint32_t ksc = 1u << log2;
  st->ksc_log2 = log2;
  st->steps = (steps_total + ksc - 1) / ksc;
  st->qpw_wg = (nquads + num_cus - 1) / num_cus;
  st->wgs = (nquads + st->qpw_wg - 1) / st->qpw_wg;
  // quad slots: as few waves as reach the same quads per wave (28 quads on 16 slots: 14 slots of 2)
  const uint32_t max_slots = 16 / ksc, per_slot = (st->qpw_wg + max_slots - 1) / max_slots;
  st->nslots = (st->qpw_wg + per_slot - 1) / per_slot;
  *lds = (size_t)bpc_pad * 128 + (size_t)bpc_pad * 8 + (size_t)st->qpw_wg * ksc * 16 + 64 + 64;
  return *lds <= 150 * 1024;
}

int launch_chain(ihipStream_t* s, int device, int fmt, const ChainStageDev* stages_dev, uint32_t nstages, uint32_t grid, size_t lds,
                 uint32_t* clear_ptr, uint32_t clear_words, uint32_t spin_limit, uint32_t* fault_flag) {
  if (fmt != MGN_FMT_Q4) return (int)hipErrorInvalidValue;
  static std::atomic<uint64_t> big_lds_done{0};
  if (lds > 64 * 1024)
    if (int e = enable_big_lds(chain_kernel_q4, device, big_lds_done)) return e;
  hipLaunchKernelGGL(chain_kernel_q4, dim3(grid), dim3(1024), lds, s, stages_dev, nstages, clear_ptr, clear_words, spin_limit, fault_flag);
  MGN_HIP_LAUNCH_CHECK();
  return 0;
}

}  // namespace mgn
