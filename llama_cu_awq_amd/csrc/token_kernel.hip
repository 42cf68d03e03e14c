// One launch per token: a persistent kernel that runs the whole network for one
// position (every layer's QKV+RoPE, attention, O-projection, gate/up+SiLU,
// down-projection, then the classifier and the greedy sampler).
//
// Why: batch-1 decode is a chain of ~10 small dependent steps per layer.  As
// separate launches each step pays kernel start-up and drain (~3.5 us measured
// on MI355X), several times the 1-7 us its weights take to stream.  Here one
// workgroup per CU stays resident for the whole token and the steps are
// separated by a grid barrier built from flags in device memory.
//
// Structure of a workgroup (768 threads):
//   * 8 streaming waves.  Each owns a ring of D slots in LDS and keeps D
//     1-KB "units" of packed weights in flight with direct global->LDS loads
//     (global_load_lds_dwordx4).  A unit is one 64-lane pass over one weight
//     row.  The sequence of units a wave will ever need is fixed when the
//     launch starts (weights do not depend on activations), so loads run ahead
//     of the consumer ACROSS steps and layers: while the workgroup waits at a
//     grid barrier the next step's weights keep arriving.
//   * 4 helper waves.  They never have weight loads outstanding, so their own
//     loads return at once: they combine the per-unit partial sums, apply the
//     step's epilogue (RoPE, residual, SiLU*up, argmax), publish the results,
//     run the grid barrier, stage the next step's input vector in LDS
//     (applying RMSNorm), and compute attention for the head the workgroup owns.
//
// Cross-workgroup data (x, q, attention output, hidden vector, the KV row of
// the current position) is written and read with agent-scope accesses, which
// bypass the non-coherent per-XCD L2, so no cache write-back/invalidate is
// needed inside the kernel.
//
// Arithmetic and rounding points are those of the reference kernels
// (gpu_kernels.h:72-105 RMSNorm, :179-283 int4 products and epilogues, :340-363
// RoPE, :150-176/:365-409/:287-337 attention, :117-147 classifier, :456-501
// argmax) in the reference's per-token order (llama2_q4.cu:430-538).
#include "common.hpp"
#include "token_kernel.hpp"

namespace tk {

// Phase descriptors are read through the constant address space so that they come in over the scalar data
// path and never enter the streaming waves' vector-memory counter.
typedef const Phase __attribute__((address_space(4)))* PhasePtr;

#define TK_AGENT __HIP_MEMORY_SCOPE_AGENT

__device__ __forceinline__ uint32_t ld_u32(const uint32_t* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, TK_AGENT); }
__device__ __forceinline__ void st_u32(uint32_t* p, uint32_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, TK_AGENT); }
__device__ __forceinline__ void st_u16(uint16_t* p, uint16_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, TK_AGENT); }

// 16-byte agent-scope load; the caller waits (wait_vm0) before using the result.
__device__ __forceinline__ void ld_x4_agent(u32x4& v, const void* p) {
    asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(p) : "memory");
}
// Direct global->LDS loads (lane L writes its 16 / 4 bytes at lds_off + 16*L / 4*L).  Issued as inline assembly
// so that the compiler's wait-count bookkeeping never sees them: the streaming waves manage vmcnt themselves.
__device__ __forceinline__ void dma16_nt(const void* gptr, uint32_t lds_off) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt" ::"s"(lds_off), "v"(gptr) : "memory");
}
__device__ __forceinline__ void dma4(const void* gptr, uint32_t lds_off) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(lds_off), "v"(gptr) : "memory");
}
__device__ __forceinline__ void wait_vm0() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// Workgroup barrier that does NOT wait for outstanding global loads (the streaming waves keep theirs in flight).
__device__ __forceinline__ void wg_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

__device__ __forceinline__ void wait_ring(int depth) {
    // at most 2*(depth-1) newer loads may remain outstanding: the oldest unit (2 loads) has landed
    switch (depth) {
        case 4: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
        case 5: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
        case 6: asm volatile("s_waitcnt vmcnt(10)" ::: "memory"); break;
        case 7: asm volatile("s_waitcnt vmcnt(12)" ::: "memory"); break;
        case 8: asm volatile("s_waitcnt vmcnt(14)" ::: "memory"); break;
        case 9: asm volatile("s_waitcnt vmcnt(16)" ::: "memory"); break;
        case 10: asm volatile("s_waitcnt vmcnt(18)" ::: "memory"); break;
        case 11: asm volatile("s_waitcnt vmcnt(20)" ::: "memory"); break;
        case 12: asm volatile("s_waitcnt vmcnt(22)" ::: "memory"); break;
        case 13: asm volatile("s_waitcnt vmcnt(24)" ::: "memory"); break;
        case 14: asm volatile("s_waitcnt vmcnt(26)" ::: "memory"); break;
        case 15: asm volatile("s_waitcnt vmcnt(28)" ::: "memory"); break;
        default: asm volatile("s_waitcnt vmcnt(30)" ::: "memory"); break;  // 16
    }
}

// ---------------------------------------------------------------- grid barrier
// Executed by helper wave 0 (64 lanes).  Every workgroup publishes the epoch in
// its own flag; up to 8 leader workgroups (one per XCD when dispatch is
// round-robin) each watch all flags and then publish the epoch in their own
// release line; every workgroup watches the release line of leader (id mod 8).
// Two store->load hops.  A wait that exceeds the spin limit sets the error word
// and returns false; the caller makes the whole workgroup leave the kernel.
__device__ bool grid_barrier(Sync* s, uint32_t epoch, int G, int lane, long long spin_limit, int* err_host) {
    const int wg = blockIdx.x;
    const int nlead = G < 8 ? G : 8;
    if (lane == 0) st_u32(&s->flags[wg], epoch);
    const long long t0 = wall_clock64();
    if (wg < nlead) {
        while (true) {
            bool ok = true;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int i = lane + 64 * k;
                const uint32_t v = i < G ? ld_u32(&s->flags[i]) : epoch;
                ok = ok && ((int)(v - epoch) >= 0);
            }
            if (__all(ok)) break;
            if (ld_u32((const uint32_t*)&s->error) != 0 || wall_clock64() - t0 > spin_limit) {
                if (lane == 0) {
                    st_u32((uint32_t*)&s->error, 1u);
                    __hip_atomic_store(err_host, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                }
                return false;
            }
        }
        if (lane == 0) st_u32(&s->release[wg * 32], epoch);
        return true;
    }
    const uint32_t* rel = &s->release[(wg % nlead) * 32];
    while (true) {
        const uint32_t v = ld_u32(rel);
        if ((int)(v - epoch) >= 0) return true;
        if (wall_clock64() - t0 > spin_limit) {
            if (lane == 0) {
                st_u32((uint32_t*)&s->error, 1u);
                __hip_atomic_store(err_host, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            }
            return false;
        }
        __builtin_amdgcn_s_sleep(1);
    }
}

// ---------------------------------------------------------------- unit addressing
// The units of a phase are split into NSW contiguous ranges, one per streaming wave.
__device__ __forceinline__ void unit_range(int U, int w, int& ubeg, int& uend) {
    ubeg = (U * w) / NSW;
    uend = (U * (w + 1)) / NSW;
}

// 32 consecutive K elements: sum (q - z) * x with the 1024-offset trick (see chunk constants in staging).
__device__ __forceinline__ float chunk_dot(const u32x4 w, const float zf, const u32x4 (&xq)[4], const float A, const float B,
                                           const uint32_t magic) {
    float acc0 = fmaf(-zf, A, -B), acc1 = 0.0f;
#pragma unroll
    for (int qi = 0; qi < 4; qi++) {
        const uint32_t d = w[qi];
        const uint32_t d8 = d >> 8;
        acc0 = dot2((d & 0x000F000Fu) | magic, xq[qi][0], acc0);
        acc1 = dot2((d & 0x00F000F0u) | magic, xq[qi][1], acc1);
        acc0 = dot2((d8 & 0x000F000Fu) | magic, xq[qi][2], acc0);
        acc1 = dot2((d8 & 0x00F000F0u) | magic, xq[qi][3], acc1);
    }
    return fmaf(acc1, 0.0625f, acc0);  // the high nibbles enter 16 times too large; the activations are never scaled
}

// Consume one landed unit: returns this lane's contribution to the row's dot product.
__device__ __forceinline__ float consume_unit(int kind, int nchunks, int pass, int lane, const char* slot, const u32x4* xs,
                                              const float2* ab, uint32_t magic) {
    const int c = pass * 64 + lane;
    float part = 0.0f;
    if (kind == KIND_CLS) {
        if (c < nchunks) {
            const u32x4 w = reinterpret_cast<const u32x4*>(slot)[lane];
            const u32x4 xv = xs[c];
#pragma unroll
            for (int i = 0; i < 4; i++) part = dot2(w[i], xv[i], part);
        }
        return part;
    }
    if (c < nchunks) {
        const u32x4 w = reinterpret_cast<const u32x4*>(slot)[lane];
        const uint16_t sbits = reinterpret_cast<const uint16_t*>(slot + 1024)[lane >> 2];
        const uint32_t zw = reinterpret_cast<const uint32_t*>(slot + 1024 + 32)[lane >> 5];
        const float zf = (float)((zw >> (((lane >> 2) & 7) * 4)) & 0xFu);
        u32x4 xq[4];
#pragma unroll
        for (int qi = 0; qi < 4; qi++) xq[qi] = xs[qi * nchunks + c];
        const float2 cab = ab[c];
        part = half_bits_to_float(sbits) * chunk_dot(w, zf, xq, cab.x, cab.y, magic);
    }
    return part;
}

// ---------------------------------------------------------------- helper work
// Helper thread id ht in [0, 256).

// Stage the phase's input vector in LDS.  Executes exactly two workgroup barriers.
__device__ void stage_input(const Args& a, PhasePtr P, int ht, int lane, int hw, u32x4* xs, float2* ab, float* red, int pos) {
    const bool is_helper = true;
    constexpr int MAXP = 10;
    u32x4 piece[MAXP];
    const int n8 = P->K >> 3;
    float ss = 0.0f;
    if (is_helper) {
        const uint16_t* src;
        if (P->in_sel == IN_EMBED) {
            const int token = a.tokens_dev[pos];
            src = a.embed + (size_t)token * a.dim;
        } else {
            src = P->in_sel == IN_X ? a.x : (P->in_sel == IN_XB ? a.xb : a.hb);
        }
#pragma unroll
        for (int i = 0; i < MAXP; i++) {
            const int e = ht + 256 * i;
            piece[i] = u32x4{0u, 0u, 0u, 0u};
            if (e < n8) ld_x4_agent(piece[i], src + (size_t)e * 8);
        }
        wait_vm0();
        if (P->norm_w) {
            float part = 0.0f;
#pragma unroll
            for (int i = 0; i < MAXP; i++) {
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const h16x2 h = as_h2(piece[i][k]);
                    const float x0 = (float)h[0], x1 = (float)h[1];
                    part = fmaf(x0, x0, part);
                    part = fmaf(x1, x1, part);
                }
            }
            part = wave_sum(part);
            if (lane == 0) red[hw] = part;
        }
    }
    wg_barrier();
    if (is_helper) {
        if (P->norm_w) {
            ss = (red[0] + red[1]) + (red[2] + red[3]);
            ss /= (float)P->K;
            ss += 1e-5f;
            ss = 1.0f / sqrtf(ss);
        }
        const u32x4* wg = reinterpret_cast<const u32x4*>(P->norm_w);
        const int total = P->kind == KIND_CLS ? n8 : P->C * 4;
#pragma unroll
        for (int i = 0; i < MAXP; i++) {
            const int e = ht + 256 * i;
            u32x4 v = piece[i];
            if (P->norm_w && e < n8) {
                const u32x4 wv = wg[e];
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const h16x2 h = as_h2(v[k]);
                    const h16x2 hw2 = as_h2(wv[k]);
                    h16x2 o;
                    o[0] = (h16_t)((float)h[0] * (ss * (float)hw2[0]));
                    o[1] = (h16_t)((float)h[1] * (ss * (float)hw2[1]));
                    v[k] = as_u32(o);
                }
            }
            if (P->kind == KIND_CLS) {
                if (e < total) xs[e] = v;
            } else {
                // (h0,h1)(h2,h3)(h4,h5)(h6,h7) -> (h0,h4)(h1,h5)(h2,h6)(h3,h7)
                const h16x2 p0 = as_h2(__builtin_amdgcn_perm(v[2], v[0], 0x05040100u));
                const h16x2 p1 = as_h2(__builtin_amdgcn_perm(v[2], v[0], 0x07060302u));
                const h16x2 p2 = as_h2(__builtin_amdgcn_perm(v[3], v[1], 0x05040100u));
                const h16x2 p3 = as_h2(__builtin_amdgcn_perm(v[3], v[1], 0x07060302u));
                const float even = ((float)p0[0] + (float)p0[1]) + ((float)p2[0] + (float)p2[1]);
                const float odd = ((float)p1[0] + (float)p1[1]) + ((float)p3[0] + (float)p3[1]);
                // even positions meet 1024 + q, odd positions (1024 + 16 q) / 16 = 64 + q
                float sa = even + odd;
                float sb = fmaf(0.0625f, odd, even);
                sa += dpp_mov<0xB1>(sa);
                sa += dpp_mov<0x4E>(sa);
                sb += dpp_mov<0xB1>(sb);
                sb += dpp_mov<0x4E>(sb);
                if (e < total) {
                    xs[(e & 3) * P->C + (e >> 2)] = u32x4{as_u32(p0), as_u32(p1), as_u32(p2), as_u32(p3)};
                    if ((e & 3) == 0) ab[e >> 2] = make_float2(sa, 1024.0f * sb);
                }
            }
        }
    }
    wg_barrier();
}

__device__ __forceinline__ float row_total(const float* partial, int r, int P) {
    float s = 0.0f;
    for (int p = 0; p < P; p++) s += partial[r * P + p];
    return s;
}

__device__ __forceinline__ void rope_pair(float& v0, float& v1, int i, int head_size, int pos, float theta) {
    const int head_dim = (i * 2) % head_size;
    const float freq = 1.0f / powf(theta, head_dim / (float)head_size);
    const float val = pos * freq;
    const float fcr = cosf(val);
    const float fci = sinf(val);
    float a0, a1;
    rope_rotate(v0, v1, fcr, fci, a0, a1);
    v0 = a0;
    v1 = a1;
}

// Epilogue of a streaming phase (helper threads only; no workgroup barrier inside).
__device__ void epilogue(const Args& a, PhasePtr P, int g, int ht, int lane, int hw, const float* partial, uint16_t* xres,
                         int pos) {
    switch (P->kind) {
        case KIND_QKV: {
            const int half_hs = a.head_size >> 1;
            const int kv_dim = a.n_kv_heads * a.head_size;
            const size_t row_off = (size_t)P->kv_layer_off + (size_t)pos * kv_dim;
            if (ht < P->ppw + P->kpw) {
                const bool isq = ht < P->ppw;
                const int j = isq ? ht : ht - P->ppw;
                const int r0 = isq ? 2 * j : 2 * P->ppw + 2 * j;
                // the reference stores q/k as fp16 and RoPE reads them back
                float v0 = half_bits_to_float(float_to_half_bits(row_total(partial, r0, P->P)));
                float v1 = half_bits_to_float(float_to_half_bits(row_total(partial, r0 + 1, P->P)));
                const int p = g * (isq ? P->ppw : P->kpw) + j;
                const int head = p / half_hs, i = p % half_hs;
                rope_pair(v0, v1, i, a.head_size, pos, a.rope_theta);
                uint16_t* dst = isq ? a.q + (size_t)head * a.head_size : a.key_cache + row_off + (size_t)head * a.head_size;
                st_u16(dst + i, float_to_half_bits(v0));
                st_u16(dst + i + half_hs, float_to_half_bits(v1));
            } else if (ht < P->ppw + P->kpw + P->vpw) {
                const int t = ht - P->ppw - P->kpw;
                const float v = row_total(partial, 2 * P->ppw + 2 * P->kpw + t, P->P);
                st_u16(a.value_cache + row_off + (size_t)g * P->vpw + t, float_to_half_bits(v));
            }
            break;
        }
        case KIND_OPROJ:
        case KIND_DOWN:
            if (ht < P->rows_per_wg) {
                float v = row_total(partial, ht, P->P);
                v += half_bits_to_float(xres[ht]);  // residual, gpu_count = 1
                const uint16_t h = float_to_half_bits(v);
                xres[ht] = h;
                st_u16(a.x + (size_t)g * P->rows_per_wg + ht, h);
            }
            break;
        case KIND_FFN:
            if (ht < (P->rows_per_wg >> 1)) {
                float gv = row_total(partial, 2 * ht, P->P);
                const float uv = row_total(partial, 2 * ht + 1, P->P);
                gv *= 1.0f / (1.0f + expf(-gv));
                st_u16(a.hb + (size_t)g * (P->rows_per_wg >> 1) + ht, float_to_half_bits(gv * uv));
            }
            break;
        case KIND_CLS:
            if (hw == 0) {  // one wave: logits of this workgroup's rows and their maximum (lowest index on ties)
                float best = -INFINITY;
                int best_i = 0x7FFFFFFF;
                for (int r = lane; r < P->rows_per_wg; r += 64) {
                    const int n = g * P->rows_per_wg + r;
                    if (n < P->N) {
                        const uint16_t h = float_to_half_bits(row_total(partial, r, P->P));
                        a.logits[n] = h;
                        const float v = half_bits_to_float(h);
                        if (v > best) {
                            best = v;
                            best_i = n;
                        }
                    }
                }
                for (int off = 32; off > 0; off >>= 1) {
                    const float ov = __shfl_xor(best, off);
                    const int oi = __shfl_xor(best_i, off);
                    if (ov > best || (ov == best && oi < best_i)) {
                        best = ov;
                        best_i = oi;
                    }
                }
                if (lane == 0) {
                    st_u32(&a.sync->amax_bits[g], __builtin_bit_cast(uint32_t, best));
                    st_u32((uint32_t*)&a.sync->amax_idx[g], (uint32_t)best_i);
                }
            }
            break;
        default:
            break;
    }
}

// Attention for head h over positions 0..pos by the 4 helper waves (reference: llama2_q4.cu:410-427).
// Executes four workgroup barriers; non-helper waves only take the barriers.
template <int LP>
__device__ void attention_head(const Args& a, PhasePtr P, int h, int ht, int lane, int hw, int pos, float* sc, float* red,
                               float* acc_lds) {
    const bool is_helper = true;
    constexpr int PW = 64 / LP;
    const int size = pos + 1;
    const int hs = a.head_size;
    const int kv_dim = a.n_kv_heads * hs;
    const int kv_mul = a.n_heads / a.n_kv_heads;
    const int j = lane % LP, pr = lane / LP;
    const size_t base = (size_t)P->kv_layer_off + (size_t)(h / kv_mul) * hs + j * 8;
    const float alpha = (float)(1.0 / sqrt((double)hs));
    const int stride_t = NHW * PW;
    const int tfirst = hw * PW + pr;
    if (is_helper) {
        u32x4 qv;
        ld_x4_agent(qv, a.q + (size_t)h * hs + j * 8);
        wait_vm0();
        for (int t0 = tfirst; t0 - pr - hw * PW < size; t0 += 4 * stride_t) {  // wave-uniform trip count
            u32x4 kv[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int t = t0 + k * stride_t;
                if (t < size) ld_x4_agent(kv[k], a.key_cache + base + (size_t)t * kv_dim);
            }
            wait_vm0();
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int t = t0 + k * stride_t;
                float s = 0.0f;
                if (t < size) {
#pragma unroll
                    for (int i = 0; i < 4; i++) s = dot2(kv[k][i], qv[i], s);
                }
                s = group_sum<LP>(s);
                if (j == 0 && t < size) sc[t] = half_bits_to_float(float_to_half_bits(s * alpha));
            }
        }
    }
    wg_barrier();  // 1: scores in LDS
    float m = 0.0f, sum = 0.0f;
    if (is_helper) {
        m = (size < 1024) ? 0.0f : -INFINITY;  // the reference's idle-lane seed
        for (int t = ht; t < size; t += 256) m = fmaxf(m, sc[t]);
        m = wave_max(m);
        if (lane == 0) red[hw] = m;
    }
    wg_barrier();  // 2
    if (is_helper) {
        m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        for (int t = ht; t < size; t += 256) sum += expf(sc[t] - m);
        sum = wave_sum(sum);
        if (lane == 0) red[4 + hw] = sum;
    }
    wg_barrier();  // 3
    if (is_helper) {
        sum = (red[4] + red[5]) + (red[6] + red[7]);
        float acc[8];
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] = 0.0f;
        for (int t0 = tfirst; t0 - pr - hw * PW < size; t0 += 4 * stride_t) {
            u32x4 vv[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int t = t0 + k * stride_t;
                if (t < size) ld_x4_agent(vv[k], a.value_cache + base + (size_t)t * kv_dim);
            }
            wait_vm0();
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int t = t0 + k * stride_t;
                if (t < size) {
                    const float e = expf(sc[t] - m);
                    const float p = half_bits_to_float(float_to_half_bits(e / sum));
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const h16x2 hv = as_h2(vv[k][i]);
                        acc[2 * i] = fmaf((float)hv[0], p, acc[2 * i]);
                        acc[2 * i + 1] = fmaf((float)hv[1], p, acc[2 * i + 1]);
                    }
                }
            }
        }
#pragma unroll
        for (int i = 0; i < 8; i++)
            for (int off = LP; off < 64; off <<= 1) acc[i] += __shfl_xor(acc[i], off);
        if (pr == 0) {
#pragma unroll
            for (int i = 0; i < 8; i++) acc_lds[hw * 256 + j * 8 + i] = acc[i];
        }
    }
    wg_barrier();  // 4
    if (is_helper && ht < hs) {
        const float total = (acc_lds[ht] + acc_lds[256 + ht]) + (acc_lds[512 + ht] + acc_lds[768 + ht]);
        st_u16(a.xb + (size_t)h * hs + ht, float_to_half_bits(total));
    }
}

// ---------------------------------------------------------------- the kernel
// Workgroup-barrier schedule, identical for both wave classes (they run separate code so that the compiler's
// wait-count bookkeeping of the helpers' loads and stores can never leak into the streaming loop):
//   streaming phase : S1 S2 (input staged) | work | B3 (partials complete) | B4 (helper stores done) | B5 (grid barrier done)
//   attention phase : 4 barriers inside attention_head if the workgroup owns a head | B4 | B5
//   argmax phase    : B4   (last phase: no grid barrier)
// After B5 every wave reads the abort flag and leaves if a grid barrier timed out.
struct LdsMap {
    u32x4* xs;
    float2* ab;
    float* partial;
    float* red;
    int* abort_flag;
    uint16_t* xres;
    float* acc_lds;
    float* sc;
};

__device__ __forceinline__ bool owns_head(const Args& a, int g, int& h) {
    const int heads_stride = a.G / a.n_heads;
    h = g / heads_stride;
    return (g % heads_stride == 0) && (h < a.n_heads);
}

__device__ void stream_main(const Args& a, PhasePtr phases, int nphases, int wave, int lane, int g, char* lds, const LdsMap& m) {
    uint32_t magic = 0x64006400u;
    asm("" : "+v"(magic));
    const int depth = a.depth;
    const char* ring = lds + a.lds_ring + (size_t)wave * depth * UNIT_BYTES;
    const uint32_t ring_off = (uint32_t)(uintptr_t)lds + a.lds_ring + wave * depth * UNIT_BYTES;  // LDS byte address

    // ---- load cursor: walks this wave's fixed unit sequence D units ahead of the consumer.
    // Everything it needs about its phase lives in scalar registers (plain locals: no struct, no array,
    // so nothing can end up in scratch memory, whose accesses would count against vmcnt).
    int lph = -1;            // phase of the load cursor; nphases = sequence exhausted
    int lu = 0, luend = 0;   // next unit and end of this wave's range in that phase
    int lr = 0, lpass = 0;   // stacked row and pass of the next unit
    int l_kind = 0, l_passes = 1, l_nchunks = 0, l_sh = 0, l_pzh = 0, l_row_dwords = 0, l_rows = 0, l_N = 0;
    int l_ppw = 0, l_kpw = 0, l_vpw = 0;
    const uint32_t *l_w0 = nullptr, *l_w1 = nullptr, *l_w2 = nullptr;
    const uint32_t *l_z0 = nullptr, *l_z1 = nullptr, *l_z2 = nullptr;
    const uint16_t *l_s0 = nullptr, *l_s1 = nullptr, *l_s2 = nullptr;
    const uint32_t* r_w = nullptr;  // pointers of the row the cursor is in
    const uint32_t* r_z = nullptr;
    const uint16_t* r_s = nullptr;
    int r_valid_for = -1;
    int i_pass = 0;  // pass of the unit to issue (kept after the sequence is exhausted)

    auto seek = [&]() {  // move to the next phase in which this wave has units
        while (true) {
            lph++;
            if (lph >= nphases) return;
            PhasePtr P = phases + lph;
            const int kind = P->kind;
            if (kind == KIND_ATTN || kind == KIND_ARGMAX) continue;
            const int passes = P->P;
            unit_range(P->rows_per_wg * passes, wave, lu, luend);
            if (lu >= luend) continue;
            l_kind = kind;
            l_passes = passes;
            l_nchunks = kind == KIND_CLS ? (P->K >> 3) : P->C;
            l_sh = P->sh;
            l_pzh = P->pzh;
            l_row_dwords = kind == KIND_CLS ? (P->K >> 1) : P->C * 4;
            l_rows = P->rows_per_wg;
            l_N = P->N;
            l_ppw = P->ppw;
            l_kpw = P->kpw;
            l_vpw = P->vpw;
            l_w0 = P->w[0];
            l_w1 = P->w[1];
            l_w2 = P->w[2];
            l_z0 = P->z[0];
            l_z1 = P->z[1];
            l_z2 = P->z[2];
            l_s0 = P->s[0];
            l_s1 = P->s[1];
            l_s2 = P->s[2];
            lr = lu / passes;
            lpass = lu - lr * passes;
            r_valid_for = -1;
            return;
        }
    };
    auto row_pointers = [&](int r) {  // stacked row r of this workgroup -> matrix row
        int m = 0, n = 0;
        if (l_kind == KIND_QKV) {
            const int sh = a.half_head_shift;
            const int half_mask = (1 << sh) - 1;
            if (r < 2 * l_ppw) {  // Q: pairs (i, i + head/2)
                const int p = g * l_ppw + (r >> 1);
                n = ((p >> sh) << (sh + 1)) + (p & half_mask) + ((r & 1) << sh);
            } else if (r < 2 * l_ppw + 2 * l_kpw) {
                const int rr = r - 2 * l_ppw;
                const int p = g * l_kpw + (rr >> 1);
                n = ((p >> sh) << (sh + 1)) + (p & half_mask) + ((rr & 1) << sh);
                m = 1;
            } else {
                n = g * l_vpw + (r - 2 * l_ppw - 2 * l_kpw);
                m = 2;
            }
        } else if (l_kind == KIND_FFN) {
            n = g * (l_rows >> 1) + (r >> 1);
            m = r & 1;  // 0 gate, 1 up
        } else {  // OPROJ, DOWN, CLS
            n = g * l_rows + r;
            if (n >= l_N) n = l_N - 1;  // rows past the end are recomputed and ignored by the epilogue
        }
        const uint32_t* bw = l_w0;
        const uint32_t* bz = l_z0;
        const uint16_t* bs = l_s0;
        if (m == 1) {
            bw = l_w1;
            bz = l_z1;
            bs = l_s1;
        } else if (m == 2) {
            bw = l_w2;
            bz = l_z2;
            bs = l_s2;
        }
        r_w = bw + (size_t)n * l_row_dwords;
        r_z = bz + (size_t)n * l_pzh;
        r_s = bs + (size_t)n * l_sh;
    };
    // Request the next unit into ring slot `slot`: 1 KB of weights + 40 bytes of scales/zeros, always exactly two
    // load instructions; once the sequence is exhausted the last unit is requested again (harmless).
    auto issue_next = [&](int slot) {
        if (lph < nphases) {
            if (lr != r_valid_for) {
                row_pointers(lr);
                r_valid_for = lr;
            }
            i_pass = lpass;
        }
        if (r_w != nullptr) {
            const uint32_t dst = __builtin_amdgcn_readfirstlane(ring_off + slot * UNIT_BYTES);
            const int c = i_pass * 64 + lane;
            if (c < l_nchunks) dma16_nt(reinterpret_cast<const u32x4*>(r_w) + c, dst);
            if (l_kind == KIND_CLS) {
                if (lane == 0) dma4(r_w, dst + 1024);
            } else {
                // lanes 0..7: 16 scales of this pass as 8 dwords; lanes 8..9: the 2 zero-point dwords of this pass
                const uint32_t* mp = nullptr;
                if (lane < 8) {
                    if (i_pass * 16 + 2 * lane < l_sh) mp = reinterpret_cast<const uint32_t*>(r_s + i_pass * 16) + lane;
                } else if (lane < 10) {
                    if (i_pass * 2 + (lane - 8) < l_pzh) mp = r_z + i_pass * 2 + (lane - 8);
                }
                if (mp) dma4(mp, dst + 1024);
            }
        }
        if (lph < nphases) {
            lu++;
            lpass++;
            if (lpass == l_passes) {
                lpass = 0;
                lr++;
            }
            if (lu == luend) seek();  // leaves the l_* state untouched when nothing is left
        }
    };

    seek();
    for (int i = 0; i < depth; i++) issue_next(i);

    int cslot = 0;
    for (int ph = 0; ph < nphases; ph++) {
        PhasePtr P = phases + ph;
        const int kind = P->kind;
        if (kind != KIND_ATTN && kind != KIND_ARGMAX) {
            const int passes = P->P;
            const int nchunks = kind == KIND_CLS ? (P->K >> 3) : P->C;
            int ubeg, uend;
            unit_range(P->rows_per_wg * passes, wave, ubeg, uend);
            int r = ubeg / passes, pass = ubeg - r * passes;
            int seg_begin = pass;  // first pass of the current row that this wave covers
            float acc = 0.0f;
            wg_barrier();  // S1
            wg_barrier();  // S2: input staged
            for (int u = ubeg; u < uend; u++) {
                wait_ring(depth);
                acc += consume_unit(kind, nchunks, pass, lane, ring + cslot * UNIT_BYTES, m.xs, m.ab, magic);
                if (pass == passes - 1 || u == uend - 1) {
                    // this wave's share of row r: the sum goes to the slot of its last pass, zero to the others
                    const float tot = wave_sum(acc);
                    const int nslots = pass - seg_begin + 1;
                    if (lane < nslots) m.partial[r * passes + seg_begin + lane] = (lane == nslots - 1) ? tot : 0.0f;
                    acc = 0.0f;
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // slot fully read before it is refilled
                issue_next(cslot);
                cslot = (cslot + 1 == depth) ? 0 : cslot + 1;
                pass++;
                if (pass == passes) {
                    pass = 0;
                    seg_begin = 0;
                    r++;
                }
            }
            wg_barrier();  // B3
        } else if (kind == KIND_ATTN) {
            int h;
            if (owns_head(a, g, h)) {
                wg_barrier();
                wg_barrier();
                wg_barrier();
                wg_barrier();
            }
        }
        wg_barrier();  // B4
        if (ph + 1 < nphases) {
            wg_barrier();  // B5
            if (*m.abort_flag) break;
        }
    }
    wait_vm0();  // loads still in flight target this workgroup's LDS
}

__device__ void helper_main(const Args& a, PhasePtr phases, int nphases, int hw, int lane, int g, const LdsMap& m, int pos) {
    const int ht = hw * 64 + lane;
    if (ht == 0) *m.abort_flag = 0;
    {   // residual rows of this workgroup start as the embedding of the current token
        const int rpw = a.dim / a.G;
        if (ht < rpw) {
            const int token = a.tokens_dev[pos];
            m.xres[ht] = a.embed[(size_t)token * a.dim + (size_t)g * rpw + ht];
        }
    }
    uint32_t epoch = a.sync->epoch_base;
    const bool tracing = a.trace != nullptr && g == 0 && ht == 0;
    for (int ph = 0; ph < nphases; ph++) {
        PhasePtr P = phases + ph;
        const int kind = P->kind;
        if (tracing) a.trace[ph * 5 + 0] = wall_clock64();
        if (kind != KIND_ATTN && kind != KIND_ARGMAX) {
            stage_input(a, P, ht, lane, hw, m.xs, m.ab, m.red, pos);  // S1, S2
            if (tracing) a.trace[ph * 5 + 1] = wall_clock64();
            wg_barrier();                                            // B3: partial sums complete
            if (tracing) a.trace[ph * 5 + 2] = wall_clock64();
            epilogue(a, P, g, ht, lane, hw, m.partial, m.xres, pos);
            wait_vm0();
        } else if (kind == KIND_ATTN) {
            int h;
            if (owns_head(a, g, h)) {
                switch (a.head_size) {
                    case 64: attention_head<8>(a, P, h, ht, lane, hw, pos, m.sc, m.red, m.acc_lds); break;
                    case 128: attention_head<16>(a, P, h, ht, lane, hw, pos, m.sc, m.red, m.acc_lds); break;
                    default: attention_head<32>(a, P, h, ht, lane, hw, pos, m.sc, m.red, m.acc_lds); break;
                }
                wait_vm0();
            }
        } else if (g == 0 && hw == 0) {  // KIND_ARGMAX: reduce the per-workgroup maxima, advance the position
            float best = -INFINITY;
            int best_i = 0x7FFFFFFF;
            for (int i = lane; i < a.G; i += 64) {
                const float v = __builtin_bit_cast(float, ld_u32(&a.sync->amax_bits[i]));
                const int idx = (int)ld_u32((const uint32_t*)&a.sync->amax_idx[i]);
                if (v > best || (v == best && idx < best_i)) {
                    best = v;
                    best_i = idx;
                }
            }
            for (int off = 32; off > 0; off >>= 1) {
                const float ov = __shfl_xor(best, off);
                const int oi = __shfl_xor(best_i, off);
                if (ov > best || (ov == best && oi < best_i)) {
                    best = ov;
                    best_i = oi;
                }
            }
            if (lane == 0) {
                if (best_i == 0x7FFFFFFF) best_i = 0;
                const int token_pos = pos + 1;
                typedef int __attribute__((address_space(1))) * gint_ptr;  // keep these global (not flat) stores
                if (a.write_token) {
                    __hip_atomic_store((gint_ptr)(uintptr_t)(a.tokens_host + token_pos), best_i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                    a.tokens_dev[token_pos] = best_i;
                }
                __hip_atomic_store((gint_ptr)(uintptr_t)a.pos_host, token_pos, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                *a.pos_dev = token_pos;
                a.sync->epoch_base = epoch;  // the next launch continues the epoch sequence
            }
        }
        wg_barrier();  // B4: this phase's stores are complete
        if (tracing) a.trace[ph * 5 + 3] = wall_clock64();
        if (ph + 1 < nphases) {
            epoch++;
            if (hw == 0) {
                if (!grid_barrier(a.sync, epoch, a.G, lane, a.spin_limit, a.err_host) && lane == 0) *m.abort_flag = 1;
            }
            wg_barrier();  // B5
            if (tracing) a.trace[ph * 5 + 4] = wall_clock64();
            if (*m.abort_flag) break;
        }
    }
}

__global__ __launch_bounds__(NT) void token_kernel(const Args a) {
    extern __shared__ char lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = blockIdx.x;
    PhasePtr phases = (PhasePtr)(uintptr_t)a.phases;
    LdsMap m;
    m.xs = reinterpret_cast<u32x4*>(lds + a.lds_xs);
    m.ab = reinterpret_cast<float2*>(lds + a.lds_ab);
    m.partial = reinterpret_cast<float*>(lds + a.lds_part);
    m.red = reinterpret_cast<float*>(lds + a.lds_misc);              // 8 floats
    m.abort_flag = reinterpret_cast<int*>(lds + a.lds_misc + 32);    // 1 int
    m.xres = reinterpret_cast<uint16_t*>(lds + a.lds_misc + 64);     // this workgroup's rows of the residual stream
    m.acc_lds = reinterpret_cast<float*>(lds + a.lds_part);          // attention reuses the partial area (4 x 256 floats)
    m.sc = reinterpret_cast<float*>(lds + a.lds_xs);                 // attention scores reuse the input area
    if (wave < NSW) {
        stream_main(a, phases, a.nphases, wave, lane, g, lds, m);
    } else {
        const int pos = *a.pos_dev;
        helper_main(a, phases, a.nphases, wave - NSW, lane, g, m, pos);
    }
}

}  // namespace tk

int tk_launch(hipStream_t stream, const tk::Args& args, size_t lds_bytes) {
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)tk::token_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) {
            awq_set_error("hipFuncSetAttribute(token_kernel) failed: %s", hipGetErrorString(e));
            return AWQ_ERR_HIP;
        }
        attr_set = true;
    }
    hipLaunchKernelGGL(tk::token_kernel, dim3(args.G), dim3(tk::NT), lds_bytes, stream, args);
    return awq_check_launch("token_kernel");
}
