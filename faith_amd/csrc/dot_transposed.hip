// McCormick bounds of a dot product in the reference's transposed layout on fp32 MFMA.
//
// The layout (Transformer_Verification_Code/Verifiers/Bounds.py:1279-1290, :1319-1329; HandTunedKernels/kernel.cpp:133-241):
// coefficients [T, L, K, D_in] with the perturbation coordinate m contiguous and K the reduction axis, result
// z [T, Lx, Ly, D_in],
//     z[i, j, m] = sum_k  x[i, k, m] a[j, k]  +  b[i, k] y[j, k, m]        (a, b: concrete intervals split by sign).
// For a FIXED i the first sum is a matrix product over k of the interval matrix a [Ly, K] with the slab
// x[i] [K, D_in]: rows j, columns m.  For a FIXED j the second is the product of b [Lx, K] with y[j] [K, D_in]:
// rows i, columns m.  The two do not share a tile -- which is why the natural-layout kernels do not serve here and
// this layout ran on the vector ALU -- but each alone is an MFMA problem whose operands need no re-layout:
//   * the slab is the B operand, lane (n, k-half) asking for element [k][m0 + n]: a wavefront's load is two runs of
//     128 contiguous bytes, straight from global memory into the register the MFMA reads (each value feeds the
//     MFMAs of every row block: up to 16 per load);
//   * the intervals are the A operand, kept in LDS for the whole batch element as [k][row] (lanes along rows:
//     conflict-free) and split by sign as they are read;
//   * the accumulators hold rows x 32 columns m per wavefront: register r of a block is row 8 (r / 4) + 4 (lane / 32)
//     + r % 4, lanes run along m -- the contiguous axis of z, so a store is again two runs of 128 bytes.
// Two launches.  The y terms go first and write z: P = sum b (y_l + y_u) and Q = sum |b| (y_l - y_u) serve both
// sides, z_l = (P + Q) / 2, z_u = (P - Q) / 2 -- two products, as on the natural-layout path.  The x terms (four
// products per k pair: a_l+, a_l-, a_u+, a_u-) then take what the first launch left in the cache as the initial
// value of their accumulators -- a load straight into the registers the MFMAs add to, requested one row block ahead --
// and store the result: one fp32 accumulation per side, the y terms first, and no pass that only adds.
// In the second launch a wavefront works through the row blocks of its tile one at a time (two accumulators; the
// slab comes from the cache again for each block: 8 KB per wavefront): the registers this leaves free hold the next
// block's initial values and the slab values ahead of the MFMAs.
#include "dot_transposed.h"

namespace {

using faith::DotTransposedArgs;

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int NTHREADS = 256;

__device__ __forceinline__ floatx16 mfma(float a, float b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ __amdgpu_buffer_rsrc_t window(const void *base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ float ld1(__amdgpu_buffer_rsrc_t r, unsigned thread_off, unsigned uniform_off) {
    return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, thread_off, uniform_off, 0));
}
__device__ __forceinline__ void st1(float v, __amdgpu_buffer_rsrc_t r, unsigned thread_off, unsigned uniform_off, int nt) {
    if (nt) __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), r, thread_off, uniform_off, 2 /* non-temporal */);
    else __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), r, thread_off, uniform_off, 0);
}
// one instruction each: this file is compiled with -fno-honor-nans (see dot.hip)
__device__ __forceinline__ float pos1(float v) { return __builtin_fmaxf(v, 0.f); }
__device__ __forceinline__ float neg1(float v) { return __builtin_fminf(v, 0.f); }

struct PassArgs {
    const float *s_lo, *s_up;    // coefficients of the object whose row is fixed: [T, Lo, K, D]
    const float *a1, *a2;        // intervals of the other object: [T, R, K] (y terms: a1 = x_l, a2 unused)
    float *zl, *zu;              // [T, Lx, Ly, D]
    int T, Lo, R, K, D, Lx, Ly;
    int m_blocks;                // blocks of 128 coordinates: ceil(D / 128)
    int tiles, per_workgroup;    // T * Lo * m_blocks tiles, dealt in runs of per_workgroup
};

// YTERMS = true : y terms, fixed row o = j of y, rows r = i: writes z[i = r, j = o].
// YTERMS = false: x terms, fixed row o = i of x, rows r = j: adds to z[i = o, j = r] (accumulators start from it).
// CH: k pairs fetched ahead of the MFMAs (K % (2 CH) == 0; sixteen measured no faster than eight).
// NB: 32-row blocks a wavefront multiplies at a time (R % (32 NB) == 0): each value of the slab then feeds 2 NB or
// 4 NB MFMAs.
template <bool YTERMS, int CH, int NB>
__global__ void __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(2, 2)))
dot_transposed_pass(const PassArgs g) {
    extern __shared__ float lds[];                         // [YTERMS ? 1 : 2][K][R + 1]
    const int tid = threadIdx.x;
    const int lane = tid % 64, wv = __builtin_amdgcn_readfirstlane(tid / 64);
    const int fi = lane % 32, fh = lane / 32;
    const int RP = g.R + 1;                                // odd pitch: the transposing fill is conflict-free too
    float *A1 = lds, *A2 = lds + g.K * RP;

    const int first = blockIdx.x * g.per_workgroup;
    const int last = min(first + g.per_workgroup, g.tiles);
    const int half = g.K / 2;
    const unsigned kstep = (unsigned)g.D * 4u;             // one step in k, bytes
    const size_t slab = (size_t)g.K * g.D;                 // floats of one row's slab
    const size_t zt = (size_t)g.Lx * g.Ly * g.D;           // floats of one batch element of z
    // one step of the row index r in z, bytes: z[i, j, m] with r = i (y terms) or r = j (x terms)
    const unsigned rstep = YTERMS ? (unsigned)g.Ly * kstep : kstep;
    int held = -1;                                         // batch element whose intervals are in LDS
    for (int tile = first; tile < last; ++tile) {
        int n = tile;
        const int mb = n % g.m_blocks;  n /= g.m_blocks;
        const int o = n % g.Lo;
        const int t = n / g.Lo;
        if (t != held) {
            if (held >= 0) __syncthreads();                // every wavefront is done with the old intervals
            // [R][K] in memory -> [K][R + 1] in LDS, 16 bytes per load and four loads per array in flight before
            // the first is stored (one at a time, the fill is a chain of as many memory latencies as it has steps)
            const float4 *s1 = reinterpret_cast<const float4 *>(g.a1 + (size_t)t * g.R * g.K);
            const float4 *s2 = YTERMS ? nullptr : reinterpret_cast<const float4 *>(g.a2 + (size_t)t * g.R * g.K);
            const int k4 = g.K / 4, n4 = g.R * k4;
            constexpr int U = 4;
            for (int base = tid; base < n4; base += NTHREADS * U) {
                float4 v1[U], v2[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int e = base + u * NTHREADS;
                    if (e < n4) {
                        v1[u] = s1[e];
                        if (!YTERMS) v2[u] = s2[e];
                    }
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int e = base + u * NTHREADS;
                    if (e < n4) {
                        const int r = e / k4, k = 4 * (e % k4);
                        float *d1 = A1 + k * RP + r;
                        d1[0] = v1[u].x;  d1[RP] = v1[u].y;  d1[2 * RP] = v1[u].z;  d1[3 * RP] = v1[u].w;
                        if (!YTERMS) {
                            float *d2 = A2 + k * RP + r;
                            d2[0] = v2[u].x;  d2[RP] = v2[u].y;  d2[2 * RP] = v2[u].z;  d2[3 * RP] = v2[u].w;
                        }
                    }
                }
            }
            __syncthreads();
            held = t;
        }
        const int m0 = mb * 128 + wv * 32;
        if (m0 >= g.D) continue;                           // a wavefront without coordinates (no barrier below)

        // the slab of row o: lane (n = fi, k half = fh) reads [fh * K / 2 + s][m0 + fi] in step s
        const size_t row = ((size_t)t * g.Lo + o) * slab;
        const __amdgpu_buffer_rsrc_t w1 = window(g.s_lo + row, (unsigned)(slab * 4)), w2 = window(g.s_up + row, (unsigned)(slab * 4));
        const unsigned vs = (unsigned)(fh * half) * kstep + (unsigned)(m0 + fi) * 4u;
        const int ka = fh * half;                          // this lane's first k in the interval matrix
        // z of this batch element; the tile's fixed index and the lane's own part of the row index and column go
        // into the lane's offset, the rest of the row index is a scalar per register
        const __amdgpu_buffer_rsrc_t wzl = window(g.zl + (size_t)t * zt, (unsigned)(zt * 4)), wzu = window(g.zu + (size_t)t * zt, (unsigned)(zt * 4));
        const unsigned vz = (YTERMS ? (unsigned)o * kstep : (unsigned)o * (unsigned)g.Ly * kstep) + (unsigned)(4 * fh) * rstep +
                            (unsigned)(m0 + fi) * 4u;
        auto zrow = [&](int r0, int r) { return (unsigned)(r0 + 8 * (r / 4) + r % 4) * rstep; };

        floatx16 c1[NB], c2[NB], n1[NB], n2[NB];
        if (!YTERMS) {
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    c1[b][r] = ld1(wzl, vz, zrow(32 * b, r));
                    c2[b][r] = ld1(wzu, vz, zrow(32 * b, r));
                }
        }
        for (int r0 = 0; r0 < g.R; r0 += 32 * NB) {
            if (YTERMS) {
#pragma unroll
                for (int b = 0; b < NB; ++b)
#pragma unroll
                    for (int r = 0; r < 16; ++r) c1[b][r] = c2[b][r] = 0.f;
            } else if (r0 + 32 * NB < g.R) {
                // the next blocks' initial values: on their way while these blocks are multiplied
#pragma unroll
                for (int b = 0; b < NB; ++b)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        n1[b][r] = ld1(wzl, vz, zrow(r0 + 32 * (NB + b), r));
                        n2[b][r] = ld1(wzu, vz, zrow(r0 + 32 * (NB + b), r));
                    }
            }
            float p1[CH], p2[CH], q1[CH], q2[CH];
            auto fetch = [&](float (&u)[CH], float (&v)[CH], int s0) {
#pragma unroll
                for (int i = 0; i < CH; ++i) {
                    u[i] = ld1(w1, vs, (unsigned)(s0 + i) * kstep);
                    v[i] = ld1(w2, vs, (unsigned)(s0 + i) * kstep);
                }
            };
            auto multiply = [&](const float (&u)[CH], const float (&v)[CH], int s0) {
                // the chunk's interval values first, all of them: one LDS latency per chunk instead of one per k pair
                const float *a1 = A1 + (ka + s0) * RP + r0 + fi, *a2 = A2 + (ka + s0) * RP + r0 + fi;
                float al[NB][CH], au[NB][YTERMS ? 1 : CH];
#pragma unroll
                for (int i = 0; i < CH; ++i)
#pragma unroll
                    for (int b = 0; b < NB; ++b) {
                        al[b][i] = a1[i * RP + 32 * b];
                        if (!YTERMS) au[b][i] = a2[i * RP + 32 * b];
                    }
                __builtin_amdgcn_sched_barrier(0);     // (left to itself the compiler moves each read down to its MFMA)
#pragma unroll
                for (int i = 0; i < CH; ++i) {
                    if (YTERMS) {
                        const float ys = u[i] + v[i], yd = u[i] - v[i];
#pragma unroll
                        for (int b = 0; b < NB; ++b) {
                            c1[b] = mfma(al[b][i], ys, c1[b]);
                            c2[b] = mfma(__builtin_fabsf(al[b][i]), yd, c2[b]);
                        }
                    } else {
#pragma unroll
                        for (int b = 0; b < NB; ++b) {
                            c1[b] = mfma(pos1(al[b][i]), u[i], c1[b]);
                            c2[b] = mfma(pos1(au[b][YTERMS ? 0 : i]), v[i], c2[b]);
                        }
#pragma unroll
                        for (int b = 0; b < NB; ++b) {
                            c1[b] = mfma(neg1(al[b][i]), v[i], c1[b]);
                            c2[b] = mfma(neg1(au[b][YTERMS ? 0 : i]), u[i], c2[b]);
                        }
                    }
                }
            };
            fetch(p1, p2, 0);
            for (int s0 = 0; s0 < half; s0 += 2 * CH) {
                if (s0 + CH < half) fetch(q1, q2, s0 + CH);
                __builtin_amdgcn_sched_barrier(0);         // the fetch goes first
                multiply(p1, p2, s0);
                if (s0 + CH < half) {
                    if (s0 + 2 * CH < half) fetch(p1, p2, s0 + 2 * CH);
                    __builtin_amdgcn_sched_barrier(0);
                    multiply(q1, q2, s0 + CH);
                }
            }
            // ---- results: register r of block b is row r0 + 32 b + 8 (r / 4) + 4 fh + r % 4, column m0 + fi
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    if (YTERMS) {
                        const float p = c1[b][r], q = c2[b][r];
                        st1(0.5f * (p + q), wzl, vz, zrow(r0 + 32 * b, r), 0);      // read again by the second launch: left in the cache
                        st1(0.5f * (p - q), wzu, vz, zrow(r0 + 32 * b, r), 0);
                    } else {
                        st1(c1[b][r], wzl, vz, zrow(r0 + 32 * b, r), 1);
                        st1(c2[b][r], wzu, vz, zrow(r0 + 32 * b, r), 1);
                    }
                }
            if (!YTERMS) {
#pragma unroll
                for (int b = 0; b < NB; ++b) {
                    c1[b] = n1[b];
                    c2[b] = n2[b];
                }
            }
        }
    }
}

template <bool YTERMS>
bool launch_pass(const PassArgs &p, hipStream_t st) {
    const size_t lds = (size_t)(YTERMS ? 1 : 2) * p.K * (p.R + 1) * sizeof(float);
    const dim3 gd((unsigned)((p.tiles + p.per_workgroup - 1) / p.per_workgroup)), bd(NTHREADS);
    // y terms: every row block at once where the registers hold them (each slab value is then loaded once; 190
    // against 194 us with two blocks and 207 with one, whole operator at 128 x 128 x 64, dim_in 256).  x terms: one
    // block at a time, the next block's initial values on their way meanwhile (two at a time measured no faster).
    if (YTERMS && p.R % 128 == 0) {
        if (!faith::reserve_lds(dot_transposed_pass<YTERMS, 8, 4>, lds)) return false;
        hipLaunchKernelGGL((dot_transposed_pass<YTERMS, 8, 4>), gd, bd, lds, st, p);
    } else if (YTERMS && p.R % 64 == 0) {
        if (!faith::reserve_lds(dot_transposed_pass<YTERMS, 8, 2>, lds)) return false;
        hipLaunchKernelGGL((dot_transposed_pass<YTERMS, 8, 2>), gd, bd, lds, st, p);
    } else {
        if (!faith::reserve_lds(dot_transposed_pass<YTERMS, 8, 1>, lds)) return false;
        hipLaunchKernelGGL((dot_transposed_pass<YTERMS, 8, 1>), gd, bd, lds, st, p);
    }
    return true;
}

PassArgs pass_args(const DotTransposedArgs &a, bool yterms) {
    PassArgs p{};
    p.s_lo = yterms ? a.ylw : a.xlw;  p.s_up = yterms ? a.yuw : a.xuw;
    p.a1 = yterms ? a.x_l : a.y_l;    p.a2 = yterms ? nullptr : a.y_u;
    p.zl = a.zlw;  p.zu = a.zuw;
    p.T = a.T;  p.Lo = yterms ? a.Ly : a.Lx;  p.R = yterms ? a.Lx : a.Ly;
    p.K = a.K;  p.D = a.D;  p.Lx = a.Lx;  p.Ly = a.Ly;
    p.m_blocks = (a.D + 127) / 128;
    p.tiles = a.T * p.Lo * p.m_blocks;
    // two workgroups per CU (registers), each a run of consecutive tiles: they share the batch element, whose
    // intervals stay in LDS
    const int resident = 2 * faith::compute_units();
    p.per_workgroup = (p.tiles + resident - 1) / resident;
    return p;
}

}  // namespace

namespace faith {

bool dot_transposed_mfma_takes(int Lx, int Ly, int K, int D) {
    const long long lds_x = 2LL * K * (Ly + 1) * 4, lds_y = 1LL * K * (Lx + 1) * 4;
    return Lx % 32 == 0 && Ly % 32 == 0 && D % 32 == 0 && K % (2 * 8) == 0 && lds_x <= 80 * 1024 && lds_y <= 80 * 1024 &&
           (long long)K * D * 4 < 0x7fffffffLL && (long long)Lx * Ly * D * 4 < 0x7fffffffLL;
}

bool dot_transposed_mfma_launch(const DotTransposedArgs &a, hipStream_t stream) {
    const PassArgs px = pass_args(a, false), py = pass_args(a, true);
    // both kernels' LDS is settled before the first launch
    const size_t lx = 2 * (size_t)px.K * (px.R + 1) * sizeof(float), ly = (size_t)py.K * (py.R + 1) * sizeof(float);
    if (lx > 160 * 1024 || ly > 160 * 1024) return false;
    if (!launch_pass<true>(py, stream)) return false;      // the y terms write z, the x terms add to it
    return launch_pass<false>(px, stream);
}

}  // namespace faith
