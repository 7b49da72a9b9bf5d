/*
 * dr_oracle.c -- CPU restatement of deepRacin's CNN layer arithmetic.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker the HIP kernels are compared against (tests/, the smoke test and the
 * cpu_baseline leg of the benchmark).  Nothing in the product library links, loads or calls it.
 *
 * Every function restates, in plain scalar fp32 C, the loop nest and accumulation order of the
 * reference's OpenCL kernel for that layer (citations are into the reference tree).  Where the
 * reference kernel is wrong or undefined the function follows the documented contract instead and
 * says so.  `mad(a,b,c)` of the reference may or may not be fused under its build flags
 * (-cl-mad-enable -cl-fast-relaxed-math, src/dR_clwrap.c:516); this restatement uses unfused
 * multiply-add; the difference is far inside the 1e-4 parity tolerance.
 *
 * Pinning (what each function is checked against in tests/test_oracle_pins.py):
 *   oracle_conv_direct    closed-form fp64 correlation, torch.nn.functional.conv2d, delta filter,
 *                         all-ones border counts, brute force with odd sizes and stride 2
 *   oracle_wino_*         Lavin-Gray identity on random 4x4/3x3, equality with oracle_conv_direct
 *   oracle_conv1x1        fp64 einsum
 *   oracle_pool           torch max_pool2d/avg_pool2d(ceil_mode) on explicitly zero-padded input
 *   oracle_fc             fp64 GEMV with the HWC permutation, torch linear
 *   oracle_softmax        scipy.special.softmax
 *   oracle_normalize      numpy mean / std in fp64 (closed form), constant-offset and scaling identities
 *   whole network         the reference's stored SqueezeNet v1.1 + tiger.png -> 292, puzzle.png -> 611
 *   stride > 1 conv       header formula only (include/dR_nodes_conv2d.h:47-54); the reference's
 *                         generated kernel ignores the stride, so no reference run could pin it.
 *
 * Parallelism: OpenMP over output channels / rows, the same axes the OpenCL work-items span.
 * Tensors are [C][H][W] fp32, x fastest.
 */
#include <float.h>
#include <math.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define DR_API __attribute__((visibility("default")))

/* Kernels/dR_helper.cl:15-28 sampleZeroPaddedFloat */
static inline float sample0(const float* img, size_t offset, int x, int y, int W, int H) {
    if (x < 0 || x >= W || y < 0 || y >= H) return 0.0f;
    return img[offset + (size_t)y * W + x];
}

static inline float act(float v, int relu) {
    /* ReLU is clamp(v, 0, FLT_MAX) in every reference kernel (e.g. Kernels/dR_winograd2.cl:232-239) */
    if (!relu) return v;
    return v < 0.0f ? 0.0f : (v > FLT_MAX ? FLT_MAX : v);
}

DR_API int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

DR_API void oracle_set_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/*
 * Direct convolution: generated kernel of src/dR_nodes_conv2d.c:481-773.
 *   out = 0; for c: { s = 0; for j,i: s = mad(sample(in,c,x+i-p,y+j-q), w[c][o][j][i], s); out += s }
 *   out = act(out + b)
 * w is [I][O][kh][kw] (:617 indexes gFilter[c*k*k*O + o*k*k + tap]).
 * Stride: the generated kernel never uses it; this function follows include/dR_nodes_conv2d.h:47-54,
 * i.e. the window of output (x,y) is centred on input (x*sx, y*sy) and the output is (W/sx, H/sy).
 */
DR_API void oracle_conv_direct(const float* in, const float* w, const float* bias, float* out,
                               int W, int H, int I, int O, int kw, int kh, int sx, int sy, int relu) {
    const int Wo = W / sx, Ho = H / sy, px = kw / 2, py = kh / 2;
#pragma omp parallel for collapse(2) schedule(static)
    for (int o = 0; o < O; ++o)
        for (int y = 0; y < Ho; ++y)
            for (int x = 0; x < Wo; ++x) {
                float acc = 0.0f;
                for (int c = 0; c < I; ++c) {
                    float s = 0.0f;
                    const float* f = w + ((size_t)c * O + o) * kh * kw;
                    for (int j = 0; j < kh; ++j)
                        for (int i = 0; i < kw; ++i)
                            s = sample0(in, (size_t)c * W * H, x * sx + i - px, y * sy + j - py, W, H) * f[j * kw + i] + s;
                    acc += s;
                }
                if (bias) acc = acc + bias[o];
                out[((size_t)o * Ho + y) * Wo + x] = act(acc, relu);
            }
}

/*
 * Winograd filter transform: dR_conv2d_winograd_fillBuffers, src/dR_nodes_conv2d.c:1162-1240.
 * U[c][o] = G g G^T with dR_matmul / dR_matmulT (src/dR_core.c:677-723: sum starts at 0.0 and adds
 * every product, zeros included), then re-laid [I][O][16] -> [I][16][O].
 */
DR_API void oracle_wino_filter(const float* w, float* U, int I, int O) {
    static const float G[12] = { 1.0f, 0.0f, 0.0f, 0.5f, 0.5f, 0.5f, 0.5f, -0.5f, 0.5f, 0.0f, 0.0f, 1.0f };
    for (int c = 0; c < I; ++c)
        for (int o = 0; o < O; ++o) {
            const float* g = w + ((size_t)c * O + o) * 9;
            float t[12], u[16];
            for (int r = 0; r < 4; ++r)
                for (int j = 0; j < 3; ++j) {
                    float s = 0.0f;
                    for (int k = 0; k < 3; ++k) s += G[r * 3 + k] * g[k * 3 + j];
                    t[r * 3 + j] = s;
                }
            for (int r = 0; r < 4; ++r)
                for (int q = 0; q < 4; ++q) {
                    float s = 0.0f;
                    for (int k = 0; k < 3; ++k) s += t[r * 3 + k] * G[q * 3 + k];
                    u[r * 4 + q] = s;
                }
            for (int k = 0; k < 16; ++k) U[((size_t)c * 16 + k) * O + o] = u[k];
        }
}

/*
 * Winograd F(2x2,3x3) convolution: kernel conv2dwinograd2, Kernels/dR_winograd2.cl:23-254.
 * U is the reference layout [I][16][O].  Per 2x2 output tile with origin (ox,oy):
 *   d = 4x4 window at (ox-1, oy-1), zero padded                                  (:72-100)
 *   V = B^T d B: left factor first (:72-100), then right factor (:135-157)
 *   M[k] = sum_c mad(V_c[k], U[c][k][o], M[k]),  c ascending                      (:180-189)
 *   Y = A^T M A: right factor first (:198-205), then left factor (:214-217)
 *   Y += b[o]; clamp; store the in-bounds part of the tile                        (:222-251)
 */
DR_API void oracle_conv_winograd(const float* in, const float* U, const float* bias, float* out,
                                 int W, int H, int I, int O, int relu) {
    const int tilesX = (W + 1) / 2, tilesY = (H + 1) / 2;
    const size_t plane = (size_t)W * H;
    const size_t nt = (size_t)tilesX * tilesY;
    /* V for all tiles and channels: [tile][c][16] */
    float* V = (float*)malloc(nt * I * 16 * sizeof(float));
#pragma omp parallel for schedule(static)
    for (int ty = 0; ty < tilesY; ++ty)
        for (int tx = 0; tx < tilesX; ++tx)
            for (int c = 0; c < I; ++c) {
                const int x0 = 2 * tx - 1, y0 = 2 * ty - 1;
                float d[16], m[16];
                for (int r = 0; r < 4; ++r)
                    for (int q = 0; q < 4; ++q) d[4 * r + q] = sample0(in, c * plane, x0 + q, y0 + r, W, H);
                for (int q = 0; q < 4; ++q) {
                    m[q]      =  d[q]     - d[8 + q];
                    m[4 + q]  =  d[4 + q] + d[8 + q];
                    m[8 + q]  = -d[4 + q] + d[8 + q];
                    m[12 + q] = -d[4 + q] + d[12 + q];
                }
                float* v = V + (((size_t)ty * tilesX + tx) * I + c) * 16;
                for (int r = 0; r < 4; ++r) {
                    const float t1 = m[4 * r + 1];
                    v[4 * r + 0] =  m[4 * r + 0] - m[4 * r + 2];
                    v[4 * r + 1] =  m[4 * r + 1] + m[4 * r + 2];
                    v[4 * r + 2] = -t1 + m[4 * r + 2];
                    v[4 * r + 3] = -t1 + m[4 * r + 3];
                }
            }
#pragma omp parallel for collapse(2) schedule(static)
    for (int o = 0; o < O; ++o)
        for (int ty = 0; ty < tilesY; ++ty)
            for (int tx = 0; tx < tilesX; ++tx) {
                const float* v = V + ((size_t)ty * tilesX + tx) * I * 16;
                float m[16];
                for (int k = 0; k < 16; ++k) m[k] = 0.0f;
                for (int c = 0; c < I; ++c)
                    for (int k = 0; k < 16; ++k) m[k] = v[c * 16 + k] * U[((size_t)c * 16 + k) * O + o] + m[k];
                float s[8];
                s[0] = m[0] + m[1] + m[2];    s[1] = m[1] - m[2] + m[3];
                s[2] = m[4] + m[5] + m[6];    s[3] = m[5] - m[6] + m[7];
                s[4] = m[8] + m[9] + m[10];   s[5] = m[9] - m[10] + m[11];
                s[6] = m[12] + m[13] + m[14]; s[7] = m[13] - m[14] + m[15];
                float y00 = s[0] + s[2] + s[4], y01 = s[1] + s[3] + s[5];
                float y10 = s[2] - s[4] + s[6], y11 = s[3] - s[5] + s[7];
                if (bias) { y00 += bias[o]; y01 += bias[o]; y10 += bias[o]; y11 += bias[o]; }
                const int ox = 2 * tx, oy = 2 * ty;
                float* po = out + o * plane + (size_t)oy * W + ox;
                po[0] = act(y00, relu);
                if (ox + 1 < W) po[1] = act(y01, relu);
                if (oy + 1 < H) {
                    po[W] = act(y10, relu);
                    if (ox + 1 < W) po[W + 1] = act(y11, relu);
                }
            }
    free(V);
}

/*
 * 1x1 convolution: Kernels/dR_conv2d1x1.cl:4-53 after the [I][O] -> [O][I] re-layout of
 * src/dR_nodes_conv2d.c:1696-1716.  out = 0; for c: out += in[c,p] * w[o][c]; out += b; clamp.
 * w here is the caller's [I][O] array.
 */
DR_API void oracle_conv1x1(const float* in, const float* w, const float* bias, float* out,
                           int P, int I, int O, int relu) {
#pragma omp parallel for schedule(static)
    for (int o = 0; o < O; ++o)
        for (int p = 0; p < P; ++p) {
            float acc = 0.0f;
            for (int c = 0; c < I; ++c) acc += in[(size_t)c * P + p] * w[(size_t)c * O + o];
            if (bias) acc += bias[o];
            out[(size_t)o * P + p] = act(acc, relu);
        }
}

/*
 * Pooling: generated kernel of src/dR_nodes_pooling.c:277-401, shape rule :186-224.
 * Window anchored at (x*stx, y*sty, z*stz); scan z, y, x ascending; x/y outside the image read 0.0f.
 * max: r = -FLT_MAX; r = max(r, v).   average: r = 0; r += v; r / (sx*sy*sz).
 * The reference does not bound-check z (reads the neighbouring channel / past the buffer); here a
 * z outside the tensor reads 0.0f.  argmax (may be NULL): flat input index of the first maximum,
 * -1 when the maximum is a padding zero -- an addition of this build, the reference has no index
 * output.
 */
DR_API void oracle_pool(const float* in, float* out, int* argmax, int W, int H, int C,
                        int sx, int sy, int sz, int stx, int sty, int stz, int type) {
    const int Wo = (W + stx - 1) / stx, Ho = (H + sty - 1) / sty, Co = (C + stz - 1) / stz;
#pragma omp parallel for schedule(static)
    for (int zo = 0; zo < Co; ++zo)
        for (int yo = 0; yo < Ho; ++yo)
            for (int xo = 0; xo < Wo; ++xo) {
                float r = type == 0 ? -FLT_MAX : 0.0f;
                int where = -1;
                for (int dz = 0; dz < sz; ++dz)
                    for (int dy = 0; dy < sy; ++dy)
                        for (int dx = 0; dx < sx; ++dx) {
                            const int x = xo * stx + dx, y = yo * sty + dy, z = zo * stz + dz;
                            const int inside = x < W && y < H && z < C;
                            const int flat = (z * H + y) * W + x;
                            const float v = inside ? in[flat] : 0.0f;
                            if (type == 0) { if (v > r) { r = v; where = inside ? flat : -1; } }
                            else r += v;
                        }
                const size_t idx = ((size_t)zo * Ho + yo) * Wo + xo;
                out[idx] = type == 0 ? r : r / (float)(sx * sy * sz);
                if (argmax && type == 0) argmax[idx] = where;
            }
}

/*
 * Fully connected: matrixVectorMultFirst / matrixVectorMultSecond, Kernels/dR_fcl.cl:59-120.
 *   xh[k] = in[(k%C)*W*H + (k/C/W)*W + (k/C)%W]            (mapToDepthMajor, dR_helper.cl:131-142)
 *   part[p][n] = sum_{i<Psz} Wt[(p*Psz+i)][n] * xh[p*Psz+i]   sequential, sum += a*b
 *   y[n] = act(sum_p part[p][n] + b[n])
 * Psz is device dependent in the reference (src/dR_nodes_fc.c:129-176) and its second kernel uses
 * K/Psz partitions (integer division, :249), silently dropping a ragged tail; this restatement sums
 * ALL of K (ceil(K/Psz) partitions), which is what the layer is documented to compute.
 */
DR_API void oracle_fc(const float* in, const float* Wt, const float* bias, float* y,
                      int W, int H, int C, int N, int relu, int Psz) {
    const int K = W * H * C;
    if (Psz <= 0 || Psz > K) Psz = K;
    const int parts = (K + Psz - 1) / Psz;
    float* xh = (float*)malloc((size_t)K * sizeof(float));
    for (int k = 0; k < K; ++k) {
        const int z = k % C, x = (k / C) % W, yy = (k / C) / W;
        xh[k] = in[(size_t)z * W * H + (size_t)yy * W + x];
    }
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n) {
        float total = 0.0f;
        for (int p = 0; p < parts; ++p) {
            float s = 0.0f;
            const int k1 = (p + 1) * Psz < K ? (p + 1) * Psz : K;
            for (int k = p * Psz; k < k1; ++k) s += Wt[(size_t)k * N + n] * xh[k];
            total += s;
        }
        if (bias) total += bias[n];
        y[n] = act(total, relu);
    }
    free(xh);
}

/*
 * Softmax: dR_softmax_compute, src/dR_nodes_math.c:620-678: e = exp(x) (computeExp,
 * Kernels/dR_math.cl:295-305); S = sequential fp32 sum on the host; y = e * (1/S) (mulScalar,
 * :216-227).  No max subtraction.
 */
DR_API void oracle_softmax(const float* x, float* y, int n) {
    float S = 0.0f;
    for (int i = 0; i < n; ++i) { y[i] = expf(x[i]); }
    for (int i = 0; i < n; ++i) S += y[i];
    const float inv = 1 / S;
    for (int i = 0; i < n; ++i) y[i] = y[i] * inv;
}

/* Box copy dst[z+dz0][y+dy0][x+dx0] = src[z+sz0][y+sy0][x+sx0]: the arithmetic-free part of Concat
 * (src/dR_nodes_transform.c:468-553) and Slice (extractSlice, Kernels/dR_transform.cl:5-24). */
DR_API void oracle_copy3d(const float* src, int sW, int sH, int sx0, int sy0, int sz0,
                          float* dst, int dW, int dH, int dx0, int dy0, int dz0, int w, int h, int c) {
    for (int z = 0; z < c; ++z)
        for (int y = 0; y < h; ++y)
            memcpy(dst + ((size_t)(z + dz0) * dH + (y + dy0)) * dW + dx0,
                   src + ((size_t)(z + sz0) * sH + (y + sy0)) * sW + sx0, (size_t)w * sizeof(float));
}

/* addScalar ... powScalar, Kernels/dR_math.cl:170-341; op numbering of dR_ElemWise1OperationType. */
DR_API void oracle_scalar_op(const float* x, float* y, size_t n, int op, float s) {
    for (size_t i = 0; i < n; ++i) {
        const float v = x[i];
        switch (op) {
            case 0: y[i] = v + s; break;
            case 1: y[i] = v - s; break;
            case 2: y[i] = v * s; break;
            case 3: y[i] = v / s; break;
            case 4: y[i] = logf(v); break;
            case 5: y[i] = expf(v); break;
            case 6: y[i] = sqrtf(v); break;
            case 7: y[i] = s; break;
            default: y[i] = powf(v, s); break;
        }
    }
}

/* One pass of `getAvg` / `getSumDev` (Kernels/dR_helper.cl:315-471) over one channel plane of
 * gW x gH values: work-groups of 16 x 8, each loads its values (0 outside the plane; `first`:
 * (v - avg)^2 instead of v) and adds them with the halving tree lsum[lid] += lsum[lid + half],
 * lid = ly*16 + lx.  One result per work-group, written row-major into `out`. */
static void norm_tree_pass(const float* in, float* out, int gW, int gH, int first, float avg) {
    const int ngx = (gW + 15) / 16, ngy = (gH + 7) / 8;
    for (int gyb = 0; gyb < ngy; ++gyb)
        for (int gxb = 0; gxb < ngx; ++gxb) {
            float lsum[128];
            for (int ly = 0; ly < 8; ++ly)
                for (int lx = 0; lx < 16; ++lx) {
                    const int gx = gxb * 16 + lx, gy = gyb * 8 + ly;
                    float v = 0.0f;
                    if (gx < gW && gy < gH) {
                        v = in[gy * gW + gx];
                        if (first) { const float d = v - avg; v = d * d; }
                    }
                    lsum[ly * 16 + lx] = v;
                }
            for (int half = 64; half >= 1; half >>= 1)
                for (int lid = 0; lid < half; ++lid) lsum[lid] += lsum[lid + half];
            out[gyb * ngx + gxb] = lsum[0];
        }
}

/* Sum of one channel plane by repeated tree passes until one work-group is left
 * (src/dR_nodes_misc.c:1206-1258, 1312-1368). */
static float norm_plane_sum(const float* plane, int W, int H, int dev, float avg, float* t1, float* t2) {
    const float* in = plane;
    float* out = t1;
    int gW = W, gH = H, first = dev;
    for (;;) {
        norm_tree_pass(in, out, gW, gH, first, avg);
        const int ngx = (gW + 15) / 16, ngy = (gH + 7) / 8;
        if (ngx * ngy == 1) return out[0];
        in = out;
        out = (out == t1) ? t2 : t1;
        gW = ngx; gH = ngy; first = 0;
    }
}

/* Normalization node, src/dR_nodes_misc.c:1163-1446: per-channel tree sums, a sequential host sum
 * over the channels, mean = sum / (W*H*C); the same again for (x - mean)^2 and dev = sqrt(sum / n);
 * then y = x + (targetMean - mean) [type 0], x * (1 / (dev / targetDev)) [type 1] or both [type 2]
 * (`addScalar`, `mulScalar`, `addMulScalar`, Kernels/dR_math.cl:100-144).  The reference sizes its
 * two scratch buffers for a single channel; this restatement gives every channel its own passes,
 * which is what the kernel's indexing intends. */
DR_API void oracle_normalize(const float* x, float* y, int W, int H, int C, int type, float targetMean, float targetDev) {
    const size_t plane = (size_t)W * H, n = plane * C;
    const int ng = ((W + 15) / 16) * ((H + 7) / 8);
    float* t1 = (float*)malloc(sizeof(float) * (size_t)ng);
    float* t2 = (float*)malloc(sizeof(float) * (size_t)ng);
    float sum = 0.0f;
    for (int c = 0; c < C; ++c) sum += norm_plane_sum(x + c * plane, W, H, 0, 0.0f, t1, t2);
    const float gavg = sum / (float)n;
    float gdev = 1.0f;
    if (type == 1 || type == 2) {
        sum = 0.0f;
        for (int c = 0; c < C; ++c) sum += norm_plane_sum(x + c * plane, W, H, 1, gavg, t1, t2);
        gdev = (float)sqrt(sum / (float)n);
    }
    free(t1);
    free(t2);
    const float add = -(gavg - targetMean), mul = 1.0f / (gdev / targetDev);
    for (size_t i = 0; i < n; ++i) {
        if (type == 0) y[i] = x[i] + add;
        else if (type == 1) y[i] = x[i] * mul;
        else y[i] = (x[i] + add) * mul;
    }
}
