"""numpy restatements of the reference's in-tree nested-loop references (test infrastructure).

Every function cites the reference lines it restates.  Pins (what fixes each function's
behaviour independently of this file) are exercised in tests/test_oracle.py.
"""
import numpy as np


def gemm_accumulate(A, B, C):
    """C + A.B, row-major.  Reference: tests/wrapper_test_167.cpp:21-28 (Halide::Buffer indices
    are flipped there: C_ref(i, j) += A(k, j) * B(i, k) is C[j][i] += A[j][k] * B[k][i]).
    Accumulation order is k ascending from the initial C, in fp32, like the reference loop."""
    out = C.astype(np.float32).copy()
    K = A.shape[1]
    for k in range(K):
        out += np.outer(A[:, k], B[k, :]).astype(np.float32)
    return out


def sgemm(A, B, C, alpha, beta):
    """alpha*A.B + beta*C.  Reference: tests/wrapper_test_162.cpp:28-35 and
    benchmarks/linear_algebra/blas/level3/sgemm/cpu/sgemm_wrapper.cpp:166-169."""
    acc = np.zeros((A.shape[0], B.shape[1]), dtype=np.float32)
    for k in range(A.shape[1]):
        acc += np.outer(A[:, k], B[k, :]).astype(np.float32)
    return (np.float32(alpha) * acc + np.float32(beta) * C.astype(np.float32)).astype(np.float32)


def transpose(A):
    """Reference: tests/wrapper_test_168.cpp:8-19."""
    return np.ascontiguousarray(A.T)


def alloc_in_time_loop_expected(steps, px, qx):
    """What tests/programs/alloc_in_time_loop.cpp must leave in its two buffers: every time slice
    overwritten by its fill expression (structure of the reference's tests/wrapper_test_197.cpp:8-41,
    which expects constant fills; here the fill depends on the indices so that a wrong index or a
    skipped slice shows)."""
    t = np.arange(steps)[:, None, None]
    p0, p1 = np.arange(px)[None, :, None], np.arange(px)[None, None, :]
    q0, q1 = np.arange(qx)[None, :, None], np.arange(qx)[None, None, :]
    P = (7 + p0 * 100 + p1 + t).astype(np.int32)
    Q = (-3 + q0 - q1 * 2 + t).astype(np.int32)
    return P, Q


def sgemm_strided(Abuf, Bbuf, Cbuf, M, N, K, alpha, beta, ldA, ldB, ldC, offA, offB, offC, tA, tB):
    """Row-major GEMM on flat buffers with leading dimensions, element offsets and optional
    transposition, as tiramisu_cublas_sgemm defines them (tiramisu_cuda_wrappers.cpp:74-115):
    ld == 0 means tightly packed."""
    if ldA == 0:
        ldA = M if tA else K
    if ldB == 0:
        ldB = K if tB else N
    if ldC == 0:
        ldC = N
    out = Cbuf.copy().ravel()
    a, b = Abuf.ravel(), Bbuf.ravel()
    real = Cbuf.dtype.type              # float32, or float64 for tiramisu_cublas_dgemm (:117-162)
    for m in range(M):
        for n in range(N):
            acc = real(0)
            for k in range(K):
                av = a[offA + (k * ldA + m if tA else m * ldA + k)]
                bv = b[offB + (n * ldB + k if tB else k * ldB + n)]
                acc = real(acc + real(av * bv))
            idx = offC + m * ldC + n
            out[idx] = real(alpha) * acc + (real(beta) * out[idx] if beta != 0 else real(0))
    return out.reshape(Cbuf.shape)


def heat2d(grid, steps, boundary_other=None):
    """STEPS sweeps of out = 0.2*(c + n + s + w + e) over the interior of a square grid on two
    ping-pong planes; returns both planes as the un-tiled program leaves them (plane t % 2 holds
    step t).  Association and rounding follow the program text in tiramisu_amd/programs/heat2d.cpp
    -- ((((c+n)+s)+w)+e)*0.2f in fp32 -- which is the 5-point form of the reference's
    benchmarks/halide/heat2d_tiramisu.cpp:52-86 with the benchmark configuration's coefficients, iterated in time like
    benchmarks/halide/heat3d_tiramisu.cpp:27-45.  `boundary_other` is the initial content of
    plane 1 (its boundary cells are read by even steps); zeros if omitted."""
    g = grid.astype(np.float32)
    planes = np.zeros((2,) + g.shape, np.float32)
    planes[0] = g
    if boundary_other is not None:
        planes[1] = boundary_other
    c02 = np.float32(0.2)
    for t in range(1, steps + 1):
        src, dst = planes[(t - 1) % 2], planes[t % 2]
        acc = src[1:-1, 1:-1] + src[:-2, 1:-1]
        acc = acc + src[2:, 1:-1]
        acc = acc + src[1:-1, :-2]
        acc = acc + src[1:-1, 2:]
        dst[1:-1, 1:-1] = acc * c02
    return planes


def row_filter(image, taps):
    """out[r, c] = sum_t image[r, c + t] * taps[t] in fp32, products added left to right: the loop
    nest of tests/programs/taps_in_constant_memory.cpp (a one-dimensional pass of the reference's
    benchmarks/halide/gaussiangpu_tiramisu.cpp:46-57)."""
    n = taps.shape[0]
    width = image.shape[1] - n + 1
    acc = image[:, 0:width] * taps[0]
    for t in range(1, n):
        acc = acc + image[:, t:t + width] * taps[t]
    return acc.astype(np.float32)


def resample_bilinear(src):
    """The bilinear resampling of tests/programs/resample_bilinear.cpp (the structure of the
    reference's benchmarks/halide/warp_affinegpu_tiramisu.cpp:55-76: affine sample position, floor,
    clamped neighbours, two horizontal and one vertical interpolation), in fp32, operation by
    operation as the program text has them."""
    f = np.float32
    h, w = src.shape
    y = np.arange(h, dtype=np.float32)[:, None]
    x = np.arange(w, dtype=np.float32)[None, :]
    fy = (y * f(0.96875) + x * f(0.0625)) - f(1.5)
    fx = (x * f(0.96875) - y * f(0.0625)) + f(2.25)
    y0 = np.floor(fy).astype(np.int32)
    x0 = np.floor(fx).astype(np.int32)
    wy = fy - np.floor(fy)
    wx = fx - np.floor(fx)
    ya, yc = np.clip(y0, 0, h - 1), np.clip(y0 + 1, 0, h - 1)
    xa, xc = np.clip(x0, 0, w - 1), np.clip(x0 + 1, 0, w - 1)
    s = src.astype(np.float32)
    p00, p01, p10, p11 = s[ya, xa], s[ya, xc], s[yc, xa], s[yc, xc]
    top = p00 + (p01 - p00) * wx
    bottom = p10 + (p11 - p10) * wx
    return (top + (bottom - top) * wy).astype(np.float32)


def ref_cvtcolor_gpu(rgb):
    """What the reference's benchmarks/halide/cvtcolorgpu_tiramisu.cpp:26-57 computes: planar RGB
    uint8 [3][M][N] to gray, (r*4899 + g*9617 + b*1868 + 2^13) >> 14 in uint32, cast to uint8."""
    r, g, b = (rgb[c].astype(np.uint32) for c in range(3))
    v = r * np.uint32(4899) + g * np.uint32(9617) + b * np.uint32(1868)
    return ((v + (np.uint32(1) << np.uint32(13))) >> np.uint32(14)).astype(np.uint8)


def ref_gaussian_gpu(img, kx, ky):
    """benchmarks/halide/gaussiangpu_tiramisu.cpp:44-55: out[c][j][i] = uint8(sum_k ky[k] * gx[c][j+k][i])
    with gx[c][j][i] = sum_k float(img[c][j][i+k]) * kx[k] (inlined), both sums started from 0.f and
    added in order, for i < N-5, j < M-5 of a uint8 image [C][M][N]."""
    f = np.float32
    C, M, N = img.shape
    x = img.astype(np.float32)
    gx = np.zeros((C, M, N - 5), np.float32)
    for k in range(5):
        gx = gx + x[:, :, k:k + N - 5] * f(kx[k])
    acc = np.zeros((C, M - 5, N - 5), np.float32)
    for k in range(5):
        acc = acc + gx[:, k:k + M - 5, :] * f(ky[k])
    return acc.astype(np.uint8)


def ref_heat2d_gpu(grid):
    """benchmarks/halide/heat2dgpu_tiramisu.cpp:37-52: one sweep out = 0.3*c + 0.4*(s + e + n + w) on
    the interior of a square fp32 grid, border cells set to 0 (terms added in the program's order:
    row below, column right, row above, column left)."""
    f = np.float32
    g = grid.astype(np.float32)
    out = np.zeros_like(g)
    s = ((g[2:, 1:-1] + g[1:-1, 2:]) + g[:-2, 1:-1]) + g[1:-1, :-2]
    out[1:-1, 1:-1] = g[1:-1, 1:-1] * f(0.3) + s * f(0.4)
    return out


def _shifted(plane, r, dy, dx):
    """View of the interior (margin r) of `plane` displaced by (dy, dx)."""
    ny, nx = plane.shape
    return plane[r + dy:ny - r + dy, r + dx:nx - r + dx]


def stencil_box9(planes, steps):
    """`steps` sweeps of the weighted 3x3 box of tests/programs/stencil_shapes.cpp (box9) on a
    ping-pong pair of planes (the iterated form of a 3x3 blur such as the reference's
    benchmarks/halide/blurxy_tiramisu.cpp); fp32 operations in the order of the program text:
    c*0.25 + (((n+s)+w)+e)*0.125 + (((nw+ne)+sw)+se)*0.0625.  Both planes are given and returned:
    boundary cells (margin 1) keep the caller's values."""
    p = planes.astype(np.float32).copy()
    f = np.float32
    for t in range(1, steps + 1):
        s, d = p[(t - 1) % 2], p[t % 2]
        g = lambda dy, dx: _shifted(s, 1, dy, dx)
        axis = ((g(-1, 0) + g(1, 0)) + g(0, -1)) + g(0, 1)
        diag = ((g(-1, -1) + g(-1, 1)) + g(1, -1)) + g(1, 1)
        d[1:-1, 1:-1] = (g(0, 0) * f(0.25) + axis * f(0.125)) + diag * f(0.0625)
    return p


def stencil_far2(planes, steps):
    """`steps` sweeps of the radius-2 stencil of tests/programs/stencil_shapes.cpp (far2):
    c*0.5 + (((n2+s2)+w2)+e2)*0.0625 + (ne+sw)*0.125 with a fixed margin of 2 cells."""
    p = planes.astype(np.float32).copy()
    f = np.float32
    for t in range(1, steps + 1):
        s, d = p[(t - 1) % 2], p[t % 2]
        g = lambda dy, dx: _shifted(s, 2, dy, dx)
        far = ((g(-2, 0) + g(2, 0)) + g(0, -2)) + g(0, 2)
        diag = g(-1, 1) + g(1, -1)
        d[2:-2, 2:-2] = (g(0, 0) * f(0.5) + far * f(0.0625)) + diag * f(0.125)
    return p


def stencil_loops(planes, steps, radius, taps):
    """Brute-force pin of the two functions above (tiny planes): `taps` is a list of
    (weight, [(dy, dx), ...]) groups, each group summed left to right, scaled, and the scaled
    groups added left to right."""
    p = planes.astype(np.float32).copy()
    ny, nx = p.shape[1:]
    for t in range(1, steps + 1):
        s, d = p[(t - 1) % 2], p[t % 2]
        for y in range(radius, ny - radius):
            for x in range(radius, nx - radius):
                total = None
                for weight, cells in taps:
                    acc = np.float32(s[y + cells[0][0], x + cells[0][1]])
                    for dy, dx in cells[1:]:
                        acc = np.float32(acc + s[y + dy, x + dx])
                    acc = np.float32(acc * np.float32(weight))
                    total = acc if total is None else np.float32(total + acc)
                d[y, x] = total
    return p


def heat2d_loops(grid, steps):
    """The same sweep as plain Python loops (tiny grids only): the brute-force pin of heat2d()."""
    n = grid.shape[0]
    planes = np.zeros((2, n, n), np.float32)
    planes[0] = grid
    c02 = np.float32(0.2)
    for t in range(1, steps + 1):
        s, d = planes[(t - 1) % 2], planes[t % 2]
        for y in range(1, n - 1):
            for x in range(1, n - 1):
                v = np.float32(s[y, x] + s[y - 1, x])
                v = np.float32(v + s[y + 1, x])
                v = np.float32(v + s[y, x - 1])
                v = np.float32(v + s[y, x + 1])
                d[y, x] = np.float32(v * c02)
    return planes


def conv2d_bias_relu(in_pad, w, bias):
    """out[n,co,y,x] = max(0, bias[co] + sum_{ci,ky,kx} in_pad[n,ci,y+ky,x+kx] * w[co,ci,ky,kx]) on an
    input the caller has already padded (reference: benchmarks/DNN/layers/convolution/direct/cpu/
    conv_layer_generator_tiramisu.cpp:19-21 pads the same way; loop nest of
    benchmarks/auto-scheduler_benchmarks/convolution/convolution_generator.cpp:17-25; ReLU of
    benchmarks/DNN/layers/relu/cpu/relu_layer_generator_tiramisu.cpp:20).  Accumulates in float64 and
    rounds once, so it is the exact value for integer-valued data and the reference point for
    tolerance checks otherwise."""
    N, CI, HP, WP = in_pad.shape
    CO, _, KH, KW = w.shape
    H, W = HP - KH + 1, WP - KW + 1
    acc = np.zeros((N, CO, H, W), np.float64) + bias.astype(np.float64)[None, :, None, None]
    for ky in range(KH):
        for kx in range(KW):
            win = in_pad[:, :, ky:ky + H, kx:kx + W].astype(np.float64)
            acc += np.einsum("nchw,oc->nohw", win, w[:, :, ky, kx].astype(np.float64))
    return np.maximum(acc, 0.0).astype(np.float32)


def conv2d_bias_relu_loops(in_pad, w, bias):
    """Seven nested loops in the program's order, fp32 accumulation (tiny shapes only)."""
    N, CI, HP, WP = in_pad.shape
    CO, _, KH, KW = w.shape
    H, W = HP - KH + 1, WP - KW + 1
    out = np.zeros((N, CO, H, W), np.float32)
    for n in range(N):
        for co in range(CO):
            for y in range(H):
                for x in range(W):
                    a = np.float32(bias[co])
                    for ci in range(CI):
                        for ky in range(KH):
                            for kx in range(KW):
                                a = np.float32(a + np.float32(in_pad[n, ci, y + ky, x + kx] * w[co, ci, ky, kx]))
                    out[n, co, y, x] = a if a > 0 else np.float32(0)
    return out


def lstm(weights, biases, x, real=np.float32):
    """Stacked LSTM forward pass in fp32 (or in `real`) with numpy matrix products.
    weights[L, 2, 4H, H] (slot 0 = input weights W, slot 1 = recurrent weights R), biases[L, 4H],
    x[S, B, H]; gate order i, f, z, o in the 4H rows; zero initial h and c; returns y[S, B, H], the
    hidden state of the last layer.  Restates benchmarks/DNN/blocks/LSTM/cpu/generator.cpp:31-60 with
    the library variant's packing (gpu_lib/generator.cpp:69-70, :78-79, :84-87)."""
    L, _, H4, H = weights.shape
    S, B, _ = x.shape
    f32 = real
    h_prev = np.zeros((L, B, H), f32)
    c_prev = np.zeros((L, B, H), f32)
    y = np.zeros((S, B, H), f32)
    one = f32(1)
    for m in range(S):
        below = x[m].astype(f32)
        for l in range(L):
            g = biases[l][None, :] + below @ weights[l, 0].T + h_prev[l] @ weights[l, 1].T
            g = g.astype(f32)
            i = one / (one + np.exp(-g[:, 0:H]))
            f = one / (one + np.exp(-g[:, H:2 * H]))
            z = np.tanh(g[:, 2 * H:3 * H])
            o = one / (one + np.exp(-g[:, 3 * H:4 * H]))
            c = (i * z + f * c_prev[l]).astype(f32)
            h = (np.tanh(c) * o).astype(f32)
            c_prev[l], h_prev[l] = c, h
            below = h
        y[m] = below
    return y



def ref_convolution_gpu(img, kernel):
    """benchmarks/halide/convolutiongpu_tiramisu.cpp:47-56, :69, :95-117: 3x3 filter of a planar uint8
    image [3][M][N] staged through an 18x18 LDS tile (the staging does not change the values):
    out[c][j][i] = uint8(0.f + sum over _j, then _i, of float(img[c][j+_j][i+_i]) * kernel[_j][_i]),
    for i < N-2, j < M-2 (kernel(_i,_j) reads kernel_gpu[_j][_i], a plain copy of the host kernel)."""
    f = np.float32
    C, M, N = img.shape
    x = img.astype(np.float32)
    acc = np.zeros((C, M - 2, N - 2), np.float32)
    for _j in range(3):
        for _i in range(3):
            acc = acc + x[:, _j:_j + M - 2, _i:_i + N - 2] * f(kernel[_j][_i])
    return acc.astype(np.uint8)


def ref_fusion_gpu(img):
    """benchmarks/halide/fusiongpu_tiramisu.cpp:36-41: f = 255 - in, g = 2*in, h = f + g, k = f - g on
    uint8, every value stored as uint8 (arithmetic modulo 256)."""
    x = img.astype(np.int32)
    f = (255 - x) % 256
    g = (2 * x) % 256
    return f.astype(np.uint8), g.astype(np.uint8), ((f + g) % 256).astype(np.uint8), ((f - g) % 256).astype(np.uint8)


def ref_rgbyuv420_gpu(rgb):
    """benchmarks/halide/rgbyuv420gpu_tiramisu.cpp:37-50: planar RGB uint8 [3][M][N] (M, N even) to a
    full-resolution y and half-resolution u, v taken at even pixels.  int32 arithmetic as the
    generated C computes it: % is the remainder of truncating division (sign of the dividend),
    and the conversion to uint8 is modulo 256."""
    r, g, b = (rgb[c].astype(np.int32) for c in range(3))
    y = np.fmod(66 * r + 129 * g + 25 * b + 128, 256) + 16
    r2, g2, b2 = r[::2, ::2], g[::2, ::2], b[::2, ::2]
    u = np.fmod(-38 * r2 - 74 * g2 + 112 * b2 + 128, 256) + 128
    v = np.fmod(112 * r2 - 94 * g2 - 18 * b2 + 128, 256) + 128
    return tuple((a % 256).astype(np.uint8) for a in (y, u, v))


def ref_warp_affine_gpu(img):
    """benchmarks/halide/warp_affinegpu_tiramisu.cpp:44-80, literally: with every coefficient 0.1f,
    o_r = 0.1*i + 0.1*j + 0.1 (the program's o_c has the same value), r = c = o_r - floor(o_r), both
    coordinates are floor(o_r) (:63-64), clamped to [0, N] for rows and [0, M] for columns, and
    out[j][i] = mix(mix(A00, A01, r), mix(A10, A11, r), c) with mix(x, y, a) = x*(1-a) + y*a and
    in(r, c) read at img[c][r].  fp32 throughout; img is uint8 [M][N]."""
    f = np.float32
    M, N = img.shape
    j, i = np.meshgrid(np.arange(M, dtype=np.float32), np.arange(N, dtype=np.float32), indexing="ij")
    o = (f(0.1) * i + f(0.1) * j).astype(np.float32) + f(0.1)
    fl = np.floor(o).astype(np.float32)
    frac = (o - fl).astype(np.float32)
    coord = fl.astype(np.int32)
    rows = lambda v: np.clip(v, 0, N)
    cols = lambda v: np.clip(v, 0, M)
    at = lambda rr, cc: img[cc, rr].astype(np.float32)
    a00, a01 = at(rows(coord), cols(coord)), at(rows(coord), cols(coord + 1))
    a10, a11 = at(rows(coord + 1), cols(coord)), at(rows(coord + 1), cols(coord + 1))
    one = f(1.0)
    mix = lambda x, y, a: (x * (one - a)).astype(np.float32) + (y * a).astype(np.float32)
    return mix(mix(a00, a01, frac), mix(a10, a11, frac), frac).astype(np.float32)


def ref_edge_gpu(img):
    """benchmarks/halide/edgegpu_tiramisu.cpp:25-31, :47-49, in place on a planar uint8 image [3][M][N]:
    R = (ring of the 8 neighbours of the 3x3 window at (i, j)) / 8 for i < N-2, j < M-2 -- in uint8
    arithmetic: the operands are uint8 expressions, so the sum wraps modulo 256 before the division,
    as in the Halide program the reference checks this benchmark against (edgegpu_ref.cpp:10-18;
    tests/test_56.cpp + wrapper_test_56.cpp pin the same rule for a uint8 blur) -- then Img(i, j) = (R(i+1,j+1) - R(i+2,j)) + (R(i+2,j+1) - R(i+1,j)) stored as uint8.  R is
    defined for indices below N-2 / M-2 only, so the result is fixed for i < N-4, j < M-4; returns
    that region, [3][M-4][N-4]."""
    x = img.astype(np.int32)
    C, M, N = img.shape
    s = lambda dj, di: x[:, dj:dj + M - 2, di:di + N - 2]          # Img(i+di, j+dj)
    R = ((s(0, 0) + s(1, 0) + s(2, 0) + s(0, 1) + s(2, 1) + s(0, 2) + s(1, 2) + s(2, 2)) % 256) // 8
    t = lambda dj, di: R[:, dj:dj + M - 4, di:di + N - 4]          # R(i+di, j+dj)
    out = (t(1, 1) - t(0, 2)) + (t(1, 2) - t(0, 1))
    return (out % 256).astype(np.uint8)


def lstm_gpu_packing(weights, biases, x):
    """The stacked LSTM of lstm() on buffers packed the way the reference's GPU generators pack them
    (benchmarks/DNN/blocks/LSTM/gpu/reference_generator.cpp:100-111 and gpu/generator.cpp:123-126, :256-257):
    weight slot 0 holds the recurrent matrices R and slot 1 the input matrices W, and the 4H rows
    are ordered i, z, o, f.  Restated by re-packing into lstm()'s layout (slot 0 = W, slot 1 = R;
    rows i, f, z, o).  Pinned by the reference's own naive program, compiled unchanged
    (tests/test_reference_generators.py: test_naive_lstm_program_pins_the_packing)."""
    H = weights.shape[3]
    blocks = [0, 3, 1, 2]                      # lstm()'s i, f, z, o taken from i, z, o, f
    rows = np.concatenate([np.arange(b * H, (b + 1) * H) for b in blocks])
    repacked = np.ascontiguousarray(weights[:, ::-1][:, :, rows, :])
    return lstm(repacked, np.ascontiguousarray(biases[:, rows]), x)
