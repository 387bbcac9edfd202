/*
 * TEST INFRASTRUCTURE ONLY - sequential CPU restatement of the reference's
 * kernels, one plain loop nest per kernel, for REAL = float or double
 * (included twice by seq_oracle.c).  Nothing in the product links or loads it.
 *
 * Each function follows the per-element arithmetic of the cited reference
 * kernel literally: same floor (-1e9), same strict comparisons, same order of
 * summation, multiply-then-add without contraction (build with
 * -ffp-contract=off).  Dense operands: a (B,M,K), b (B,K,N); the reference
 * names them a_size = M, in_size = K, b_size = N.
 */

#define A3(p, d1, d2, i, j, k) (p)[((size_t)(i) * (d1) + (j)) * (d2) + (k)]

/* matmul_cuda_forward_kernel, matmul_cuda_kernel.cu:13-45 */
void FN(logbmm_fwd)(const REAL* a, const REAL* b, REAL* out, REAL* maxes, int B, int M, int K, int N) {
  for (int n = 0; n < B; ++n)
    for (int row = 0; row < M; ++row)
      for (int col = 0; col < N; ++col) {
        REAL val = 0, m = (REAL)-1e9;
        for (int i = 0; i < K; ++i) {
          REAL v = A3(a, M, K, n, row, i) + A3(b, K, N, n, i, col);
          if (v > m) m = v;
        }
        for (int i = 0; i < K; ++i) {
          REAL v = A3(a, M, K, n, row, i) + A3(b, K, N, n, i, col);
          val += EXP(v - m);
        }
        A3(out, M, N, n, row, col) = LOG(val) + m;
        if (maxes) A3(maxes, M, N, n, row, col) = m;
      }
}

/* max_cuda_forward_kernel :47-75 (prod = 0) and prod_max_cuda_forward_kernel :124-152 (prod = 1) */
void FN(maxbmm_fwd)(const REAL* a, const REAL* b, REAL* out, int32_t* idx, int B, int M, int K, int N, int prod) {
  for (int n = 0; n < B; ++n)
    for (int row = 0; row < M; ++row)
      for (int col = 0; col < N; ++col) {
        REAL m = (REAL)-1e9;
        int ind = -1;
        for (int i = 0; i < K; ++i) {
          REAL x = A3(a, M, K, n, row, i), y = A3(b, K, N, n, i, col);
          REAL v = prod ? x * y : x + y;
          if (v > m) { m = v; ind = i; }
        }
        A3(out, M, N, n, row, col) = m;
        A3(idx, M, N, n, row, col) = ind;
      }
}

/* sample_cuda_forward_kernel :77-121; `rnd` is the (B,M,N) uniform tensor the
 * reference draws with torch::rand (:517); idx keeps its zero fill when the
 * scan never brackets rnd. */
void FN(samplebmm_fwd)(const REAL* a, const REAL* b, const REAL* rnd, REAL* out, int32_t* idx, int B, int M, int K, int N) {
  FN(logbmm_fwd)(a, b, out, NULL, B, M, K, N);
  for (int n = 0; n < B; ++n)
    for (int row = 0; row < M; ++row)
      for (int col = 0; col < N; ++col) {
        REAL total = 0, r = A3(rnd, M, N, n, row, col);
        A3(idx, M, N, n, row, col) = 0;
        for (int i = 0; i < K; ++i) {
          REAL v = A3(a, M, K, n, row, i) + A3(b, K, N, n, i, col) - A3(out, M, N, n, row, col);
          if (total < r && total + EXP(v) > r) { A3(idx, M, N, n, row, col) = i; break; }
          total += EXP(v);
        }
      }
}

/* matmul_cuda_backward_kernel_A :159-184 and _B :190-217 (the latter is what
 * the reference's transposed second call computes, genmul.py:38-41). */
void FN(logbmm_bwd)(const REAL* a, const REAL* b, const REAL* part, const REAL* maxes, const REAL* g,
                    REAL* grad_a, REAL* grad_b, int B, int M, int K, int N) {
  for (int n = 0; n < B; ++n)
    for (int row = 0; row < M; ++row)
      for (int col = 0; col < K; ++col) {
        REAL val = 0;
        for (int k = 0; k < N; ++k) {
          REAL m = A3(maxes, M, N, n, row, k);
          val += (EXP(A3(a, M, K, n, row, col) + A3(b, K, N, n, col, k) - m) /
                  EXP(A3(part, M, N, n, row, k) - m)) * A3(g, M, N, n, row, k);
        }
        A3(grad_a, M, K, n, row, col) = val;
      }
  for (int n = 0; n < B; ++n)
    for (int row = 0; row < K; ++row)
      for (int col = 0; col < N; ++col) {
        REAL val = 0;
        for (int k = 0; k < M; ++k) {
          REAL m = A3(maxes, M, N, n, k, col);
          REAL v = EXP(A3(a, M, K, n, k, row) + A3(b, K, N, n, row, col) - m);
          val += (v / EXP(A3(part, M, N, n, k, col) - m)) * A3(g, M, N, n, k, col);
        }
        A3(grad_b, K, N, n, row, col) = val;
      }
}

/* matmul_cuda_backbackward_kernel_A :220-258, _B :261-303, _C :305-331 -
 * the literal quartic loops; u = grad_output_a (cotangent of grad_a). */
void FN(logbmm_bwdbwd)(const REAL* a, const REAL* b, const REAL* part, const REAL* maxes, const REAL* g,
                       const REAL* u, REAL* grad_a, REAL* grad_b, REAL* grad_g, int B, int M, int K, int N) {
  for (int n = 0; n < B; ++n)
    for (int row = 0; row < M; ++row)
      for (int col = 0; col < K; ++col) {
        REAL val = 0;
        for (int k = 0; k < N; ++k) {
          REAL m = A3(maxes, M, N, n, row, k);
          REAL z = EXP(A3(part, M, N, n, row, k) - m);
          REAL s = EXP(A3(a, M, K, n, row, col) + A3(b, K, N, n, col, k) - m) / z;
          REAL inner = 0;
          for (int k2 = 0; k2 < K; ++k2) {
            REAL s2 = EXP(A3(a, M, K, n, row, k2) + A3(b, K, N, n, k2, k) - m) / z;
            REAL v = (col == k2) ? s - s * s2 : -s * s2;
            inner += v * A3(u, M, K, n, row, k2);
          }
          val += inner * A3(g, M, N, n, row, k);
        }
        A3(grad_a, M, K, n, row, col) = val;
      }
  for (int n = 0; n < B; ++n)
    for (int row = 0; row < K; ++row)
      for (int col = 0; col < N; ++col) {
        REAL val = 0;
        for (int k = 0; k < M; ++k) {
          REAL m = A3(maxes, M, N, n, k, col);
          REAL z = EXP(A3(part, M, N, n, k, col) - m);
          REAL s = EXP(A3(a, M, K, n, k, row) + A3(b, K, N, n, row, col) - m) / z;
          REAL inner = 0;
          for (int k2 = 0; k2 < K; ++k2) {
            REAL s2 = EXP(A3(a, M, K, n, k, k2) + A3(b, K, N, n, k2, col) - m) / z;
            REAL v = (row == k2) ? s - s * s2 : -s * s2;
            inner += v * A3(u, M, K, n, k, k2);
          }
          val += inner * A3(g, M, N, n, k, col);
        }
        A3(grad_b, K, N, n, row, col) = val;
      }
  for (int n = 0; n < B; ++n)
    for (int row = 0; row < M; ++row)
      for (int col = 0; col < N; ++col) {
        REAL val = 0, m = A3(maxes, M, N, n, row, col);
        for (int k = 0; k < K; ++k)
          val += (EXP(A3(a, M, K, n, row, k) + A3(b, K, N, n, k, col) - m) /
                  EXP(A3(part, M, N, n, row, col) - m)) * A3(u, M, K, n, row, k);
        A3(grad_g, M, N, n, row, col) = val;
      }
}

/* max_cuda_backward_kernel_A/_B :336-395 (prod = 0), prod_max_cuda_backward_kernel_A/_B
 * :399-456 (prod = 1).  The reference receives idx as a float tensor and
 * compares `col == part`; an int32 compare is the same test. */
void FN(argmax_bwd)(const REAL* a, const REAL* b, const int32_t* idx, const REAL* g,
                    REAL* grad_a, REAL* grad_b, int B, int M, int K, int N, int prod) {
  for (int n = 0; n < B; ++n)
    for (int row = 0; row < M; ++row)
      for (int col = 0; col < K; ++col) {
        REAL val = 0;
        for (int k = 0; k < N; ++k)
          if (col == A3(idx, M, N, n, row, k)) {
            if (prod) { REAL t = A3(b, K, N, n, col, k) * A3(g, M, N, n, row, k); val += t; }
            else val += A3(g, M, N, n, row, k);
          }
        A3(grad_a, M, K, n, row, col) = val;
      }
  for (int n = 0; n < B; ++n)
    for (int row = 0; row < K; ++row)
      for (int col = 0; col < N; ++col) {
        REAL val = 0;
        for (int k = 0; k < M; ++k)
          if (row == A3(idx, M, N, n, k, col)) {
            if (prod) { REAL t = A3(a, M, K, n, k, row) * A3(g, M, N, n, k, col); val += t; }
            else val += A3(g, M, N, n, k, col);
          }
        A3(grad_b, K, N, n, row, col) = val;
      }
}

/* ------------------------------------------------------------------ banded
 * banded_cuda_forward_kernel_mul, banded_cuda_kernel.cu:13-100.  out / idx /
 * maxes are zero-filled first, as the host code does (:373-387). mode 0 log,
 * 1 max, 3 (+,*). */
void FN(band_fwd)(const REAL* a, int a_lu, int a_lb, const REAL* b, int b_lu, int b_lb,
                  REAL* out, int32_t* indices, REAL* maxes, int B, int n, int mode) {
  const int result_lu = a_lu + b_lb, result_lb = a_lb + b_lu;
  const int self_width = a_lu + a_lb + 1, b_width = b_lu + b_lb + 1;
  const int W = result_lu + result_lb + 1;
  for (size_t e = 0; e < (size_t)B * n * W; ++e) { out[e] = 0; if (indices) indices[e] = 0; if (maxes) maxes[e] = 0; }
  for (int batch = 0; batch < B; ++batch)
    for (int i = 0; i < n; ++i)
      for (int j = 0; j < W; ++j) {
        const int o = i + (j - result_lu);
        if (o < 0 || o >= n) continue;
        if (mode == 1) {
          REAL m = (REAL)-1e9; int ind = -1;
          for (int k = 0; k < self_width; ++k) {
            int pos = i + (k - a_lu), k2 = (pos - o) + b_lu;
            if (k2 < 0 || k2 >= b_width) continue;
            if (pos < 0 || pos >= n) continue;
            REAL v = A3(a, n, self_width, batch, i, k) + A3(b, n, b_width, batch, o, k2);
            if (v > m) { m = v; ind = k; }
          }
          A3(out, n, W, batch, i, j) = m;
          A3(indices, n, W, batch, i, j) = ind;
        } else if (mode == 3) {
          REAL val = 0;
          for (int k = 0; k < self_width; ++k) {
            int pos = i + (k - a_lu), k2 = (pos - o) + b_lu;
            if (k2 < 0 || k2 >= b_width) continue;
            if (pos < 0 || pos >= n) continue;
            REAL t = A3(a, n, self_width, batch, i, k) * A3(b, n, b_width, batch, o, k2);
            val += t;
          }
          A3(out, n, W, batch, i, j) = val;
        } else {
          REAL val = 0, m = (REAL)-1e9;
          for (int k = 0; k < self_width; ++k) {
            int pos = i + (k - a_lu);
            if (pos < 0 || pos >= n) continue;
            int k2 = (pos - o) + b_lu;
            if (k2 < 0 || k2 >= b_width) continue;
            REAL v = A3(a, n, self_width, batch, i, k) + A3(b, n, b_width, batch, o, k2);
            if (v > m) m = v;
          }
          for (int k = 0; k < self_width; ++k) {
            int pos = i + (k - a_lu);
            if (pos < 0 || pos >= n) continue;
            int k2 = (pos - o) + b_lu;
            if (k2 < 0 || k2 >= b_width) continue;
            val += EXP(A3(a, n, self_width, batch, i, k) + A3(b, n, b_width, batch, o, k2) - m);
          }
          A3(out, n, W, batch, i, j) = LOG(val) + m;
          if (maxes) A3(maxes, n, W, batch, i, j) = m;
        }
      }
}

/* Banded sample product.  The reference's band kernel has modes 0, 1 and 3 only
 * (banded_cuda_kernel.cu:42, 65, 76), so there is no reference function to follow line
 * by line: this is its dense sampling rule (sample_cuda_forward_kernel,
 * matmul_cuda_kernel.cu:107-118: walk the terms in ascending order, take the first one
 * with total < r && total + exp(v - out) > r) applied to the term list of a band cell
 * (banded_cuda_kernel.cu:32-51, ascending k with the two range tests).  out = banded
 * log-sum-exp (mode 0 above); indices[i][j] = the chosen k (index into a's band, as
 * mode 1 stores it); a cell whose walk never brackets r keeps the first term of its
 * list, cells outside the matrix keep the zero fill.  `rnd` is (B, n, W). */
void FN(band_sample_fwd)(const REAL* a, int a_lu, int a_lb, const REAL* b, int b_lu, int b_lb,
                         const REAL* rnd, REAL* out, int32_t* indices, int B, int n) {
  const int result_lu = a_lu + b_lb, result_lb = a_lb + b_lu;
  const int self_width = a_lu + a_lb + 1, b_width = b_lu + b_lb + 1;
  const int W = result_lu + result_lb + 1;
  FN(band_fwd)(a, a_lu, a_lb, b, b_lu, b_lb, out, indices, NULL, B, n, 0);
  for (int batch = 0; batch < B; ++batch)
    for (int i = 0; i < n; ++i)
      for (int j = 0; j < W; ++j) {
        const int o = i + (j - result_lu);
        if (o < 0 || o >= n) continue;
        REAL total = 0, r = A3(rnd, n, W, batch, i, j);
        int first = -1, hit = -1;
        for (int k = 0; k < self_width; ++k) {
          int pos = i + (k - a_lu), k2 = (pos - o) + b_lu;
          if (k2 < 0 || k2 >= b_width) continue;
          if (pos < 0 || pos >= n) continue;
          if (first < 0) first = k;
          REAL v = A3(a, n, self_width, batch, i, k) + A3(b, n, b_width, batch, o, k2) - A3(out, n, W, batch, i, j);
          if (total < r && total + EXP(v) > r) { hit = k; break; }
          total += EXP(v);
        }
        A3(indices, n, W, batch, i, j) = hit >= 0 ? hit : first;
      }
}

/* banded_cuda_backward_kernel_mul :104-152: gradient with respect to the FIRST
 * operand; `part` is out (mode 0) or the arg-max as REAL (mode 1); grad_a is
 * zero-filled first (:436). */
void FN(band_bwd_first)(const REAL* a, int a_lu, int a_lb, const REAL* b, int b_lu, int b_lb,
                        const REAL* part, const REAL* g, REAL* grad_a, int B, int n, int mode) {
  const int result_lu = a_lu + b_lb, result_lb = a_lb + b_lu;
  const int aw = a_lu + a_lb + 1, bw = b_lu + b_lb + 1;
  const int gradout_width = result_lu + result_lb + 1;
  for (size_t e = 0; e < (size_t)B * n * aw; ++e) grad_a[e] = 0;
  for (int batch = 0; batch < B; ++batch)
    for (int i = 0; i < n; ++i)
      for (int j = 0; j < aw; ++j) {
        const int o = i + (j - a_lu);
        if (!(o >= 0 && o < n)) continue;
        REAL val = 0;
        for (int k = 0; k < gradout_width; ++k) {
          const int pos = i + (k - result_lu);
          const int k2 = (o - pos) + b_lu;
          if (k2 < 0 || k2 >= bw) continue;
          if (pos < 0 || pos >= n) continue;
          if (mode == 3) {
            REAL t = A3(b, n, bw, batch, pos, k2) * A3(g, n, gradout_width, batch, i, k);
            val += t;
          } else if (mode == 1) {
            REAL v = (j == A3(part, n, gradout_width, batch, i, k)) ? 1 : 0;
            REAL t = v * A3(g, n, gradout_width, batch, i, k);
            val += t;
          } else {
            REAL v = A3(a, n, aw, batch, i, j) + A3(b, n, bw, batch, pos, k2) - A3(part, n, gradout_width, batch, i, k);
            REAL t = EXP(v) * A3(g, n, gradout_width, batch, i, k);
            val += t;
          }
        }
        A3(grad_a, n, aw, batch, i, j) = val;
      }
}

/* banded_cuda_backbackward_kernel_A :154-223, _B :225-301, _C :304-350
 * (literal; u = grad_output_a).  Outputs are zero-filled first (:466,:492,:516). */
void FN(band_bwdbwd)(const REAL* a, int a_lu, int a_lb, const REAL* b, int b_lu, int b_lb,
                     const REAL* g, const REAL* part, const REAL* maxes, const REAL* u,
                     REAL* grad_a, REAL* grad_b, REAL* grad_grad, int B, int n) {
  const int result_lu = a_lu + b_lb, result_lb = a_lb + b_lu;
  const int aw = a_lu + a_lb + 1, b_width = b_lu + b_lb + 1;
  const int gw = result_lu + result_lb + 1;
  for (size_t e = 0; e < (size_t)B * n * aw; ++e) grad_a[e] = 0;
  for (size_t e = 0; e < (size_t)B * n * b_width; ++e) grad_b[e] = 0;
  for (size_t e = 0; e < (size_t)B * n * gw; ++e) grad_grad[e] = 0;
  for (int batch = 0; batch < B; ++batch)
    for (int i = 0; i < n; ++i)
      for (int j = 0; j < aw; ++j) {
        const int o = i + (j - a_lu);
        if (!(o >= 0 && o < n)) continue;
        REAL a_val = A3(a, n, aw, batch, i, j), val = 0;
        for (int k = 0; k < gw; ++k) {
          const int pos = i + (k - result_lu);
          const int k2 = (o - pos) + b_lu;
          if (k2 < 0 || k2 >= b_width) continue;
          if (pos < 0 || pos >= n) continue;
          REAL b_val = A3(b, n, b_width, batch, pos, k2);
          REAL mx = A3(maxes, n, gw, batch, i, k);
          REAL z = EXP(A3(part, n, gw, batch, i, k) - mx);
          REAL s = EXP(a_val + b_val - mx) / z, inner = 0;
          const int o2 = i + (k - result_lu);
          for (int m = 0; m < aw; ++m) {
            const int pos_in = i + (m - a_lu);
            int m2 = (pos_in - o2) + b_lu;
            if (m2 < 0 || m2 >= b_width) continue;
            if (pos_in < 0 || pos_in >= n) continue;
            REAL s2 = EXP(A3(a, n, aw, batch, i, m) + A3(b, n, b_width, batch, o2, m2) - mx) / z;
            REAL v = (j == m) ? s - s * s2 : -s * s2;
            inner += v * A3(u, n, aw, batch, i, m);
          }
          val += inner * A3(g, n, gw, batch, i, k);
        }
        A3(grad_a, n, aw, batch, i, j) = val;
      }
  for (int batch = 0; batch < B; ++batch)
    for (int pos = 0; pos < n; ++pos)
      for (int k2 = 0; k2 < b_width; ++k2) {
        const int check = pos + (k2 - b_lu);
        if (!(check < n && check >= 0)) continue;
        REAL b_val = A3(b, n, b_width, batch, pos, k2), val = 0;
        for (int k = 0; k < gw; ++k) {
          const int i = pos - (k - result_lu);
          const int j = k2 + pos - b_lu - (i - a_lu);
          if (j < 0 || j >= aw) continue;
          if (i < 0 || i >= n) continue;
          REAL a_val = A3(a, n, aw, batch, i, j);
          REAL mx = A3(maxes, n, gw, batch, i, k);
          REAL z = EXP(A3(part, n, gw, batch, i, k) - mx);
          REAL s = EXP(a_val + b_val - mx) / z, inner = 0;
          const int o2 = i + (k - result_lu);
          for (int m = 0; m < aw; ++m) {
            const int pos_in = i + (m - a_lu);
            int m2 = (pos_in - o2) + b_lu;
            if (m2 < 0 || m2 >= b_width) continue;
            if (pos_in < 0 || pos_in >= n) continue;
            REAL s2 = EXP(A3(a, n, aw, batch, i, m) + A3(b, n, b_width, batch, o2, m2) - mx) / z;
            REAL v = (j == m) ? s - s * s2 : -s * s2;
            inner += v * A3(u, n, aw, batch, i, m);
          }
          val += inner * A3(g, n, gw, batch, i, k);
        }
        A3(grad_b, n, b_width, batch, pos, k2) = val;
      }
  for (int batch = 0; batch < B; ++batch)
    for (int i = 0; i < n; ++i)
      for (int j = 0; j < gw; ++j) {
        const int o = i + (j - result_lu);
        if (!(o >= 0 && o < n)) continue;
        REAL val = 0, mx = A3(maxes, n, gw, batch, i, j);
        for (int k = 0; k < aw; ++k) {
          int pos = i + (k - a_lu), k2 = (pos - o) + b_lu;
          if (k2 < 0 || k2 >= b_width) continue;
          if (pos < 0 || pos >= n) continue;
          val += (EXP(A3(a, n, aw, batch, i, k) + A3(b, n, b_width, batch, o, k2) - mx) /
                  EXP(A3(part, n, gw, batch, i, j) - mx)) * A3(u, n, aw, batch, i, k);
        }
        A3(grad_grad, n, gw, batch, i, j) = val;
      }
}

#undef A3
