// linalg.hip — cholesky, triangular_solve, qr, eigh / eigvalsh, svd, eig / eigvals
// (backend_intf.ml:625-720; packages/nx/lib/backend_c/nx_c_tri.c, nx_c_qr.c,
// nx_c_eigh.c, nx_c_svd.c, nx_c_eig.c; bindings nx_backend.ml:550-707).
//
// What is kept from the reference: shapes and dtypes of every result (S and the
// Hermitian eigenvalues are float64, the general eigenpairs complex128, factors
// carry the input dtype), the batch convention (the last two dims are the
// matrix), cholesky reading the lower triangle and returning L or U = L^H with
// the other triangle zero (nx_c_tri.c:11-16, 222-262), the substitution order and
// the exact-zero-pivot rule of triangular_solve (nx_c_tri.c:88-118), the LAPACK
// reflector convention of qr (real beta = -sign(re alpha) |x|, A = Q R with
// Q = H_0 H_1 ..., nx_c_qr.c:24-31), eigh reading the lower triangle and
// returning ascending eigenvalues (nx_c_eigh.c:14-21), descending singular
// values, unit-norm eigenvectors of eig (nx_c_eig.c:56-62), and the three
// numeric failures with the reference's status strings (nx_c_linalg.h:29-36).
// Arithmetic is double (or complex double) for every storage dtype; the
// reference computes f32 storage in f32, so results here are at least as close
// to the exact factors. Eigenvectors and singular vectors are determined up to a
// unit phase per vector, which is not fixed by either implementation.
//
// How it runs: correctness first, one workgroup per matrix of the batch, the
// matrix in a contiguous double-precision workspace (the strided, any-dtype
// operands are brought in and results sent out by nxh_cast).
//   cholesky      left-looking columns, one row per lane
//   tri. solve    right-looking substitution, all right-hand sides in parallel
//   qr            Householder columns, one wave per trailing column
//   eigh          two-sided Jacobi with a round-robin ordering: n/2 disjoint
//                 rotations per round, applied as a column phase and a row phase
//   svd           one-sided Jacobi on the columns (round-robin, one wave per pair),
//                 then Householder QR of the orthogonalised columns for U
//   eig           complex Hessenberg reduction, explicit single-shift QR with
//                 deflation (the scheme nx_c_eig.c:43-55 names), back-substitution

#include "nxh_common.hpp"

namespace {

constexpr int LA_THREADS = 256;
constexpr int LA_MAX_N = 4096;  // rotation tables of the Jacobi kernels live in LDS
enum { LA_OK = 0, LA_NOT_PD = 1, LA_SINGULAR = 2, LA_NO_CONVERGE = 3 };

const char *const LA_MESSAGES[] = {"", "matrix is not positive definite", "triangular matrix is singular",
                                   "eigenvalue iteration did not converge"};

// ── scalars: double and complex double behind one interface ─────────────────
template <class T>
struct Sc;
template <>
struct Sc<double> {
  __device__ __forceinline__ static double conj(double x) { return x; }
  __device__ __forceinline__ static double re(double x) { return x; }
  __device__ __forceinline__ static double im(double) { return 0.0; }
  __device__ __forceinline__ static double abs2(double x) { return x * x; }
  __device__ __forceinline__ static double make(double r, double) { return r; }
  __device__ __forceinline__ static double scale(double x, double r) { return x * r; }
};
template <>
struct Sc<c64> {
  __device__ __forceinline__ static c64 conj(c64 x) { return {x.re, -x.im}; }
  __device__ __forceinline__ static double re(c64 x) { return x.re; }
  __device__ __forceinline__ static double im(c64 x) { return x.im; }
  __device__ __forceinline__ static double abs2(c64 x) { return x.re * x.re + x.im * x.im; }
  __device__ __forceinline__ static c64 make(double r, double i) { return {r, i}; }
  __device__ __forceinline__ static c64 scale(c64 x, double r) { return {x.re * r, x.im * r}; }
};

__device__ __forceinline__ double wave_sum(double v) {
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}
__device__ __forceinline__ c64 wave_sum(c64 v) { return {wave_sum(v.re), wave_sum(v.im)}; }

// Sum over the workgroup; every lane gets it. `scratch` holds one T per wave.
template <class T>
__device__ T block_sum(T v, T *scratch) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
  __syncthreads();
  T total = scratch[0];
  for (int w = 1; w < (int)(blockDim.x >> 6); w++) total = total + scratch[w];
  return total;
}

__device__ __forceinline__ void raise(int *status, int code) { atomicMax(status, code); }

// ── cholesky ────────────────────────────────────────────────────────────────
// Row-major n x n per block. Column j of L from the lower triangle of A and the
// finished columns to its left; a pivot that is not > 0 (NaN included) stops the
// matrix (nx_c_tri.c:15-16).
template <class T>
__global__ __launch_bounds__(LA_THREADS) void cholesky_kernel(T *all, int n, int upper, int *status) {
  using S = Sc<T>;
  T *A = all + (size_t)blockIdx.x * n * n;
  __shared__ int failed;
  if (threadIdx.x == 0) failed = 0;
  for (int j = 0; j < n; j++) {
    for (int i = j + threadIdx.x; i < n; i += blockDim.x) {
      T s = A[(size_t)i * n + j];
      const T *ri = A + (size_t)i * n, *rj = A + (size_t)j * n;
      for (int k = 0; k < j; k++) s = s - ri[k] * S::conj(rj[k]);
      A[(size_t)i * n + j] = s;
    }
    __syncthreads();
    const double d = S::re(A[(size_t)j * n + j]);
    if (threadIdx.x == 0 && !(d > 0.0)) failed = 1;
    __syncthreads();
    if (failed) {
      if (threadIdx.x == 0) raise(status, LA_NOT_PD);
      return;
    }
    const double l = sqrt(d);
    for (int i = j + threadIdx.x; i < n; i += blockDim.x)
      A[(size_t)i * n + j] = i == j ? S::make(l, 0.0) : S::scale(A[(size_t)i * n + j], 1.0 / l);
    __syncthreads();
  }
  // the other triangle: zero for L; for U the conjugate transpose moves there first
  for (int64_t e = threadIdx.x; e < (int64_t)n * n; e += blockDim.x) {
    const int i = (int)(e / n), k = (int)(e % n);
    if (i <= k) continue;
    if (upper) {
      A[(size_t)k * n + i] = S::conj(A[e]);
      A[e] = S::make(0.0, 0.0);
    } else {
      A[(size_t)k * n + i] = S::make(0.0, 0.0);
    }
  }
}

// ── triangular solve ────────────────────────────────────────────────────────
// X (n x nrhs) holds B and is solved in place against op(A), op = conjugate
// transpose when `transpose`. Forward iff upper == transpose (nx_c_tri.c:103-118).
template <class T>
__global__ __launch_bounds__(LA_THREADS) void trsm_kernel(const T *a_all, T *x_all, int n, int nrhs, int upper,
                                                         int transpose, int unit, int *status) {
  using S = Sc<T>;
  const T *A = a_all + (size_t)blockIdx.x * n * n;
  T *X = x_all + (size_t)blockIdx.x * n * nrhs;
  const bool forward = (upper != 0) == (transpose != 0);
  for (int ii = 0; ii < n; ii++) {
    const int i = forward ? ii : n - 1 - ii;
    if (!unit) {
      T diag = A[(size_t)i * n + i];
      if (transpose) diag = S::conj(diag);
      if (diag == S::make(0.0, 0.0)) {  // uniform: every lane reads the same element
        if (threadIdx.x == 0) raise(status, LA_SINGULAR);
        return;
      }
      for (int j = threadIdx.x; j < nrhs; j += blockDim.x) X[(size_t)i * nrhs + j] = X[(size_t)i * nrhs + j] / diag;
      __syncthreads();
    }
    const int rest = n - 1 - ii;  // rows not yet solved
    for (int64_t e = threadIdx.x; e < (int64_t)rest * nrhs; e += blockDim.x) {
      const int rr = (int)(e / nrhs), j = (int)(e % nrhs);
      const int r = forward ? i + 1 + rr : i - 1 - rr;
      const T m = transpose ? S::conj(A[(size_t)i * n + r]) : A[(size_t)r * n + i];
      X[(size_t)r * nrhs + j] = X[(size_t)r * nrhs + j] - m * X[(size_t)i * nrhs + j];
    }
    __syncthreads();
  }
}

// ── Householder QR on column-major storage ──────────────────────────────────
// At[c * m + i] = A[i][c]. On return the upper trapezoid holds R, the reflector
// tails sit below the diagonal, tau[j] beside them (nx_c_qr.c:44-80).
template <class T>
__device__ void householder_factor(T *At, int m, int n, T *tau, T *scratch) {
  using S = Sc<T>;
  const int k = m < n ? m : n;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, waves = blockDim.x >> 6;
  for (int j = 0; j < k; j++) {
    T *col = At + (size_t)j * m;
    double part = 0.0;
    for (int i = j + 1 + threadIdx.x; i < m; i += blockDim.x) part += S::abs2(col[i]);
    const double xnorm2 = block_sum(part, (double *)scratch);
    const T alpha = col[j];
    __syncthreads();
    if (xnorm2 == 0.0) {
      if (threadIdx.x == 0) tau[j] = S::make(0.0, 0.0);
      continue;
    }
    const double alphr = S::re(alpha), anorm = sqrt(S::abs2(alpha) + xnorm2);
    const double beta = alphr >= 0.0 ? -anorm : anorm;
    const T t = S::make((beta - alphr) / beta, -S::im(alpha) / beta);
    const T scal = alpha - S::make(beta, 0.0);
    for (int i = j + 1 + threadIdx.x; i < m; i += blockDim.x) col[i] = col[i] / scal;
    if (threadIdx.x == 0) {
      col[j] = S::make(beta, 0.0);
      tau[j] = t;
    }
    __syncthreads();
    const T tauc = S::conj(t);  // the factorisation applies H_j^H
    for (int c = j + 1 + wave; c < n; c += waves) {
      T *cc = At + (size_t)c * m;
      T w = lane == 0 ? cc[j] : S::make(0.0, 0.0);
      for (int i = j + 1 + lane; i < m; i += 64) w = w + S::conj(col[i]) * cc[i];
      w = tauc * wave_sum(w);
      if (lane == 0) cc[j] = cc[j] - w;
      for (int i = j + 1 + lane; i < m; i += 64) cc[i] = cc[i] - col[i] * w;
    }
    __syncthreads();
  }
}

// Q = H_0 H_1 ... H_{k-1} applied to the first nq columns of the identity, in
// column-major Qt (nq columns of m rows).
template <class T>
__device__ void householder_form_q(const T *At, const T *tau, int m, int k, T *Qt, int nq) {
  using S = Sc<T>;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, waves = blockDim.x >> 6;
  for (int64_t e = threadIdx.x; e < (int64_t)nq * m; e += blockDim.x)
    Qt[e] = (e / m) == (e % m) ? S::make(1.0, 0.0) : S::make(0.0, 0.0);
  __syncthreads();
  for (int j = k - 1; j >= 0; j--) {
    const T *v = At + (size_t)j * m;
    const T t = tau[j];
    if (!(t == S::make(0.0, 0.0))) {
      for (int c = j + wave; c < nq; c += waves) {
        T *qc = Qt + (size_t)c * m;
        T w = lane == 0 ? qc[j] : S::make(0.0, 0.0);
        for (int i = j + 1 + lane; i < m; i += 64) w = w + S::conj(v[i]) * qc[i];
        w = t * wave_sum(w);
        if (lane == 0) qc[j] = qc[j] - w;
        for (int i = j + 1 + lane; i < m; i += 64) qc[i] = qc[i] - v[i] * w;
      }
    }
    __syncthreads();
  }
}

template <class T>
__global__ __launch_bounds__(LA_THREADS) void qr_kernel(T *at_all, T *qt_all, T *tau_all, int m, int n, int nq) {
  using S = Sc<T>;
  __shared__ T scratch[LA_THREADS / 64];
  const int k = m < n ? m : n;
  T *At = at_all + (size_t)blockIdx.x * m * n;
  T *Qt = qt_all + (size_t)blockIdx.x * m * nq;
  T *tau = tau_all + (size_t)blockIdx.x * k;
  householder_factor(At, m, n, tau, scratch);
  householder_form_q(At, tau, m, k, Qt, nq);
  for (int64_t e = threadIdx.x; e < (int64_t)n * m; e += blockDim.x)
    if ((e % m) > (e / m)) At[e] = S::make(0.0, 0.0);  // below the diagonal: R's zeros
}

// ── round-robin pairing ─────────────────────────────────────────────────────
// N even players, N - 1 rounds, pair t of round r. An index >= n is the bye of an
// odd n.
__device__ __forceinline__ void round_robin(int N, int r, int t, int *p, int *q) {
  int a, b;
  if (t == 0) {
    a = N - 1;
    b = r;
  } else {
    a = (r + t) % (N - 1);
    b = (r - t + (N - 1)) % (N - 1);
  }
  *p = a < b ? a : b;
  *q = a < b ? b : a;
}

// The rotation J = [[c, sp], [-conj(sp), c]] on the index pair (p, q) that
// annihilates the (p, q) element g of a Hermitian 2 x 2 block with diagonal
// (app, aqq): J^H [[app, g], [conj(g), aqq]] J is diagonal.
template <class T>
__device__ __forceinline__ void jacobi_rotation(double app, double aqq, T g, double *c, T *sp) {
  using S = Sc<T>;
  const double g2 = S::abs2(g);
  if (!(g2 > 1e-300)) {
    *c = 1.0;
    *sp = S::make(0.0, 0.0);
    return;
  }
  const double ga = sqrt(g2);
  const double zeta = (aqq - app) / (2.0 * ga);
  const double t = (zeta >= 0.0 ? 1.0 : -1.0) / (fabs(zeta) + sqrt(1.0 + zeta * zeta));
  const double cc = 1.0 / sqrt(1.0 + t * t);
  *c = cc;
  *sp = S::scale(g, t * cc / ga);
}

// Ascending order, ties by position (nx_c_eigh.c:21): eigenvalue k goes to its
// rank, its eigenvector column with it.
template <class T>
__device__ void eigh_sort_block(const T *A, const T *V, T *Vs, double *w, int n, int wantv) {
  using S = Sc<T>;
  for (int k = threadIdx.x; k < n; k += blockDim.x) {
    const double wk = S::re(A[(size_t)k * n + k]);
    int rank = 0;
    for (int j = 0; j < n; j++) {
      const double wj = S::re(A[(size_t)j * n + j]);
      rank += (wj < wk) || (wj == wk && j < k);
    }
    w[rank] = wk;
    if (wantv)
      for (int i = 0; i < n; i++) Vs[(size_t)i * n + rank] = V[(size_t)i * n + k];
  }
}

// ── eigh: two-sided Jacobi ──────────────────────────────────────────────────
// A (row-major, overwritten), V (row-major; the eigenvectors when wantv), sorted
// results to w (n doubles) and Vs (row-major, column k = eigenvector of w[k]).
template <class T>
__global__ __launch_bounds__(LA_THREADS) void eigh_kernel(T *a_all, T *v_all, T *vs_all, double *w_all, int n, int wantv,
                                                         int *status) {
  using S = Sc<T>;
  extern __shared__ double lds_raw[];
  const int N = (n + 1) & ~1, P = N / 2;
  double *rc = lds_raw;        // P cosines
  T *rs = (T *)(rc + P);       // P sines with phase
  __shared__ double scratch[LA_THREADS / 64];
  T *A = a_all + (size_t)blockIdx.x * n * n;
  T *V = v_all + (size_t)blockIdx.x * n * n;
  T *Vs = vs_all + (size_t)blockIdx.x * n * n;
  double *w = w_all + (size_t)blockIdx.x * n;
  // the lower triangle is the matrix (nx_c_eigh.c:14)
  for (int64_t e = threadIdx.x; e < (int64_t)n * n; e += blockDim.x) {
    const int i = (int)(e / n), j = (int)(e % n);
    if (i < j) A[e] = S::conj(A[(size_t)j * n + i]);
    if (wantv) V[e] = i == j ? S::make(1.0, 0.0) : S::make(0.0, 0.0);
  }
  __syncthreads();
  for (int64_t e = threadIdx.x; e < n; e += blockDim.x) A[(size_t)e * n + e] = S::make(S::re(A[(size_t)e * n + e]), 0.0);
  __syncthreads();
  bool converged = n < 2;
  for (int sweep = 0; sweep < 60 && !converged; sweep++) {
    double off = 0.0, all = 0.0;
    for (int64_t e = threadIdx.x; e < (int64_t)n * n; e += blockDim.x) {
      const double a2 = S::abs2(A[e]);
      all += a2;
      if (e / n != e % n) off += a2;
    }
    off = block_sum(off, scratch);
    all = block_sum(all, scratch);
    if (!(all == all) || !(off == off)) break;  // NaN in the matrix: never converges
    if (off <= all * 1e-29 * n) {  // off-diagonal norm at rounding level of the whole
      converged = true;
      break;
    }
    for (int r = 0; r < N - 1; r++) {
      for (int t = threadIdx.x; t < P; t += blockDim.x) {
        int p, q;
        round_robin(N, r, t, &p, &q);
        double c = 1.0;
        T sp = S::make(0.0, 0.0);
        if (q < n) jacobi_rotation(S::re(A[(size_t)p * n + p]), S::re(A[(size_t)q * n + q]), A[(size_t)p * n + q], &c, &sp);
        rc[t] = c;
        rs[t] = sp;
      }
      __syncthreads();
      // columns: X <- X J for A and V
      for (int64_t e = threadIdx.x; e < (int64_t)P * n; e += blockDim.x) {
        const int t = (int)(e / n), i = (int)(e % n);
        int p, q;
        round_robin(N, r, t, &p, &q);
        if (q >= n) continue;
        const double c = rc[t];
        const T sp = rs[t];
        if (c == 1.0 && sp == S::make(0.0, 0.0)) continue;
        T x = A[(size_t)i * n + p], y = A[(size_t)i * n + q];
        A[(size_t)i * n + p] = S::scale(x, c) - S::conj(sp) * y;
        A[(size_t)i * n + q] = sp * x + S::scale(y, c);
        if (wantv) {
          x = V[(size_t)i * n + p];
          y = V[(size_t)i * n + q];
          V[(size_t)i * n + p] = S::scale(x, c) - S::conj(sp) * y;
          V[(size_t)i * n + q] = sp * x + S::scale(y, c);
        }
      }
      __syncthreads();
      // rows: A <- J^H A
      for (int64_t e = threadIdx.x; e < (int64_t)P * n; e += blockDim.x) {
        const int t = (int)(e / n), j = (int)(e % n);
        int p, q;
        round_robin(N, r, t, &p, &q);
        if (q >= n) continue;
        const double c = rc[t];
        const T sp = rs[t];
        if (c == 1.0 && sp == S::make(0.0, 0.0)) continue;
        const T x = A[(size_t)p * n + j], y = A[(size_t)q * n + j];
        A[(size_t)p * n + j] = S::scale(x, c) - sp * y;
        A[(size_t)q * n + j] = S::conj(sp) * x + S::scale(y, c);
      }
      __syncthreads();
    }
  }
  if (!converged) {
    if (threadIdx.x == 0) raise(status, LA_NO_CONVERGE);
    return;
  }
  eigh_sort_block(A, V, Vs, w, n, wantv);
}

// Columns by descending norm (ties by position) into Gs / Vs; `norms` holds nn doubles.
template <class T>
__device__ void svd_sort_block(const T *G, const T *V, T *Gs, T *Vs, int mm, int nn, double *norms, int *status) {
  using S = Sc<T>;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, waves = blockDim.x >> 6;
  for (int c = wave; c < nn; c += waves) {
    double a = 0.0;
    for (int i = lane; i < mm; i += 64) a += S::abs2(G[(size_t)c * mm + i]);
    a = wave_sum(a);
    if (lane == 0) {
      norms[c] = a;
      // a NaN or infinity in the matrix stops no rotation and orders nowhere: the iteration has not converged
      if (!(a - a == 0.0)) raise(status, LA_NO_CONVERGE);
    }
  }
  __syncthreads();
  for (int c = wave; c < nn; c += waves) {
    const double a = norms[c];
    int rank = 0;
    for (int j = 0; j < nn; j++) rank += (norms[j] > a) || (norms[j] == a && j < c);
    for (int i = lane; i < mm; i += 64) Gs[(size_t)rank * mm + i] = G[(size_t)c * mm + i];
    for (int i = lane; i < nn; i += 64) Vs[(size_t)rank * nn + i] = V[(size_t)c * nn + i];
  }
}

// ── svd: one-sided Jacobi ───────────────────────────────────────────────────
// Gt: nn columns of mm rows (mm >= nn), orthogonalised in place; Vt: the
// accumulated rotations, column-major nn x nn. Sorted by descending column norm
// into Gs / Vs.
template <class T>
__global__ __launch_bounds__(LA_THREADS) void svd_jacobi_kernel(T *g_all, T *v_all, T *gs_all, T *vs_all, int mm, int nn,
                                                               int *status) {
  using S = Sc<T>;
  extern __shared__ double norms[];  // nn column norms for the final ordering
  __shared__ int rotated;
  T *G = g_all + (size_t)blockIdx.x * mm * nn;
  T *V = v_all + (size_t)blockIdx.x * nn * nn;
  T *Gs = gs_all + (size_t)blockIdx.x * mm * nn;
  T *Vs = vs_all + (size_t)blockIdx.x * nn * nn;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, waves = blockDim.x >> 6;
  const int N = (nn + 1) & ~1, P = N / 2;
  for (int64_t e = threadIdx.x; e < (int64_t)nn * nn; e += blockDim.x)
    V[e] = (e / nn) == (e % nn) ? S::make(1.0, 0.0) : S::make(0.0, 0.0);
  __syncthreads();
  // two columns count as orthogonal when |<p, q>| <= tol |p| |q|, tol at the rounding level of a dot product of mm terms
  const double tol = fmax(1e-15, 8.0 * 2.220446049250313e-16 * sqrt((double)mm)), tol2 = tol * tol;
  bool converged = false;
  for (int sweep = 0; sweep < 60 && !converged; sweep++) {
    if (threadIdx.x == 0) rotated = 0;
    __syncthreads();
    for (int r = 0; r < N - 1; r++) {
      for (int t = wave; t < P; t += waves) {
        int p, q;
        round_robin(N, r, t, &p, &q);
        if (q >= nn) continue;
        T *gp = G + (size_t)p * mm, *gq = G + (size_t)q * mm;
        double a = 0.0, b = 0.0;
        T g = S::make(0.0, 0.0);
        for (int i = lane; i < mm; i += 64) {
          const T x = gp[i], y = gq[i];
          a += S::abs2(x);
          b += S::abs2(y);
          g = g + S::conj(x) * y;
        }
        a = wave_sum(a);
        b = wave_sum(b);
        g = wave_sum(g);
        const double g2 = S::abs2(g);
        if (!(g2 > tol2 * a * b) || !(g2 > 1e-300)) continue;  // orthogonal to working precision (or NaN)
        double c;
        T sp;
        jacobi_rotation(a, b, g, &c, &sp);
        if (lane == 0) rotated = 1;
        for (int i = lane; i < mm; i += 64) {
          const T x = gp[i], y = gq[i];
          gp[i] = S::scale(x, c) - S::conj(sp) * y;
          gq[i] = sp * x + S::scale(y, c);
        }
        T *vp = V + (size_t)p * nn, *vq = V + (size_t)q * nn;
        for (int i = lane; i < nn; i += 64) {
          const T x = vp[i], y = vq[i];
          vp[i] = S::scale(x, c) - S::conj(sp) * y;
          vq[i] = sp * x + S::scale(y, c);
        }
      }
      __syncthreads();
    }
    converged = rotated == 0;
    __syncthreads();
  }
  if (!converged) {
    if (threadIdx.x == 0) raise(status, LA_NO_CONVERGE);
    return;
  }
  svd_sort_block(G, V, Gs, Vs, mm, nn, norms, status);
}

// After the QR of the sorted, orthogonal columns: R's diagonal carries the
// singular values with a unit phase, which moves into the columns of Q.
template <class T>
__global__ __launch_bounds__(LA_THREADS) void svd_finish_kernel(const T *rt_all, T *qt_all, double *s_all, int mm, int nn, int nq) {
  using S = Sc<T>;
  const T *Rt = rt_all + (size_t)blockIdx.x * mm * nn;
  T *Qt = qt_all + (size_t)blockIdx.x * mm * nq;
  double *s = s_all + (size_t)blockIdx.x * nn;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, waves = blockDim.x >> 6;
  for (int j = wave; j < nn; j += waves) {
    const T d = Rt[(size_t)j * mm + j];
    const double a = sqrt(S::abs2(d));
    if (lane == 0) s[j] = a;
    if (a > 0.0) {
      const T phase = S::scale(d, 1.0 / a);
      for (int i = lane; i < mm; i += 64) Qt[(size_t)j * mm + i] = Qt[(size_t)j * mm + i] * phase;
    }
  }
}

// ── the same Jacobi iterations over the whole device ────────────────────────
// One workgroup per matrix leaves 255 of 256 compute units idle when the batch is
// small and the matrix is not: above 64 rows each phase of a round is a launch of
// its own over every (matrix, pair, row) item, the host reads one convergence
// counter per sweep, and a matrix that has converged is skipped by later rounds.
template <class T>
__global__ __launch_bounds__(LA_THREADS) void eigh_wide_prepare(T *a_all, T *v_all, int n, int wantv, int64_t total) {
  using S = Sc<T>;
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= total) return;
  const int64_t nn2 = (int64_t)n * n;
  T *A = a_all + (e / nn2) * nn2;
  const int i = (int)((e % nn2) / n), j = (int)(e % n);
  if (i < j) A[(size_t)i * n + j] = S::conj(A[(size_t)j * n + i]);  // the lower triangle is never written here
  else if (i == j) A[(size_t)i * n + i] = S::make(S::re(A[(size_t)i * n + i]), 0.0);
  if (wantv) v_all[e] = i == j ? S::make(1.0, 0.0) : S::make(0.0, 0.0);
}

template <class T>
__global__ __launch_bounds__(LA_THREADS) void eigh_wide_check(const T *a_all, int n, int *done, int *remaining, int *status) {
  using S = Sc<T>;
  __shared__ double scratch[LA_THREADS / 64];
  if (done[blockIdx.x]) return;
  const T *A = a_all + (size_t)blockIdx.x * n * n;
  double off = 0.0, all = 0.0;
  for (int64_t e = threadIdx.x; e < (int64_t)n * n; e += blockDim.x) {
    const double a2 = S::abs2(A[e]);
    all += a2;
    if (e / n != e % n) off += a2;
  }
  off = block_sum(off, scratch);
  all = block_sum(all, scratch);
  if (threadIdx.x != 0) return;
  if (!(all == all) || !(off == off)) {
    raise(status, LA_NO_CONVERGE);
    done[blockIdx.x] = 1;
  } else if (off <= all * 1e-29 * n) {
    done[blockIdx.x] = 1;
  } else {
    atomicAdd(remaining, 1);
  }
}

template <class T>
__global__ __launch_bounds__(LA_THREADS) void eigh_wide_params(const T *a_all, double *rc_all, T *rs_all, const int *done, int n,
                                                              int N, int r, int64_t total) {
  using S = Sc<T>;
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= total) return;
  const int P = N / 2, t = (int)(e % P);
  const int64_t b = e / P;
  if (done[b]) return;
  const T *A = a_all + (size_t)b * n * n;
  int p, q;
  round_robin(N, r, t, &p, &q);
  double c = 1.0;
  T sp = S::make(0.0, 0.0);
  if (q < n) jacobi_rotation(S::re(A[(size_t)p * n + p]), S::re(A[(size_t)q * n + q]), A[(size_t)p * n + q], &c, &sp);
  rc_all[e] = c;
  rs_all[e] = sp;
}

// ROWS = false: X <- X J on the columns of A and V; ROWS = true: A <- J^H A.
template <class T, bool ROWS>
__global__ __launch_bounds__(LA_THREADS) void eigh_wide_rotate(T *a_all, T *v_all, const double *rc_all, const T *rs_all,
                                                              const int *done, int n, int N, int r, int wantv, int64_t total) {
  using S = Sc<T>;
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= total) return;
  const int P = N / 2;
  // rows: neighbouring lanes take neighbouring columns i of the row pair. Columns:
  // neighbouring lanes take the pairs of one row i, which together cover that row
  // exactly once (a lane per row would stride the whole matrix)
  const int i = ROWS ? (int)(e % n) : (int)((e / P) % n), t = ROWS ? (int)((e / n) % P) : (int)(e % P);
  const int64_t b = e / ((int64_t)n * P);
  if (done[b]) return;
  int p, q;
  round_robin(N, r, t, &p, &q);
  if (q >= n) return;
  const double c = rc_all[b * P + t];
  const T sp = rs_all[b * P + t];
  if (c == 1.0 && sp == S::make(0.0, 0.0)) return;
  T *A = a_all + (size_t)b * n * n;
  if (ROWS) {
    const T x = A[(size_t)p * n + i], y = A[(size_t)q * n + i];
    A[(size_t)p * n + i] = S::scale(x, c) - sp * y;
    A[(size_t)q * n + i] = S::conj(sp) * x + S::scale(y, c);
  } else {
    T x = A[(size_t)i * n + p], y = A[(size_t)i * n + q];
    A[(size_t)i * n + p] = S::scale(x, c) - S::conj(sp) * y;
    A[(size_t)i * n + q] = sp * x + S::scale(y, c);
    if (wantv) {
      T *V = v_all + (size_t)b * n * n;
      x = V[(size_t)i * n + p];
      y = V[(size_t)i * n + q];
      V[(size_t)i * n + p] = S::scale(x, c) - S::conj(sp) * y;
      V[(size_t)i * n + q] = sp * x + S::scale(y, c);
    }
  }
}

template <class T>
__global__ __launch_bounds__(LA_THREADS) void eigh_wide_sort(const T *a_all, const T *v_all, T *vs_all, double *w_all, int n,
                                                            int wantv) {
  const size_t m = (size_t)blockIdx.x * n * n;
  eigh_sort_block(a_all + m, v_all + m, vs_all + m, w_all + (size_t)blockIdx.x * n, n, wantv);
}

template <class T>
__global__ __launch_bounds__(LA_THREADS) void svd_wide_init(T *v_all, int nn, int64_t total) {
  using S = Sc<T>;
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= total) return;
  const int64_t w = e % ((int64_t)nn * nn);
  v_all[e] = (w / nn) == (w % nn) ? S::make(1.0, 0.0) : S::make(0.0, 0.0);
}

// One round: a wave per (matrix, pair).
template <class T>
__global__ __launch_bounds__(LA_THREADS) void svd_wide_round(T *g_all, T *v_all, int mm, int nn, int N, int r, int64_t pairs,
                                                            int *rotated) {
  using S = Sc<T>;
  const int lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (item >= pairs) return;
  const int P = N / 2, t = (int)(item % P);
  const int64_t b = item / P;
  int p, q;
  round_robin(N, r, t, &p, &q);
  if (q >= nn) return;
  T *gp = g_all + ((size_t)b * nn + p) * mm, *gq = g_all + ((size_t)b * nn + q) * mm;
  double a = 0.0, bb = 0.0;
  T g = S::make(0.0, 0.0);
  for (int i = lane; i < mm; i += 64) {
    const T x = gp[i], y = gq[i];
    a += S::abs2(x);
    bb += S::abs2(y);
    g = g + S::conj(x) * y;
  }
  a = wave_sum(a);
  bb = wave_sum(bb);
  g = wave_sum(g);
  const double tol = fmax(1e-15, 8.0 * 2.220446049250313e-16 * sqrt((double)mm)), g2 = S::abs2(g);
  if (!(g2 > tol * tol * a * bb) || !(g2 > 1e-300)) return;
  double c;
  T sp;
  jacobi_rotation(a, bb, g, &c, &sp);
  if (lane == 0) atomicAdd(rotated, 1);
  for (int i = lane; i < mm; i += 64) {
    const T x = gp[i], y = gq[i];
    gp[i] = S::scale(x, c) - S::conj(sp) * y;
    gq[i] = sp * x + S::scale(y, c);
  }
  T *vp = v_all + ((size_t)b * nn + p) * nn, *vq = v_all + ((size_t)b * nn + q) * nn;
  for (int i = lane; i < nn; i += 64) {
    const T x = vp[i], y = vq[i];
    vp[i] = S::scale(x, c) - S::conj(sp) * y;
    vq[i] = sp * x + S::scale(y, c);
  }
}

template <class T>
__global__ __launch_bounds__(LA_THREADS) void svd_wide_sort(const T *g_all, const T *v_all, T *gs_all, T *vs_all, int mm, int nn,
                                                           int *status) {
  extern __shared__ double norms[];
  const size_t g = (size_t)blockIdx.x * mm * nn, v = (size_t)blockIdx.x * nn * nn;
  svd_sort_block(g_all + g, v_all + v, gs_all + g, vs_all + v, mm, nn, norms, status);
}

__global__ void la_fill_int(int *p, int count, int value) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) p[i] = value;
}

// ── triangular solve over the whole device ──────────────────────────────────
// Row i of the solution (one launch), then its elimination from the rows not yet
// solved (another), for every matrix and right-hand side at once.
template <class T>
__global__ __launch_bounds__(LA_THREADS) void trsm_wide_scale(const T *a_all, T *x_all, int n, int nrhs, int i, int transpose,
                                                             int64_t total, int *status) {
  using S = Sc<T>;
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= total) return;
  const int64_t b = e / nrhs;
  const int j = (int)(e % nrhs);
  T diag = a_all[(size_t)b * n * n + (size_t)i * n + i];
  if (transpose) diag = S::conj(diag);
  if (diag == S::make(0.0, 0.0)) {
    if (j == 0) raise(status, LA_SINGULAR);
    return;
  }
  T *x = x_all + (size_t)b * n * nrhs + (size_t)i * nrhs + j;
  *x = *x / diag;
}

template <class T>
__global__ __launch_bounds__(LA_THREADS) void trsm_wide_eliminate(const T *a_all, T *x_all, int n, int nrhs, int i, int rest,
                                                                 int forward, int transpose, int64_t total) {
  using S = Sc<T>;
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= total) return;
  const int j = (int)(e % nrhs), rr = (int)((e / nrhs) % rest);
  const int64_t b = e / ((int64_t)nrhs * rest);
  const int r = forward ? i + 1 + rr : i - 1 - rr;
  const T *A = a_all + (size_t)b * n * n;
  T *X = x_all + (size_t)b * n * nrhs;
  const T m = transpose ? S::conj(A[(size_t)i * n + r]) : A[(size_t)r * n + i];
  X[(size_t)r * nrhs + j] = X[(size_t)r * nrhs + j] - m * X[(size_t)i * nrhs + j];
}

// ── cholesky and qr over the whole device ───────────────────────────────────
// Column j of every matrix in one launch, a wave per (matrix, row >= j): the
// lanes split the dot product along the finished columns (contiguous in the
// row-major matrix). Every wave recomputes row j's own dot product for the pivot
// instead of waiting for it.
template <class T>
__global__ __launch_bounds__(LA_THREADS) void cholesky_wide_column(T *all, double *diag_all, int n, int j, int64_t waves_total,
                                                                  int *status) {
  using S = Sc<T>;
  const int lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (item >= waves_total) return;
  const int rows = n - j, i = j + (int)(item % rows);
  T *A = all + (size_t)(item / rows) * n * n;
  const T *ri = A + (size_t)i * n, *rj = A + (size_t)j * n;
  T s = S::make(0.0, 0.0);
  double dj = 0.0;
  for (int k = lane; k < j; k += 64) {
    const T ljk = rj[k];
    s = s + ri[k] * S::conj(ljk);
    dj += S::abs2(ljk);
  }
  s = wave_sum(s);
  const double d = S::re(rj[j]) - wave_sum(dj);
  if (!(d > 0.0)) {
    if (i == j && lane == 0) raise(status, LA_NOT_PD);
    return;  // later columns see an unfinished factor; the call fails as a whole
  }
  const double l = sqrt(d);
  if (lane != 0) return;
  // the pivot is kept aside until the end: the other waves of this launch still read A[j][j]
  if (i == j) diag_all[(item / rows) * n + j] = l;
  else A[(size_t)i * n + j] = S::scale(A[(size_t)i * n + j] - s, 1.0 / l);
}

template <class T>
__global__ __launch_bounds__(LA_THREADS) void cholesky_wide_finish(T *all, const double *diag_all, int n, int upper,
                                                                  int64_t total) {
  using S = Sc<T>;
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= total) return;
  const int64_t nn2 = (int64_t)n * n;
  T *A = all + (e / nn2) * nn2;
  const int i = (int)((e % nn2) / n), k = (int)(e % n);
  if (i == k) A[(size_t)i * n + i] = S::make(diag_all[(e / nn2) * n + i], 0.0);
  if (i <= k) return;
  if (upper) {
    A[(size_t)k * n + i] = S::conj(A[(size_t)i * n + k]);
    A[(size_t)i * n + k] = S::make(0.0, 0.0);
  } else {
    A[(size_t)k * n + i] = S::make(0.0, 0.0);
  }
}

// Reflector of column j (one workgroup per matrix), then its application to the
// trailing columns (a wave per (matrix, column)).
template <class T>
__global__ __launch_bounds__(LA_THREADS) void qr_wide_reflect(T *at_all, T *tau_all, int m, int n, int k, int j) {
  using S = Sc<T>;
  __shared__ double scratch[LA_THREADS / 64];
  T *col = at_all + ((size_t)blockIdx.x * n + j) * m;
  T *tau = tau_all + (size_t)blockIdx.x * k;
  double part = 0.0;
  for (int i = j + 1 + threadIdx.x; i < m; i += blockDim.x) part += S::abs2(col[i]);
  const double xnorm2 = block_sum(part, scratch);
  const T alpha = col[j];
  __syncthreads();
  if (xnorm2 == 0.0) {
    if (threadIdx.x == 0) tau[j] = S::make(0.0, 0.0);
    return;
  }
  const double alphr = S::re(alpha), anorm = sqrt(S::abs2(alpha) + xnorm2);
  const double beta = alphr >= 0.0 ? -anorm : anorm;
  const T scal = alpha - S::make(beta, 0.0);
  for (int i = j + 1 + threadIdx.x; i < m; i += blockDim.x) col[i] = col[i] / scal;
  if (threadIdx.x == 0) {
    col[j] = S::make(beta, 0.0);
    tau[j] = S::make((beta - alphr) / beta, -S::im(alpha) / beta);
  }
}

// X (column-major, `cols` columns of m rows per matrix) <- (I - t v v^H) X on the
// columns from `first` on, v the reflector stored below the diagonal of column j
// of At; t = conj(tau_j) while factoring, tau_j while forming Q.
template <class T>
__global__ __launch_bounds__(LA_THREADS) void qr_wide_apply(const T *at_all, const T *tau_all, T *x_all, int m, int n, int k, int j,
                                                           int cols, int first, int conj_tau, int64_t waves_total) {
  using S = Sc<T>;
  const int lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (item >= waves_total) return;
  const int span = cols - first, c = first + (int)(item % span);
  const int64_t b = item / span;
  T t = tau_all[(size_t)b * k + j];
  if (t == S::make(0.0, 0.0)) return;
  if (conj_tau) t = S::conj(t);
  const T *v = at_all + ((size_t)b * n + j) * m;
  T *xc = x_all + ((size_t)b * cols + c) * m;
  T w = lane == 0 ? xc[j] : S::make(0.0, 0.0);
  for (int i = j + 1 + lane; i < m; i += 64) w = w + S::conj(v[i]) * xc[i];
  w = t * wave_sum(w);
  if (lane == 0) xc[j] = xc[j] - w;
  for (int i = j + 1 + lane; i < m; i += 64) xc[i] = xc[i] - v[i] * w;
}

template <class T>
__global__ __launch_bounds__(LA_THREADS) void qr_wide_identity(T *qt_all, int m, int nq, int64_t total) {
  using S = Sc<T>;
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= total) return;
  const int64_t w = e % ((int64_t)m * nq);
  qt_all[e] = (w / m) == (w % m) ? S::make(1.0, 0.0) : S::make(0.0, 0.0);
}

// R's zeros: below the diagonal of every matrix (where the reflectors were).
template <class T>
__global__ __launch_bounds__(LA_THREADS) void qr_wide_clear(T *at_all, int m, int n, int64_t total) {
  using S = Sc<T>;
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= total) return;
  const int i = (int)(e % m), c = (int)((e / m) % n);
  if (i > c) at_all[e] = S::make(0.0, 0.0);
}

// conj in place (V^H from a column-major V; U'^H likewise)
template <class T>
__global__ void conj_kernel(T *x, int64_t count) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) x[i] = Sc<T>::conj(x[i]);
}

// ── eig: complex Hessenberg + shifted QR ────────────────────────────────────
__device__ __forceinline__ double cabs1(c64 z) { return fabs(z.re) + fabs(z.im); }
__device__ __forceinline__ double cabs2(c64 z) { return hypot(z.re, z.im); }
__device__ __forceinline__ c64 csqrt_principal(c64 z) {
  if (z.re == 0.0 && z.im == 0.0) return {0.0, 0.0};
  const double t = sqrt((fabs(z.re) + hypot(z.re, z.im)) * 0.5);
  if (z.re >= 0.0) return {t, z.im / (2.0 * t)};
  return {fabs(z.im) / (2.0 * t), copysign(t, z.im)};
}

// G = [[c, s], [-conj(s), c]] with G [a; b] = [r; 0]. Every lane of the workgroup
// computes it at every step of a QR sweep, on the chain from one rotation to the
// next: the moduli come from one square root each after a common power-of-two
// scaling (exact, and safe against overflow of the squares) instead of three
// calls of hypot.
__device__ __forceinline__ void givens(c64 a, c64 b, double *c, c64 *s) {
  const double m = fmax(fmax(fabs(a.re), fabs(a.im)), fmax(fabs(b.re), fabs(b.im)));
  if (!(m > 0.0) || !(m < __builtin_inf())) {  // all zero, or not finite: no rotation (NaNs surface in the convergence test)
    *c = 1.0;
    *s = {0.0, 0.0};
    return;
  }
  const int e = -ilogb(m);
  a = {ldexp(a.re, e), ldexp(a.im, e)};
  b = {ldexp(b.re, e), ldexp(b.im, e)};
  const double a2 = a.re * a.re + a.im * a.im, b2 = b.re * b.re + b.im * b.im;
  if (b2 == 0.0) {
    *c = 1.0;
    *s = {0.0, 0.0};
  } else if (a2 == 0.0) {
    const double nb = sqrt(b2);
    *c = 0.0;
    *s = {b.re / nb, -b.im / nb};
  } else {
    const double na = sqrt(a2), inv = 1.0 / sqrt(a2 + b2);
    *c = na * inv;
    const c64 ph = {a.re / na, a.im / na};
    const c64 t = ph * c64{b.re, -b.im};
    *s = {t.re * inv, t.im * inv};
  }
}

// H (row-major n x n, overwritten by the triangular Schur factor), Q (the Schur
// vectors when wantv), Y (workspace for the back-substitution, column-major),
// eigenvalues to w, unit-norm eigenvectors to Vout (row-major).
__global__ __launch_bounds__(LA_THREADS) void eig_kernel(c64 *h_all, c64 *q_all, c64 *y_all, c64 *w_all, c64 *v_all, int n,
                                                        int wantv, int *status) {
  extern __shared__ double lds_raw[];
  c64 *vec = (c64 *)lds_raw;     // n: a reflector, then the sines of one QR sweep
  c64 *sub = vec + n;            // n: the subdiagonal as a QR sweep found it
  double *cs = (double *)(sub + n);  // n cosines
  __shared__ c64 s_pivot[2];
  __shared__ c64 scratch[LA_THREADS / 64];
  __shared__ int s_lo, s_hi, s_its, s_total, s_state;
  __shared__ c64 s_mu;
  c64 *H = h_all + (size_t)blockIdx.x * n * n;
  c64 *Q = q_all + (size_t)blockIdx.x * n * n;
  c64 *Y = y_all + (size_t)blockIdx.x * n * n;
  c64 *w = w_all + (size_t)blockIdx.x * n;
  c64 *Vout = v_all + (size_t)blockIdx.x * n * n;
  const c64 zero = {0.0, 0.0}, one = {1.0, 0.0};
  if (wantv) {
    for (int64_t e = threadIdx.x; e < (int64_t)n * n; e += blockDim.x) Q[e] = (e / n) == (e % n) ? one : zero;
  }
  __syncthreads();
  // Hessenberg form: P = I - beta v v^H (Hermitian and unitary) per column, H <- P H P, Q <- Q P
  for (int k = 0; k + 2 < n; k++) {
    double part = 0.0;
    for (int i = k + 1 + threadIdx.x; i < n; i += blockDim.x) {
      const c64 x = H[(size_t)i * n + k];
      vec[i] = x;
      part += x.re * x.re + x.im * x.im;
    }
    const double norm2 = block_sum(part, (double *)scratch);
    const c64 x0 = H[(size_t)(k + 1) * n + k];
    const double below = norm2 - (x0.re * x0.re + x0.im * x0.im);
    __syncthreads();
    if (!(below > 0.0)) continue;  // already Hessenberg in this column (uniform)
    const double norm = sqrt(norm2), a0 = cabs2(x0);
    const c64 ph = a0 > 0.0 ? c64{x0.re / a0, x0.im / a0} : one;
    const c64 v0 = x0 + c64{ph.re * norm, ph.im * norm};
    const double beta = 2.0 / (norm2 - (x0.re * x0.re + x0.im * x0.im) + (v0.re * v0.re + v0.im * v0.im));
    if (threadIdx.x == 0) vec[k + 1] = v0;
    __syncthreads();
    // left: rows k+1.., every column j; lanes over j
    for (int j = threadIdx.x; j < n; j += blockDim.x) {
      c64 s = zero;
      for (int i = k + 1; i < n; i++) s = s + c64{vec[i].re, -vec[i].im} * H[(size_t)i * n + j];
      s = {s.re * beta, s.im * beta};
      for (int i = k + 1; i < n; i++) H[(size_t)i * n + j] = H[(size_t)i * n + j] - vec[i] * s;
    }
    __syncthreads();
    // right: columns k+1.., every row i of H and of Q; lanes over i
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
      c64 *row = H + (size_t)i * n;
      c64 s = zero;
      for (int j = k + 1; j < n; j++) s = s + row[j] * vec[j];
      s = {s.re * beta, s.im * beta};
      for (int j = k + 1; j < n; j++) row[j] = row[j] - s * c64{vec[j].re, -vec[j].im};
      if (wantv) {
        row = Q + (size_t)i * n;
        s = zero;
        for (int j = k + 1; j < n; j++) s = s + row[j] * vec[j];
        s = {s.re * beta, s.im * beta};
        for (int j = k + 1; j < n; j++) row[j] = row[j] - s * c64{vec[j].re, -vec[j].im};
      }
    }
    __syncthreads();
    for (int i = k + 2 + threadIdx.x; i < n; i += blockDim.x) H[(size_t)i * n + k] = zero;
    __syncthreads();
  }
  // shifted QR with deflation (the discipline of nx_c_eig.c:47-52)
  if (threadIdx.x == 0) {
    s_hi = n - 1;
    s_its = 0;
    s_total = 0;
    s_state = 0;
  }
  __syncthreads();
  const double eps = 2.220446049250313e-16;
  while (true) {
    if (threadIdx.x == 0) {
      int hi = s_hi;
      s_state = 0;
      while (hi >= 0) {
        int l = hi;
        while (l > 0) {
          const double sub = cabs1(H[(size_t)l * n + l - 1]);
          double scale = cabs1(H[(size_t)(l - 1) * n + l - 1]) + cabs1(H[(size_t)l * n + l]);
          if (scale == 0.0) scale = 1.0;
          if (sub <= eps * scale) {
            H[(size_t)l * n + l - 1] = zero;
            break;
          }
          l--;
        }
        if (l == hi) {  // one eigenvalue has converged
          hi--;
          s_its = 0;
          continue;
        }
        s_lo = l;
        break;
      }
      s_hi = hi;
      if (hi < 0) {
        s_state = 1;  // done
      } else if (s_total >= 30 * n || !(cabs1(H[(size_t)hi * n + hi]) == cabs1(H[(size_t)hi * n + hi]))) {
        s_state = 2;  // no convergence (or NaN)
      } else {
        // Wilkinson shift from the trailing 2 x 2; exceptional shifts at 10 and 20
        const c64 a = H[(size_t)(hi - 1) * n + hi - 1], b = H[(size_t)(hi - 1) * n + hi];
        const c64 c = H[(size_t)hi * n + hi - 1], d = H[(size_t)hi * n + hi];
        c64 mu;
        if (s_its == 10 || s_its == 20) {
          mu = {cabs1(c) + (hi >= 2 ? cabs1(H[(size_t)(hi - 1) * n + hi - 2]) : 0.0) + d.re, d.im};
        } else {
          const c64 half = {0.5, 0.0};
          const c64 tr = (a + d) * half, det = (a - d) * half * ((a - d) * half) + b * c;
          const c64 root = csqrt_principal(det);
          const c64 m1 = tr + root, m2 = tr - root;
          mu = cabs2(m1 - d) <= cabs2(m2 - d) ? m1 : m2;
        }
        s_mu = mu;
        s_its++;
        s_total++;
      }
    }
    __syncthreads();
    if (s_state == 1) break;
    if (s_state == 2) {
      if (threadIdx.x == 0) raise(status, LA_NO_CONVERGE);
      return;
    }
    const int lo = s_lo, hi = s_hi;
    const c64 mu = s_mu;
    // values only: the active block is enough; with vectors the whole Schur factor is updated
    const int col_end = wantv ? n : hi + 1, row_begin = wantv ? 0 : lo;
    for (int i = lo + threadIdx.x; i <= hi; i += blockDim.x) H[(size_t)i * n + i] = H[(size_t)i * n + i] - mu;
    __syncthreads();
    // G_k ... G_lo (H - mu): rotation k needs the pivot H[k][k] as the rotations before it
    // left it, and nothing else that changes: the subdiagonal is still the sweep's
    // original (kept in LDS), and a lane that owns column j carries row k's element
    // of its column from step to step in a register, so the only memory on the
    // chain from one rotation to the next is a two-slot mailbox in LDS for the
    // pivot. Row k + 1 of a column is read one step ahead of its use.
    {
      constexpr int CPT = LA_MAX_N / 2 / LA_THREADS;  // columns per lane
      c64 carry[CPT], ynext[CPT];
      for (int k = lo + threadIdx.x; k < hi; k += blockDim.x) sub[k] = H[(size_t)(k + 1) * n + k];
#pragma unroll
      for (int m = 0; m < CPT; m++) {
        const int j = threadIdx.x + m * LA_THREADS;
        carry[m] = ynext[m] = zero;
        if (j >= lo && j < col_end) {
          carry[m] = H[(size_t)lo * n + j];
          ynext[m] = H[(size_t)(lo + 1) * n + j];
        }
      }
      if (threadIdx.x == 0) s_pivot[lo & 1] = H[(size_t)lo * n + lo];
      for (int k = lo; k < hi; k++) {
        __syncthreads();
        double c;
        c64 s;
        givens(s_pivot[k & 1], sub[k], &c, &s);
        if (threadIdx.x == 0) {
          cs[k] = c;
          vec[k] = s;
        }
#pragma unroll
        for (int m = 0; m < CPT; m++) {
          const int j = threadIdx.x + m * LA_THREADS;
          if (j < k || j >= col_end) continue;
          const c64 x = carry[m], y = ynext[m];
          if (k + 2 <= hi && j >= k + 1) ynext[m] = H[(size_t)(k + 2) * n + j];
          H[(size_t)k * n + j] = c64{x.re * c, x.im * c} + s * y;
          const c64 low = c64{y.re * c, y.im * c} - c64{s.re, -s.im} * x;
          carry[m] = low;
          if (j == k) H[(size_t)(k + 1) * n + k] = low;
          if (j == k + 1) s_pivot[(k + 1) & 1] = low;
        }
      }
#pragma unroll
      for (int m = 0; m < CPT; m++) {
        const int j = threadIdx.x + m * LA_THREADS;
        if (j >= hi && j < col_end) H[(size_t)hi * n + j] = carry[m];
      }
      __syncthreads();
    }
    // R G_lo^H G_{lo+1}^H ...: row i takes the rotations in order, no lane depends on
    // another. The element that moves along the row stays in a register and the
    // row is read eight elements ahead, so that no rotation waits for memory.
    auto rotate_row = [&](c64 *row, int kstart) {
      c64 x = row[kstart];
      for (int k = kstart; k < hi; k += 8) {
        c64 yb[8];
#pragma unroll
        for (int u = 0; u < 8; u++)
          if (k + u < hi) yb[u] = row[k + 1 + u];
#pragma unroll
        for (int u = 0; u < 8; u++) {
          if (k + u >= hi) break;
          const double c = cs[k + u];
          const c64 s = vec[k + u];
          row[k + u] = c64{x.re * c, x.im * c} + yb[u] * c64{s.re, -s.im};
          x = c64{yb[u].re * c, yb[u].im * c} - x * s;
        }
      }
      row[hi] = x;
    };
    for (int i = row_begin + threadIdx.x; i <= hi; i += blockDim.x) rotate_row(H + (size_t)i * n, i - 1 > lo ? i - 1 : lo);
    if (wantv)
      for (int i = threadIdx.x; i < n; i += blockDim.x) rotate_row(Q + (size_t)i * n, lo);
    __syncthreads();
    for (int i = lo + threadIdx.x; i <= hi; i += blockDim.x) H[(size_t)i * n + i] = H[(size_t)i * n + i] + mu;
    __syncthreads();
  }
  for (int k = threadIdx.x; k < n; k += blockDim.x) w[k] = H[(size_t)k * n + k];
  if (!wantv) return;
  // eigenvectors of the triangular factor by back-substitution, one per lane
  double part = 0.0;
  for (int64_t e = threadIdx.x; e < (int64_t)n * n; e += blockDim.x)
    if (e / n <= e % n) part = fmax(part, cabs1(H[e]));
  __syncthreads();
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = zero;
  for (int o = 32; o > 0; o >>= 1) part = fmax(part, __shfl_xor(part, o));
  __syncthreads();
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6].re = part;
  __syncthreads();
  double tnorm = 0.0;
  for (int i = 0; i < (int)(blockDim.x >> 6); i++) tnorm = fmax(tnorm, scratch[i].re);
  const double smin = fmax(eps * tnorm, 1e-300);
  for (int k = threadIdx.x; k < n; k += blockDim.x) {
    c64 *y = Y + (size_t)k * n;
    const c64 lam = H[(size_t)k * n + k];
    for (int i = k + 1; i < n; i++) y[i] = zero;
    y[k] = one;
    for (int i = k - 1; i >= 0; i--) {
      c64 s = zero;
      for (int j = i + 1; j <= k; j++) s = s - H[(size_t)i * n + j] * y[j];
      c64 d = H[(size_t)i * n + i] - lam;
      if (cabs1(d) < smin) d = {smin, 0.0};
      y[i] = s / d;
    }
  }
  __syncthreads();
  // V = Q Y, then unit 2-norm columns (nx_c_eig.c:56)
  for (int64_t e = threadIdx.x; e < (int64_t)n * n; e += blockDim.x) {
    const int i = (int)(e / n), k = (int)(e % n);
    const c64 *y = Y + (size_t)k * n, *qr = Q + (size_t)i * n;
    c64 s = zero;
    for (int j = 0; j <= k; j++) s = s + qr[j] * y[j];
    Vout[e] = s;
  }
  __syncthreads();
  for (int k = threadIdx.x; k < n; k += blockDim.x) {
    double a = 0.0;
    for (int i = 0; i < n; i++) {
      const c64 x = Vout[(size_t)i * n + k];
      a += x.re * x.re + x.im * x.im;
    }
    a = a > 0.0 ? 1.0 / sqrt(a) : 1.0;
    for (int i = 0; i < n; i++) {
      const c64 x = Vout[(size_t)i * n + k];
      Vout[(size_t)i * n + k] = {x.re * a, x.im * a};
    }
  }
}

// ── host side ───────────────────────────────────────────────────────────────
static inline bool la_float(int dt) {
  return dt == NXH_F16 || dt == NXH_BF16 || dt == NXH_F32 || dt == NXH_F64 || dt == NXH_F8E4M3 || dt == NXH_F8E5M2;
}
static inline bool la_complex(int dt) { return dt == NXH_C32 || dt == NXH_C64; }

// A contiguous tensor over `data` with the batch dims of `like` and the given
// matrix dims; `transposed` describes the same logical matrix stored column-major.
static nxh_tensor workspace_tensor(const nxh_tensor *like, void *data, int dtype, int64_t rows, int64_t cols, bool transposed,
                                   int trailing = 2) {
  nxh_tensor t{};
  t.data = data;
  t.dtype = dtype;
  const int nb = like->ndim - 2;
  t.ndim = nb + trailing;
  t.offset = 0;
  int64_t stride = trailing == 2 ? rows * cols : rows;
  for (int d = nb - 1; d >= 0; d--) {
    t.shape[d] = like->shape[d];
    t.strides[d] = stride;
    stride *= like->shape[d];
  }
  if (trailing == 2) {
    t.shape[nb] = rows;
    t.shape[nb + 1] = cols;
    t.strides[nb] = transposed ? 1 : cols;
    t.strides[nb + 1] = transposed ? rows : 1;
  } else {
    t.shape[nb] = rows;
    t.strides[nb] = 1;
  }
  return t;
}

struct Work {  // device blocks of one call, returned to the allocator on every path
  nxh_context *ctx;
  std::vector<void *> blocks;
  explicit Work(nxh_context *c) : ctx(c) {}
  ~Work() {
    for (void *p : blocks) (void)nxh_free(ctx, p);
  }
  int get(size_t bytes, void **out) {
    if (int rc = nxh_alloc(ctx, bytes ? bytes : 16, out)) return rc;
    blocks.push_back(*out);
    return NXH_OK;
  }
};

// The status word of the factorisation kernels, beside the gather flag.
static int *la_status(nxh_context *ctx) { return ctx->fault_flag + 1; }

static int la_begin(nxh_context *ctx, const char *op) {
  std::lock_guard<std::mutex> g(ctx->mu);
  if (ctx->capture) return nxh_fail(NXH_FAILURE, op, "factorisations report numeric failures by waiting for the stream: not recorded into a graph");
  NXH_HIP(op, hipSetDevice(ctx->device));
  return NXH_OK;
}

// Waits for the kernels of this call and turns their status into the reference's failure.
static int la_collect(nxh_context *ctx, const char *op) {
  std::lock_guard<std::mutex> g(ctx->mu);
  NXH_HIP(op, hipGetLastError());
  int *host = ctx->fault_flag_host + 1;
  NXH_HIP(op, hipMemcpyAsync(host, la_status(ctx), sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
  NXH_HIP(op, hipStreamSynchronize(ctx->stream));
  const int code = *host;
  if (code == LA_OK) return NXH_OK;
  *host = 0;
  NXH_HIP(op, hipMemcpyAsync(la_status(ctx), host, sizeof(int), hipMemcpyHostToDevice, ctx->stream));
  NXH_HIP(op, hipStreamSynchronize(ctx->stream));
  return nxh_fail(NXH_FAILURE, op, LA_MESSAGES[code <= LA_NO_CONVERGE ? code : LA_NO_CONVERGE]);
}

// One int of device memory as it is once the queued work has run (a stream wait).
static int la_read_int(nxh_context *ctx, const char *op, const int *dev, int *out) {
  std::lock_guard<std::mutex> g(ctx->mu);
  int *host = ctx->fault_flag_host + 2;
  NXH_HIP(op, hipMemcpyAsync(host, dev, sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
  NXH_HIP(op, hipStreamSynchronize(ctx->stream));
  *out = *host;
  return NXH_OK;
}

static inline unsigned la_blocks(int64_t items, int per_block = LA_THREADS) { return (unsigned)((items + per_block - 1) / per_block); }
constexpr int LA_WIDE_FROM = 65;  // rows from which the Jacobi iterations run as device-wide launches

template <class T>
static int eigh_wide(nxh_context *ctx, const char *op, Work &work, int64_t batch, int n, int wantv, T *A, T *V, T *Vs, double *W) {
  const int N = (n + 1) & ~1, P = N / 2;
  const int64_t elems = batch * n * n, rots = batch * P, items = rots * n;
  if (items / LA_THREADS > 0x7fffffffLL) return nxh_fail(NXH_FAILURE, op, "too many elements for one launch");
  void *flags, *rc, *rs;
  int rcode;
  if ((rcode = work.get((size_t)(batch + 1) * sizeof(int), &flags)) || (rcode = work.get((size_t)rots * sizeof(double), &rc)) ||
      (rcode = work.get((size_t)rots * sizeof(T), &rs)))
    return rcode;
  int *counter = (int *)flags, *done = counter + 1;
  {
    std::lock_guard<std::mutex> g(ctx->mu);
    hipLaunchKernelGGL(la_fill_int, dim3(la_blocks(batch + 1)), dim3(LA_THREADS), 0, ctx->stream, counter, (int)(batch + 1), 0);
    hipLaunchKernelGGL(eigh_wide_prepare<T>, dim3(la_blocks(elems)), dim3(LA_THREADS), 0, ctx->stream, A, V, n, wantv, elems);
  }
  bool converged = false;
  for (int sweep = 0; sweep < 60 && !converged; sweep++) {
    {
      std::lock_guard<std::mutex> g(ctx->mu);
      hipLaunchKernelGGL(la_fill_int, dim3(1), dim3(64), 0, ctx->stream, counter, 1, 0);
      hipLaunchKernelGGL(eigh_wide_check<T>, dim3((unsigned)batch), dim3(LA_THREADS), 0, ctx->stream, (const T *)A, n, done, counter,
                         la_status(ctx));
    }
    int remaining = 0;
    if ((rcode = la_read_int(ctx, op, counter, &remaining))) return rcode;
    if (remaining == 0) {
      converged = true;
      break;
    }
    std::lock_guard<std::mutex> g(ctx->mu);
    for (int r = 0; r < N - 1; r++) {
      hipLaunchKernelGGL(eigh_wide_params<T>, dim3(la_blocks(rots)), dim3(LA_THREADS), 0, ctx->stream, (const T *)A, (double *)rc,
                         (T *)rs, (const int *)done, n, N, r, rots);
      hipLaunchKernelGGL((eigh_wide_rotate<T, false>), dim3(la_blocks(items)), dim3(LA_THREADS), 0, ctx->stream, A, V,
                         (const double *)rc, (const T *)rs, (const int *)done, n, N, r, wantv, items);
      hipLaunchKernelGGL((eigh_wide_rotate<T, true>), dim3(la_blocks(items)), dim3(LA_THREADS), 0, ctx->stream, A, V,
                         (const double *)rc, (const T *)rs, (const int *)done, n, N, r, wantv, items);
    }
    NXH_HIP(op, hipGetLastError());
  }
  if (!converged) return nxh_fail(NXH_FAILURE, op, LA_MESSAGES[LA_NO_CONVERGE]);
  std::lock_guard<std::mutex> g(ctx->mu);
  hipLaunchKernelGGL(eigh_wide_sort<T>, dim3((unsigned)batch), dim3(LA_THREADS), 0, ctx->stream, (const T *)A, (const T *)V, Vs, W, n,
                     wantv);
  return NXH_OK;
}

template <class T>
static int svd_wide(nxh_context *ctx, const char *op, Work &work, int64_t batch, int mm, int nn, T *G, T *V, T *Gs, T *Vs) {
  const int N = (nn + 1) & ~1, P = N / 2;
  const int64_t pairs = batch * P, vcount = batch * nn * nn;
  void *flags;
  int rcode;
  if ((rcode = work.get(sizeof(int), &flags))) return rcode;
  int *counter = (int *)flags;
  {
    std::lock_guard<std::mutex> g(ctx->mu);
    hipLaunchKernelGGL(svd_wide_init<T>, dim3(la_blocks(vcount)), dim3(LA_THREADS), 0, ctx->stream, V, nn, vcount);
  }
  bool converged = false;
  for (int sweep = 0; sweep < 60 && !converged; sweep++) {
    {
      std::lock_guard<std::mutex> g(ctx->mu);
      hipLaunchKernelGGL(la_fill_int, dim3(1), dim3(64), 0, ctx->stream, counter, 1, 0);
      for (int r = 0; r < N - 1; r++)
        hipLaunchKernelGGL(svd_wide_round<T>, dim3(la_blocks(pairs, LA_THREADS / 64)), dim3(LA_THREADS), 0, ctx->stream, G, V, mm, nn,
                           N, r, pairs, counter);
      NXH_HIP(op, hipGetLastError());
    }
    int rotated = 0;
    if ((rcode = la_read_int(ctx, op, counter, &rotated))) return rcode;
    converged = rotated == 0;
  }
  if (!converged) return nxh_fail(NXH_FAILURE, op, LA_MESSAGES[LA_NO_CONVERGE]);
  std::lock_guard<std::mutex> g(ctx->mu);
  hipLaunchKernelGGL(svd_wide_sort<T>, dim3((unsigned)batch), dim3(LA_THREADS), (size_t)nn * 8, ctx->stream, (const T *)G, (const T *)V,
                     Gs, Vs, mm, nn, la_status(ctx));
  return NXH_OK;
}

template <class T>
static int trsm_wide(nxh_context *ctx, const char *op, int64_t batch, int n, int nrhs, int upper, int transpose, int unit, const T *A,
                     T *X) {
  const int forward = (upper != 0) == (transpose != 0);
  std::lock_guard<std::mutex> g(ctx->mu);
  for (int ii = 0; ii < n; ii++) {
    const int i = forward ? ii : n - 1 - ii, rest = n - 1 - ii;
    if (!unit)
      hipLaunchKernelGGL(trsm_wide_scale<T>, dim3(la_blocks(batch * nrhs)), dim3(LA_THREADS), 0, ctx->stream, A, X, n, nrhs, i,
                         transpose, batch * nrhs, la_status(ctx));
    const int64_t items = batch * rest * nrhs;
    if (items > 0)
      hipLaunchKernelGGL(trsm_wide_eliminate<T>, dim3(la_blocks(items)), dim3(LA_THREADS), 0, ctx->stream, A, X, n, nrhs, i, rest,
                         forward, transpose, items);
  }
  NXH_HIP(op, hipGetLastError());
  return NXH_OK;
}

template <class T>
static int cholesky_wide(nxh_context *ctx, const char *op, Work &work, int64_t batch, int n, int upper, T *A) {
  void *diag;
  if (int rc = work.get((size_t)(batch * n) * sizeof(double), &diag)) return rc;
  std::lock_guard<std::mutex> g(ctx->mu);
  for (int j = 0; j < n; j++) {
    const int64_t waves = batch * (n - j);
    hipLaunchKernelGGL(cholesky_wide_column<T>, dim3(la_blocks(waves, LA_THREADS / 64)), dim3(LA_THREADS), 0, ctx->stream, A,
                       (double *)diag, n, j, waves, la_status(ctx));
  }
  const int64_t total = batch * n * n;
  hipLaunchKernelGGL(cholesky_wide_finish<T>, dim3(la_blocks(total)), dim3(LA_THREADS), 0, ctx->stream, A, (const double *)diag, n,
                     upper, total);
  NXH_HIP(op, hipGetLastError());
  return NXH_OK;
}

// Householder QR of `batch` column-major m x n matrices At, Q's first nq columns to Qt.
template <class T>
static int run_qr(nxh_context *ctx, const char *op, int64_t batch, int m, int n, int nq, T *At, T *Qt, T *tau) {
  std::lock_guard<std::mutex> g(ctx->mu);
  if (std::max(m, n) < LA_WIDE_FROM) {
    hipLaunchKernelGGL(qr_kernel<T>, dim3((unsigned)batch), dim3(LA_THREADS), 0, ctx->stream, At, Qt, tau, m, n, nq);
    NXH_HIP(op, hipGetLastError());
    return NXH_OK;
  }
  const int k = std::min(m, n), per = LA_THREADS / 64;
  for (int j = 0; j < k; j++) {
    hipLaunchKernelGGL(qr_wide_reflect<T>, dim3((unsigned)batch), dim3(LA_THREADS), 0, ctx->stream, At, tau, m, n, k, j);
    const int64_t waves = batch * (n - j - 1);
    if (waves > 0)
      hipLaunchKernelGGL(qr_wide_apply<T>, dim3(la_blocks(waves, per)), dim3(LA_THREADS), 0, ctx->stream, (const T *)At, (const T *)tau,
                         At, m, n, k, j, n, j + 1, 1, waves);
  }
  const int64_t qcount = batch * m * nq;
  if (qcount > 0) hipLaunchKernelGGL(qr_wide_identity<T>, dim3(la_blocks(qcount)), dim3(LA_THREADS), 0, ctx->stream, Qt, m, nq, qcount);
  for (int j = k - 1; j >= 0; j--) {
    const int64_t waves = batch * (nq - j);
    if (waves > 0)
      hipLaunchKernelGGL(qr_wide_apply<T>, dim3(la_blocks(waves, per)), dim3(LA_THREADS), 0, ctx->stream, (const T *)At, (const T *)tau,
                         Qt, m, n, k, j, nq, j, 0, waves);
  }
  const int64_t acount = batch * m * n;
  if (acount > 0) hipLaunchKernelGGL(qr_wide_clear<T>, dim3(la_blocks(acount)), dim3(LA_THREADS), 0, ctx->stream, At, m, n, acount);
  NXH_HIP(op, hipGetLastError());
  return NXH_OK;
}

struct Problem {
  int64_t batch, rows, cols;
  bool cx;
  int wdt;       // NXH_F64 or NXH_C64
  size_t esize;  // of the compute type
};

static int la_problem(const char *op, const nxh_tensor *x, bool square, Problem *p) {
  if (int rc = nxh_check_tensor(op, x)) return rc;
  if (!la_float(x->dtype) && !la_complex(x->dtype)) return nxh_fail(NXH_FAILURE, op, "linalg requires a float or complex dtype");
  if (x->ndim < 2) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  p->rows = x->shape[x->ndim - 2];
  p->cols = x->shape[x->ndim - 1];
  if (square && p->rows != p->cols) return nxh_fail(NXH_INVALID_ARGUMENT, op, "matrix must be square");
  p->batch = 1;
  for (int d = 0; d < x->ndim - 2; d++) p->batch *= x->shape[d];
  p->cx = la_complex(x->dtype);
  p->wdt = p->cx ? NXH_C64 : NXH_F64;
  p->esize = p->cx ? 16 : 8;
  if (p->batch > 0x7fffffffLL) return nxh_fail(NXH_FAILURE, op, "too many matrices for one launch");
  return NXH_OK;
}

static int same_dims(const char *op, const nxh_tensor *t, const nxh_tensor *like, int64_t rows, int64_t cols) {
  if (t->ndim != like->ndim || t->shape[t->ndim - 2] != rows || t->shape[t->ndim - 1] != cols)
    return nxh_fail(NXH_INVALID_ARGUMENT, op, "operand shapes are incompatible");
  for (int d = 0; d < t->ndim - 2; d++)
    if (t->shape[d] != like->shape[d]) return nxh_fail(NXH_INVALID_ARGUMENT, op, "operand shapes are incompatible");
  return NXH_OK;
}

// The casts that carry operands in and results out report their own paths: the
// factorisation's is set last.
struct PathAtExit {
  const char *name;
  ~PathAtExit() { nxh_set_path(name); }
};

#define LA_LAUNCH(ctx, kernel, blocks, lds, ...)                                                        \
  do {                                                                                                  \
    std::lock_guard<std::mutex> g_((ctx)->mu);                                                          \
    hipLaunchKernelGGL(kernel, dim3((unsigned)(blocks)), dim3(LA_THREADS), (lds), (ctx)->stream, __VA_ARGS__); \
  } while (0)

}  // namespace

// nx_c_tri.c:303-400, 564-578
NXH_EXPORT int nxh_cholesky(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x, int upper) {
  NXH_DEFER_BARRIER(ctx, out);
  const char *op = "cholesky";
  if (!ctx || !out || !x) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  Problem p;
  int rc = la_problem(op, x, true, &p);
  if (!rc) rc = nxh_check_tensor(op, out);
  if (!rc && out->dtype != x->dtype) rc = nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  if (!rc) rc = same_dims(op, out, x, p.rows, p.cols);
  if (rc) return rc;
  const int64_t n = p.rows;
  if (p.batch == 0 || n == 0) return NXH_OK;
  // one factorisation at a time per context: they share the status word and its host slot
  std::lock_guard<std::mutex> whole_call(ctx->call_mu);
  if ((rc = la_begin(ctx, op))) return rc;
  Work work(ctx);
  void *A;
  if ((rc = work.get((size_t)(p.batch * n * n) * p.esize, &A))) return rc;
  nxh_tensor wa = workspace_tensor(x, A, p.wdt, n, n, false);
  if ((rc = nxh_cast(ctx, &wa, x))) return rc;
  PathAtExit path{n >= LA_WIDE_FROM ? "cholesky_columns_wide" : "cholesky_columns"};
  if (n >= LA_WIDE_FROM) {
    rc = p.cx ? cholesky_wide<c64>(ctx, op, work, p.batch, (int)n, upper, (c64 *)A)
              : cholesky_wide<double>(ctx, op, work, p.batch, (int)n, upper, (double *)A);
    if (rc) return rc;
  } else if (p.cx) {
    LA_LAUNCH(ctx, cholesky_kernel<c64>, p.batch, 0, (c64 *)A, (int)n, upper, la_status(ctx));
  } else {
    LA_LAUNCH(ctx, cholesky_kernel<double>, p.batch, 0, (double *)A, (int)n, upper, la_status(ctx));
  }
  if ((rc = la_collect(ctx, op))) return rc;
  return nxh_cast(ctx, out, &wa);
}

// nx_c_tri.c:459-562, 580-600. `b` and `out` are matrices of right-hand sides
// (the binding reshapes a vector to one column, nx_backend.ml:598-611).
// flags: bit 0 upper, bit 1 transpose (conjugate transpose for complex), bit 2 unit diagonal.
NXH_EXPORT int nxh_triangular_solve(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *a, const nxh_tensor *b,
                                    int flags) {
  NXH_DEFER_BARRIER(ctx, out);
  const char *op = "triangular_solve";
  if (!ctx || !out || !a || !b) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  Problem p;
  int rc = la_problem(op, a, true, &p);
  if (!rc) rc = nxh_check_tensor(op, out);
  if (!rc) rc = nxh_check_tensor(op, b);
  if (rc) return rc;
  if (b->dtype != a->dtype || out->dtype != a->dtype) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  if (b->ndim != a->ndim) return nxh_fail(NXH_INVALID_ARGUMENT, op, "operand shapes are incompatible");
  const int64_t n = p.rows, nrhs = b->shape[b->ndim - 1];
  if ((rc = same_dims(op, b, a, n, nrhs)) || (rc = same_dims(op, out, a, n, nrhs))) return rc;
  if (p.batch == 0 || n == 0 || nrhs == 0) return NXH_OK;
  // one factorisation at a time per context: they share the status word and its host slot
  std::lock_guard<std::mutex> whole_call(ctx->call_mu);
  if ((rc = la_begin(ctx, op))) return rc;
  Work work(ctx);
  void *A, *X;
  if ((rc = work.get((size_t)(p.batch * n * n) * p.esize, &A))) return rc;
  if ((rc = work.get((size_t)(p.batch * n * nrhs) * p.esize, &X))) return rc;
  nxh_tensor wa = workspace_tensor(a, A, p.wdt, n, n, false);
  nxh_tensor wx = workspace_tensor(b, X, p.wdt, n, nrhs, false);
  if ((rc = nxh_cast(ctx, &wa, a)) || (rc = nxh_cast(ctx, &wx, b))) return rc;
  PathAtExit path{n >= LA_WIDE_FROM ? "triangular_substitution_wide" : "triangular_substitution"};
  const int up = flags & 1, tr = (flags >> 1) & 1, unit = (flags >> 2) & 1;
  if (n >= LA_WIDE_FROM) {
    if (p.batch * n * nrhs / LA_THREADS > 0x7fffffffLL) return nxh_fail(NXH_FAILURE, op, "too many elements for one launch");
    rc = p.cx ? trsm_wide<c64>(ctx, op, p.batch, (int)n, (int)nrhs, up, tr, unit, (const c64 *)A, (c64 *)X)
              : trsm_wide<double>(ctx, op, p.batch, (int)n, (int)nrhs, up, tr, unit, (const double *)A, (double *)X);
    if (rc) return rc;
  } else if (p.cx) LA_LAUNCH(ctx, trsm_kernel<c64>, p.batch, 0, (const c64 *)A, (c64 *)X, (int)n, (int)nrhs, up, tr, unit, la_status(ctx));
  else LA_LAUNCH(ctx, trsm_kernel<double>, p.batch, 0, (const double *)A, (double *)X, (int)n, (int)nrhs, up, tr, unit, la_status(ctx));
  if ((rc = la_collect(ctx, op))) return rc;
  return nxh_cast(ctx, out, &wx);
}

// nx_c_qr.c; nx_backend.ml:613-626. q is [..., m, k] (reduced) or [..., m, m]; r is
// [..., k, n] or [..., m, n], k = min(m, n).
NXH_EXPORT int nxh_qr(nxh_context *ctx, const nxh_tensor *q, const nxh_tensor *r, const nxh_tensor *x, int reduced) {
  NXH_DEFER_BARRIER(ctx, q, r);
  const char *op = "qr";
  if (!ctx || !q || !r || !x) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  Problem p;
  int rc = la_problem(op, x, false, &p);
  if (!rc) rc = nxh_check_tensor(op, q);
  if (!rc) rc = nxh_check_tensor(op, r);
  if (rc) return rc;
  if (q->dtype != x->dtype || r->dtype != x->dtype) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  const int64_t m = p.rows, n = p.cols, k = std::min(m, n);
  const int64_t nq = reduced ? k : m, rr = reduced ? k : m;
  if ((rc = same_dims(op, q, x, m, nq)) || (rc = same_dims(op, r, x, rr, n))) return rc;
  if (p.batch == 0) return NXH_OK;
  if (m == 0 || n == 0) {  // nothing to factor: Q is the identity (if it has elements), R is empty
    if (m == 0 || nq == 0) return NXH_OK;
  }
  // one factorisation at a time per context: they share the status word and its host slot
  std::lock_guard<std::mutex> whole_call(ctx->call_mu);
  if ((rc = la_begin(ctx, op))) return rc;
  Work work(ctx);
  void *At, *Qt, *tau;
  if ((rc = work.get((size_t)(p.batch * m * n) * p.esize, &At))) return rc;
  if ((rc = work.get((size_t)(p.batch * m * nq) * p.esize, &Qt))) return rc;
  if ((rc = work.get((size_t)(p.batch * k) * p.esize, &tau))) return rc;
  nxh_tensor wa = workspace_tensor(x, At, p.wdt, m, n, true);
  if (n > 0 && (rc = nxh_cast(ctx, &wa, x))) return rc;
  PathAtExit path{std::max(m, n) >= LA_WIDE_FROM ? "qr_householder_wide" : "qr_householder"};
  rc = p.cx ? run_qr<c64>(ctx, op, p.batch, (int)m, (int)n, (int)nq, (c64 *)At, (c64 *)Qt, (c64 *)tau)
            : run_qr<double>(ctx, op, p.batch, (int)m, (int)n, (int)nq, (double *)At, (double *)Qt, (double *)tau);
  if (rc) return rc;
  nxh_tensor wq = workspace_tensor(x, Qt, p.wdt, m, nq, true);
  if ((rc = nxh_cast(ctx, q, &wq))) return rc;
  if (n == 0 || rr == 0) return NXH_OK;
  // R: the first rr rows of the m x n trapezoid
  nxh_tensor wr = wa;
  wr.shape[wr.ndim - 2] = rr;
  return nxh_cast(ctx, r, &wr);
}

// nx_c_eigh.c:1492-1500, 1765-; nx_backend.ml:628-649. v may be null (eigvalsh).
NXH_EXPORT int nxh_eigh(nxh_context *ctx, const nxh_tensor *w, const nxh_tensor *v, const nxh_tensor *x) {
  NXH_DEFER_BARRIER(ctx, w, v);
  const char *op = v ? "eigh" : "eigvalsh";
  if (!ctx || !w || !x) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  Problem p;
  int rc = la_problem(op, x, true, &p);
  if (!rc) rc = nxh_check_tensor(op, w);
  if (!rc && v) rc = nxh_check_tensor(op, v);
  if (rc) return rc;
  const int64_t n = p.rows;
  if (w->dtype != NXH_F64 || (v && v->dtype != x->dtype)) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  if (w->ndim != x->ndim - 1 || w->shape[w->ndim - 1] != n) return nxh_fail(NXH_INVALID_ARGUMENT, op, "operand shapes are incompatible");
  for (int d = 0; d < x->ndim - 2; d++)
    if (w->shape[d] != x->shape[d]) return nxh_fail(NXH_INVALID_ARGUMENT, op, "operand shapes are incompatible");
  if (v && (rc = same_dims(op, v, x, n, n))) return rc;
  if (n > LA_MAX_N) return nxh_fail(NXH_FAILURE, op, "matrix too large (the limit is 4096)");
  if (p.batch == 0 || n == 0) return NXH_OK;
  // one factorisation at a time per context: they share the status word and its host slot
  std::lock_guard<std::mutex> whole_call(ctx->call_mu);
  if ((rc = la_begin(ctx, op))) return rc;
  Work work(ctx);
  void *A, *V = nullptr, *Vs = nullptr, *W;
  const size_t mat = (size_t)(p.batch * n * n) * p.esize;
  if ((rc = work.get(mat, &A)) || (rc = work.get((size_t)(p.batch * n) * 8, &W))) return rc;
  if (v && ((rc = work.get(mat, &V)) || (rc = work.get(mat, &Vs)))) return rc;
  nxh_tensor wa = workspace_tensor(x, A, p.wdt, n, n, false);
  if ((rc = nxh_cast(ctx, &wa, x))) return rc;
  PathAtExit path{n >= LA_WIDE_FROM ? "eigh_jacobi_wide" : "eigh_jacobi"};
  const size_t lds = (size_t)((n + 1) / 2) * (8 + p.esize);
  if (n >= LA_WIDE_FROM) {
    rc = p.cx ? eigh_wide<c64>(ctx, op, work, p.batch, (int)n, v ? 1 : 0, (c64 *)A, (c64 *)V, (c64 *)Vs, (double *)W)
              : eigh_wide<double>(ctx, op, work, p.batch, (int)n, v ? 1 : 0, (double *)A, (double *)V, (double *)Vs, (double *)W);
    if (rc) return rc;
  } else if (p.cx) {
    LA_LAUNCH(ctx, eigh_kernel<c64>, p.batch, lds, (c64 *)A, (c64 *)V, (c64 *)Vs, (double *)W, (int)n, v ? 1 : 0, la_status(ctx));
  } else {
    LA_LAUNCH(ctx, eigh_kernel<double>, p.batch, lds, (double *)A, (double *)V, (double *)Vs, (double *)W, (int)n, v ? 1 : 0, la_status(ctx));
  }
  if ((rc = la_collect(ctx, op))) return rc;
  nxh_tensor ww = workspace_tensor(x, W, NXH_F64, n, 0, false, 1);
  if ((rc = nxh_cast(ctx, w, &ww))) return rc;
  if (!v) return NXH_OK;
  nxh_tensor wv = workspace_tensor(x, Vs, p.wdt, n, n, false);
  return nxh_cast(ctx, v, &wv);
}

// nx_c_svd.c; nx_backend.ml:651-677. u is [..., m, k] or [..., m, m], s [..., k]
// float64 descending, vt [..., k, n] or [..., n, n]; k = min(m, n).
NXH_EXPORT int nxh_svd(nxh_context *ctx, const nxh_tensor *u, const nxh_tensor *s, const nxh_tensor *vt, const nxh_tensor *x) {
  NXH_DEFER_BARRIER(ctx, u, s, vt);
  const char *op = "svd";
  if (!ctx || !u || !s || !vt || !x) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  Problem p;
  int rc = la_problem(op, x, false, &p);
  if (!rc) rc = nxh_check_tensor(op, u);
  if (!rc) rc = nxh_check_tensor(op, s);
  if (!rc) rc = nxh_check_tensor(op, vt);
  if (rc) return rc;
  const int64_t m = p.rows, n = p.cols, k = std::min(m, n);
  if (u->dtype != x->dtype || vt->dtype != x->dtype || s->dtype != NXH_F64) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  if (u->ndim != x->ndim || vt->ndim != x->ndim || s->ndim != x->ndim - 1)
    return nxh_fail(NXH_INVALID_ARGUMENT, op, "operand shapes are incompatible");
  const int64_t ucols = u->shape[u->ndim - 1], vrows = vt->shape[vt->ndim - 2];
  const bool full = ucols == m && vrows == n && !(m == n);
  if (!((ucols == k && vrows == k) || (ucols == m && vrows == n))) return nxh_fail(NXH_INVALID_ARGUMENT, op, "operand shapes are incompatible");
  if ((rc = same_dims(op, u, x, m, ucols)) || (rc = same_dims(op, vt, x, vrows, n))) return rc;
  if (s->shape[s->ndim - 1] != k) return nxh_fail(NXH_INVALID_ARGUMENT, op, "operand shapes are incompatible");
  for (int d = 0; d < x->ndim - 2; d++)
    if (s->shape[d] != x->shape[d]) return nxh_fail(NXH_INVALID_ARGUMENT, op, "operand shapes are incompatible");
  if (k > LA_MAX_N) return nxh_fail(NXH_FAILURE, op, "matrix too large (the limit is 4096 on the shorter side)");
  if (p.batch == 0) return NXH_OK;
  if (k == 0) return nxh_fail(NXH_INVALID_ARGUMENT, op, "empty matrix");
  // one factorisation at a time per context: they share the status word and its host slot
  std::lock_guard<std::mutex> whole_call(ctx->call_mu);
  if ((rc = la_begin(ctx, op))) return rc;
  // G = x (m >= n) or x^H (m < n): mm rows >= nn columns, column-major
  const bool flip = m < n;
  const int64_t mm = flip ? n : m, nn = flip ? m : n;
  const int64_t nq = full ? mm : nn;  // columns of the long-side factor
  Work work(ctx);
  void *G, *V, *Gs, *Vs, *Qt, *tau, *S;
  const size_t gsz = (size_t)(p.batch * mm * nn) * p.esize, vsz = (size_t)(p.batch * nn * nn) * p.esize;
  if ((rc = work.get(gsz, &G)) || (rc = work.get(vsz, &V)) || (rc = work.get(gsz, &Gs)) || (rc = work.get(vsz, &Vs)) ||
      (rc = work.get((size_t)(p.batch * mm * nq) * p.esize, &Qt)) || (rc = work.get((size_t)(p.batch * nn) * p.esize, &tau)) ||
      (rc = work.get((size_t)(p.batch * nn) * 8, &S)))
    return rc;
  // column-major G of x is x's row-major transpose; of x^H it is conj(x) laid out row-major
  nxh_tensor wg = flip ? workspace_tensor(x, G, p.wdt, m, n, false) : workspace_tensor(x, G, p.wdt, m, n, true);
  if ((rc = nxh_cast(ctx, &wg, x))) return rc;
  PathAtExit path{std::min(m, n) >= LA_WIDE_FROM ? "svd_jacobi_wide" : "svd_jacobi"};
  const int64_t gcount = p.batch * mm * nn;
  if (flip && p.cx) {
    std::lock_guard<std::mutex> g_(ctx->mu);
    hipLaunchKernelGGL(conj_kernel<c64>, dim3((unsigned)((gcount + 255) / 256)), dim3(256), 0, ctx->stream, (c64 *)G, gcount);
  }
  const size_t lds = (size_t)nn * 8;
  if (nn >= LA_WIDE_FROM) {
    rc = p.cx ? svd_wide<c64>(ctx, op, work, p.batch, (int)mm, (int)nn, (c64 *)G, (c64 *)V, (c64 *)Gs, (c64 *)Vs)
              : svd_wide<double>(ctx, op, work, p.batch, (int)mm, (int)nn, (double *)G, (double *)V, (double *)Gs, (double *)Vs);
    if (rc) return rc;
  }
  if (p.cx) {
    if (nn < LA_WIDE_FROM)
      LA_LAUNCH(ctx, svd_jacobi_kernel<c64>, p.batch, lds, (c64 *)G, (c64 *)V, (c64 *)Gs, (c64 *)Vs, (int)mm, (int)nn, la_status(ctx));
    if ((rc = run_qr<c64>(ctx, op, p.batch, (int)mm, (int)nn, (int)nq, (c64 *)Gs, (c64 *)Qt, (c64 *)tau))) return rc;
    LA_LAUNCH(ctx, svd_finish_kernel<c64>, p.batch, 0, (const c64 *)Gs, (c64 *)Qt, (double *)S, (int)mm, (int)nn, (int)nq);
  } else {
    if (nn < LA_WIDE_FROM)
      LA_LAUNCH(ctx, svd_jacobi_kernel<double>, p.batch, lds, (double *)G, (double *)V, (double *)Gs, (double *)Vs, (int)mm, (int)nn, la_status(ctx));
    if ((rc = run_qr<double>(ctx, op, p.batch, (int)mm, (int)nn, (int)nq, (double *)Gs, (double *)Qt, (double *)tau))) return rc;
    LA_LAUNCH(ctx, svd_finish_kernel<double>, p.batch, 0, (const double *)Gs, (double *)Qt, (double *)S, (int)mm, (int)nn, (int)nq);
  }
  if ((rc = la_collect(ctx, op))) return rc;
  nxh_tensor ws = workspace_tensor(x, S, NXH_F64, k, 0, false, 1);
  if ((rc = nxh_cast(ctx, s, &ws))) return rc;
  // G V = Q diag: x = Q S V^H (m >= n), or x^H = Q S V^H, x = V S Q^H (m < n)
  const int64_t vcount = p.batch * nn * nn, qcount = p.batch * mm * nq;
  if (!flip) {
    nxh_tensor wq = workspace_tensor(x, Qt, p.wdt, m, nq, true);  // U = Q
    if ((rc = nxh_cast(ctx, u, &wq))) return rc;
    if (p.cx) {  // Vt[j][i] = conj(V[i][j]) = conj of the column-major storage read row-major
      std::lock_guard<std::mutex> g_(ctx->mu);
      hipLaunchKernelGGL(conj_kernel<c64>, dim3((unsigned)((vcount + 255) / 256)), dim3(256), 0, ctx->stream, (c64 *)Vs, vcount);
    }
    nxh_tensor wv = workspace_tensor(x, Vs, p.wdt, nn, nn, false);
    return nxh_cast(ctx, vt, &wv);
  }
  nxh_tensor wv = workspace_tensor(x, Vs, p.wdt, nn, nn, true);  // U = V
  if ((rc = nxh_cast(ctx, u, &wv))) return rc;
  if (p.cx) {
    std::lock_guard<std::mutex> g_(ctx->mu);
    hipLaunchKernelGGL(conj_kernel<c64>, dim3((unsigned)((qcount + 255) / 256)), dim3(256), 0, ctx->stream, (c64 *)Qt, qcount);
  }
  nxh_tensor wq = workspace_tensor(x, Qt, p.wdt, nq, mm, false);  // Vt = Q^H
  return nxh_cast(ctx, vt, &wq);
}

// nx_c_eig.c; nx_backend.ml:679-707. w [..., n] and v [..., n, n] are complex128;
// v may be null (eigvals).
NXH_EXPORT int nxh_eig(nxh_context *ctx, const nxh_tensor *w, const nxh_tensor *v, const nxh_tensor *x) {
  NXH_DEFER_BARRIER(ctx, w, v);
  const char *op = v ? "eig" : "eigvals";
  if (!ctx || !w || !x) return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  Problem p;
  int rc = la_problem(op, x, true, &p);
  if (!rc) rc = nxh_check_tensor(op, w);
  if (!rc && v) rc = nxh_check_tensor(op, v);
  if (rc) return rc;
  const int64_t n = p.rows;
  if (w->dtype != NXH_C64 || (v && v->dtype != NXH_C64)) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  if (w->ndim != x->ndim - 1 || w->shape[w->ndim - 1] != n) return nxh_fail(NXH_INVALID_ARGUMENT, op, "operand shapes are incompatible");
  for (int d = 0; d < x->ndim - 2; d++)
    if (w->shape[d] != x->shape[d]) return nxh_fail(NXH_INVALID_ARGUMENT, op, "operand shapes are incompatible");
  if (v && (rc = same_dims(op, v, x, n, n))) return rc;
  if (n > LA_MAX_N / 2) return nxh_fail(NXH_FAILURE, op, "matrix too large (the limit is 2048)");
  if (p.batch == 0 || n == 0) return NXH_OK;
  // one factorisation at a time per context: they share the status word and its host slot
  std::lock_guard<std::mutex> whole_call(ctx->call_mu);
  if ((rc = la_begin(ctx, op))) return rc;
  Work work(ctx);
  void *H, *Q = nullptr, *Y = nullptr, *W, *V = nullptr;
  const size_t mat = (size_t)(p.batch * n * n) * 16;
  if ((rc = work.get(mat, &H)) || (rc = work.get((size_t)(p.batch * n) * 16, &W))) return rc;
  if (v && ((rc = work.get(mat, &Q)) || (rc = work.get(mat, &Y)) || (rc = work.get(mat, &V)))) return rc;
  nxh_tensor wh = workspace_tensor(x, H, NXH_C64, n, n, false);
  if ((rc = nxh_cast(ctx, &wh, x))) return rc;
  PathAtExit path{"eig_hessenberg_qr"};
  {
    static std::once_flag once;
    static hipError_t attr = hipSuccess;
    std::call_once(once, [&] {
      attr = hipFuncSetAttribute((const void *)eig_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, LA_MAX_N / 2 * 40);
    });
    NXH_HIP(op, attr);
  }
  LA_LAUNCH(ctx, eig_kernel, p.batch, (size_t)n * 40, (c64 *)H, (c64 *)Q, (c64 *)Y, (c64 *)W, (c64 *)V, (int)n, v ? 1 : 0, la_status(ctx));
  if ((rc = la_collect(ctx, op))) return rc;
  nxh_tensor ww = workspace_tensor(x, W, NXH_C64, n, 0, false, 1);
  if ((rc = nxh_cast(ctx, w, &ww))) return rc;
  if (!v) return NXH_OK;
  nxh_tensor wv = workspace_tensor(x, V, NXH_C64, n, n, false);
  return nxh_cast(ctx, v, &wv);
}
