/*
 * CPU oracle for the tensor-transpose path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker that the GPU library is compared against; nothing
 * in the shipped library links, loads or calls it.  It restates, in plain C,
 * the element mapping that the reference defines for a transpose and that its
 * own tester recomputes on the GPU:
 *
 *   - layout and permutation semantics: reference src/TensorTester.cu:151-170
 *     (calcTensorConv: input stride ct of output rank j is the input stride of
 *     rank permutation[j]) and src/TensorTester.cu:56-70 (an output element at
 *     compact output position p comes from the input position
 *     sum_j ((p / c_j) % d_j) * ct_j);
 *   - dimension order "dim[0] fastest" and odim[j] = dim[permutation[j]]:
 *     reference README.md:95-97 and src/cutt_bench.cpp:789-792;
 *   - the rank-fusing rule of src/cuttplan.cpp:63-126 (reduceRanks);
 *   - the check pattern of src/TensorTester.cu:33-37 (data[i] = i as 32-bit
 *     words, so an 8-byte element k holds words 2k, 2k+1).
 *
 * How each function is pinned (see tests/test_oracle.py):
 *   oracle_transpose      - against numpy.transpose on Fortran-ordered arrays
 *                           (an independent library routine), the README shape
 *                           example, hand-worked 2x3 and 2x3x4 cases, identity
 *                           == copy, permutation followed by its inverse ==
 *                           identity, rank-2 (1,0) == matrix transpose.
 *   oracle_transpose_mt   - bit-equal to oracle_transpose on random shapes.
 *   oracle_reduce_ranks   - the hand-derivable cases of src/cutt_test.cpp:
 *                           245-366 and the invariant that transposing the
 *                           fused problem gives the same bytes.
 *   oracle_check_pattern  - agrees with oracle_transpose of the pattern.
 */
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_MAX_RANK 64

/* Input strides (dim[0] fastest) of every rank. */
static void input_strides(int rank, const int *dim, int64_t *cI) {
  int64_t c = 1;
  for (int r = 0; r < rank; r++) {
    cI[r] = c;
    c *= dim[r];
  }
}

/*
 * Copy output elements [o0, o1) of the transposed tensor.  The output is
 * walked in its own linear order with an odometer over the output multi-index;
 * the matching input offset is kept incrementally.
 */
static void transpose_range(int rank, const int *dim, const int *perm,
                            size_t elemSize, const char *in, char *out,
                            int64_t o0, int64_t o1) {
  int64_t cI[ORACLE_MAX_RANK];
  int64_t strideOfOut[ORACLE_MAX_RANK]; /* input stride of output rank j */
  int odim[ORACLE_MAX_RANK];
  int idx[ORACLE_MAX_RANK];
  input_strides(rank, dim, cI);
  for (int j = 0; j < rank; j++) {
    odim[j] = dim[perm[j]];
    strideOfOut[j] = cI[perm[j]];
  }
  /* decompose o0 */
  int64_t rem = o0, ipos = 0;
  for (int j = 0; j < rank; j++) {
    idx[j] = (int)(rem % odim[j]);
    rem /= odim[j];
    ipos += idx[j] * strideOfOut[j];
  }
  for (int64_t o = o0; o < o1; o++) {
    memcpy(out + (size_t)o * elemSize, in + (size_t)ipos * elemSize, elemSize);
    /* advance odometer */
    int j = 0;
    while (j < rank) {
      idx[j]++;
      ipos += strideOfOut[j];
      if (idx[j] < odim[j]) break;
      ipos -= (int64_t)odim[j] * strideOfOut[j];
      idx[j] = 0;
      j++;
    }
  }
}

static int64_t volume(int rank, const int *dim) {
  int64_t v = 1;
  for (int r = 0; r < rank; r++) v *= dim[r];
  return v;
}

/* Single-thread index-loop transpose.  elemSize is arbitrary (4 and 8 used). */
int oracle_transpose(int rank, const int *dim, const int *perm, size_t elemSize,
                     const void *in, void *out) {
  if (rank < 1 || rank > ORACLE_MAX_RANK) return 1;
  transpose_range(rank, dim, perm, elemSize, (const char *)in, (char *)out, 0,
                  volume(rank, dim));
  return 0;
}

/* ---- multithreaded CPU transpose: the reported CPU baseline ------------- */

typedef struct {
  int rank;
  const int *dim;
  const int *perm;
  size_t elemSize;
  const char *in;
  char *out;
  int64_t o0, o1;
  /* blocked path */
  int blocked;
  int64_t task0, task1;
} mt_job;

/*
 * Blocked path: when the leading rank moves (perm[0] != 0) the tensor is a
 * batch of 2-D transposes between input rank 0 and output rank 0.  Tiles of
 * BT x BT elements keep both the reads and the writes inside a few cache
 * lines.  Tasks enumerate (tile along output rank 0, all remaining ranks in
 * output order); each task then loops over tiles along input rank 0.
 */
#define BT 32

static void blocked_tasks(const mt_job *job) {
  const int rank = job->rank;
  const int *dim = job->dim, *perm = job->perm;
  int64_t cI[ORACLE_MAX_RANK] = {0}, cO[ORACLE_MAX_RANK] = {0};
  input_strides(rank, dim, cI);
  /* output stride of output rank j */
  int64_t c = 1;
  for (int j = 0; j < rank; j++) {
    cO[j] = c;
    c *= dim[perm[j]];
  }
  const int k = perm[0];          /* input rank that becomes output rank 0 */
  int jm = 0;                     /* output rank that holds input rank 0 */
  for (int j = 0; j < rank; j++) if (perm[j] == 0) jm = j;
  const int dM = dim[0], dK = dim[k];
  const int64_t inStrideK = cI[k], outStrideM = cO[jm];
  const int ntK = (dK + BT - 1) / BT;
  /* remaining output ranks (all j except 0 and jm) */
  int rest[ORACLE_MAX_RANK], nrest = 0;
  for (int j = 1; j < rank; j++) if (j != jm) rest[nrest++] = j;
  const size_t es = job->elemSize;
  for (int64_t t = job->task0; t < job->task1; t++) {
    int64_t rem = t;
    const int tk = (int)(rem % ntK);
    rem /= ntK;
    int64_t ibase = 0, obase = 0;
    for (int q = 0; q < nrest; q++) {
      const int j = rest[q];
      const int d = dim[perm[j]];
      const int i = (int)(rem % d);
      rem /= d;
      ibase += i * cI[perm[j]];
      obase += i * cO[j];
    }
    const int k0 = tk * BT, k1 = (k0 + BT < dK) ? k0 + BT : dK;
    for (int m0 = 0; m0 < dM; m0 += BT) {
      const int m1 = (m0 + BT < dM) ? m0 + BT : dM;
      if (es == 8) {
        const uint64_t *src = (const uint64_t *)job->in;
        uint64_t *dst = (uint64_t *)job->out;
        for (int m = m0; m < m1; m++)
          for (int kk = k0; kk < k1; kk++)
            dst[obase + kk + m * outStrideM] = src[ibase + m + kk * inStrideK];
      } else if (es == 4) {
        const uint32_t *src = (const uint32_t *)job->in;
        uint32_t *dst = (uint32_t *)job->out;
        for (int m = m0; m < m1; m++)
          for (int kk = k0; kk < k1; kk++)
            dst[obase + kk + m * outStrideM] = src[ibase + m + kk * inStrideK];
      } else {
        for (int m = m0; m < m1; m++)
          for (int kk = k0; kk < k1; kk++)
            memcpy(job->out + (size_t)(obase + kk + m * outStrideM) * es,
                   job->in + (size_t)(ibase + m + kk * inStrideK) * es, es);
      }
    }
  }
}

static void *mt_worker(void *arg) {
  const mt_job *job = (const mt_job *)arg;
  if (job->blocked)
    blocked_tasks(job);
  else
    transpose_range(job->rank, job->dim, job->perm, job->elemSize, job->in,
                    job->out, job->o0, job->o1);
  return NULL;
}

/*
 * Multithreaded transpose on nthreads host threads.  Returns 0 on success.
 * Uses the cache-blocked path when the leading rank moves, otherwise splits
 * the output range evenly (rows along rank 0 are then plain copies).
 */
int oracle_transpose_mt(int rank, const int *dim, const int *perm,
                        size_t elemSize, const void *in, void *out,
                        int nthreads) {
  if (rank < 1 || rank > ORACLE_MAX_RANK || nthreads < 1) return 1;
  if (nthreads > 1024) nthreads = 1024;
  const int64_t vol = volume(rank, dim);
  const int blocked = (rank >= 2 && perm[0] != 0);
  int64_t ntask = 0;
  if (blocked) {
    const int dK = dim[perm[0]];
    ntask = (int64_t)((dK + BT - 1) / BT) * (vol / ((int64_t)dim[0] * dK));
  }
  pthread_t *th = (pthread_t *)malloc(sizeof(pthread_t) * nthreads);
  mt_job *jobs = (mt_job *)malloc(sizeof(mt_job) * nthreads);
  if (!th || !jobs) { free(th); free(jobs); return 2; }
  for (int t = 0; t < nthreads; t++) {
    mt_job *j = &jobs[t];
    j->rank = rank; j->dim = dim; j->perm = perm; j->elemSize = elemSize;
    j->in = (const char *)in; j->out = (char *)out;
    j->blocked = blocked;
    j->o0 = vol * t / nthreads;
    j->o1 = vol * (t + 1) / nthreads;
    j->task0 = ntask * t / nthreads;
    j->task1 = ntask * (t + 1) / nthreads;
  }
  int started = 0, rc = 0;
  for (int t = 1; t < nthreads; t++) {
    if (pthread_create(&th[t], NULL, mt_worker, &jobs[t]) != 0) { rc = 3; break; }
    started = t;
  }
  if (rc == 0) mt_worker(&jobs[0]);
  for (int t = 1; t <= started; t++) pthread_join(th[t], NULL);
  free(th); free(jobs);
  return rc;
}

/* ---- rank fusing (reference src/cuttplan.cpp:63-126) --------------------- */

/*
 * Runs of output ranks whose input ranks are consecutive (perm[i] ==
 * perm[i-1] + 1) are fused into one rank.  Writes the fused dims (in input
 * order) and the renumbered permutation; returns the fused rank.
 */
int oracle_reduce_ranks(int rank, const int *dim, const int *perm, int *redDim,
                        int *redPerm) {
  int groupFirst[ORACLE_MAX_RANK]; /* first input rank of every group, output order */
  int groupVol[ORACLE_MAX_RANK];
  int n = 0;
  for (int i = 0; i < rank; i++) {
    if (i > 0 && perm[i] == perm[i - 1] + 1) {
      groupVol[n - 1] *= dim[perm[i]];
    } else {
      groupFirst[n] = perm[i];
      groupVol[n] = dim[perm[i]];
      n++;
    }
  }
  /* new input-rank number of a group = number of groups that start earlier */
  for (int g = 0; g < n; g++) {
    int id = 0;
    for (int h = 0; h < n; h++) if (groupFirst[h] < groupFirst[g]) id++;
    redPerm[g] = id;
    redDim[id] = groupVol[g];
  }
  return n;
}

/* ---- closed-form check of the "value = linear index" pattern ------------- */

/* Fill words[i] = i (reference src/TensorTester.cu:33-37). */
void oracle_fill_pattern(uint32_t *words, size_t nwords) {
  for (size_t i = 0; i < nwords; i++) words[i] = (uint32_t)i;
}

/*
 * Checks a transposed pattern buffer: output element p must hold the value
 * of the input element it comes from.  Returns -1 if all match, otherwise the
 * first failing output position.
 */
int64_t oracle_check_pattern(int rank, const int *dim, const int *perm,
                             size_t elemSize, const void *out) {
  const int64_t vol = volume(rank, dim);
  int64_t cI[ORACLE_MAX_RANK];
  input_strides(rank, dim, cI);
  const int wordsPer = (int)(elemSize / 4);
  const uint32_t *w = (const uint32_t *)out;
  for (int64_t p = 0; p < vol; p++) {
    int64_t rem = p, src = 0;
    for (int j = 0; j < rank; j++) {
      const int d = dim[perm[j]];
      src += (rem % d) * cI[perm[j]];
      rem /= d;
    }
    for (int k = 0; k < wordsPer; k++)
      if (w[p * wordsPer + k] != (uint32_t)(src * wordsPer + k)) return p;
  }
  return -1;
}
