/* A plain C99 caller of the public headers: compiled and run by tests/test_c_abi.py on a machine
 * without a GPU.  It only takes paths that return before any HIP call. */
#include <stdio.h>

#include "cutt.h"
#include "cutt_ext.h"

int main(void) {
  int dim[3] = {31, 17, 45}, perm[3] = {2, 0, 1};
  int bad[3] = {2, 2, 1};
  int redDim[4], redPerm[4];
  int dim4[4] = {24, 330, 64, 147}, perm4[4] = {1, 0, 2, 3};
  cuttHandle h = 0;
  cuttPlanInfo info;
  void* list;
  int n, best;

  /* the enum keeps the reference's values */
  if (CUTT_SUCCESS != 0 || CUTT_INVALID_PLAN != 1 || CUTT_INVALID_PARAMETER != 2 || CUTT_INVALID_DEVICE != 3 ||
      CUTT_INTERNAL_ERROR != 4 || CUTT_UNDEFINED_ERROR != 5)
    return 10;
  /* input checks come before any device access */
  if (cuttPlan(&h, 3, dim, perm, 3, 0) != CUTT_INVALID_PARAMETER) return 11;
  if (cuttPlan(&h, 1, dim, perm, 4, 0) != CUTT_INVALID_PARAMETER) return 12;
  if (cuttPlan(&h, 3, dim, bad, 8, 0) != CUTT_INVALID_PARAMETER) return 13;
  if (cuttPlan(0, 3, dim, perm, 8, 0) != CUTT_INVALID_PARAMETER) return 14;
  if (cuttPlanMeasure(&h, 3, dim, perm, 8, 0, (void*)dim, (void*)dim) != CUTT_INVALID_PARAMETER) return 15;
  if (cuttExecuteNoAlloc(3, dim, perm, 3, 0, (void*)dim, (void*)perm) != CUTT_INVALID_PARAMETER) return 27;
  if (cuttExecuteNoAlloc(3, dim, bad, 8, 0, (void*)dim, (void*)perm) != CUTT_INVALID_PARAMETER) return 28;
  if (cuttExecuteNoAlloc(3, dim, perm, 8, 0, (void*)dim, (void*)dim) != CUTT_INVALID_PARAMETER) return 29;
  if (cuttExecute(123456u, (void*)dim, (void*)perm) != CUTT_INVALID_PLAN) return 16;
  if (cuttDestroy(123456u) != CUTT_INVALID_PLAN) return 17;
  if (cuttGetPlanInfo(123456u, &info) != CUTT_INVALID_PLAN) return 18;
  /* rank fusing: (24,330,64,147) with (1,0,2,3) fuses its last two ranks */
  if (cuttReduceRanks(4, dim4, perm4, redDim, redPerm) != 3) return 19;
  if (redDim[0] != 24 || redDim[1] != 330 || redDim[2] != 64 * 147) return 20;
  if (redPerm[0] != 1 || redPerm[1] != 0 || redPerm[2] != 2) return 21;
  /* candidate lists need no GPU */
  list = cuttCandidatesCreate(3, dim, perm, 8);
  if (!list) return 22;
  n = cuttCandidatesCount(list);
  best = cuttCandidatesBest(list);
  if (n < 1 || best < 0 || best >= n) return 23;
  if (cuttCandidatesInfo(list, best, &info) != 0) return 24;
  if (info.method < CUTT_METHOD_TRIVIAL || info.method > CUTT_METHOD_TILEDCOPY) return 25;
  cuttCandidatesFree(list);
  cuttSetMethodOverride(CUTT_METHOD_TILED);
  if (cuttGetMethodOverride() != CUTT_METHOD_TILED) return 26;
  cuttSetMethodOverride(0);
  cuttClearPlanCache();
  printf("c abi ok, %d candidates, best method %d\n", n, info.method);
  return 0;
}
