/* A C99 client of the public header: builds against tbruntime_amd.h alone, links the shared library and
 * drives the error paths that need no GPU.  Exit code 0 = everything behaved as documented. */
#include "tbruntime_amd.h"

#include <stdio.h>
#include <string.h>

int main(int argc, char **argv) {
  intptr_t options, runner, forest;
  int64_t info[6];
  double initial = 0.0;
  if (argc < 2) return 2;
  options = CreateCompilerOptions();
  if (!options) return 3;
  Set_batchSize(options, 16);
  Set_tileSize(options, 1);
  /* a missing model: 0 and a message, no abort */
  runner = CreateInferenceRunner("/nonexistent/model.json", "", options);
  if (runner != 0 || strstr(tbmi_last_error(), "cannot open") == NULL) return 4;
  /* host-only inspection works without a device */
  forest = tbmi_load_forest(argv[1], "xgboost_json", 0);
  if (!forest) { fprintf(stderr, "%s\n", tbmi_last_error()); return 5; }
  if (tbmi_forest_info(forest, info, &initial) != 0 || info[0] <= 0 || info[1] <= 0) return 6;
  printf("trees=%lld features=%lld classes=%lld initial=%g devices=%d\n", (long long)info[0], (long long)info[1],
         (long long)info[2], initial, (int)tbmi_device_count());
  tbmi_delete_forest(forest);
  /* null handles are refused with a message */
  if (tbmi_run_device(0, NULL, NULL, 4) != -1 || strstr(tbmi_last_error(), "null") == NULL) return 7;
  if (tbmi_device_count() == 0) { /* no GPU here: creating a runner must fail loudly, never fall back */
    runner = CreateInferenceRunner(argv[1], "", options);
    if (runner != 0 || strstr(tbmi_last_error(), "no HIP device") == NULL) return 8;
  }
  DeleteCompilerOptions(options);
  return 0;
}
