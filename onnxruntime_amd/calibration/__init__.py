"""Calibration builds of the library and the small drivers the planners' constants and the profile summaries come
from.  Nothing here is loaded by the operator: the product library has none of the switches below compiled in.

  python -m onnxruntime_amd.calibration.build [--tag T] [-D NAME[=VALUE] ...] [--only SRC.hip,...]
      builds onnxruntime_amd/calibration/libmnb_calibration[_T].so: every source with -DMNB_TUNING_HOOKS (the planners
      then read their decisions from the environment: the names in run.ENV_KEYS), the sources named by --only also with the -D switches
      (ablations: MNB_ABLATE_NO_LOADS, MNB_ABLATE_NO_MATH, MNB_ABLATE_NO_REDUCE; MNB_SPLIT_FENCES=1)
  python -m onnxruntime_amd.calibration.run one  LIB M N K BITS BLOCK ZP [--launches N] [--copies C]
      launches one problem N times (for rocprofv3 --kernel-trace / --pmc); the variant comes from the environment
  python -m onnxruntime_amd.calibration.run ab   "LIB[;LIB...]" "ENV[;ENV...]" "M,N,K,BITS,BLOCK[,ZP[,COPIES]][;...]"
      alternating timing of libraries x environment variants on the same problems (HIP graphs of 20 launches, or of
      COPIES launches over as many copies of the packed matrix: weights from HBM rather than the Infinity Cache);
      ENV is KEY=VALUE[+KEY=VALUE...], empty for none; reports whether outputs are bit-identical to the first variant
  python -m onnxruntime_amd.calibration.run stamps LIB M N K BITS BLOCK ZP [COPIES]
      anatomy of a direct decode launch (M <= 16) from a library built with --tag stamps -D MNB_STAMPS --only
      mnb_skinny.hip (names the decode kernel's four translation units): every wavefront's readings of the 100 MHz counter at seven points of its life
LIB is a path or the word `product`.
"""
