#!/bin/bash
# Builds the reference's standalone evaluator from the sources under /root/reference into
# oracle/_ref/ (git-ignored): 1. the vendored flatc (contrib/libs/flatbuffers), 2. the headers it
# generates from the reference's own .fbs schemas, 3. catboost/libs/standalone_evaluator/evaluator.cpp
# + oracle/ref_main.cpp. Nothing of the reference is copied into the repository.
set -euo pipefail
HERE="$(cd "$(dirname "$0")" && pwd)"
R=/root/reference
OUT="$HERE/_ref"
FB="$R/contrib/libs/flatbuffers"
[ -d "$R/catboost" ] || { echo "reference tree not mounted, nothing to do"; exit 0; }
mkdir -p "$OUT/obj" "$OUT/gen"
if [ ! -x "$OUT/flatc" ]; then
  ls "$FB"/src/*.cpp "$FB"/grpc/src/compiler/*.cc | xargs -P8 -I{} sh -c \
    'g++ -std=c++17 -O1 -w -I'"$FB"'/include -I'"$FB"'/grpc -I'"$FB"' -c {} -o '"$OUT"'/obj/$(basename {}).o'
  g++ "$OUT"/obj/*.o -o "$OUT/flatc"
  rm -rf "$OUT/obj"
fi
"$OUT/flatc" -c --gen-mutable --reflect-names -o "$OUT/gen" -I "$R" \
  "$R/catboost/libs/helpers/flatbuffers/guid.fbs" \
  "$R/catboost/libs/model/flatbuffers/features.fbs" \
  "$R/catboost/libs/model/flatbuffers/ctr_data.fbs" \
  "$R/catboost/libs/model/flatbuffers/model.fbs"
g++ -std=c++17 -O2 -w -I "$OUT/gen" -I "$R" -I "$FB/include" -I "$R/catboost/libs/standalone_evaluator" \
  -include cstring "$HERE/ref_main.cpp" "$R/catboost/libs/standalone_evaluator/evaluator.cpp" -o "$OUT/standalone_eval"
echo "built $OUT/standalone_eval"
# the exponent of the prediction types (fmath::expd_v, AVX2 path as on the hosts this runs on)
g++ -std=c++17 -O2 -mavx2 -w -I "$R" "$HERE/ref_fmath_main.cpp" -o "$OUT/fmath_exp"
echo "built $OUT/fmath_exp"
# the CTR calculator of exported models (model_export/resources/ctr_structs.cpp + ctr_calcer.cpp)
g++ -std=c++17 -O2 -w -I "$R" "$HERE/ref_ctr_main.cpp" -o "$OUT/ctr_calc"
echo "built $OUT/ctr_calc"
# models that the reference holds as exported C++ code (canonical outputs of its export tests)
CANON="$R/catboost/python-package/ut/medium/canondata"
g++ -std=c++20 -O1 -w -DWITH_CATS=1 "-DMODEL_SOURCE=\"$CANON/test.test_cpp_export_with_cat_features_CPU_/model.cpp\"" \
  "$HERE/ref_export_main.cpp" -o "$OUT/export_cat"
g++ -std=c++20 -O1 -w -DWITH_CATS=0 "-DMODEL_SOURCE=\"$CANON/test.test_cpp_export_no_cat_features_CPU_/model.cpp\"" \
  "$HERE/ref_export_main.cpp" -o "$OUT/export_nocat"
echo "built $OUT/export_cat $OUT/export_nocat"
