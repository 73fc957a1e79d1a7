"""Copies the small `.espdl` DATA files that the reference's own tests and examples hold, each with
embedded test inputs and expected outputs, into tests/golden/espdl/ so that the GPU box (which has no
copy of the reference) can load them.  They are model containers (weights + known-answer vectors), not
source code.  Run in the development container:  python tests/golden/copy_espdl_fixtures.py

  test_apps/esp-dl/models/{c,esp32s3,esp32p4}/Gemm/*.espdl   one int8 Gemm each, three targets
  examples/tutorial/how_to_run_model/main/models/{s3,p4}/model.espdl   three chained int8 Gemms
  examples/tutorial/how_to_deploy_streaming_model/test_streaming_model/main/models/{esp32s3,esp32p4}/model.espdl
      a Conv1d network: dense and dilated depthwise Conv1d, Sigmoid tables, Mul, Add, AveragePool,
      Transpose, Slice, Flatten, Gemm; and streaming_model.espdl beside it, the same network with StreamingCache
      nodes for chunk-by-chunk inference
"""
import glob
import os
import shutil

REF = "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "espdl")


def main():
    os.makedirs(OUT, exist_ok=True)
    n = 0
    for target in ("c", "esp32s3", "esp32p4"):
        for src in sorted(glob.glob(os.path.join(REF, "test_apps/esp-dl/models", target, "Gemm", "*.espdl"))):
            shutil.copyfile(src, os.path.join(OUT, "gemm_%s_%s" % (target, os.path.basename(src))))
            n += 1
    for target in ("s3", "p4"):
        src = os.path.join(REF, "examples/tutorial/how_to_run_model/main/models", target, "model.espdl")
        shutil.copyfile(src, os.path.join(OUT, "gemm_chain_%s.espdl" % target))
        n += 1
    for target in ("esp32s3", "esp32p4"):
        src = os.path.join(REF, "examples/tutorial/how_to_deploy_streaming_model/test_streaming_model/main/models",
                           target, "model.espdl")
        shutil.copyfile(src, os.path.join(OUT, "conv1d_net_%s.espdl" % target))
        n += 1
        # the same network exported for frame-by-frame use: StreamingCache nodes in front of every windowed operator
        shutil.copyfile(src.replace("model.espdl", "streaming_model.espdl"),
                        os.path.join(OUT, "conv1d_net_streaming_%s.espdl" % target))
        n += 1
    print("copied", n, "files to", OUT)


if __name__ == "__main__":
    main()
