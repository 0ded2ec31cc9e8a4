"""Generate and compile (on the CPU, ahead of any GPU run) the Session code of every network the GPU tests
and the benchmark execute: the reference's Gemm / Conv / MaxPool fixtures, the fp32 MLP, the CNN in fp32
and the int8 CNN. Output: sofie_amd/generated/{<name>.hxx, <name>.dat, run_<name>}.

    python tests/build_generated.py
"""
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

import models  # noqa: E402
import random_graphs  # noqa: E402
from oracle import oracle  # noqa: E402
from sofie_amd import emit  # noqa: E402


def all_specs(with_large=True):
    specs = [models.fixture_spec(n)[0] for n in models.FIXTURES]
    specs.append(models.mlp_spec()[0])
    specs.append(models.cnn_f32_spec(8))
    specs.append(models.qcnn_spec(oracle, 8))
    specs.append(models.qdq_conv_spec())
    specs.append(models.convbn_spec())
    specs.append(models.functor_spec())
    specs.append(models.stacked_spec())
    specs.append(models.conv1d_spec())
    specs.append(models.conv3d_spec())
    specs.append(models.pool1d_spec())
    specs.append(models.pool3d_spec())
    specs.append(models.qcnn_rt_spec(oracle))
    specs.append(models.cnn_f32_rt_spec())
    specs.append(models.two_heads_spec()[0])
    specs.append(models.mixed_outputs_spec()[0])
    specs.append(models.mlp_nosession_spec()[0])
    # graphs with seeded random attributes (tests/random_graphs.py)
    specs += [random_graphs.float_graph(seed)[0] for seed in random_graphs.FLOAT_SEEDS]
    specs += [random_graphs.quantized_graph(seed, oracle)[0] for seed in random_graphs.QUANT_SEEDS]
    if with_large:
        specs.append(models.qcnn_spec(oracle, 4096, "qcnn_b4096"))
    return specs


def main():
    emit.build_emitter()
    for spec in all_specs():
        hxx, dat, res = spec.generate()
        exe = spec.compile_runner()
        if spec.name == "convbn":
            # the same tensors as typed binary records: the compiled runner reads either file
            import shutil
            sub = os.path.join(emit.GEN_DIR, "binary")
            _, binf, _ = models.convbn_spec().generate(sub, binary_weight_file=True)
            shutil.copyfile(binf, os.path.join(emit.GEN_DIR, "convbn.bin"))
            shutil.rmtree(sub)
        if spec.name == "functor4":
            emit.compile_example("run_functor.cxx", spec.name, "run_functor")
        if spec.name in ("qcnn_b4096", "qcnn_rt", "cnn_f32_rt"):
            os.remove(dat)      # same tensors as qcnn.dat / cnn_f32.dat: the runner is pointed at that file
        print("%-28s %s" % (spec.name, res.stdout.strip().split(", ")[-1]))
    # The fp32 networks once more as code for the host cores (Options::kHostCode), for the test that compares the two
    # emissions on a GPU box and for the benchmark's CPU baseline: sofie_amd/generated/host/run_host_<name>. They
    # read the weight files written above.
    host_dir = os.path.join(emit.GEN_DIR, "host")
    for spec in (models.mlp_spec()[0], models.cnn_f32_spec(8), models.cnn_f32_spec(256, "cnn_f32_b256"), models.qcnn_spec(oracle, 8)):
        _, dat, res = spec.generate(host_dir, host_code=True)
        emit.compile_host_runner(spec.name, host_dir)
        os.remove(dat)
        print("%-28s host code, %s" % (spec.name, res.stdout.strip().split(", ")[-1]))
    return 0


if __name__ == "__main__":
    sys.exit(main())
