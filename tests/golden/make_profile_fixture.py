"""Writes tests/golden/mi355x_resnet50/: the two profile files that
orion_amd.profiling.capture_profile produced on an MI355X for the headline pair
(ResNet-50 inference batch 4 bf16, 371 kernels; ResNet-50 training batch 32 fp32
SGD, 713 kernels), kernel names cut to 32 characters to keep the fixture small.

    python tests/golden/make_profile_fixture.py <dir holding the captured profiles>

(<dir> is the ``profiles`` directory a ``capture_profile.fill_job`` run on the
GPU leaves behind, e.g. under bench.py's --workdir.)
tests/test_c1_cpu_plumbing.py replays the policy over them in virtual time.
"""

import csv
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
FILES = {"resnet50_4_bf16_inf_fwd": "hp_resnet50_bs4_bf16_inference.csv",
         "resnet50_32_fp32_train_fb1": "be_resnet50_bs32_fp32_training.csv"}


def main(src):
    out = os.path.join(HERE, "mi355x_resnet50")
    os.makedirs(out, exist_ok=True)
    for name, short in FILES.items():
        with open(os.path.join(src, name)) as f:
            rows = list(csv.reader(f))
        with open(os.path.join(out, short), "w") as f:
            f.write(",".join(rows[0]) + "\n")
            for r in rows[1:]:
                f.write(",".join([r[0][:32].replace(" ", "_")] + r[1:]) + "\n")
        print(short, len(rows) - 1, "rows")


if __name__ == "__main__":
    main(sys.argv[1])
