"""Writes tests/golden/<model>_kernel_roles.json (models: resnet152, mobilenet, alexnet, vgg, resnet18, inception, bert): for every
kernel of the reference's resource/<model>/<model>.cu the names of its parameters in signature order (TVM names
inputs `placeholder*` and the result after what it computes, e.g. `T_relu`).  The GPU test
that runs the reference's own kernels needs to know which argument is the output; the
signatures are the only place that says so.  Run in the build container, where the reference
tree is mounted:  python tests/golden/make_kernel_roles.py [/root/reference] [model ...]"""
import json
import os
import re
import sys

ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
for model in (sys.argv[2:] or ["resnet152", "mobilenet", "alexnet", "vgg", "resnet18", "inception", "bert"]):
    src = open(os.path.join(ref, "resource", model, model + ".cu")).read()
    roles = {}
    for m in re.finditer(r'extern "C" __global__ void (?:__launch_bounds__\(\d+\) )?(\w+)\(([^)]*)\)', src):
        roles[m.group(1)] = [a.replace("__restrict__", " ").replace("*", " ").split()[-1]
                             for a in m.group(2).split(",")]
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), model + "_kernel_roles.json")
    json.dump(roles, open(out, "w"), indent=0, sort_keys=True)
    print(model, len(roles), "kernels ->", out)
