"""Extracts the 1-D and 3-D golden vectors of the reference's ReferenceConvFwd test into
reference_convnd_fwd_vectors.json (numbers only: problem parameters and expected outputs).

    python tests/golden/make_convnd_vectors.py [/root/reference]

Reads test/reference_conv_fwd/reference_conv_fwd.cpp as text; nothing of the reference is compiled,
imported or run. The 2-D cases of the same file are in reference_conv_fwd_vectors.json.
"""
import json
import os
import re
import sys

ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
src = open(os.path.join(ref, "test/reference_conv_fwd/reference_conv_fwd.cpp")).read()
tests = re.split(r"\nTEST\(ReferenceConvolutionFWD, ", src)[1:]
cases = []
for t in tests:
    name = t[:t.index(")")]
    if "Conv1D" not in name and "Conv3D" not in name:
        continue
    # a test body may hold several problems: each starts at "params.num_dim_spatial_" or reuses the
    # previous params with some fields overwritten
    fields = {}
    pos = 0
    for m in re.finditer(r"params\.(\w+?)_\s*=\s*(?:std::vector<ck::index_t>)?\{?([0-9, ]+)\}?;|"
                         r"run_reference_convolution_forward<(\d),[^;]*?>\(\s*params(?:,\s*ck::utils::FillMonotonicSeq<float>\{([0-9.f, ]+)\})?\);|"
                         r"std::vector<std::size_t> ref_dims\{([0-9, ]+)\};|"
                         r"std::vector<float> ref_data\{([^}]*)\};|"
                         r"(?!x)x(unused)|"
                         r"\"Error[^\"]*incorrect results!\"(?:,\s*([0-9.e-]+)f,\s*([0-9.e-]+)f)?\)", t):
        if m.group(1):
            vals = [int(v) for v in m.group(2).replace(" ", "").split(",") if v]
            fields[m.group(1)] = vals if len(vals) > 1 or m.group(1) not in ("num_dim_spatial", "N", "K", "C") else vals[0]
        elif m.group(3):
            fields["ndim"] = int(m.group(3))
            step = m.group(4)
            fields["fill"] = [float(v.strip().rstrip("f")) for v in step.split(",")] if step else [0.0, 1.0]
            fields["layout"] = "channels_first" if re.search(r"convolution::(NCDHW|NCW)\b", m.group(0)) else "channels_last"
        elif m.group(5):
            fields["out_dims"] = [int(v) for v in m.group(5).replace(" ", "").split(",")]
        elif m.group(6) is not None:
            fields["expected"] = [float(v) for v in m.group(6).replace("\n", " ").split(",") if v.strip()]
        else:
            c = dict(name=name, ndim=fields["ndim"], layout=fields["layout"], fill_start_step=fields["fill"],
                     N=fields["N"], K=fields["K"], C=fields["C"], filter=fields["filter_spatial_lengths"],
                     input=fields["input_spatial_lengths"], strides=fields["conv_filter_strides"],
                     dilations=fields["conv_filter_dilations"], left_pads=fields["input_left_pads"],
                     right_pads=fields["input_right_pads"], out_dims_nk_spatial=fields["out_dims"],
                     rtol=float(m.group(8)) if m.group(8) else 1e-5, atol=float(m.group(9)) if m.group(9) else 3e-6,
                     expected=fields["expected"])
            for k in ("filter", "input", "strides", "dilations", "left_pads", "right_pads"):
                if not isinstance(c[k], list):
                    c[k] = [c[k]]
            cases.append(c)
out = {"_source": "expected outputs held by the reference's own test test/reference_conv_fwd/reference_conv_fwd.cpp:"
                  "156-392 (1-D NWC and 3-D NCDHW cases); input = start, start + step, ... in the layout's memory "
                  "order, every weight = 0.5, fp32; outputs listed in the output layout's memory order "
                  "(NWK / NKDHW); tolerances are those the reference test passes to check_err "
                  "(default rtol 1e-5, atol 3e-6)",
       "cases": cases}
dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_convnd_fwd_vectors.json")
json.dump(out, open(dst, "w"), indent=1)
print(len(cases), "cases ->", dst)
for c in cases:
    print(c["name"], c["ndim"], c["layout"], c["fill_start_step"], c["N"], c["K"], c["C"], c["input"], c["filter"], c["strides"],
          c["dilations"], c["left_pads"], c["out_dims_nk_spatial"], len(c["expected"]), c["rtol"], c["atol"])
