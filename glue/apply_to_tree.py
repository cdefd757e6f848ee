"""Adds the HIP backend to an apache/singa source tree.

    python glue/apply_to_tree.py /path/to/singa

copies the glue sources of this directory to where the build expects them and makes the few
edits to existing files that a third backend needs (the lang tag, the Context fields, the
Graph's event pair, the dispatch switches of tensor.cc, the build option).  Every edit is an
insertion behind an anchor line that must be found exactly once; a tree where an anchor is
missing is left untouched and the script says which one.  Running it twice is harmless (edits
that are already there are skipped).

What it does NOT touch: python/singa/autograd.py, the operation headers and every CUDA / CPU
source.  The SWIG interface additions are printed at the end (src/api/*.i need SWIG to take
effect; they are a dozen lines).
"""
import os
import re
import shutil
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(HERE)

# (source in this repository, destination in the SINGA tree)
COPIES = [
    ("glue/hip_gpu.h", "include/singa/core/hip_gpu.h"),
    ("glue/hip_gpu.cc", "src/core/device/hip_gpu.cc"),
    ("glue/tensor_math_hip.h", "src/core/tensor/tensor_math_hip.h"),
    ("glue/operation_hip.h", "src/model/operation/operation_hip.h"),
    ("glue/operation_hip.cc", "src/model/operation/operation_hip.cc"),
    ("include/singa_hip.h", "include/singa_hip.h"),
]

MARK = "USE_HIP"


class EditError(RuntimeError):
    pass


def _insert(text, anchor_regex, addition, where, what, count=1, pick=0):
    """Inserts `addition` before / after the `pick`-th of the lines matching `anchor_regex`, of which
    there must be exactly `count`."""
    lines = text.split("\n")
    hits = [i for i, line in enumerate(lines) if re.search(anchor_regex, line)]
    if len(hits) != count:
        raise EditError("%s: expected %d line(s) matching %r, found %d" % (what, count, anchor_regex, len(hits)))
    add = addition.rstrip("\n").split("\n")
    at = hits[pick] if where == "before" else hits[pick] + 1
    lines[at:at] = add
    return "\n".join(lines)


def edit_core_proto(text):
    # value 3 is free and fits the (dtype << 3) + lang hash of TYPE_LANG_SWITCH
    if re.search(r"\bkHip\b", text):
        return text
    return _insert(text, r"^\s*kOpencl\s*=\s*2;", "  kHip = 3;", "after", "core.proto LangType")


def edit_common_h(text):
    if "hip_stream" in text:
        return text
    text = _insert(text, r"^\}\s*Opencl;", "/// To implement functions using the MI355X library (singa_hip.h)\n"
                   "typedef struct _Hip {\n} Hip;", "after", "common.h lang::Opencl")
    ctx = ("#ifdef USE_HIP\n"
           "  // the device behind this context (sgh_device*), its stream (hipStream_t), the state of the\n"
           "  // counter-based random fills, and the scratch of Dot / Sum with the word their host results\n"
           "  // are copied back from\n"
           "  struct sgh_device *hip_device = nullptr;\n"
           "  void *hip_stream = nullptr;\n"
           "  unsigned long long hip_rng_seed = 0, hip_rng_offset = 0;\n"
           "  void *hip_reduce_ws = nullptr;\n"
           "  size_t hip_reduce_ws_bytes = 0;\n"
           "  void *hip_reduce_result = nullptr;\n"
           "#endif  // USE_HIP\n")
    text = _insert(text, r"^\s*std::mt19937 random_generator;", ctx, "after", "common.h Context")
    return _insert(text, r"^namespace singa \{", "struct sgh_device;", "before", "common.h namespace", count=1)


def edit_scheduler_h(text):
    if "hip_start_" in text:
        return text
    ev = ("#ifdef USE_HIP\n"
          "  ::sgh_event *hip_start_ = nullptr;\n"
          "  ::sgh_event *hip_end_ = nullptr;\n"
          "  friend class HipGPU;\n"
          "#endif  // USE_HIP\n")
    # (two classes of the header keep a `time_elapsed_`: Node, the first, is the one that gets the events)
    text = _insert(text, r"^\s*float time_elapsed_ = 0;", ev, "after", "scheduler.h Node", count=2, pick=0)
    return _insert(text, r"^namespace singa \{", "struct sgh_event;", "before", "scheduler.h namespace")


def edit_device_h(text):
    if "hip_gpu.h" in text:
        return text
    # behind the last class of the header, so that HipGPU sees Device and Platform complete
    return _insert(text, r"^#endif\s*//\s*SINGA_CORE_DEVICE_H_", "#ifdef USE_HIP\n#include \"singa/core/hip_gpu.h\"\n#endif  // USE_HIP\n",
                   "before", "device.h tail")


_CASE1 = """      case ((%(dt)s << _SwitchShift) + kHip): {               \\
        typedef %(ct)s DType;                                  \\
        typedef lang::Hip Lang;                                \\
        { __VA_ARGS__ }                                        \\
        break;                                                 \\
      }                                                        \\"""

_CASE2 = """      case (((%(l)s) << _SwitchShift * 2) + (%(r)s << _SwitchShift) +    \\
            kHip): {                                                           \\
        typedef %(lt)s LDType;                                                 \\
        typedef %(rt)s RDType;                                                 \\
        typedef lang::Hip Lang;                                                \\
        { __VA_ARGS__ }                                                        \\
        break;                                                                 \\
      }                                                                        \\"""


def edit_tensor_cc(text):
    if "tensor_math_hip.h" in text:
        return text
    text = _insert(text, r'^#include "\./tensor_math_opencl\.h"', '#include "./tensor_math_hip.h"', "after", "tensor.cc includes")
    def pad(block, width):   # continuation backslashes in the macro's own column
        return "\n".join(l.rstrip("\\").rstrip().ljust(width) + "\\" for l in block.split("\n"))

    one = "\n".join(_CASE1 % {"dt": dt, "ct": ct} for dt, ct in
                    (("kFloat32", "float"), ("kFloat16", "half_float::half"), ("kInt", "int")))
    two = "\n".join(_CASE2 % {"l": l, "r": r, "lt": lt, "rt": rt} for l, r, lt, rt in
                    (("kFloat16", "kFloat32", "half_float::half", "float"),
                     ("kFloat32", "kFloat16", "float", "half_float::half"),
                     ("kFloat32", "kInt", "float", "int"), ("kInt", "kFloat32", "int", "float")))
    # the `default:` line of each of the two switch macros, told apart by its indentation width
    lines = text.split("\n")
    out, state = [], None
    for line in lines:
        if line.startswith("#define TYPE_TYPE_LANG_SWITCH"):
            state = "two"
        elif line.startswith("#define TYPE_LANG_SWITCH"):
            state = "one"
        if state and re.match(r"^\s*default:\s*\\$", line):
            out.extend((pad(two, 79) if state == "two" else pad(one, 63)).split("\n"))
            state = None
        out.append(line)
    text = "\n".join(out)
    if text.count("kHip") != 7:
        raise EditError("tensor.cc: the two dispatch macros were not found as expected")
    return text


def edit_config_in(text):
    if MARK in text:
        return text
    return _insert(text, r"^#cmakedefine USE_OPENCL", "\n#cmakedefine USE_HIP", "after", "singa_config.h.in")


def edit_cmakelists(text):
    if MARK in text:
        return text
    add = ('OPTION(USE_HIP "Use the MI355X backward engine (libsinga_hip.so)" OFF)\n'
           "IF(USE_HIP)\n"
           "  FIND_LIBRARY(SINGA_HIP_LIB singa_hip PATHS ${SINGA_HIP_ROOT}/singa_amd/lib)\n"
           "  LIST(APPEND SINGA_LINKER_LIBS ${SINGA_HIP_LIB})\n"
           "ENDIF()\n")
    return _insert(text, r"^OPTION\(USE_OPENCL\b", add, "after", "CMakeLists.txt options")


EDITS = [
    ("src/proto/core.proto", edit_core_proto),
    ("include/singa/core/common.h", edit_common_h),
    ("include/singa/core/scheduler.h", edit_scheduler_h),
    ("include/singa/core/device.h", edit_device_h),
    ("src/core/tensor/tensor.cc", edit_tensor_cc),
    ("cmake/Templates/singa_config.h.in", edit_config_in),
    ("CMakeLists.txt", edit_cmakelists),
]

SWIG_NOTES = """
SWIG interface additions (src/api), to be made by hand:
  core_device.i       %include / declare under `#if USE_HIP`:
                        int GetNumHipGPUs();
                        std::vector<std::shared_ptr<Device>> CreateHipGPUsOn(const std::vector<int>&);
                      python/singa/device.py gains create_hip_gpu_on(id) = singa.CreateHipGPUsOn([id])[0]
                      (autograd.py stays as it is: it tests `device.id() == -1` for the host).
  model_operation.i   `#if USE_HIP` beside `#if USE_CUDNN` (:121-191): the same class and function
                      declarations, taken from src/model/operation/operation_hip.h, plus the fused
                      functions of its last section for callers that want them.
  config.i.in         #define USE_HIP @USE_HIP@, and USE_CUDA reported true if python/singa/device.py
                      is to keep its `singa.USE_CUDA` gate unchanged.
"""


def apply(tree, quiet=False):
    """Applies copies and edits to `tree`; returns the list of files written."""
    planned = []
    for rel, fn in EDITS:
        path = os.path.join(tree, rel)
        if not os.path.exists(path):
            raise EditError("missing file in the tree: " + rel)
        with open(path) as f:
            old = f.read()
        new = fn(old)
        if new != old:
            planned.append((path, new))
    written = []
    for path, new in planned:   # nothing is written unless every edit succeeded
        with open(path, "w") as f:
            f.write(new)
        written.append(path)
    for src, dst in COPIES:
        target = os.path.join(tree, dst)
        os.makedirs(os.path.dirname(target), exist_ok=True)
        shutil.copyfile(os.path.join(REPO, src), target)
        written.append(target)
    if not quiet:
        for w in written:
            print("wrote", os.path.relpath(w, tree))
        print(SWIG_NOTES)
    return written


if __name__ == "__main__":
    if len(sys.argv) != 2 or not os.path.isdir(sys.argv[1]):
        sys.exit(__doc__)
    try:
        apply(sys.argv[1])
    except EditError as e:
        sys.exit("not applied: %s" % e)
