"""Type-checks the OpenVINO plugin shim against the developer headers of an OpenVINO source tree.

The shim needs libopenvino to link and run, which this repository does not ship; where a source tree is
present (OPENVINO_SRC, default /root/reference) this script runs `g++ -fsyntax-only` over
ovfcc_plugin.cpp so that every override matches the interface it claims to implement.  Without a tree it
does nothing.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))


def main() -> int:
    src = os.environ.get("OPENVINO_SRC", "/root/reference")
    marker = os.path.join(src, "src", "inference", "dev_api", "openvino", "runtime", "iplugin.hpp")
    if not os.path.exists(marker):
        print("check_syntax: no OpenVINO source tree, skipped")
        return 0
    inc = ["src/core/include", "src/core/dev_api", "src/inference/include", "src/inference/dev_api",
           "src/common/transformations/include", "src/common/util/include", "src/common/itt/include"]
    cmd = ["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-I" + os.path.join(ROOT, "include")]
    cmd += ["-I" + os.path.join(src, i) for i in inc]
    cmd.append(os.path.join(HERE, "ovfcc_plugin.cpp"))
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        print(res.stderr[-6000:])
        return 1
    print("check_syntax: ovfcc_plugin.cpp type-checks against", src)
    return 0


if __name__ == "__main__":
    sys.exit(main())
