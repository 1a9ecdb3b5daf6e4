"""Builds zero-tvm_amd/js/ztvm_napi.node: the N-API addon over libztvm_hip.so (g++, no node-gyp needed)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "ztvm_napi.node")
NODE_INCLUDE = os.environ.get("NODE_INCLUDE", "/usr/include/node")


def build():
    if not os.path.exists(os.path.join(NODE_INCLUDE, "node_api.h")):
        raise RuntimeError("node_api.h not found under %s" % NODE_INCLUDE)
    libdir = os.path.join(os.path.dirname(HERE), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-DNAPI_VERSION=6", "-DNODE_GYP_MODULE_NAME=ztvm_napi",
           "-I", NODE_INCLUDE, os.path.join(HERE, "addon.cc"), "-o", OUT, "-L", libdir, "-lztvm_hip",
           "-Wl,-rpath,$ORIGIN/../lib"]
    subprocess.check_call(cmd)
    return OUT


if __name__ == "__main__":
    print(build())
