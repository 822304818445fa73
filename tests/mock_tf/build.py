"""Builds the mock TensorFlow host used by the plugin tests (g++, no GPU code)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))


def build():
    out = os.path.join(HERE, "libmock_tf.so")
    subprocess.run(["g++", "-O1", "-g", "-std=c++17", "-fPIC", "-shared", "-Wall", "-I", os.path.join(ROOT, "include"),
                    os.path.join(HERE, "mock_tf.cc"), "-o", out, "-ldl"], check=True)
    arena = os.path.join(HERE, "libarena_test.so")
    subprocess.run(["g++", "-O1", "-g", "-std=c++17", "-fPIC", "-shared", "-Wall",
                    "-I", os.path.join(ROOT, "intel-extension-for-tensorflow_amd", "plugin"),
                    os.path.join(HERE, "arena_test_lib.cc"), "-o", arena], check=True)
    return out


if __name__ == "__main__":
    print(build())
