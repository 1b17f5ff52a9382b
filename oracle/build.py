"""Build oracle/_build/liboracle.so from the C restatements (test infrastructure)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "_build", "liboracle.so")
SOURCES = ["we_oracle.c", "we_aniso_oracle.c", "geo_attn_oracle.c"]


def build(force: bool = True) -> str:
    if not force and os.path.exists(LIB):
        return LIB
    os.makedirs(os.path.join(HERE, "_build"), exist_ok=True)
    cmd = ["gcc", "-O2", "-fPIC", "-fopenmp", "-fno-fast-math", "-ffp-contract=off",
           "-Wall", "-Wextra", "-shared", "-o", LIB] + [os.path.join(HERE, s) for s in SOURCES] + ["-lm"]
    subprocess.run(cmd, check=True, cwd=HERE)
    return LIB


if __name__ == "__main__":
    print(build())
