"""Writes the model-file fixtures of tests/golden/model_file/ with the
REFERENCE's own classes: oracle/_ref/ref_model_file (built by `make -C oracle
ref` where the reference checkout is present) writes the example program and
parameters as a meta-version-1 and a meta-version-2 "<name>.nb" file, and
dumps each as text.  The fixtures are data: two small binary files and what
the reference's reader makes of them.

    python tests/golden/make_model_file_golden.py
"""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
TOOL = os.path.join(ROOT, "oracle", "_ref", "ref_model_file")
OUT = os.path.join(ROOT, "tests", "golden", "model_file")


def main():
    if not os.path.exists(TOOL):
        raise SystemExit("oracle/_ref/ref_model_file is not built (needs the reference checkout): make -C oracle ref")
    os.makedirs(OUT, exist_ok=True)
    for meta in (1, 2):
        nb = os.path.join(OUT, "ref_example_v%d.nb" % meta)
        subprocess.run([TOOL, "write-example", nb, str(meta)], check=True)
        dump = subprocess.run([TOOL, "dump", nb], check=True, stdout=subprocess.PIPE).stdout
        with open(os.path.join(OUT, "ref_example_v%d.dump.txt" % meta), "wb") as f:
            f.write(dump)
        print(nb, os.path.getsize(nb), "bytes")


if __name__ == "__main__":
    main()
