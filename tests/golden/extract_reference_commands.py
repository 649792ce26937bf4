"""Writes fusilli_amd/bench/reference_commands.txt: the argument lists of every
add_fusilli_benchmark(...) entry of the reference's benchmarks/CMakeLists.txt
(:49-392), one command per line in the format of test_commands.txt.  Entries
the reference has commented out (it disables them for a compiler issue of its
own backend) are kept and marked in their comment line.  Run once in the
container that holds the reference; the output is committed data.

    python tests/golden/extract_reference_commands.py [/root/reference]
"""
import os
import re
import sys


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    src = os.path.join(ref, "benchmarks", "CMakeLists.txt")
    text = open(src).read()
    out = ["# Benchmark commands of the reference's benchmarks/CMakeLists.txt "
           "(add_fusilli_benchmark entries), extracted by "
           "extract_reference_commands.py"]
    # an entry may be commented out line by line with "# "
    pat = re.compile(
        r"^(?P<c>#\s*)?add_fusilli_benchmark\(\s*\n(?P<body>(?:.*\n)*?)^(?:#\s*)?\)",
        re.M)
    for m in pat.finditer(text):
        body = re.sub(r"^#\s?", "", m.group("body"), flags=re.M)
        name = re.search(r"NAME\s+(\S+)", body).group(1)
        args = body.split("ARGS", 1)[1]
        args = " ".join(args.replace('"', "").split())
        out.append("")
        out.append(f"# {name}" + ("  (disabled in the reference)" if m.group("c") else ""))
        out.append(args)
    root = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    with open(os.path.join(root, "fusilli_amd", "bench", "reference_commands.txt"), "w") as f:
        f.write("\n".join(out) + "\n")
    print(f"{(len(out) - 1) // 3} commands")


if __name__ == "__main__":
    main()
