"""TEST INFRASTRUCTURE.  Builds tests/lite_stub/_build/libprovider_harness.so: the MindSpore Lite provider
(mindspore_amd/provider/mi355x_provider.cc) compiled against the stand-in Lite API of this directory, together with a
harness that plays the scheduler, linked against libmi355x_int8.so."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
OUT = os.path.join(HERE, "_build", "libprovider_harness.so")
REFERENCE = "/root/reference"


def build_harness():
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    subprocess.check_call([
        "g++", "-std=c++17", "-O1", "-fPIC", "-shared", "-pthread", "-Wall", "-I" + HERE, "-I" + os.path.join(ROOT, "include"),
        os.path.join(HERE, "harness.cc"), "-L" + os.path.join(ROOT, "mindspore_amd"), "-lmi355x_int8",
        "-Wl,-rpath,$ORIGIN/../../../mindspore_amd", "-o", OUT])
    return OUT


def syntax_check_against_reference_headers():
    """The provider against the reference's own public headers (include/api, mindspore/lite/include, mindapi); only the
    flatc-generated schema header is the stand-in.  Returns compiler output ('' = clean) or None without the tree."""
    if not os.path.isdir(os.path.join(REFERENCE, "include", "api")):
        return None
    out = ""
    for src in ("mi355x_provider.cc", "mi355x_allocator.h"):
        cmd = ["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-I" + REFERENCE,
               "-I" + os.path.join(REFERENCE, "mindspore", "lite"), "-I" + os.path.join(REFERENCE, "mindspore", "core"),
               "-I" + HERE, "-I" + os.path.join(ROOT, "include"), "-x", "c++",
               os.path.join(ROOT, "mindspore_amd", "provider", src)]
        p = subprocess.run(cmd, capture_output=True, text=True)
        if p.returncode != 0 or p.stderr.strip():
            out += (p.stdout + p.stderr).strip() + "\n"
    return out.strip()


if __name__ == "__main__":
    print(build_harness())
    print("reference headers:", repr(syntax_check_against_reference_headers()))
