"""TEST INFRASTRUCTURE.  Builds tests/lite_stub/_build/libprovider_harness.so: the MindSpore Lite provider
(mindspore_amd/provider/mi355x_provider.cc) compiled against the stand-in Lite API of this directory, together with a
harness that plays the scheduler, linked against libmi355x_int8.so."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
OUT = os.path.join(HERE, "_build", "libprovider_harness.so")
REFERENCE = "/root/reference"


# The reference's own kernel registry: three sources that compile against the stand-in API headers of this directory
# (they only store and hand back the creator functors) plus the reference's public registration header.
REAL_REGISTRY_HEADER = os.path.join(REFERENCE, "mindspore", "lite", "include", "registry", "register_kernel.h")
REAL_REGISTRY_SOURCES = [os.path.join(REFERENCE, "mindspore", "lite", "src", p) for p in (
    "registry/register_kernel.cc", "registry/register_kernel_impl.cc", "common/log.cc")]


def real_registry_available():
    return all(os.path.exists(p) for p in [REAL_REGISTRY_HEADER] + REAL_REGISTRY_SOURCES)


def build_harness():
    """With the reference tree present the harness is linked with the reference's own RegisterKernel /
    RegistryKernelImpl (compiled from where they lie); without it, with the stand-in table of
    include/registry/register_kernel.h.  ph_registry_is_real() tells which one a built harness holds."""
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    cmd = ["g++", "-std=c++17", "-O1", "-fPIC", "-shared", "-pthread", "-Wall", "-I" + HERE,
           "-I" + os.path.join(ROOT, "include")]
    sources = [os.path.join(HERE, "harness.cc")]
    if real_registry_available():
        cmd += ["-DPH_REAL_REGISTRY_HEADER=\"%s\"" % REAL_REGISTRY_HEADER, "-I" + os.path.join(REFERENCE, "mindspore", "lite"),
                "-I" + REFERENCE, "-I" + os.path.join(REFERENCE, "mindspore", "core")]
        sources += REAL_REGISTRY_SOURCES
    subprocess.check_call(cmd + sources + ["-L" + os.path.join(ROOT, "mindspore_amd"), "-lmi355x_int8",
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
