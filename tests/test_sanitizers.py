"""AddressSanitizer + UndefinedBehaviorSanitizer builds of the CPU-side C and C++ (the oracle and the host-side
layer framework), run on dry-run networks and small awkward shapes.  Host code only: nothing here touches a GPU."""
import os
import shutil
import subprocess

import numpy as np
import pytest

from nebula_amd import zoo
from nebula_amd.net import Network

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SAN = ["-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer", "-g", "-O1", "-static-libasan"]
ENV = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:halt_on_error=1", UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")

pytestmark = pytest.mark.skipif(shutil.which("gcc") is None or shutil.which("g++") is None, reason="needs gcc and g++")


def run(cmd, **kw):
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=600, **kw)
    assert out.returncode == 0, "%s\n--- stdout\n%s\n--- stderr\n%s" % (" ".join(cmd), out.stdout[-3000:], out.stderr[-6000:])
    return out.stdout


def test_oracle_under_asan_ubsan(tmp_path):
    exe = str(tmp_path / "oracle_driver")
    run(["gcc", "-std=c11"] + SAN + ["-pthread", "-fno-fast-math", "-ffp-contract=off", "-I", os.path.join(ROOT, "oracle"),
         "-o", exe, os.path.join(ROOT, "tests", "sanitize", "oracle_driver.c"), os.path.join(ROOT, "oracle", "nebula_oracle.c"),
         "-lm", "-ldl"])
    assert run([exe], env=ENV).strip() == "ok"


@pytest.fixture(scope="module")
def host_driver(tmp_path_factory):
    """The host-side framework compiled with the sanitizers into one executable (it links the uninstrumented HIP
    library for the symbols a dry-run network never calls)."""
    d = tmp_path_factory.mktemp("san")
    exe = str(d / "host_driver")
    host = os.path.join(ROOT, "nebula_amd", "host")
    libdir = os.path.join(ROOT, "nebula_amd", "lib")
    srcs = [os.path.join(host, f) for f in sorted(os.listdir(host)) if f.endswith(".cc")]
    run(["g++", "-std=c++11"] + SAN + ["-D__HIP_PLATFORM_AMD__", "-I", "/opt/rocm/include", "-I", os.path.join(ROOT, "include"),
         "-I", host, "-o", exe, os.path.join(ROOT, "tests", "sanitize", "host_driver.cc")] + srcs +
        ["-L", libdir, "-lnebula_hip", "-L", "/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib"])
    return exe


EXTRA = {
    "mixed": ("[net]\nbatch=2\nheight=19\nwidth=19\nchannels=3\nfuse_shortcut=1\npool_index=1\n"
              "[convolutional]\nbatch_normalize=1\nfilters=8\nsize=3\nstride=1\npadding=1\nactivation=leaky\n"
              "[convolutional]\nfilters=8\nsize=1\nstride=1\npadding=0\nactivation=linear\n[shortcut]\nhops=2\nactivation=relu\n"
              "[maxpool]\nsize=3\nstride=2\n[avgpool]\nsize=2\nstride=2\npadding=0\n[dropout]\nprobability=0.5\n"
              "[connected]\nbatch_normalize=1\noutput=7\nactivation=tanh\n[softmax]\n[cost]\ntype=l2\n"),
    "recurrent": ("[net]\nbatch=3\ninput_size=10\ntime_steps=4\nlast_step_only=1\n[rnn]\nbatch_normalize=1\noutput=12\nactivation=relu\n"
                  "[lstm]\nbatch_normalize=1\noutput=8\nactivation=linear\n[dropout]\nprobability=0.1\n[connected]\noutput=5\nactivation=linear\n[softmax]\n"),
}


# the networks with hundreds of megabytes of connected-layer weights run the same code as the rest and only make the
# instrumented run slow
NETS = [n for n in sorted(zoo.WORKLOADS) if n not in ("vgg16", "mlp", "dbn", "alexnet")] + sorted(EXTRA)


@pytest.mark.parametrize("name", NETS)
def test_host_framework_under_asan_ubsan(host_driver, tmp_path, name):
    cfg = EXTRA[name] if name in EXTRA else zoo.WORKLOADS[name](2)
    with Network(cfg, device=-1) as net:
        floats = sum(f[2] for f in net.weight_layout())
        layers = net.num_layers
    (tmp_path / "network.cfg").write_text(cfg)
    rng = np.random.default_rng(len(name))
    # large nets: a constant-filled stream keeps the file cheap to make; the driver compares it byte for byte anyway
    blob = rng.standard_normal(floats).astype(np.float32) if floats < (1 << 22) else np.full(floats, 0.25, np.float32)
    blob.tofile(str(tmp_path / "in.wgh"))
    out = run([host_driver, str(tmp_path / "network.cfg"), str(tmp_path / "in.wgh"), str(tmp_path / "scratch.wgh")], env=ENV)
    assert out.split() == ["ok", str(layers), str(floats)]
