"""The C-ABI library loads (no GPU needed) and exports every symbol include/nebula_hip.h declares."""
import ctypes as C
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared():
    text = open(os.path.join(ROOT, "include", "nebula_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nbl_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_exported_and_bound():
    from nebula_amd import hip
    names = declared()
    assert len(names) >= 30
    l = hip.lib()
    for n in names:
        assert hasattr(l, n), "library does not export " + n
    assert set(names) == set(hip.SIGNATURES), set(names) ^ set(hip.SIGNATURES)
    assert b"gfx950" in l.nbl_version()


def test_no_device_is_reported_not_crashed():
    from nebula_amd import hip
    l = hip.lib()
    import subprocess, sys
    # creating a context in a child keeps a CPU-only runner safe from any driver noise
    code = ("import ctypes as C, sys; sys.path.insert(0, %r); from nebula_amd import hip; l = hip.lib(); p = C.c_void_p(); "
            "rc = l.nbl_ctx_create(0, C.byref(p)); print(rc, l.nbl_last_error(None).decode())") % ROOT
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    rc = int(out.stdout.split()[0])
    assert rc in (0, -5, -2)          # 0 on a GPU box, NBL_ENODEVICE (or a HIP error) without one
    # pure host helpers work anywhere
    assert l.nbl_pool_out_dim(55, 2, 0) == 27 and l.nbl_pool_out_dim(112, 2, 0) == 56
    assert l.nbl_conv_out_dim(227, 11, 4, 0) == 55 and l.nbl_conv_out_dim(224, 7, 2, 3) == 112
    assert l.nbl_conv2d_num_variants() >= 1
    assert l.nbl_conv2d_variant_name(l.nbl_conv2d_num_variants()) == b"strip" and l.nbl_conv2d_variant_name(-1) is None
    assert l.nbl_conv2d_variant_name(0) == b"128x128"


def test_layers_library_exports_and_reports_missing_device():
    import subprocess, sys
    from nebula_amd import net
    text = open(os.path.join(ROOT, "include", "nebula_layers.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(nbl_net_[a-z0-9_]+)\s*\(", text)))
    l = net.lib()
    for n in names:
        assert hasattr(l, n), "library does not export " + n
    assert set(names) == set(net.SIGNATURES)
    code = ("import sys; sys.path.insert(0, %r); from nebula_amd.net import Network, NetworkError\n"
            "try:\n    Network('[net]\\nbatch=1\\nheight=4\\nwidth=4\\nchannels=1\\n[softmax]\\n'); print('created')\n"
            "except NetworkError as e:\n    print('error:', e)\n") % ROOT
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    assert out.stdout.startswith("created") or "device context" in out.stdout
