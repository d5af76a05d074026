"""Runs the C++ test executables of the host API (tests/cpp/*_test.cpp -> tests/cpp/bin/).

host_cpu_test needs no GPU (tokenizer, prompt templates, argument errors); the *_gpu_test executables drive
the engine, sampler, state cache and backend against device memory and are marked gpu.  Each executable
prints one line per case and exits non-zero if any case failed.
"""
import os
import subprocess

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(REPO, "tests", "cpp", "bin")


def _exe(name):
    path = os.path.join(BIN, name)
    if not os.path.exists(path):
        from rwkv_lightning_cuda_amd import build
        if not os.path.exists(build.LIB_PATH):
            build.build_all()
        if not os.path.exists(build.HOST_LIB_PATH):
            build.build_host()
        build.build_host_tests()
    return path


def _run(name, *extra):
    proc = subprocess.run([_exe(name), REPO, *extra], capture_output=True, text=True, timeout=300)
    report = proc.stdout[-4000:] + proc.stderr[-2000:]
    assert proc.returncode == 0, "%s exited with %d:\n%s" % (name, proc.returncode, report)
    assert " 0 failed" in proc.stdout, report
    return proc.stdout


def test_host_cpu():
    out = _run("host_cpu_test")
    assert "ok   tokenizer_round_trips" in out
    assert "ok   prompt_templates" in out
    assert "ok   admission_is_first_come_first_served" in out


def test_host_library_exports_the_api():
    """librwkv_host.so loads without a GPU and defines the classes of include/*.hpp."""
    import ctypes
    from rwkv_lightning_cuda_amd import build
    _exe("host_cpu_test")
    ctypes.CDLL(build.LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    ctypes.CDLL(build.HOST_LIB_PATH)
    syms = subprocess.run(["nm", "-DC", "--defined-only", build.HOST_LIB_PATH], capture_output=True, text=True).stdout
    for needle in ("rwkv7_server::InferenceEngine::batch_generate(",
                   "rwkv7_server::InferenceEngine::batch_generate_stream(",
                   "rwkv7_server::InferenceEngine::generate_from_logits_stream(",
                   "rwkv7_server::InferenceEngine::prefill_prompt(",
                   "rwkv7_server::InferenceEngine::format_openai_prompt(",
                   "rwkv7_server::StateCacheManager::put_state(",
                   "rwkv7_server::StateCacheManager::get_state(",
                   "rwkv7_server::StateCacheManager::delete_state_from_any_level(",
                   "rwkv7_server::PrefillAdmissionController::acquire(",
                   "rwkv7_server::PrefillAdmissionController::snapshot(",
                   "rwkv7_server::ModelBackend::forward_prefill(",
                   "rwkv7_server::ModelBackend::forward_decode(",
                   "rwkv7_server::ModelBackend::copy_state_slice(",
                   "rwkv7_server::ModelBackend::query_prefill_capacity(",
                   "rwkv7_server::TrieTokenizer::encode(",
                   "rwkv7_server::make_sampler_penalties(",
                   "rwkv7_server::sample_batch_repetition_temperature_topk_topp("):
        assert needle in syms, needle


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["sampler_gpu_test", "engine_gpu_test", "state_cache_gpu_test", "backend_gpu_test"])
def test_host_gpu(name, tmp_path):
    extra = [str(tmp_path / "sessions.db")] if name == "state_cache_gpu_test" else []
    _run(name, *extra)


# ---------------------------------------------------------------------------------------- checkpoint reader
def _fixture_module():
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_pth_fixture", os.path.join(REPO, "tests", "golden", "make_pth_fixture.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_checkpoint_reader_cpu():
    """Archive reader (the reference's own test among the cases), scalar conversions over every bit pattern, and the
    committed checkpoint written by torch.save against its manifest - whole-file and on-demand reading."""
    out = _run("pth_cpu_test")
    for case in ("stored_zip_whole_and_on_demand_agree", "zip64_records", "damaged_and_unsupported_archives",
                 "scalar_conversions_over_every_bf16_pattern", "checkpoint_written_by_torch_save", "hostile_pickles"):
        assert "ok   " + case in out


def test_untrusted_input_code_under_sanitizers(tmp_path):
    """The code that reads bytes it did not write - the checkpoint's ZIP directory and pickle, the vocabulary file, prompt
    text - built with g++ -fsanitize=address,undefined (host code only: the sources are compiled into the test
    executables instead of coming from librwkv_host.so) and run over the same cases, among them the damaged pickles
    of pth_cpu_test (cut short, bytes replaced, dimensions blown up).  A read or write outside a buffer, a signed
    overflow or a misaligned access ends the run with a report."""
    from rwkv_lightning_cuda_amd import build
    _exe("host_cpu_test")
    cxx = os.environ.get("CXX", "g++")
    probe = subprocess.run([cxx, "-fsanitize=address,undefined", "-x", "c++", "-", "-o", str(tmp_path / "probe")],
                           input="int main(){return 0;}", capture_output=True, text=True)
    if probe.returncode != 0:
        pytest.skip("this compiler has no sanitizer runtimes: " + probe.stderr[-200:])
    host = os.path.join(REPO, "rwkv_lightning_cuda_amd", "host")
    flags = ["-std=c++17", "-O1", "-g", "-fno-omit-frame-pointer", "-fsanitize=address,undefined",
             "-fno-sanitize-recover=all", "-I" + os.path.join(REPO, "include"), "-I" + os.path.join(REPO, "tests", "cpp")]
    link = ["-L" + build.PKG_DIR, "-lrwkv_hip", "-ldl", "-pthread", "-Wl,-rpath," + build.PKG_DIR]
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=0:abort_on_error=0",
               UBSAN_OPTIONS="print_stacktrace=1")
    for name, sources in (("pth_cpu_test", ["pth_archive.cpp", "pth_tensor.cpp"]),
                          ("host_cpu_test", sorted(f for f in os.listdir(host) if f.endswith(".cpp")))):
        exe = str(tmp_path / (name + "_san"))
        cmd = [cxx] + flags + [os.path.join(REPO, "tests", "cpp", name + ".cpp")] + [os.path.join(host, f) for f in sources] + \
              ["-o", exe] + link
        proc = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
        assert proc.returncode == 0, proc.stderr[-3000:]
        run = subprocess.run([exe, REPO], capture_output=True, text=True, timeout=600, env=env)
        report = run.stdout[-3000:] + run.stderr[-3000:]
        assert run.returncode == 0, "%s under sanitizers exited with %d:\n%s" % (name, run.returncode, report)
        assert " 0 failed" in run.stdout, report
        assert "runtime error" not in run.stderr and "AddressSanitizer" not in run.stderr, report
        if name == "pth_cpu_test":
            assert "ok   hostile_pickles" in run.stdout


@pytest.mark.parametrize("variant", ["ordered_with_metadata", "plain_dict", "many_small_tensors"])
def test_checkpoint_reader_on_fresh_torch_checkpoints(variant, tmp_path):
    """Checkpoints written by this interpreter's torch.save right now (not the committed file): an OrderedDict with
    _metadata, a plain dict, and a few hundred small tensors (memo indices beyond one byte: LONG_BINPUT / LONG_BINGET)."""
    torch = pytest.importorskip("torch")
    import collections
    fx = _fixture_module()
    if variant == "many_small_tensors":
        g = torch.Generator().manual_seed(5)
        sd = collections.OrderedDict(("t.%d" % i, torch.randn((3, 1 + i % 5), generator=g).to(torch.bfloat16)) for i in range(400))
    else:
        sd = fx.state_dict(dict(L=1, C=64, H=1, F=128, V=16, Rw=8, Ra=8, Rg=8, Rv=8), seed=77)
        sd.update(fx.reader_stress_entries())
    pth, manifest = str(tmp_path / "fresh.pth"), str(tmp_path / "fresh.manifest")
    if variant == "plain_dict":
        torch.save(dict(sd), pth)
        fx.write_manifest(manifest, sd)
    else:
        fx.write_checkpoint(pth, manifest, sd, with_metadata=(variant == "ordered_with_metadata"))
    out = _run("pth_cpu_test", pth, manifest)
    assert "ok   checkpoint_written_by_torch_save" in out


def _weights_from_state_dict(sd, dims, orc):
    """The checkpoint's tensors in the layout of rwkv_lightning_cuda_amd.model.synth_weights (numpy fp16), converted
    on the host: bf16 -> fp16 is exact for these values, LoRA matrices transposed, the embedding through ln0 (oracle)."""
    import numpy as np
    import torch

    def bits(t):
        return t.contiguous().view(torch.int16).numpy().astype(np.uint16)

    def f16(name, transpose=False):
        b = bits(sd[name])
        b = b.reshape(b.shape[0], -1) if b.ndim == 2 else b.reshape(1, -1)
        out = orc.bf16_to_f16(b, transpose=transpose)
        return out if sd[name].dim() == 2 else out.reshape(-1)

    w = {"emb_ln0": orc.emb_ln0(bits(sd["emb.weight"]), bits(sd["blocks.0.ln0.weight"]), bits(sd["blocks.0.ln0.bias"])),
         "ln_out_w": f16("ln_out.weight"), "ln_out_b": f16("ln_out.bias"), "head": f16("head.weight"), "layers": []}
    vec = {"ln1_w": "ln1.weight", "ln1_b": "ln1.bias", "ln2_w": "ln2.weight", "ln2_b": "ln2.bias", "x_r": "att.x_r",
           "x_w": "att.x_w", "x_k": "att.x_k", "x_v": "att.x_v", "x_a": "att.x_a", "x_g": "att.x_g", "w0": "att.w0",
           "a0": "att.a0", "v0": "att.v0", "k_k": "att.k_k", "k_a": "att.k_a", "r_k": "att.r_k", "lnx_w": "att.ln_x.weight",
           "lnx_b": "att.ln_x.bias", "ffn_x_k": "ffn.x_k"}
    mats = {"att_r": "att.receptance.weight", "att_k": "att.key.weight", "att_v": "att.value.weight",
            "att_o": "att.output.weight", "ffn_key": "ffn.key.weight", "ffn_value": "ffn.value.weight"}
    for l in range(dims.L):
        p = "blocks.%d." % l
        lw = {k: f16(p + n).reshape(-1) for k, n in vec.items()}
        for k in ("w", "a", "g", "v"):
            lw[k + "1"] = f16(p + "att.%s1" % k, transpose=True)   # [C,R] in the file -> [R,C]
            lw[k + "2"] = f16(p + "att.%s2" % k, transpose=True)   # [R,C] in the file -> [C,R]
        for k, n in mats.items():
            lw[k] = f16(p + n)
        w["layers"].append(lw)
    return w


@pytest.mark.gpu
def test_checkpoint_backend_gpu(tmp_path, gpu, orc):
    """ModelBackend("<file>.pth") end to end: whole-file and on-demand loading agree bitwise, the w8 suffix
    quantises on load, load errors - and its logits for a fixed prompt against two other routes to the same weights:
    the Python binding fed with host-converted tensors (same kernels: tight), and the CPU oracle (parity bar)."""
    torch = pytest.importorskip("torch")
    import numpy as np
    hip = gpu
    from rwkv_lightning_cuda_amd.model import HipModel, ModelDims, Session, State
    pth = os.path.join(REPO, "tests", "golden", "rwkv7_tiny.pth")
    dump = str(tmp_path / "logits.bin")
    out = _run("pth_backend_gpu_test", pth, dump)
    for case in ("checkpoint_whole_and_on_demand_give_the_same_model", "weight_format_suffix_quantises_on_load", "load_errors"):
        assert "ok   " + case in out

    fx = _fixture_module()
    d = fx.tiny_dims()
    dims = ModelDims(**d)
    sd = torch.load(pth, weights_only=True)   # written by tests/golden/make_pth_fixture.py
    weights = _weights_from_state_dict(sd, dims, orc)
    got = np.fromfile(dump, np.float32).reshape(3, dims.V)
    prompt = np.array([[(3 + 7 * i) % dims.V for i in range(11)]])
    steps = [np.array([[5 % dims.V]]), np.array([[17 % dims.V]])]

    gmodel = HipModel.from_host_weights(dims, weights, hip.FMT_F16)
    sess = Session(gmodel)
    st = State(dims, 1)
    lg = hip.DeviceArray((1, dims.V), np.float32)
    rows = []
    for toks in [prompt] + steps:
        sess.forward(toks, st, lg)
        rows.append(lg.numpy()[0].copy())
    sess.close()
    same_kernels = np.stack(rows)
    # the only difference between the two routes is emb+ln0 (device kernel vs oracle): a few fp16 ulps of the input
    assert np.max(np.abs(got - same_kernels)) <= 2e-2 * np.max(np.abs(same_kernels))

    om = orc.Model(dims, weights, orc.FMT_F16)
    ostate = om.new_state(1)
    orows = [om.forward(toks, ostate)[0] for toks in [prompt] + steps]
    for a, b in zip(got, orows):
        cos = float(np.dot(a, b) / np.sqrt(np.dot(a, a) * np.dot(b, b)))
        assert cos >= 0.9995
        assert int(np.argmax(a)) == int(np.argmax(b))
