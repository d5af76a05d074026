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
