"""Host code under AddressSanitizer + UndefinedBehaviorSanitizer (CPU only, no GPU code involved).

`tests/host_fuzz.cpp` is compiled together with the GraphDef loader and the tokenizer (`csrc/host/Graph.cpp`,
`csrc/host/tokenization.cpp`: the two parts of the library that read files and text a caller hands in) and fed
damaged model files and arbitrary byte strings.  A read or write out of bounds, a leak, signed overflow, a
misaligned access or an exception other than the documented std::invalid_argument fails the test."""
import json
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
HOST = os.path.join(ROOT, "cubert_amd", "csrc", "host")


def _clang():
    for cand in ("/opt/rocm/llvm/bin/clang++", shutil.which("clang++")):
        if cand and os.path.exists(cand):
            return cand
    return None


@pytest.mark.timeout(600)
def test_graph_loader_and_tokenizer_under_sanitizers(tmp_path):
    clang = _clang()
    if clang is None:
        pytest.skip("no clang++ with sanitizer runtimes")
    exe = str(tmp_path / "host_fuzz")
    # (-asan-globals=0: the instrumentation of merged string literals trips the sanitizer's own ODR check at start-up
    # with this toolchain; heap and stack are what the driver is after)
    cmd = [clang, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
           "-mllvm", "-asan-globals=0", "-fno-omit-frame-pointer",
           "-I" + os.path.join(ROOT, "include"), "-I" + HOST, "-I" + os.path.join(ROOT, "cubert_amd", "csrc", "kernels"),
           os.path.join(HERE, "host_fuzz.cpp"), os.path.join(HOST, "Graph.cpp"), os.path.join(HOST, "tokenization.cpp"),
           "-o", exe]
    built = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if built.returncode != 0 and "sanitizer" in built.stdout.lower() and "not supported" in built.stdout.lower():
        pytest.skip("sanitizer runtimes not installed: " + built.stdout[-300:])
    assert built.returncode == 0, built.stdout[-3000:]

    vectors = json.load(open(os.path.join(HERE, "golden", "tokenization_vectors.json"), encoding="utf8"))
    vocab = tmp_path / "vocab.txt"
    vocab.write_text("\n".join(vectors["test_vocab"]) + "\n", encoding="utf8")
    for seed in (1, 2):
        run = subprocess.run([exe, os.path.join(HERE, "golden", "tf_style_graphdef.pb"), str(vocab),
                              str(tmp_path / "damaged.pb"), "3000", str(seed)],
                             stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
        assert run.returncode == 0, run.stdout[-4000:]
        assert "host_fuzz ok" in run.stdout, run.stdout[-2000:]
        # the damage is not all refused at the first byte: a good share of the files still load
        line = [l for l in run.stdout.splitlines() if l.startswith("graphdef:")][0]
        loaded = int(line.split("damaged files ")[1].split(" loaded")[0])
        assert loaded > 300, line
