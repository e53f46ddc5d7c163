"""The parts of bench.py's contract that need no GPU: more than one GPU is refused with a message, and nothing that is
committed reads the working folder."""
import re
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr and r.stdout.strip() == ""


def test_committed_python_reads_no_working_files():
    for path in [ROOT / "bench.py", ROOT / "__graft_entry__.py", *ROOT.glob("tests/*.py"), *ROOT.glob("oracle/*.py"),
                 *ROOT.glob("mineru-diffusion_amd/**/*.py")]:
        if path.name == Path(__file__).name:
            continue
        text = path.read_text()
        assert not re.search(r"['\"/]_work[/'\"]", text), f"{path} names the working folder"


def test_product_code_never_imports_the_oracle():
    for path in ROOT.glob("mineru-diffusion_amd/**/*.py"):
        assert not re.search(r"^\s*(import|from)\s+oracle\b", path.read_text(), flags=re.M), f"{path} imports the oracle"
