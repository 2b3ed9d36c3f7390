"""bench.py's contract that can be checked without a GPU: more than one GPU is refused with a message,
and the byte counts behind `roofline.achieved` are the wire format's (a K page-head is 32 (D + D_BOOSTED)
bytes of planes, D bytes of slot map and D (scale, zero) pairs; a V page-head 32 D bytes and 128 pairs;
kitty/kvcache/utils_kv_per_layer.py:33-59 of the reference)."""
import subprocess
import sys
import types
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))
import bench  # noqa: E402


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one-GPU" in r.stderr and not r.stdout.strip()


def _layer(D, DB, pk, pv, sink=32, qk=96, qv=96, lv=128):
    return types.SimpleNamespace(D=D, D_BOOSTED=DB, PageCount_K=pk, PageCount_V=pv, Sink_Count=sink,
                                 Q_Buffer_Count_K=qk, Q_Buffer_Count_V=qv, Local_Count_V=lv)


def test_algorithmic_bytes_of_config1():
    total, packed = bench.algorithmic_bytes(16, 32, 8, _layer(128, 32, 255, 254))
    assert packed == 16 * 8 * (5760 * 255 + 4608 * 254) == 337_821_696
    assert total == 350_666_752          # the figure the profiles and the roofline use


def test_algorithmic_bytes_follow_the_head_dimension():
    for D in (64, 256):
        DB = D // 4
        total, packed = bench.algorithmic_bytes(2, 8, 2, _layer(D, DB, 3, 2))
        k_page = 32 * (D + DB) + D + 4 * D
        v_page = 32 * D + 4 * 128
        assert packed == 2 * 2 * (3 * k_page + 2 * v_page)
        assert total == packed + 2 * 2 * (2 * D) * (2 * 32 + 96 + 96 + 128) + 2 * (2 * 8 * D * 2)
