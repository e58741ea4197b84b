"""bench.py's helpers that need no GPU: the traffic figure comes from the committed
summary of the counter runs, and only while that summary was measured on the kernel
sources of this tree."""
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench   # noqa: E402

TRAFFIC = os.path.join(ROOT, 'profiles', 'roialign_cfg2_hbm_traffic.txt')
CONV = os.path.join(ROOT, 'profiles', 'conv2d_cfg5_mfma.txt')


def test_traffic_summary_names_the_kernel_sources_of_this_tree():
    text = open(TRAFFIC).read()
    assert 'kernel sources: ' + bench.kernel_source_digest() in text, (
        'profiles/roialign_cfg2_hbm_traffic.txt was measured on other kernel sources: collect the '
        'FETCH_SIZE / WRITE_SIZE runs again (the file says how)')


def test_every_roialign_summary_names_the_kernel_sources_of_this_tree():
    import glob
    files = sorted(glob.glob(os.path.join(ROOT, 'profiles', 'roialign_*.txt')))
    assert len(files) >= 5
    for f in files:
        assert 'kernel sources: ' + bench.kernel_source_digest() in open(f).read(), (
            os.path.basename(f) + ' was measured on other kernel sources: run its command again')


def test_conv_summary_names_the_kernel_sources_of_this_tree():
    assert 'kernel sources: ' + bench.conv_source_digest() in open(CONV).read(), (
        'profiles/conv2d_cfg5_mfma.txt was measured on other Conv2D kernel sources: collect its runs again '
        '(the file says how)')


def test_traffic_is_read_from_the_summary():
    fwd = bench.measured_traffic(TRAFFIC, 'forward_blocked_kernel')
    bwd = bench.measured_traffic(TRAFFIC, 'backward_blocked_kernel')
    # one launch moves at least the algorithmic bytes of its pass (476 MB) and not several times that
    assert fwd is not None and 4.0e8 < fwd < 1.5e9
    assert bwd is not None and 4.0e8 < bwd < 1.5e9


def test_traffic_of_a_summary_for_other_sources_is_not_quoted(tmp_path):
    stale = tmp_path / 'traffic.txt'
    stale.write_text(open(TRAFFIC).read().replace(bench.kernel_source_digest(), '0' * 16))
    assert bench.measured_traffic(str(stale), 'backward_blocked_kernel') is None
    assert bench.measured_traffic(str(tmp_path / 'absent.txt'), 'backward_blocked_kernel') is None
