"""bench.py command line and the rule that the oracle is a checker, never part of the product path."""
import re
import subprocess
import sys
from pathlib import Path

REPO = Path(__file__).resolve().parent.parent


def test_more_than_one_gpu_is_refused():
    proc = subprocess.run([sys.executable, str(REPO / 'bench.py'), '--gpus', '2'], capture_output=True, text=True,
                          timeout=120)
    assert proc.returncode != 0
    assert 'one GPU' in (proc.stderr + proc.stdout)


def test_product_code_never_touches_the_oracle():
    offenders = []
    for path in (REPO / 'cuda-agent_amd').rglob('*'):
        if path.suffix in ('.py', '.hip', '.hpp', '.cpp', '.h', '.sh') and path.is_file():
            text = path.read_text(errors='replace')
            if re.search(r'^\s*(from|import)\s+oracle\b', text, flags=re.M) or 'oracle/' in text:
                offenders.append(str(path.relative_to(REPO)))
    assert not offenders, offenders


def test_bench_uses_the_oracle_only_for_the_cpu_baseline():
    src = (REPO / 'bench.py').read_text()
    lines = src.splitlines()
    for i, line in enumerate(lines):
        if re.search(r'\bfrom oracle import\b|\bimport oracle\b', line):
            # the import sits inside a function; the function's use of it is behind `cpu_baseline`
            # (or is the cpu baseline helper itself)
            head = next(l for l in reversed(lines[:i]) if l.startswith('def '))
            assert 'cpu_baseline' in head or head.startswith('def moe_cpu_baseline'), (i + 1, head)


def test_no_committed_file_reads_the_scratch_folder():
    offenders = []
    for path in list(REPO.glob('*.py')) + list((REPO / 'tests').rglob('*.py')) + \
            list((REPO / 'cuda-agent_amd').rglob('*.py')) + list((REPO / 'oracle').rglob('*.py')):
        if path.name == 'test_bench_cli.py':
            continue
        if re.search(r'''["'/]_work["'/]''', path.read_text(errors='replace')):
            offenders.append(str(path.relative_to(REPO)))
    assert not offenders, offenders


def test_measured_constants_of_bench_are_the_figures_of_the_committed_profiles():
    """bench.py carries HBM traffic and matrix-pipe occupancy as constants taken from rocprofv3 counter runs;
    each must be a figure of the committed summary it names, so that one cannot change without the other."""
    import ast
    src = (REPO / 'bench.py').read_text()
    tree = ast.parse(src)
    values = {}
    for node in tree.body:
        if isinstance(node, ast.Assign) and getattr(node.targets[0], 'id', '') in ('MEASURED_TRAFFIC', 'MEASURED_MFMA'):
            values[node.targets[0].id] = ast.literal_eval(ast.unparse(node.value).replace('dict(', 'dict(')) \
                if node.targets[0].id == 'MEASURED_TRAFFIC' else ast.unparse(node.value)
    traffic_md = (REPO / 'profiles' / 'all_workloads_hbm_traffic_pmc.md').read_text()
    # the fourth column of the summary's table ("HBM bytes (scaled)") of some row, not just any place in the file
    hbm_bytes = set()
    for row in traffic_md.splitlines():
        cells = [c.strip() for c in row.split('|')]
        if row.startswith('|') and len(cells) >= 6 and re.fullmatch(r'[\d ]+', cells[4] or 'x'):
            hbm_bytes.add(int(cells[4].replace(' ', '')))
    assert len(hbm_bytes) >= 8
    for name, nbytes in values['MEASURED_TRAFFIC'].items():
        assert nbytes in hbm_bytes, (name, nbytes)
    counters_md = (REPO / 'profiles' / 'moe_prefill_mla_matrix_core_counters_pmc.md').read_text()
    for figure in re.findall(r'mfma_busy(?:_down)?=([0-9.]+)', values['MEASURED_MFMA']):
        assert figure in counters_md, figure
