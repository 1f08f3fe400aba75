"""Host-side logic that needs no GPU: dtype tables, meta state machine, hooks, model-state flattening,
error behaviour, and that the C-ABI library loads and exports every declared symbol."""

import ctypes
import itertools
import json
import os
import re

import pytest
import torch

import msamp
from msamp import _backend
from msamp.common.dtype import Dtypes, Floating
from msamp.common.tensor import HookManager, ScalingMeta, ScalingTensor, TypeCast
from msamp.nn import FP8Linear, LinearReplacer, ScalingParameter, model_state
from msamp.nn.state import ModelState
from msamp.operators.gemm import Gemm

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = json.load(open(os.path.join(ROOT, 'tests', 'golden', 'reference_kats.json')))


def test_fp_max_table():
    k = GOLDEN['fp_max']
    assert Floating.qfp_max[Dtypes.kfloat8_e4m3] == k['e4m3']
    assert Floating.qfp_max[Dtypes.kfloat8_e5m2] == k['e5m2']
    assert Floating.qfp_max[Dtypes.kfloat16] == k['fp16']
    assert Floating.fp_maxs[torch.uint8] == k['e4m3'] and Floating.fp_maxs[torch.int8] == k['e5m2']
    assert Floating.qfp_max[Dtypes.kfloat32] == torch.finfo(torch.float32).max
    assert Floating.qfp_max[Dtypes.kbfloat16] == torch.finfo(torch.bfloat16).max


def test_dtypes():
    assert Dtypes.is_fp8_qtype(Dtypes.kfloat8_e4m3) and Dtypes.is_fp8_qtype(Dtypes.kfloat8_e5m2)
    assert not Dtypes.is_fp8_qtype(Dtypes.kfloat16)
    assert Dtypes.get_dtype_from_qtype(Dtypes.kfloat8_e4m3) == torch.uint8
    assert Dtypes.get_dtype_from_qtype(Dtypes.kfloat8_e5m2) == torch.uint8
    assert Dtypes.get_dtype_from_qtype(Dtypes.kbfloat16) == torch.bfloat16
    assert Dtypes.dtype_to_qtype[torch.int8] == Dtypes.kfloat8_e5m2
    assert [int(q) for q in (Dtypes.kfloat32, Dtypes.kfloat16, Dtypes.kbfloat16, Dtypes.kfloat8_e4m3, Dtypes.kfloat8_e5m2)] \
        == [_backend.DT_F32, _backend.DT_F16, _backend.DT_BF16, _backend.DT_E4M3, _backend.DT_E5M2]
    assert torch.randn(2).qtype == Dtypes.kfloat32


def test_warmup_truth_table():
    for c in GOLDEN['warmup_truth_table']['cases']:
        meta = ScalingMeta(Dtypes.kfloat8_e4m3, window_size=c['window'], device='cpu')
        for _ in range(c['counter']):
            meta.amax_counter += 1
        assert bool(meta.is_warmup()) == c['warmup']
        assert meta.is_in_time_scaling() == c['in_time']


def test_in_time_scaling_flag_and_context():
    meta = ScalingMeta(Dtypes.kfloat8_e4m3, device='cpu')
    assert meta.is_in_time_scaling()
    with ScalingMeta.in_time_scaling_context(False):
        assert not meta.is_in_time_scaling()
        with ScalingMeta.in_time_scaling_context(True):
            assert meta.is_in_time_scaling()
        assert not meta.is_in_time_scaling()
    assert meta.is_in_time_scaling() and ScalingMeta.in_time_scaling


def test_meta_copy_clone():
    a = ScalingMeta(Dtypes.kfloat8_e4m3, window_size=4, device='cpu')
    a.scale.fill_(8)
    a.amax[1] = 3
    a.amax_counter += 2
    b = a.clone()
    assert b is not a and b.scale.item() == 8 and b.amax[1].item() == 3 and b.amax_counter.item() == 2
    b.scale.fill_(2)
    assert a.scale.item() == 8
    c = ScalingMeta(Dtypes.kfloat8_e5m2, window_size=4, device='cpu')
    c.copy_(a)
    assert c.qtype == Dtypes.kfloat8_e4m3 and c.scale.item() == 8 and c.amax_counter.item() == 2


def test_hook_manager():
    seen = []
    hm = HookManager()
    h1 = hm.register_hook(lambda _, inp, out: seen.append((inp[0], out)))
    h2 = hm.register_hook(lambda _, inp, out: seen.append((inp[0], out)))
    x = torch.randn(2, 3)
    hm(x)
    assert len(seen) == 2 and all(i is x and o is x for i, o in seen)
    h1.remove()
    h2.remove()
    seen.clear()
    hm(x)
    assert not seen


def test_round2times():
    for value, base, expected in GOLDEN['round2times']['cases']:
        assert Gemm._round2times(value, base) == expected


def test_scaling_tensor_type_checks_and_scale_only_ops():
    meta = ScalingMeta(Dtypes.kfloat8_e4m3, device='cpu')
    with pytest.raises(TypeError):
        ScalingTensor(torch.zeros(4, dtype=torch.float16), meta)
    st = ScalingTensor(torch.zeros(4, dtype=torch.uint8), meta)
    st.mul_(2.0)
    assert meta.scale_inv.item() == 2.0
    st.div_(torch.tensor([4.0]))
    assert meta.scale_inv.item() == 0.5
    with pytest.raises(ValueError):
        st.mul_(torch.ones(2))
    assert not st.is_floating_point() and not torch.is_floating_point(st)
    assert torch.zeros_like(st).dtype == torch.uint8
    assert st.shape == (4, ) and st.numel() == 4 and len(st) == 4 and st.is_leaf and st.grad_fn is None
    assert st.isnan().sum() == 0
    st.value[1] = 127
    assert st.isnan().tolist() == [False, True, False, False]
    assert (ScalingTensor(torch.tensor([0x85], dtype=torch.uint8), meta).abs().value == 5).all()
    with pytest.raises(TypeError):
        st.copy_(torch.zeros(4))
    with pytest.raises(TypeError):
        st.to(torch.int32)
    with pytest.raises(TypeError):
        st.to(torch.float32, torch.float16)


def test_has_inf_or_nan_and_amp_unscale_on_cpu():
    meta = ScalingMeta(Dtypes.kfloat8_e4m3, device='cpu')
    st = ScalingTensor(torch.zeros(4, dtype=torch.uint8), meta)
    assert not st.has_inf_or_nan()
    found = torch.zeros(1)
    plain = torch.ones(3)
    torch._amp_foreach_non_finite_check_and_unscale_([plain], found, torch.tensor(0.5))
    assert plain.tolist() == [0.5] * 3 and found.item() == 0
    meta.amax[0] = float('inf')
    assert st.has_inf_or_nan()


def test_compute_paths_refuse_cpu_tensors():
    meta = ScalingMeta(Dtypes.kfloat8_e4m3, device='cpu')
    with pytest.raises(ValueError):
        TypeCast.cast_to_fp8(torch.randn(4), meta)
    with pytest.raises(ValueError):
        TypeCast.cast_from_fp8(torch.zeros(4, dtype=torch.uint8), meta, Dtypes.kfloat32)
    with pytest.raises(ValueError):
        _backend.fp8_transpose(torch.zeros(4, 4, dtype=torch.uint8))


def test_model_state_flatten_and_check_on_cpu():
    state = ModelState()
    model = torch.nn.Sequential(FP8Linear(4, 8), torch.nn.ReLU(), FP8Linear(8, 2))
    for m in model:
        if isinstance(m, FP8Linear):    # keep this test on the CPU whatever the box
            for meta in m.scaling_metas.values():
                meta.cpu()
    state.register_scaling_metas(model)
    flat = state.flattened_scaling_metas
    assert set(flat) == {'input', 'wgrad', 'ograd'}
    assert flat['input']['amaxs'].shape == (2, 16) and flat['wgrad']['amaxs'].shape == (2, 1)
    assert flat['ograd']['qtype'] == Dtypes.kfloat8_e5m2
    first = model[0].scaling_metas['input']
    assert first.locked
    first.amax[0] = 5.0
    first.scale.fill_(3.0)
    first.amax_counter += 1
    assert flat['input']['amaxs'][0, 0].item() == 5.0 and flat['input']['scales'][0].item() == 3.0
    assert flat['input']['amax_counters'].tolist() == [1, 0]
    state.check_metas_in_flat(model[0].scaling_metas)
    first.scale = torch.ones(())
    with pytest.raises(RuntimeError):
        state.check_metas_in_flat(model[0].scaling_metas)
    st = ScalingTensor(torch.zeros(2, dtype=torch.uint8), model[2].scaling_metas['input'])
    with pytest.raises(ValueError):
        st.data = ScalingTensor(torch.zeros(2, dtype=torch.uint8), ScalingMeta(Dtypes.kfloat8_e4m3, device='cpu'))


def test_fp8linear_structure_and_replacer_attr_compare():
    lin = FP8Linear(4, 8, use_bias=False)
    assert isinstance(lin.weight, ScalingParameter) and lin.bias is None
    assert [n for n, _ in lin.named_parameters()] == ['weight']
    assert lin.weight.dtype == torch.float16 and lin.weight._scaling_metas is lin.scaling_metas
    assert lin.scaling_metas['input'].window_size == 16 and lin.scaling_metas['wgrad'].window_size == 1
    assert lin.half() is lin and lin.weight.dtype == torch.float16
    a, b = LinearReplacer._compare_attrs(type(torch.nn.Linear(1, 1)), lin)
    assert 'scaling_metas' in b


def test_initialize_argument_checks():
    with pytest.raises(ValueError):
        msamp.initialize(object())
    with pytest.raises(ValueError):
        msamp.initialize(torch.nn.Linear(2, 2), opt_level='O3')
    model = torch.nn.Linear(2, 2)
    with pytest.raises(ValueError):
        msamp.initialize(model, torch.optim.SGD(model.parameters(), lr=0.1))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, 'include', 'msamp_hip.h')).read()
    declared = set(re.findall(r'\b(msamp_[a-z0-9_]+)\s*\(', header))
    assert declared == set(_backend.EXPORTED_SYMBOLS), declared ^ set(_backend.EXPORTED_SYMBOLS)
    lib = ctypes.CDLL(_backend.library_path())
    for name in declared:
        assert hasattr(lib, name), name
    assert _backend.load().msamp_hip_version() >= 100
    assert _backend.load().msamp_last_error() is not None


def test_adamw_descriptor_layout_matches_header():
    header = open(os.path.join(ROOT, 'include', 'msamp_hip.h')).read()
    body = header[header.index('typedef struct msamp_adamw_tensor {'):header.index('} msamp_adamw_tensor;')]
    n_ptr = len(re.findall(r'\*\s*\w+;', body))
    assert n_ptr == 14
    assert 8 * n_ptr + 8 + 12 + 12 + 8 == 8 * _backend.ADAMW_DESC_WORDS
    assert int(re.search(r'#define MSAMP_ADAMW_CHUNK (\d+)', header).group(1)) == _backend.ADAMW_CHUNK
    assert int(re.search(r'#define MSAMP_WORKSPACE_BYTES (\d+)', header).group(1)) == _backend.WORKSPACE_BYTES


def test_scale_group_layout_matches_header():
    import ctypes
    header = open(os.path.join(ROOT, 'include', 'msamp_hip.h')).read()
    body = header[header.index('typedef struct msamp_scale_group {'):header.index('} msamp_scale_group;')]
    fields = re.findall(r'(\w+);', body)
    assert fields == [name for name, _ in _backend._ScaleGroup._fields_]
    assert ctypes.sizeof(_backend._ScaleGroup) == 4 * 8 + 4 * 4
    assert int(re.search(r'#define MSAMP_MAX_SCALE_GROUPS (\d+)', header).group(1)) == _backend.MAX_SCALE_GROUPS


def test_one_pass_kernels_stay_off_under_a_process_group(monkeypatch):
    """Kernels whose workgroups wait for each other are only asked for when no other rank exists; the answer is kept
    per default process group."""
    import torch.distributed as dist
    from msamp import _backend
    assert _backend._shared_device() is False
    monkeypatch.setattr(_backend, '_default_group', lambda group=object(): group)
    monkeypatch.setattr(dist, 'get_world_size', lambda group=None: 2)
    assert _backend._shared_device() is True
    monkeypatch.setattr(dist, 'get_world_size', lambda group=None: 1)
    assert _backend._shared_device() is True    # same group: not asked again
    monkeypatch.setattr(_backend, '_default_group', lambda group=object(): group)    # another group: asked again
    assert _backend._shared_device() is False
    monkeypatch.setattr(_backend, '_default_group', lambda: None)
    assert _backend._shared_device() is False


def test_chunk_map_rows_and_cache():
    """One (item, chunk) row per BUCKET_CHUNK elements, ragged tails and empty items included; the same sizes
    return the same tensor."""
    from msamp import _backend
    c = _backend.BUCKET_CHUNK
    m = _backend.chunk_map([2 * c + 1, 0, c], 'cpu')
    assert m.dtype == torch.int32
    assert m.tolist() == [[0, 0], [0, 1], [0, 2], [2, 0]]
    assert _backend.chunk_map([2 * c + 1, 0, c], 'cpu') is m
    assert _backend.chunk_map([], 'cpu').shape[0] == 0


GEMM_PAIRS = ((5, 5), (5, 6), (6, 5), (6, 6))    # the four translation units of the Makefile: E4M3 / E5M2 operands


@pytest.fixture(scope='module')
def gemm_assembly(tmp_path_factory):
    """The GEMM kernels of every operand-format pair compiled to assembly, side by side (cross-compiles without a GPU)."""
    import shutil
    import subprocess
    hipcc = shutil.which('hipcc') or '/opt/rocm/bin/hipcc'
    if not os.path.exists(hipcc):
        pytest.skip('no hipcc here')
    src = os.path.join(os.path.dirname(_backend.__file__), '..', 'csrc')
    tmp = tmp_path_factory.mktemp('gemm_asm')
    procs = []
    for xf, yf in GEMM_PAIRS:
        # (each pair is two translation units: everything but the split-wait instantiations, and those)
        for unit, extra in (('inst', []), ('split', ['-DMSAMP_GEMM_SPLIT_UNIT'])):
            out = str(tmp / f'gemm_{unit}_{xf}{yf}.s')
            cmd = [hipcc, '--offload-arch=gfx950', '-O3', '-std=c++17', '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
                   '-Wno-unused-command-line-argument', '-Wno-inline-asm', f'-DMSAMP_XF={xf}', f'-DMSAMP_YF={yf}', *extra,
                   '--cuda-device-only', '-S', '-o', out, os.path.join(src, 'gemm_inst.hip')]
            procs.append(((xf, yf), out, subprocess.Popen(cmd, cwd=src, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
    paths = {}
    for pair, out, proc in procs:
        log = proc.communicate()[0]
        assert proc.returncode == 0, log.decode(errors='replace')[-2000:]
        paths.setdefault(pair, []).append(out)
    return paths


@pytest.mark.parametrize('pair', GEMM_PAIRS)
def test_direct_to_lds_gemm_kernels_leave_the_accumulator_registers_alone(gemm_assembly, pair):
    """The accumulators of fp8_gemm_dma_kernel live in fixed AGPRs behind the compiler's back (inline-assembly MFMAs).
    That holds only while the compiler itself uses no AGPR in those kernels (it would, to spill VGPRs) and no scratch
    memory.  Each pair of operand formats is a translation unit of its own with its own register allocation: look at
    the assembly of all four."""
    kernel, in_asm, found = None, False, {}
    for line in itertools.chain.from_iterable(open(path) for path in gemm_assembly[pair]):
        m = re.match(r'^(_Z\w+):', line)
        if m:
            kernel = m.group(1)
        elif '#ASMSTART' in line:
            in_asm = True
        elif '#ASMEND' in line:
            in_asm = False
        elif kernel and ('fp8_gemm_dma_kernel' in kernel or 'fp8_gemm_dma128_kernel' in kernel):
            c = found.setdefault(kernel, [0, 0, 0])
            if 'v_accvgpr' in line:
                c[0 if in_asm else 1] += 1
            if re.search(r'scratch_(load|store)', line):
                c[2] += 1
    # bf16 / f16 / float outputs, row- and K-major operands, both parities, the fused and the speculative cast; and the
    # kernel with 128 x 128 tiles, which keeps 64 accumulator registers the same way
    small = [k for k in found if 'fp8_gemm_dma128_kernel' in k]
    assert len(found) - len(small) >= 42 and len(small) == 9    # three output types x (row-major, Y K-major, both K-major)
    assert sum('Lb1EEEv' in k for k in found if k not in small) == 6    # the split-wait instantiations: three output types, two parities
    for name, (ours, compilers, scratch) in found.items():
        assert ours >= (320 if name in small else 512) and compilers == 0 and scratch == 0, (name, ours, compilers, scratch)


def test_entry_points_refuse_bad_arguments_before_touching_a_gpu():
    """Argument checks of the entry points run on the host before any HIP call: what they refuse, and the walk registry
    (host data only), can be tried without a GPU."""
    lib = _backend.load()
    err = lambda: lib.msamp_last_error().decode()    # noqa: E731
    # tile-walk registry: walks 0..7, -1 erases, anything else is refused
    assert lib.msamp_fp8_gemm_get_walk(4096, 8192, 1024, 0, 0) == -1
    assert lib.msamp_fp8_gemm_set_walk(4096, 8192, 1024, 0, 0, 2) == 0
    assert lib.msamp_fp8_gemm_get_walk(4096, 8192, 1024, 0, 0) == 2
    assert lib.msamp_fp8_gemm_get_walk(4096, 8192, 1024, 1, 0) == -1 and lib.msamp_fp8_gemm_get_walk(8192, 4096, 1024, 0, 0) == -1
    assert lib.msamp_fp8_gemm_set_walk(4096, 8192, 1024, 0, 0, 8) == -2 and 'walk=8' in err()
    assert lib.msamp_fp8_gemm_get_walk(4096, 8192, 1024, 0, 0) == 2
    assert lib.msamp_fp8_gemm_set_walk(4096, 8192, 1024, 0, 0, -1) == 0
    assert lib.msamp_fp8_gemm_get_walk(4096, 8192, 1024, 0, 0) == -1
    # the AdamW steps for float32 moments and for high-precision parameters
    hyper = (1e-3, 0.9, 0.999, 1e-8, 0.01, 1, 1, 0, 0)
    assert lib.msamp_adamw_f32(None, None, _backend.DT_F32, 0, None, None, *hyper, None) == 0          # nothing to do
    assert lib.msamp_adamw_f32(None, None, _backend.DT_F32, 16, None, None, *hyper, None) == -3 and 'null' in err()
    buf = (ctypes.c_float * 16)()
    p = ctypes.cast(buf, ctypes.c_void_p)
    assert lib.msamp_adamw_f32(p, p, _backend.DT_E4M3, 16, p, p, *hyper, None) == -1 and 'grad dtype' in err()
    assert lib.msamp_adamw_plain_fused(None, 0, None, 0, _backend.DT_F32, _backend.DT_F32, *hyper, 1, None) == 0
    assert lib.msamp_adamw_plain_fused(None, 3, None, 0, _backend.DT_F32, _backend.DT_F32, *hyper, 1, None) == -3
    assert lib.msamp_adamw_plain_fused(p, 3, None, 0, _backend.DT_E5M2, _backend.DT_F32, *hyper, 1, None) == -1
    assert lib.msamp_adamw_plain_fused(p, -1, None, 0, _backend.DT_F32, _backend.DT_F32, *hyper, 1, None) == -2


def test_every_tile_walk_is_a_bijection(tmp_path):
    """The function that maps a workgroup id to its output tile, taken as it stands in the kernel header and compiled for
    the host: for every grid of 1..140 x 1..140 tiles and each of the four walks (groups of rows or of columns, the
    XCD's patch turned or not -- the rules pick one, the timing at first use may pick any) every tile is taken exactly
    once."""
    import subprocess
    src = open(os.path.join(os.path.dirname(os.path.abspath(__file__)), '..', 'ms-amp_amd', 'csrc', 'gemm_kernels.cuh')).read()
    start = src.index('__device__ __forceinline__ void tile_of_id(')
    fn = src[start:src.index('\n}\n', start) + 3]
    prog = '''#include <cstdio>
#include <vector>
#define __device__
#define __forceinline__ inline
''' + fn + '''
int main() {
    long checked = 0;
    for (int tr = 1; tr <= 140; ++tr)
        for (int tc = 1; tc <= 140; ++tc)
            for (int walk = 0; walk < 4; ++walk) {
                std::vector<char> seen(tr * tc, 0);
                for (int id = 0; id < tr * tc; ++id) {
                    int r = -1, c = -1;
                    tile_of_id(id, tr, tc, walk & 1, (walk >> 1) & 1, r, c);
                    if (r < 0 || r >= tr || c < 0 || c >= tc || seen[r * tc + c]) {
                        printf("BAD %d x %d walk %d id %d -> %d %d\\n", tr, tc, walk, id, r, c);
                        return 1;
                    }
                    seen[r * tc + c] = 1;
                }
                ++checked;
            }
    printf("OK %ld\\n", checked);
    return 0;
}
'''
    cpp, exe = tmp_path / 'walk.cpp', tmp_path / 'walk'
    cpp.write_text(prog)
    subprocess.run(['g++', '-O2', '-o', str(exe), str(cpp)], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and out.stdout.strip() == 'OK 78400', out.stdout[-300:]
