"""The example set as a whole (prism_amd/examples): every program passes the perspective check and is printed,
the printed text equals the committed copies under prism_amd/examples/generated (the way the reference keeps
generated/*.cu beside its examples and compares against them in test/test_codegen.py), and the index names
every program the modules define.
"""
from prism_amd import examples
from prism_amd.hipgen import _REGISTRY


def test_fresh_text_equals_the_committed_copies():
    fresh = examples.texts()
    on_disk = {p.name: p.read_text() for p in examples.GENERATED.glob("*.hip")}
    assert sorted(fresh) == sorted(on_disk)
    changed = [name for name in fresh if fresh[name] != on_disk[name]]
    assert not changed, f"regenerate with `python -m prism_amd.examples`: {changed}"


def test_index_names_every_program_of_the_example_modules():
    examples.load()
    defined = {name for name, k in _REGISTRY.items() if getattr(k.fn, "__module__", "").startswith("prism_amd.examples.")}
    assert defined == set(examples.KERNELS) | set(examples.DEVICE_FUNCTIONS)
    for name, (module, block_size, _) in examples.KERNELS.items():
        assert _REGISTRY[name].kind == "global" and _REGISTRY[name].fn.__module__ == f"prism_amd.examples.{module}"
        assert block_size % 64 == 0
    for name, module in examples.DEVICE_FUNCTIONS.items():
        assert _REGISTRY[name].kind == "device" and _REGISTRY[name].fn.__module__ == f"prism_amd.examples.{module}"


def test_write_into_another_directory(tmp_path):
    written = examples.write(str(tmp_path))
    assert len(written) == len(examples.DEVICE_FUNCTIONS) + 2 * len(examples.KERNELS)
    assert (tmp_path / "staged_sgemm_launcher.hip").read_text().count("__syncthreads();") == 2
