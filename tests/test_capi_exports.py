"""Host-side checks that need no GPU: the C-ABI library loads, exports every symbol
include/pink_hip.h declares, validates arguments like the reference's constructors,
and its host-only helpers agree with the oracle."""
import os
import re

import numpy as np
import pytest

import oracle as O
from pink_amd import capi, synthetic

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "pink_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)          # declarations only, not comments
    declared = set(re.findall(r"\b(pink_hip_[a-z_]+)\s*\(", header))
    assert declared, "no declarations found"
    L = capi.lib()
    for name in sorted(declared):
        assert hasattr(L, name), "libpink_hip.so does not export " + name
    assert declared == set(capi.EXPORTS)
    version = int(re.search(r"#define\s+PINK_HIP_ABI_VERSION\s+(\d+)", open(os.path.join(ROOT, "include", "pink_hip.h")).read()).group(1))
    assert L.pink_hip_abi_version() == version == 2


@pytest.mark.parametrize("num_rot", [0, 3, 90, 6])
def test_num_rot_validation(num_rot):
    # test/SelfOrganizingMapTest/Trainer.cpp:22-47 : 0, 3, 90 throw; 1, 4, 720 do not
    with pytest.raises(capi.PinkError) as e:
        capi.Context(4, 1, 2, 2, num_rot, False, 2)
    assert "Number of rotations must be 1 or larger then 1 and divisible by 4" in str(e.value)
    assert e.value.status == -1


def test_ed_dim_validation():
    # SelfOrganizingMapLib/Mapper.h:63-66
    with pytest.raises(capi.PinkError) as e:
        capi.Context(4, 1, 8, 4, 4, False, 5)
    assert "Euclidean distance dimension larger than neuron dimension" in str(e.value)


def test_interpolation_validation():
    with pytest.raises(capi.PinkError) as e:
        capi.Context(4, 1, 8, 4, 8, False, 4, interpolation=capi.NEAREST_NEIGHBOR)
    assert "unknown interpolation" in str(e.value)


def test_update_factors_match_oracle():
    for w in synthetic.WORKLOADS.values():
        a = synthetic.update_factors(w)
        b = O.update_factors(w.layout, w.som_dims, w.functor, w.sigma, w.damping, -1.0)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), w.name
    a = capi.make_update_factors(capi.CARTESIAN, [3, 4], capi.STEP, 1.0, 0.0, 1.5)
    b = O.update_factors(O.CARTESIAN, [3, 4], O.STEP, 1.0, 0.0, 1.5)
    assert np.array_equal(a, b)
    assert capi.som_size(capi.HEXAGONAL, [21, 21]) == 331
    assert capi.som_size(capi.HEXAGONAL, [4, 4]) == 0       # HexagonalLayout.h:40 : odd dimensions only


def test_initial_som_matches_filler():
    w = synthetic.WORKLOADS["cfg4"]
    som = synthetic.initial_som(w, 1234)
    assert np.array_equal(som.ravel(), O.fill_random_uniform(som.size, 1234))


def test_synthetic_images_are_deterministic_and_in_range():
    for w in synthetic.WORKLOADS.values():
        a = synthetic.images(w, 5)
        b = synthetic.images(w, 5)
        assert np.array_equal(a, b)
        assert a.min() >= 0.0 and a.max() <= 1.0 and a.dtype == np.float32


def test_generated_assembly_loop_is_current():
    # pink_amd/csrc/ssd_steps.inc is what gen_ssd_steps.py writes: the build compiles the committed file
    import subprocess, sys
    csrc = os.path.join(ROOT, "pink_amd", "csrc")
    out = subprocess.run([sys.executable, os.path.join(csrc, "gen_ssd_steps.py")], check=True, capture_output=True, text=True).stdout
    with open(os.path.join(csrc, "ssd_steps.inc")) as f:
        assert f.read() == out
