"""The C++ host layer (pink::Trainer<...,true> / pink::Mapper<...,true> over the C ABI,
pink_amd/host/pink_hip_som.h) through its own test program tests/cpp/test_host.cpp."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "test_host")


def _bin():
    if not os.path.exists(BIN):
        from pink_amd import build
        build.build_host_test()
    return BIN


def test_argument_validation_needs_no_device():
    out = subprocess.run([_bin(), "args"], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stdout + out.stderr


@pytest.mark.gpu
def test_reference_known_answers_through_cpp_classes():
    out = subprocess.run([_bin(), "gpu"], capture_output=True, text=True, timeout=110)
    print(out.stdout, out.stderr, flush=True)
    assert out.returncode == 0, out.stdout + out.stderr


REF = "/root/reference"


@pytest.mark.skipif(not os.path.isdir(os.path.join(REF, "src", "SelfOrganizingMapLib")),
                    reason="reference tree not present")
def test_boundary_compiles_against_the_reference_headers(tmp_path):
    """pink_hip_som.h behind the reference's own Trainer.h / Mapper.h, as a maintainer would build it:
    g++ (no nvcc, so the reference's `true` specialisations are out, Trainer.h:25-31,198,337), the
    classes instantiated with the reference's SOM, Data and layout types.  Compile only: it guards the
    interface (member names, constructor signatures), it pins no result.  Version.h is what the
    reference's CMake writes from Version.h.in (CMakeLists.txt:120-123), here into a temporary folder."""
    template = open(os.path.join(REF, "src", "UtilitiesLib", "Version.h.in")).read()
    (tmp_path / "Version.h").write_text(template.replace("@PROJECT_VERSION@", "0").replace("@GIT_REVISION@", "0"))
    tu = tmp_path / "boundary.cpp"
    tu.write_text('''
#include "SelfOrganizingMapLib/Trainer.h"
#include "SelfOrganizingMapLib/Mapper.h"
#include "pink_hip_som.h"
using namespace pink;
template class pink::Trainer<CartesianLayout<2>, CartesianLayout<2>, float, true>;
template class pink::Trainer<HexagonalLayout, CartesianLayout<3>, float, true>;
template class pink::Mapper<CartesianLayout<2>, CartesianLayout<2>, float, true>;
template class pink::Mapper<HexagonalLayout, CartesianLayout<3>, float, true>;
void use(SOM<CartesianLayout<2>, CartesianLayout<2>, float>& som, Data<CartesianLayout<2>, float> const& image)
{
    Trainer<CartesianLayout<2>, CartesianLayout<2>, float, true> trainer(som, GaussianFunctor(1.1f, 0.2f), 0, 360, true,
        -1.0f, Interpolation::BILINEAR, 32, EuclideanDistanceShape::QUADRATIC, 256, DataType::UINT8);
    trainer(image);
    trainer.update_som();
    (void)trainer.get_update_info();
    Mapper<CartesianLayout<2>, CartesianLayout<2>, float, true> mapper(som, 0, 360, true, Interpolation::BILINEAR, 32);
    std::tuple<std::vector<float>, std::vector<uint32_t>> result = mapper(image);
    (void)result;
}
''')
    cmd = [os.environ.get("CXX", "g++"), "-std=c++17", "-fsyntax-only", "-DPINK_USE_HIP", "-I" + str(tmp_path),
           "-I" + os.path.join(REF, "src"), "-I" + os.path.join(ROOT, "include"),
           "-I" + os.path.join(ROOT, "pink_amd", "host"), str(tu)]
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-4000:]
