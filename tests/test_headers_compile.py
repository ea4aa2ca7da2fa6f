"""The public headers stand on their own: the C ABI is C99, the C++ host layer C++17, both
warning-free under -Wall -Wextra -pedantic with the host compilers (no HIP needed)."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include")


def _syntax_only(compiler, std, source, suffix, tmp_path):
    src = tmp_path / f"tu{suffix}"
    src.write_text(source)
    proc = subprocess.run([compiler, f"-std={std}", "-fsyntax-only", "-Wall", "-Wextra", "-pedantic", "-Werror",
                           f"-I{INCLUDE}", str(src)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout


def test_c_header_is_c99(tmp_path):
    _syntax_only("gcc", "c99", '#include "cubek_quant.h"\n'
                 "int main(void) { cq_scheme s = {0}; cq_tensor t = {0}; (void)t; return (int)sizeof(s) - 12; }\n",
                 ".c", tmp_path)


def test_cpp_host_layer_is_cpp17(tmp_path):
    _syntax_only("g++", "c++17", '#include "cubek_quant.hpp"\n'
                 "int main() {\n"
                 "    using namespace cubek_quant::scheme;\n"
                 "    auto s = QuantScheme::default_().with_value(QuantValue::Q4S).with_level(QuantLevel::block({32}));\n"
                 "    return s.num_quants() == 8 ? 0 : 1;\n"
                 "}\n", ".cpp", tmp_path)
