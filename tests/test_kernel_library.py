"""The kernel library's interface as far as it can be checked without a GPU: its header, the argument
lists the Python side holds, and what the recorder of step programs knows."""
import ctypes
import re
from pathlib import Path

from flambeau_amd.kernels import library
from flambeau_amd.kernels import tuned  # noqa: F401  (registers the tuned kernels' argument lists)
from flambeau_amd.sampling import device  # noqa: F401

CSRC = Path(library.__file__).resolve().parent.parent / "csrc"


def _declarations():
    """``{name: [argument type texts]}`` of every ``int fl_*(...)`` declared in api.h."""
    text = re.sub(r"//[^\n]*", "", (CSRC / "api.h").read_text())
    out = {}
    for m in re.finditer(r"\bint\s+(fl_\w+)\s*\(([^;]*?)\)\s*;", text, re.S):
        args = [a.strip() for a in m.group(2).replace("\n", " ").split(",")]
        out[m.group(1)] = [] if args == ["void"] else args
    return out


def _ctype_of(arg: str):
    if "*" in arg or arg.startswith("hipStream_t"):
        return library.P
    if arg.startswith("float"):
        return library.F
    if arg.startswith("long"):
        return library.L
    assert arg.startswith("int") or arg.startswith("unsigned"), arg
    return library.I


def test_argument_lists_follow_the_header():
    """Every argument list held on the Python side names a declared function and has its arguments' types
    (a list one argument short or long corrupts the call without any error)."""
    decl = _declarations()
    assert len(decl) > 50
    for name, types in library._SIGNATURES.items():
        assert name in decl, f"{name} is not declared in api.h"
        assert [_ctype_of(a) for a in decl[name]] == list(types), name


def test_every_launch_function_is_recordable():
    """A launch function (one whose last argument is the stream) registers itself with the recorder
    beside its definition; the recorder's own file names no kernel."""
    lib = library.load()
    decl = _declarations()
    launch = [n for n, a in decl.items() if a and a[-1].startswith("hipStream_t")]
    assert len(launch) >= 37
    lib.fl_program_knows.argtypes = [ctypes.c_char_p]
    for name in launch:
        assert lib.fl_program_knows(name.encode()) == len(decl[name]), name
        assert library.recordable(name)
    assert not library.recordable("fl_no_such_kernel") and not library.recordable("fl_attn_prefill_splits")
    program = (CSRC / "program.hip").read_text()
    body = program[program.index("namespace {"):]
    assert not re.search(r"\bfl_(?!program_|set_error|last_error)\w+", body), "program.hip names a kernel"


def test_a_launch_function_from_elsewhere_can_be_registered():
    """``fl_program_register`` takes a trampoline for a function the library has never seen; a program
    then records it by name (here the trampoline is a Python callback that notes what it was given)."""
    lib = library.load()
    seen = []
    proto = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.POINTER(library.FlArg), ctypes.c_void_p)

    def tramp(args, stream):
        seen.append((args[0].i, round(args[1].f, 3), stream))
        return 0 if args[0].i >= 0 else -7
    cb = proto(tramp)
    library._SIGNATURES["toy_launch"] = [library.I, library.F, library.P]
    try:
        library.make_recordable("toy_launch", cb)
        assert library.recordable("toy_launch")
        prog = library.Program()
        prog.append("toy_launch", (5, 0.25, None))
        prog.append("toy_launch", (-1, 1.5, None))
        prog.append("toy_launch", (9, 2.0, None))
        assert len(prog) == 3
        try:
            prog.run(1234)
            raise AssertionError("the failing call did not stop the replay")
        except library.KernelError as e:
            assert "call 1" in str(e)
        assert seen == [(5, 0.25, 1234), (-1, 1.5, 1234)]
    finally:
        del library._SIGNATURES["toy_launch"]


def test_a_function_of_another_library_registered_before_the_first_load_stays_there():
    """A part may give the argument list of its own launch function before anything has loaded the kernel
    library; loading then looks up only its own functions."""
    import subprocess
    import sys
    code = ("import ctypes\n"
            "from flambeau_amd.kernels import library\n"
            "assert library._lib is None\n"
            "library.register_signatures({'getpid': []}, library=ctypes.CDLL(None))\n"
            "library.load()\n"
            "assert library._functions['getpid']() > 0\n"
            "print('ok')\n")
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, cwd=str(CSRC.parent.parent))
    assert r.returncode == 0 and r.stdout.strip() == "ok", r.stderr


def test_the_tiled_attention_s_plan_for_few_tiles():
    """Heads per wave and parts of the keys for a batch's shape (7B head counts, 256 units): a grid of too
    few blocks is filled by parts of the keys while a part keeps a dozen stages, by fewer heads per wave
    where the keys are too few for that; the two numbers come from one plan."""
    def plan(tokens, keys):
        n_tiles = -(-tokens // 64)
        return tuned.attn_prefill_heads(n_tiles, 32, 8, 128, keys), tuned.attn_prefill_splits(n_tiles, 32, 8, 128, keys)
    assert plan(2048, 2048) == (2, 1)               # 512 blocks as it is
    assert plan(1024, 1024) == (1, 1)               # too few keys to split: one head per wave gives the blocks
    assert plan(512, 512) == (1, 1)
    assert plan(512, 8192) == (2, 4) and plan(512, 32768) == (2, 4)
    assert plan(256, 32768) == (2, 8) and plan(64, 32768) == (2, 16)
    assert plan(512, 1536) == (1, 2)
    for tokens in (64, 200, 512, 1000, 3000):
        for keys in (tokens, 2000, 9000, 70000, 262144):
            h, s = plan(tokens, max(keys, tokens))
            assert h in (1, 2) and 1 <= s <= 16
            assert s == 1 or max(keys, tokens) // 64 // s >= 10        # a part keeps its stages


def test_parts_of_k_for_products_of_17_to_64_rows():
    """One round of blocks that fills the chip as far as it goes (256 units): parts = units / blocks rounded
    down, any number; blocks of eight waves only where a block streams half a megabyte or more."""
    parts = lambda n, k: (tuned.gemm_mid_splits(64, n, k), tuned.gemm_mid_splits(64, n, k, 4, 0), tuned.gemm_mid_splits(64, n, k, 8, 0))
    assert parts(4096, 4096) == (4, 4, 4)             # 64 blocks of four waves x 4; eight waves: parts of 8 chunks at least
    assert parts(6144, 4096)[0] == 2                  # 96 blocks x 2 = 192 (x 3 would start a second round)
    assert parts(5120, 4096) == (3, 3, 4)             # 80 blocks x 3 = 240
    assert parts(5120, 32768) == (6, 3, 6)            # 40 blocks of eight waves x 6 = 240: 1.4 MB per block
    assert parts(4096, 14336)[:2] == (4, 4)
    assert parts(5120, 14336) == (6, 3, 6)            # 611 KB per block: eight waves
    assert parts(32768, 4096) == (1, 1, 1) and parts(96, 64) == (1, 1, 1)
    for n in (1000, 2048, 4096, 5120, 6144, 8192, 28672):
        for k in (512, 4096, 14336, 32768):
            for w in (0, 4, 8):
                s = tuned.gemm_mid_splits(64, n, k, w, 0)
                assert 1 <= s <= 32 and (s == 1 or (k // 128) // s >= 4)


def test_which_products_of_9_to_16_rows_leave_the_skinny_kernel():
    """Only the product that adds to the residual stream with a long K (a feed-forward's way down) goes to the
    kernel for 17 to 64 rows early; everything stays with the skinny kernel up to 8 rows."""
    assert not any(tuned.mid_preferred(m, n, k) for m in (1, 8) for n, k in ((5120, 32768), (4096, 14336), (65536, 5120)))
    assert all(tuned.mid_preferred(m, 5120, 32768) for m in (9, 12, 16))
    assert all(tuned.mid_preferred(m, 5120, 14336) for m in (9, 16))
    assert [tuned.mid_preferred(m, 4096, 14336) for m in (9, 12, 13, 16)] == [False, False, True, True]
    assert not tuned.mid_preferred(16, 65536, 5120) and not tuned.mid_preferred(16, 4096, 4096)
    assert not tuned.mid_preferred(16, 5120, 32768 + 8)          # K must be whole steps of 32 for that kernel
