"""CPU-only: the C-ABI library loads and exports every symbol the public header declares."""
import ctypes
import os
import re

from __graft_entry__ import ROOT, load_package


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "currennt_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cnt_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_header_symbols():
    capi = load_package().capi
    assert os.path.exists(capi.LIB_PATH), "build the library first: python __graft_entry__.py"
    lib = ctypes.CDLL(capi.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 10
    for n in names:
        assert hasattr(lib, n), "missing export " + n
    # the ctypes binding covers the same set
    assert sorted(capi.exported_symbols()) == names


def test_version_and_argument_errors_without_gpu():
    capi = load_package().capi
    L = capi.lib()
    assert L.cnt_version() >= 1
    # argument validation happens before any device call
    assert L.cnt_matrix_product(None, None, 1, 1, 1, None, 0, None, 0, 0) == 1
    assert b"null" in L.cnt_last_error()
    assert L.cnt_lstm_weight_count(382, 256, 0) == 655104
    assert L.cnt_lstm_weight_count(512, 512, 1) == 1576448


def test_network_file_syntax_errors_without_gpu():
    """The network file is parsed before any device call: malformed JSON and a missing 'layers' section are
    reported with the parser's message."""
    import ctypes as C

    import pytest

    capi = load_package().capi
    capi.lib()
    for text, what in (('{"layers": [', "JSON error"), ('{"layers": [{"size": 3,}]}', "JSON error"),
                       ('{"weights": {}}', "missing section 'layers'"), ('[1, 2]', "not a JSON object"),
                       ('{"layers": [{"size": 1, "name": "input", "type": "input"}]}', "needs an input layer")):
        h = C.c_void_p()
        with pytest.raises(RuntimeError, match=what):
            capi.check(capi.lib().cnt_network_create(text.encode(), 2, 10, None, C.byref(h)))


def test_truncated_network_files_are_rejected_without_gpu():
    """Every prefix of a valid network file is an error (never a crash): the reader validates as it goes."""
    import ctypes as C
    import json

    capi = load_package().capi
    L = capi.lib()
    doc = {"layers": [{"size": 3, "name": "input", "type": "input"},
                      {"size": 4, "name": "h", "type": "feedforward_tanh", "bias": 1.0},
                      {"size": 4, "name": "s", "type": "skipini", "bias": 1.0},
                      {"size": 4, "name": "post", "type": "sse"}],
           "weights": {"h": {"input": [0.5, -1e-3, 2.0e1], "bias": [1, 2], "internal": []}}}
    text = json.dumps(doc)
    for cut in range(len(text)):
        h = C.c_void_p()
        assert L.cnt_network_create(text[:cut].encode(), 2, 10, None, C.byref(h)) != 0
        assert L.cnt_last_error()
