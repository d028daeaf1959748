"""CPU checks of the boundary and the host logic: the shared library loads and exports every
entry point include/tunix_hip.h declares (no compute call is made here), the ctypes table covers
the same set with matching arity and struct sizes, argument checking works without a GPU where
it happens before any launch, and the host helpers agree with the oracle / the reference's
literal vectors."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

from oracle import utils_ref as U
from tunix_amd import _lib as L
from tunix_amd import config
from tunix_amd.generate import utils as G

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tunix_hip.h")

DECL = re.compile(r"^(?:int|int64_t|size_t|const char\*)\s+(tnx_[a-z0-9_]+)\s*\(([^;]*)\)\s*;", re.M | re.S)


def _declared():
  text = open(HEADER).read()
  text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
  out = {}
  for m in DECL.finditer(text):
    args = m.group(2).strip()
    n = 0 if args in ("", "void") else len([a for a in args.split(",") if a.strip()])
    out[m.group(1)] = n
  return out


def test_header_declares_the_expected_entry_points():
  d = _declared()
  assert len(d) >= 23
  for name in ("tnx_qlinear_lora", "tnx_gqa_attn", "tnx_qknorm_rope_kvwrite", "tnx_rmsnorm",
               "tnx_lmhead_logp", "tnx_moe_int4_gmm", "tnx_sample_topk", "tnx_grpo_ratio"):
    assert name in d


def test_library_exports_every_declared_symbol():
  assert os.path.exists(L.LIB_PATH), "libtunix_hip.so is not built (run __graft_entry__.build())"
  handle = ctypes.CDLL(L.LIB_PATH)
  for name in _declared():
    assert hasattr(handle, name), f"{name} is declared in include/tunix_hip.h but not exported"
  # and nothing beyond the declared ABI leaks out with the tnx_ prefix (tnx_set_error is the
  # library-internal error setter shared by its translation units)
  nm = subprocess.run(["nm", "-D", "--defined-only", L.LIB_PATH], capture_output=True, text=True).stdout
  exported = {ln.split()[-1] for ln in nm.splitlines() if " T " in ln and ln.split()[-1].startswith("tnx_")}
  assert exported - set(_declared()) <= {"tnx_set_error"}, exported - set(_declared())


def test_ctypes_table_matches_header():
  d = _declared()
  assert set(L.SIGNATURES) == set(d)
  for name, (_, args) in L.SIGNATURES.items():
    assert len(args) == d[name], f"{name}: header has {d[name]} parameters, ctypes table {len(args)}"


def test_version_and_argument_errors_without_gpu():
  lib = L.lib()
  # the library, the header and the ctypes binding name one and the same ABI version
  hdr = open(HEADER).read()
  major = int(re.search(r"#define TNX_ABI_VERSION_MAJOR (\d+)", hdr).group(1))
  minor = int(re.search(r"#define TNX_ABI_VERSION_MINOR (\d+)", hdr).group(1))
  assert lib.tnx_version() == (major << 16) | minor
  assert L.ABI_VERSION == (major, minor)
  cb, sb = ctypes.c_size_t(), ctypes.c_size_t()
  assert lib.tnx_qw_sizes(4096, 4096, 64, ctypes.byref(cb), ctypes.byref(sb)) == 0
  assert cb.value == 4096 * 4096 // 2
  assert sb.value == (4096 // 16) * (4096 // 128) * 2 * 16 * 2 + 16
  rc = lib.tnx_qw_sizes(100, 4096, 64, ctypes.byref(cb), ctypes.byref(sb))
  assert rc == -22 and b"128" in lib.tnx_last_error()
  with pytest.raises(ValueError, match="128"):
    L.check(rc, "qw_sizes")
  assert lib.tnx_qw_sizes(4096, 4096, 48, None, None) == -22
  assert lib.tnx_lmhead_nblocks(128256) > 0


def test_struct_layouts_match_the_header(tmp_path):
  # the descriptor structs cross the C ABI by pointer: the ctypes mirrors must have the sizes and
  # the field offsets a C compiler gives the header's structs
  pairs = {"tnx_qlinear_desc": L.QLinearDesc, "tnx_rope_desc": L.RopeDesc,
           "tnx_attn_desc": L.AttnDesc, "tnx_lmhead_desc": L.LmHeadDesc, "tnx_moe_gmm_desc": L.MoeGmmDesc}
  lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "tunix_hip.h"', 'int main(void) {']
  for cname, cls in pairs.items():
    lines.append(f'  printf("{cname} %zu\\n", sizeof({cname}));')
    for fname, _ in cls._fields_:
      lines.append(f'  printf("{cname}.{fname} %zu\\n", offsetof({cname}, {fname}));')
  lines += ['  return 0;', '}']
  src = tmp_path / "layout.c"
  src.write_text("\n".join(lines))
  exe = tmp_path / "layout"
  subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
  got = dict(ln.split() for ln in subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.splitlines())
  for cname, cls in pairs.items():
    assert int(got[cname]) == ctypes.sizeof(cls), cname
    for fname, _ in cls._fields_:
      assert int(got[f"{cname}.{fname}"]) == getattr(cls, fname).offset, f"{cname}.{fname}"


def test_host_utils_match_oracle_and_reference_vectors():
  assert [G.next_power_of_2(x) for x in (0, 2, 3, 4, 5)] == [1, 2, 4, 4, 8]
  x = np.array([1, 2, 3])
  np.testing.assert_array_equal(G.pad_to_length(x, 5, 0, left=True), U.pad_to_length(x, 5, 0, left=True))
  for ids in ([1, 2, 3, 4, 5, 6], [0, 0, 1, 2, 3, 4], [0, 1, 2, 3, 0, 0]):
    assert G.np_find_first_non_pad_idx(np.array(ids), 0) == U.find_first_non_pad_idx(np.array(ids), 0)
  for ids in ([1, 2, 3, 4, 5, -1], [1, 2, -1, 4, -1, 0], [1, 2, 3, 4, 5, 6]):
    assert G.np_find_first_eos_idx(np.array(ids), -1) == U.find_first_eos_idx(np.array(ids), -1)
  m = np.array([[1, 1, 1, 1], [0, 1, 1, 1], [1, 1, 1, 0], [0, 1, 1, 0]])
  np.testing.assert_array_equal(G.build_positions_from_mask(m), [[0, 1, 2, 3], [0, 0, 1, 2], [0, 1, 2, 2], [0, 0, 1, 1]])


def test_sampling_mode_conflict_message():
  cur = [None]
  G.check_sampling_mode_conflict(cur, "top_p")
  with pytest.raises(ValueError, match="Conflicts setting sampling_mode"):
    G.check_sampling_mode_conflict(cur, "greedy")


def test_id_tokenizer():
  t = G.IdTokenizer(100, pad_id=0, eos_id=1, bos_id=2)
  assert t.encode("5 6 7") == [5, 6, 7] and t.decode([5, 6]) == "5 6"
  assert t.dedup_bos_ids([2, 2, 2, 9]) == [2, 9]
  assert (t.pad_id(), t.eos_id(), t.bos_id()) == (0, 1, 2)


def test_config_presets():
  c = config.llama31_8b()
  assert (c.num_layers, c.embed_dim, c.hidden_dim, c.num_heads, c.num_kv_heads, c.head_dim, c.vocab_size) == (
      32, 4096, 14336, 32, 8, 128, 128256)
  assert c.qtype == config.Q_NF4 and c.group == 64 and c.lora_rank == 64
  g = config.gemma3_1b()
  assert [g.is_local_layer(i) for i in range(6)] == [True] * 5 + [False]
  assert g.rope_params(0) == (10_000.0, 1.0) and g.rope_params(5) == (1_000_000.0, 1.0)
  m = config.qwen3_30b_a3b()
  assert m.num_experts == 128 and m.num_experts_per_tok == 8
  assert "l0.e_gate" in m.quantized_names() and "l0.wq" in m.lora_names() and "l0.e_gate" not in m.lora_names()
  with pytest.raises(ValueError):
    config.ModelConfig(family="gpt2", num_layers=1, vocab_size=8, embed_dim=8, hidden_dim=8, num_heads=1,
                       num_kv_heads=1, head_dim=8)


def test_product_does_not_import_the_oracle():
  """The oracle is test infrastructure: nothing under tunix_amd/ may reference it."""
  pkg = os.path.join(ROOT, "tunix_amd")
  for dirpath, _, files in os.walk(pkg):
    for f in files:
      if f.endswith((".py", ".hip", ".h")):
        text = open(os.path.join(dirpath, f)).read()
        assert not re.search(r"^\s*(from|import)\s+oracle\b", text, re.M), os.path.join(dirpath, f)


def test_ffi_handlers_cover_the_documented_targets_and_call_declared_entry_points():
  """csrc/tunix_ffi.cc (the jax.ffi handlers, built only where jaxlib's headers exist) defines the
  twelve targets INTEGRATION.md lists and calls nothing the header does not declare."""
  src = open(os.path.join(ROOT, "tunix_amd", "csrc", "tunix_ffi.cc")).read()
  targets = set(re.findall(r"XLA_FFI_DEFINE_HANDLER_SYMBOL\((tnx_\w+_ffi)", src))
  doc = open(os.path.join(ROOT, "INTEGRATION.md")).read()
  documented = set(re.findall(r"`(tnx_\w+_ffi)`", doc))
  assert targets == documented and len(targets) == 12, (targets ^ documented)
  called = set(re.findall(r"\b(tnx_[a-z0-9_]+)\s*\(", src)) - {t for t in targets}
  assert called <= set(_declared()), called - set(_declared())


def test_binding_refuses_another_abi_version(monkeypatch):
  """A library of another major version (or an older minor one) must not be called."""
  major, minor = L.ABI_VERSION
  monkeypatch.setattr(L, "_lib", None)
  monkeypatch.setattr(L, "ABI_VERSION", (major + 1, 0))
  with pytest.raises(ImportError, match="ABI version"):
    L.lib()
  monkeypatch.setattr(L, "_lib", None)
  monkeypatch.setattr(L, "ABI_VERSION", (major, minor + 1))   # the real major, a newer minor
  with pytest.raises(ImportError, match="ABI version"):
    L.lib()


def test_missing_library_fails_loudly(monkeypatch):
  monkeypatch.setattr(L, "_lib", None)
  monkeypatch.setattr(L, "LIB_PATH", "/nonexistent/libtunix_hip.so")
  with pytest.raises(ImportError, match="no CPU fallback"):
    L.lib()


def test_sampling_plan_uses_one_predicate_for_path_and_workspace():
  """top_k None / <= 0 mean "no top-k"; top_k == V is a real top-k of the whole row in the
  reference (jax.lax.top_k(k = V), draw over sorted positions: tunix/generate/sampler.py:118-134)
  and takes the full sort whatever top_p; top_k > V raises as jax.lax.top_k does.  The same
  predicate decides the workspace: a full sort must get the full-row sort's workspace, not the
  (much smaller) segmented top-k one."""
  from tunix_amd.generate.sampler import sampling_plan
  V = 1000
  assert sampling_plan(None, 1.0, V) == (0, "head_draw")
  assert sampling_plan(0, 1.0, V) == (0, "head_draw")
  assert sampling_plan(V, 1.0, V) == (V, "fullsort")
  assert sampling_plan(V, 0.9, V) == (V, "fullsort")
  with pytest.raises(ValueError, match="top_k"):
    sampling_plan(V + 5, 0.9, V)
  assert sampling_plan(None, 0.9, V) == (0, "fullsort")
  assert sampling_plan(50, 0.9, V) == (50, "topk")
  assert sampling_plan(V - 1, 1.0, V) == (V - 1, "topk")
  lib = L.lib()
  # the library treats k >= V like k = 0 when it sizes the segmented workspace: that size is far
  # below what the full sort needs, which is why the host must not pair it with top_p < 1
  B, Vbig = 128, 128256
  small = lib.tnx_sample_topk_ws_bytes(B, Vbig, Vbig)
  assert small == lib.tnx_sample_topk_ws_bytes(B, Vbig, 0)
  assert small < 4 * B * Vbig


def test_threefry_seed_mirrors_jax_with_32_bit_integers():
  from tunix_amd.generate.sampler import _threefry_seed
  assert _threefry_seed(0) == (0, 0)
  assert _threefry_seed(7) == (0, 7)
  assert _threefry_seed(-1) == (0, 0xFFFFFFFF)
  assert _threefry_seed(-2 ** 31) == (0, 0x80000000)
  assert _threefry_seed(2 ** 32 + 5) == (0, 5)


def test_split_k_choice_of_the_decode_linears():
  """The k split the model picks per linear (host logic, no GPU): shapes that fill the device
  run unsplit, few-block shapes split up to 8 ways, and a gate|up linear stays unsplit when the
  split would save at most 7 k-tiles (its epilogue then replaces the finishing pass and the next
  linear's LoRA down-projection); the override wins over everything."""
  import types
  from tunix_amd.model import Runner
  m = Runner.__new__(Runner)
  m.split_k_override = {}
  lin = lambda name, K, N, il=False: types.SimpleNamespace(names=[f"layers.0.{name}"], K=K, N=N, interleave2=il)
  assert m._split_k(lin("wq", 4096, 6144), 128) == 5            # Llama-3.1-8B q|k|v: 48 column blocks
  assert m._split_k(lin("wo", 4096, 4096), 128) == 8
  assert m._split_k(lin("w_down", 14336, 4096), 128) == 8
  assert m._split_k(lin("w_gate", 4096, 28672, True), 128) == 1  # 224 blocks fill the device
  assert m._split_k(lin("w_gate", 1152, 13824, True), 64) == 1   # Gemma3-1B: 108 blocks, a 2-way split saves 4 k-tiles
  assert m._split_k(lin("w_gate", 4096, 2048, True), 64) == 8    # 16 blocks: the split saves 28 k-tiles
  assert m._split_k(lin("wq", 4096, 6144), 8192) == 1            # many rows
  m.split_k_override = {"w_gate": 3}
  assert m._split_k(lin("w_gate", 1152, 13824, True), 64) == 3
