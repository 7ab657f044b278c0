"""CPU-side checks of the boundary: the C-ABI library loads and exports every symbol that
include/ttmi.h declares, the pybind module and the drop-in package import, and the host
logic that needs no GPU (Tensor/DLPack semantics, allocator rounding, the npz reader, error
paths).  No compute entry point is called here.
"""
import ctypes
import os
import subprocess

import numpy as np
import pytest
import torch

from turbotransformers_amd import capi


def test_header_declares_and_library_exports_every_entry_point():
    protos = capi.parse_header()
    assert len(protos) >= 45
    lib = ctypes.CDLL(capi.LIB_PATH)
    missing = [n for n in protos if not hasattr(lib, n)]
    assert not missing, missing
    # and nothing with C linkage is exported that the header does not declare
    out = subprocess.run(["nm", "-D", "--defined-only", capi.LIB_PATH], capture_output=True, text=True).stdout
    exported = {l.split()[-1] for l in out.splitlines() if " T " in l and l.split()[-1].startswith("ttmi_")}
    assert exported == set(protos), exported ^ set(protos)


def test_every_declaration_cites_or_explains_itself():
    text = open(capi.HEADER).read()
    assert text.count("TTMI_API int") >= 40 and "extern \"C\"" in text
    assert "torch" not in text.split("*/", 1)[1].lower().replace("pytorch", "")  # no torch types in signatures


def test_error_reporting_without_a_gpu():
    lib = capi.load()
    rc = lib.ttmi_layer_norm(None, None, None, 1, 8, 1e-12, capi.F32, None)
    assert rc == -1 and b"null tensor" in lib.ttmi_last_error()
    with pytest.raises(capi.TtmiError):
        capi.check(lib.ttmi_gemm(None, None, None, 1, 1, 1, 1, 1, 1, 0, 1.0, 0.0, capi.F32, None))
    n = ctypes.c_int(-1)
    assert lib.ttmi_device_count(ctypes.byref(n)) == 0 and n.value >= 0


def test_dropin_package_surface():
    import turbo_transformers as tt
    import turbo_transformers.turbo_transformers_cxx as cxx
    for name in ("BertModel", "BertLayer", "BertEncoder", "BertAttention", "BertIntermediate", "BertOutput",
                 "BertEmbeddings", "BertPooler", "SequencePool", "PoolingType", "ReturnType", "BertModelSmartBatch",
                 "MultiHeadedAttentionSmartBatch", "AlbertModel", "AlbertLayer", "MultiHeadedAttention",
                 "PositionwiseFeedForward", "DistrillFFN", "QBertModel", "pref_guard", "nparray2tensor", "tensor2nparrayf",
                 "tensor2nparrayl", "enable_perf", "disable_perf", "set_num_threads", "reset_allocator_schema",
                 "bert_opt_mem_allocate_api"):
        assert hasattr(tt, name), name
    for name in ("Tensor", "BERTEmbedding", "BertAttention", "MultiHeadedAttention", "MultiHeadedAttentionSmartBatch",
                 "BertIntermediate", "BertOutput", "SequencePool", "BertPooler", "PrepareBertMasks", "AlbertLayer",
                 "FusedAddBiasGELU", "FusedAddBiasLayerNorm", "PositionwiseFeedForward", "DistrillFFN", "nparray2tensor", "tensor2nparrayf", "tensor2nparrayl",
                 "set_num_threads", "reset_allocator_schema", "bert_opt_mem_allocate_api", "enable_perf", "disable_perf",
                 "set_stderr_verbose_level"):
        assert hasattr(cxx, name), name
    assert cxx.config.is_compiled_with_cuda() is True
    assert callable(tt.BertModel.from_torch)


def test_tensor_dlpack_round_trip_and_ownership():
    import turbo_transformers.turbo_transformers_cxx as cxx
    t = torch.arange(24, dtype=torch.float32).reshape(2, 3, 4)
    capsule = torch.utils.dlpack.to_dlpack(t)
    tt = cxx.Tensor.from_dlpack(capsule)
    assert tt.n_dim() == 3 and [tt.shape(i) for i in range(3)] == [2, 3, 4] and tt.shape(-1) == 4
    assert tt.float_data() == t.data_ptr()            # alias, not a copy
    with pytest.raises(RuntimeError):
        tt.shape(3)
    back = torch.utils.dlpack.from_dlpack(tt.to_dlpack())
    assert back.data_ptr() == t.data_ptr() and torch.equal(back, t)
    assert tt.is_null()                               # to_dlpack released ownership
    with pytest.raises(RuntimeError):
        tt.to_dlpack()
    assert cxx.Tensor.create_empty().is_null()
    i64 = cxx.Tensor.from_dlpack(torch.utils.dlpack.to_dlpack(torch.ones(3, dtype=torch.int64)))
    with pytest.raises(RuntimeError):                 # dtype check of data<float>()
        i64.float_data()


def test_numpy_converters_on_cpu():
    import turbo_transformers.turbo_transformers_cxx as cxx
    a = np.arange(12, dtype=np.float32).reshape(3, 4)
    t = cxx.nparray2tensor(a, "CPU")
    assert np.array_equal(cxx.tensor2nparrayf(t), a)
    ids = np.arange(5, dtype=np.int64)
    assert np.array_equal(cxx.tensor2nparrayl(cxx.nparray2tensor(ids, "CPU")), ids)
    with pytest.raises(RuntimeError):
        cxx.nparray2tensor(a, "TPU")


def test_layers_reject_cpu_tensors_and_bad_shapes():
    """No CPU fallback: a layer built on host tensors refuses to run; shape checks raise."""
    import turbo_transformers.turbo_transformers_cxx as cxx
    conv = lambda x: cxx.Tensor.from_dlpack(torch.utils.dlpack.to_dlpack(x))
    inter = cxx.BertIntermediate(conv(torch.zeros(8, 32)), conv(torch.zeros(32)))
    with pytest.raises(RuntimeError, match="not on the GPU"):
        inter(conv(torch.zeros(2, 8)), cxx.Tensor.create_empty())
    with pytest.raises(RuntimeError):  # weight/bias mismatch (bert_intermediate.cpp EnforceShapeAndType)
        cxx.BertIntermediate(conv(torch.zeros(8, 32)), conv(torch.zeros(31)))
    with pytest.raises(RuntimeError):
        cxx.SequencePool("Median")
    with pytest.raises(RuntimeError):
        cxx.reset_allocator_schema("no-such-schema")
    cxx.reset_allocator_schema("naive")
    import turbo_transformers as tt
    from transformers import BertConfig, BertModel
    tiny = BertModel(BertConfig(vocab_size=10, hidden_size=8, num_hidden_layers=1, num_attention_heads=2,
                                intermediate_size=16, max_position_embeddings=8))
    with pytest.raises(RuntimeError, match="GPU"):
        tt.BertModel.from_torch(tiny, torch.device("cpu"), "turbo")
    with pytest.raises(NotImplementedError):
        tt.BertModel.from_torch(tiny, torch.device("cpu"), "onnxrt")


def test_npz_reader_matches_numpy(tmp_path):
    import turbo_transformers.turbo_transformers_cxx as cxx
    rng = np.random.default_rng(0)
    arrays = {"embeddings.word_embeddings.weight": rng.standard_normal((7, 4)).astype(np.float32),
              "pooler.dense.bias": rng.standard_normal(4).astype(np.float32),
              "half": rng.standard_normal((2, 3)).astype(np.float16),
              "ids": np.arange(6, dtype=np.int64).reshape(2, 3)}
    path = str(tmp_path / "w.npz")
    np.savez(path, **arrays)
    loaded = cxx.load_npz(path)
    assert set(loaded) == set(arrays)
    for k, v in arrays.items():
        assert loaded[k].dtype == v.dtype and np.array_equal(loaded[k], v)
    # deflated members: what numpy.savez_compressed and the reference's converter
    # (tools/convert_huggingface_bert_pytorch_to_npz.py:71) write; a larger, compressible array as well
    arrays["big"] = np.tile(rng.standard_normal(1000).astype(np.float32), 300).reshape(600, 500)
    np.savez_compressed(path, **arrays)
    loaded = cxx.load_npz(path)
    assert set(loaded) == set(arrays)
    for k, v in arrays.items():
        assert loaded[k].dtype == v.dtype and np.array_equal(loaded[k], v)
    # a truncated archive is an error, not a crash
    data = open(path, "rb").read()
    bad = str(tmp_path / "bad.npz")
    open(bad, "wb").write(data[:len(data) // 2])
    with pytest.raises(RuntimeError):
        cxx.load_npz(bad)


def test_converter_writes_the_reference_key_scheme(tmp_path):
    """tools/convert_huggingface_bert_pytorch_to_npz.py:44-71: q/k/v packed into qkv.weight [hidden, 3*hidden] and
    qkv.bias, other dense weights transposed to [in, out]; the (deflated) file reads back through the C++ loader."""
    import torch
    from transformers import BertConfig, BertModel
    import turbo_transformers.turbo_transformers_cxx as cxx
    from turbotransformers_amd.convert_huggingface_bert_to_npz import save_bert_npz
    torch.manual_seed(0)
    model = BertModel(BertConfig(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, intermediate_size=128, vocab_size=100))
    path = str(tmp_path / "m.npz")
    save_bert_npz(model, path)
    got = cxx.load_npz(path)
    sd = {k: v.detach().numpy() for k, v in model.named_parameters()}
    assert not any(".attention.self." in k for k in got)
    for i in range(2):
        p = "encoder.layer.%d." % i
        want = np.concatenate([sd[p + "attention.self.%s.weight" % x] for x in ("query", "key", "value")], 0).T
        assert np.array_equal(got[p + "attention.qkv.weight"], want) and want.shape == (64, 192)
        assert np.array_equal(got[p + "attention.qkv.bias"],
                              np.concatenate([sd[p + "attention.self.%s.bias" % x] for x in ("query", "key", "value")]))
        assert np.array_equal(got[p + "intermediate.dense.weight"], sd[p + "intermediate.dense.weight"].T)
        assert np.array_equal(got[p + "output.dense.weight"], sd[p + "output.dense.weight"].T)
        assert np.array_equal(got[p + "attention.output.dense.weight"], sd[p + "attention.output.dense.weight"].T)
    assert np.array_equal(got["pooler.dense.weight"], sd["pooler.dense.weight"].T)
    assert np.array_equal(got["embeddings.word_embeddings.weight"], sd["embeddings.word_embeddings.weight"])



def _stored_npz(path, members):
    """A zip archive of stored (uncompressed) members with the given raw bytes."""
    import zipfile
    with zipfile.ZipFile(path, "w", zipfile.ZIP_STORED) as z:
        for name, raw in members.items():
            z.writestr(name, raw)


def _npy(header_text, payload=b""):
    head = header_text.encode("latin1")
    return b"\x93NUMPY\x01\x00" + len(head).to_bytes(2, "little") + head + payload


@pytest.mark.parametrize("header", [
    "{'descr': '<f4', 'fortran_order': False, 'shape': (2, 3), }",                # payload missing
    "{'descr': '<f4', 'fortran_order': False, 'shape': (4611686018427387904, 4), }",  # product wraps around 2^64
    "{'descr': '<f4', 'fortran_order': False, 'shape': (99999999999999999999999, ), }",
    "{'descr': '<f4', 'fortran_order': False, 'shape' ",                          # no parenthesis
    "{'descr': '<f4', 'fortran_order': False }",                                   # no shape
    "{'descr': <f4, 'fortran_order': False, 'shape': (1, ), }",                    # unquoted dtype
    "{'descr': '<fx', 'fortran_order': False, 'shape': (1, ), }",                  # dtype size is not a number
    "{'descr'",                                                                    # nothing after the key
    "{'descr': '<f4', 'fortran_order':",                                           # ends inside a value
    "{'descr': '<f4', 'fortran_order': True, 'shape': (1, ), }",
    "{'descr': '<c8', 'fortran_order': False, 'shape': (1, ), }",
])
def test_npz_reader_refuses_malformed_members(tmp_path, header):
    """A malformed member ends in the loader's own error (RuntimeError), never in a crash or a C++ library exception
    of another type; a well-formed neighbour is no excuse."""
    import turbo_transformers.turbo_transformers_cxx as cxx
    path = str(tmp_path / "m.npz")
    _stored_npz(path, {"ok.npy": _npy("{'descr': '<f4', 'fortran_order': False, 'shape': (1, ), }".ljust(118) + "\n",
                                      np.float32(1).tobytes()),
                       "bad.npy": _npy(header.ljust(118) + "\n", b"\0" * 16)})
    with pytest.raises(RuntimeError):
        cxx.load_npz(path)


def test_npz_reader_refuses_sizes_beyond_the_file(tmp_path):
    import turbo_transformers.turbo_transformers_cxx as cxx
    path = str(tmp_path / "m.npz")
    np.savez(path, a=np.arange(4, dtype=np.float32))
    data = bytearray(open(path, "rb").read())
    cd = data.rfind(b"PK\x01\x02")
    data[cd + 20:cd + 28] = (0x7ffffff0).to_bytes(4, "little") * 2  # compressed and uncompressed size of the member
    open(path, "wb").write(bytes(data))
    with pytest.raises(RuntimeError):
        cxx.load_npz(path)


def test_gemm_describe_names_the_variant_without_a_device():
    """ttmi_gemm_describe runs the launchers' own selection with launching switched off, so it answers on a machine
    without a GPU: a family, the wavefronts per workgroup, the tile and the K split."""
    import ctypes
    import re
    lib = capi.load()
    buf = ctypes.create_string_buffer(64)
    args = capi.EpilogueArgs()
    args.act = capi.ACT_GELU
    for m, n, k, epi in [(32768, 3072, 768, capi.EPI_BIAS_ACT), (32768, 768, 3072, capi.EPI_NONE), (128, 768, 3072, capi.EPI_NONE),
                         (2560, 768, 3072, capi.EPI_BIAS)]:
        capi.check(lib.ttmi_gemm_describe(m, n, k, epi, ctypes.byref(args), capi.F16, buf, 64))
        assert re.fullmatch(r"(reg|dma|dma_agpr|dma3_agpr|wave)\d+w_\d+x\d+(_splitk\d+)?", buf.value.decode()), buf.value
    assert lib.ttmi_gemm_describe(128, 768, 3072, capi.EPI_NONE, None, capi.F16, buf, 4) != 0  # too small for the answer


def test_one_short_sequence_splits_k_only_where_a_second_launch_pays():
    """128 tokens: the output projection and the second FFN product (24 tiles of 64 x 64) are cut along K; the
    intermediate Linear (96 tiles) keeps bias + GELU in the GEMM in 16-bit types, where the reduction kernel's launch
    costs more than the split saves, and is cut in fp32, where it does not."""
    import ctypes
    lib = capi.load()
    buf = ctypes.create_string_buffer(64)
    args = capi.EpilogueArgs()
    args.act = capi.ACT_GELU

    def variant(m, n, k, epi, dt):
        capi.check(lib.ttmi_gemm_describe(m, n, k, epi, ctypes.byref(args), dt, buf, 64))
        return buf.value.decode()

    assert "_splitk" in variant(128, 768, 768, capi.EPI_NONE, capi.F16)
    assert "_splitk" in variant(128, 768, 3072, capi.EPI_NONE, capi.F16)
    assert variant(128, 3072, 768, capi.EPI_BIAS_ACT, capi.F16) == "wave1w_32x32"
    assert variant(128, 3072, 768, capi.EPI_BIAS_ACT, capi.BF16) == "wave1w_32x32"
    assert "_splitk" in variant(128, 3072, 768, capi.EPI_BIAS_ACT, capi.F32)


def test_up_to_128_rows_of_16_bit_operands_take_the_wavefront_kernel():
    """One wavefront per 32 x 32 tile, operand fragments straight from global memory: 16-bit types, at most 128 rows,
    K a multiple of the 128-byte step; fp32 and longer inputs stay on the LDS-tiled kernels."""
    import ctypes
    lib = capi.load()
    buf = ctypes.create_string_buffer(64)

    def variant(m, n, k, dt):
        capi.check(lib.ttmi_gemm_describe(m, n, k, capi.EPI_NONE, None, dt, buf, 64))
        return buf.value.decode()

    for m in (1, 10, 40, 128):
        assert variant(m, 2304, 768, capi.F16).startswith("wave1w_32x32")  # cut along K while its tiles are few
        assert variant(m, 2304, 768, capi.BF16).startswith("wave1w_32x32")
        assert variant(m, 768, 3072, capi.F16).startswith("wave1w_32x32_splitk")
    assert not variant(128, 2304, 768, capi.F32).startswith("wave")
    assert not variant(129, 2304, 768, capi.F16).startswith("wave")
    assert not variant(128, 2304, 776, capi.F16).startswith("wave")


def test_transposed_v_of_sequences_shorter_than_8_stays_off_the_one_wavefront_per_simd_kernel():
    """That kernel stores a group of eight rows of a transposed V that leaves its sequence element by element into
    this sequence and the next one; with fewer than 8 positions per sequence a group would touch three, so such a
    QKV projection runs on the other kernels however many rows it has."""
    import ctypes
    lib = capi.load()
    buf = ctypes.create_string_buffer(64)

    def variant(batch, seq, pitch):
        args = capi.EpilogueArgs()
        args.bias = args.q = args.k = args.v = 1 << 20  # never dereferenced: describe launches nothing
        args.seq, args.heads, args.head_dim, args.v_seq_pitch = seq, 12, 64, pitch
        capi.check(lib.ttmi_gemm_describe(batch * seq, 2304, 768, capi.EPI_QKV_SPLIT, ctypes.byref(args), capi.F16, buf, 64))
        return buf.value.decode()

    assert variant(1000, 12, 16).startswith("dma_agpr4w")
    assert variant(1500, 8, 8).startswith("dma_agpr4w")
    assert variant(2400, 5, 0).startswith("dma_agpr4w")  # row-major V: any length
    assert not variant(2400, 5, 8).startswith("dma_agpr4w")


def test_fp32_products_pick_tiles_by_rounds_over_the_compute_units():
    """fp32 is bound by the matrix pipe at every tile size, so the tile (and a cut along K) is chosen for whole
    rounds of tiles over the CUs: a few thousand rows by 768 columns run on 64 x 64 tiles where the 16-bit types take
    128 x 128, a last round that is nearly empty is filled by slices of K, large products keep the large tiles."""
    import ctypes
    lib = capi.load()
    buf = ctypes.create_string_buffer(64)

    def variant(m, n, k, dt):
        capi.check(lib.ttmi_gemm_describe(m, n, k, capi.EPI_NONE, None, dt, buf, 64))
        return buf.value.decode()

    assert variant(4000, 768, 3072, capi.F32) == "reg4w_64x64"        # 756 tiles: three rounds of 256
    assert variant(4000, 768, 3072, capi.F16) == "dma4w_128x128"
    assert variant(1600, 768, 3072, capi.F32) == "reg4w_64x64_splitk5"  # 300 tiles are 1.17 rounds: 1500 slices, six
    assert variant(1600, 768, 768, capi.F32) == "reg4w_64x64"          # K too short for the cut to pay
    assert variant(32768, 3072, 768, capi.F32) == "dma8w_256x256"
    assert variant(128, 768, 3072, capi.F32) == "reg4w_64x64_splitk10"  # one short sequence: as before
