"""The serialized mapping options and the options-cache files against a real protobuf
implementation.  The message types are built here, by hand, from the field numbers of the
reference's schemas (tc/proto/mapping_options.proto:19-96, tc/proto/compcache.proto:20-62; the
HIP options message adds fields 11-14), so the library's hand-written wire codec is read and
written by google.protobuf and not only by itself."""
import ctypes
import os
import tempfile

import pytest

import tensorcomprehensions_amd as tc
from tests.scaffolding import scaffold_query
from tensorcomprehensions_amd import _capi

pb = pytest.importorskip("google.protobuf")
from google.protobuf import descriptor_pb2, descriptor_pool, message_factory  # noqa: E402

F = descriptor_pb2.FieldDescriptorProto
REQ, OPT, REP = F.LABEL_REQUIRED, F.LABEL_OPTIONAL, F.LABEL_REPEATED


def _file():
    f = descriptor_pb2.FileDescriptorProto(name="tc_wire_test.proto", package="tc", syntax="proto2")
    e = f.enum_type.add(name="FusionStrategy")
    for name, number in (("Max", 1), ("Preserve3Coincident", 2), ("Min", 3)):
        e.value.add(name=name, number=number)

    def message(name, fields):
        m = f.message_type.add(name=name)
        for fname, number, label, ftype, type_name in fields:
            fd = m.field.add(name=fname, number=number, label=label, type=ftype)
            if type_name:
                fd.type_name = ".tc." + type_name
    U64, U32, BOOL, STR, MSG, ENUM = F.TYPE_UINT64, F.TYPE_UINT32, F.TYPE_BOOL, F.TYPE_STRING, F.TYPE_MESSAGE, F.TYPE_ENUM
    message("CudaDimProto", [("x", 1, REQ, U64, None), ("y", 2, OPT, U64, None), ("z", 3, OPT, U64, None)])
    message("SchedulerOptionsProto", [("fusion_strategy", 1, REQ, ENUM, "FusionStrategy"), ("allow_skewing", 2, REQ, BOOL, None),
                                      ("positive_orthant", 3, REQ, BOOL, None)])
    message("TilingProto", [("sizes", 1, REP, U64, None)])
    message("MappingOptionsProto", [
        ("outer_schedule_options", 1, REQ, MSG, "SchedulerOptionsProto"),
        ("intra_tile_schedule_options", 2, REQ, MSG, "SchedulerOptionsProto"),
        ("fix_parameters_before_scheduling", 3, REQ, BOOL, None), ("tiling", 4, OPT, MSG, "TilingProto"),
        ("unroll", 5, OPT, U64, None), ("tile_imperfectly_nested", 6, REQ, BOOL, None),
        ("match_library_calls", 7, REQ, BOOL, None)])
    message("HipMappingOptionsProto", [
        ("generic_mapping_options", 1, REQ, MSG, "MappingOptionsProto"), ("block", 2, REQ, MSG, "CudaDimProto"),
        ("grid", 3, REQ, MSG, "CudaDimProto"), ("use_shared_memory", 4, REQ, BOOL, None),
        ("use_private_memory", 5, REQ, BOOL, None), ("unroll_copy_shared", 6, REQ, BOOL, None),
        ("max_shared_memory", 7, OPT, U64, None), ("use_readonly_cache", 8, REQ, BOOL, None),
        ("private_depth", 9, OPT, U32, None), ("shared_depth", 10, OPT, U32, None),
        # beyond the reference's message: the CDNA4 mapper's own knobs
        ("vector_width", 11, OPT, U32, None), ("collapse_contiguous", 12, OPT, BOOL, None),
        ("use_mfma", 13, OPT, BOOL, None), ("prefetch_shared", 14, OPT, BOOL, None),
        ("reduction_blocks", 15, OPT, U32, None)])
    message("DLDataTypeProto", [("code", 1, REQ, U32, None), ("bits", 2, REQ, U32, None), ("lanes", 3, REQ, U32, None)])
    message("TensorInfoProto", [("shape", 1, REP, U64, None), ("strides", 2, REP, U64, None), ("alignment", 3, REQ, U64, None),
                                ("dtype", 4, REQ, MSG, "DLDataTypeProto")])
    message("OptionsCacheKeyProto", [("id", 1, REQ, STR, None), ("inputs", 2, REP, MSG, "TensorInfoProto"),
                                     ("outputs", 3, REP, MSG, "TensorInfoProto"), ("backend_str", 4, REQ, STR, None),
                                     ("git_version", 5, REQ, STR, None)])
    message("HipOptionsCacheValueProto", [("kernel_options", 1, REQ, MSG, "HipMappingOptionsProto"),
                                          ("recorded_runtimes", 2, REP, U64, None)])
    message("HipOptionsCacheProto", [("keys", 1, REP, MSG, "OptionsCacheKeyProto"),
                                     ("values", 2, REP, MSG, "HipOptionsCacheValueProto")])
    return f


@pytest.fixture(scope="module")
def messages():
    pool = descriptor_pool.DescriptorPool()
    pool.Add(_file())
    get = getattr(message_factory, "GetMessageClass", None)
    def cls(name):
        d = pool.FindMessageTypeByName("tc." + name)
        return get(d) if get else message_factory.MessageFactory(pool).GetPrototype(d)
    return {n: cls(n) for n in ("HipMappingOptionsProto", "HipOptionsCacheProto")}


def serialized(options_text):
    data, size = ctypes.c_void_p(), ctypes.c_size_t(0)
    _capi.check(_capi.lib().tc_options_to_serialized(options_text.encode(), ctypes.byref(data), ctypes.byref(size)))
    raw = ctypes.string_at(data.value, size.value)
    _capi.lib().tc_free(data)
    return raw


def from_serialized(raw):
    text = ctypes.c_void_p()
    _capi.check(_capi.lib().tc_options_from_serialized(raw, len(raw), ctypes.byref(text)))
    return _capi.take_string(text)


OPTIONS = ("naive;outerScheduleFusionStrategy=Max;intraTileScheduleFusionStrategy=Min;outerScheduleAllowSkewing=1;"
           "fixParametersBeforeScheduling=1;tile=1,8,2,0;unroll=128;tileImperfectlyNested=1;matchLibraryCalls=1;"
           "mapToThreads=196,2;mapToBlocks=32,64,3;useSharedMemory=1;usePrivateMemory=1;unrollCopyShared=1;"
           "maxSharedMemory=40000;useReadOnlyCache=1;privateDepth=3;sharedDepth=2;vectorWidth=4;collapseContiguous=0;"
           "useMfma=1;prefetchShared=1;reductionBlocks=8")


def test_protobuf_reads_the_serialized_options_field_by_field(messages):
    m = messages["HipMappingOptionsProto"]()
    m.ParseFromString(serialized(OPTIONS))
    assert m.IsInitialized()                                       # every required field of the schema is there
    g = m.generic_mapping_options
    assert (g.outer_schedule_options.fusion_strategy, g.outer_schedule_options.allow_skewing,
            g.outer_schedule_options.positive_orthant) == (1, True, True)
    assert (g.intra_tile_schedule_options.fusion_strategy, g.intra_tile_schedule_options.allow_skewing) == (3, False)
    assert g.fix_parameters_before_scheduling and g.tile_imperfectly_nested and g.match_library_calls
    assert list(g.tiling.sizes) == [1, 8, 2, 0] and g.unroll == 128
    assert (m.block.x, m.block.y, m.block.HasField("z")) == (196, 2, False)
    assert (m.grid.x, m.grid.y, m.grid.z) == (32, 64, 3)
    assert m.use_shared_memory and m.use_private_memory and m.unroll_copy_shared and m.use_readonly_cache
    assert (m.max_shared_memory, m.private_depth, m.shared_depth) == (40000, 3, 2)
    assert (m.vector_width, m.collapse_contiguous, m.use_mfma, m.prefetch_shared) == (4, False, True, True)
    assert m.reduction_blocks == 8
    # nothing on the wire that the schema does not name: re-serialising gives the same bytes
    assert m.SerializeToString() == serialized(OPTIONS)
    # optional fields that were never set stay absent on the wire
    plain = messages["HipMappingOptionsProto"]()
    plain.ParseFromString(serialized("naive"))
    assert not plain.HasField("max_shared_memory") and not plain.HasField("private_depth") and not plain.HasField("shared_depth")
    assert not plain.HasField("reduction_blocks")
    assert list(plain.generic_mapping_options.tiling.sizes) == [32, 32, 32] and plain.generic_mapping_options.unroll == 1


def test_the_library_reads_options_that_protobuf_serialized(messages):
    m = messages["HipMappingOptionsProto"]()
    m.ParseFromString(serialized(OPTIONS))
    # through protobuf and back: byte for byte what the library wrote, and the same option text
    assert m.SerializeToString() == serialized(OPTIONS)
    assert from_serialized(m.SerializeToString()) == from_serialized(serialized(OPTIONS))
    # a message built from nothing by protobuf
    n = messages["HipMappingOptionsProto"]()
    for sched, fusion in ((n.generic_mapping_options.outer_schedule_options, 2), (n.generic_mapping_options.intra_tile_schedule_options, 1)):
        sched.fusion_strategy, sched.allow_skewing, sched.positive_orthant = fusion, False, True
    n.generic_mapping_options.fix_parameters_before_scheduling = False
    n.generic_mapping_options.tiling.sizes.extend([4, 16])
    n.generic_mapping_options.unroll = 16
    n.generic_mapping_options.tile_imperfectly_nested = False
    n.generic_mapping_options.match_library_calls = True
    n.block.x, n.block.y = 64, 4
    n.grid.x = 500
    n.use_shared_memory, n.use_private_memory, n.unroll_copy_shared, n.use_readonly_cache = True, False, False, True
    n.shared_depth = 1
    n.vector_width, n.collapse_contiguous, n.use_mfma, n.prefetch_shared = 2, True, False, False
    n.reduction_blocks = 16
    text = from_serialized(n.SerializeToString())
    for fragment in ("outerScheduleFusionStrategy=Preserve3Coincident", "intraTileScheduleFusionStrategy=Max", "tile=4,16", "unroll=16",
                     "matchLibraryCalls=1", "mapToThreads=64,4", "mapToBlocks=500", "useSharedMemory=1", "usePrivateMemory=0",
                     "useReadOnlyCache=1", "sharedDepth=1", "vectorWidth=2", "collapseContiguous=1", "useMfma=0",
                     "reductionBlocks=16"):
        assert fragment in text.split(";"), (fragment, text)
    assert "privateDepth" not in text and "maxSharedMemory" not in text


def test_packed_repeated_fields_are_accepted():
    """`repeated uint64 sizes = 1` as a packed run (what proto3 tooling writes for this schema)."""
    raw = serialized("naive;tile=3,5,7")
    unpacked = bytes([0x08, 3, 0x08, 5, 0x08, 7])
    assert raw.count(unpacked) == 1
    packed = bytes([0x0A, 3, 3, 5, 7])
    grown = raw.replace(unpacked, packed)        # one byte shorter: fix the two enclosing lengths (tiling, generic options)
    i = grown.index(packed)
    tiling_len_at = i - 1
    assert grown[tiling_len_at] == len(unpacked) and grown[tiling_len_at - 1] == 0x22
    grown = bytearray(grown)
    grown[tiling_len_at] = len(packed)
    assert grown[0] == 0x0A
    grown[1] -= 1
    assert "tile=3,5,7" in from_serialized(bytes(grown)).split(";")


@pytest.mark.parametrize("field,value,message", [(15, 0, "reductionBlocks must be between 1 and 1024"),
                                                  (15, 5000, "reductionBlocks must be between 1 and 1024"),
                                                  (11, 3, "vector width must be 1, 2 or 4")])
def test_out_of_range_scalars_in_a_message_are_refused_like_in_the_text_form(field, value, message):
    """A foreign or damaged cache file must not plant a value the setters and the text form refuse
    (the options would print and then not parse again)."""
    raw = serialized("naive")
    tail = bytes([field << 3])
    v = value
    while True:
        tail += bytes([(v & 0x7F) | (0x80 if v > 0x7F else 0)])
        v >>= 7
        if not v:
            break
    with pytest.raises(tc.TcError) as e:
        from_serialized(raw + tail)
    assert message in str(e.value)


@pytest.mark.parametrize("damage", ["truncated", "overlong_varint", "length_past_end", "scalar_for_message"])
def test_corrupt_messages_are_refused_not_read_out_of_bounds(damage):
    raw = serialized(OPTIONS)
    bad = {"truncated": raw[:-1],
           "overlong_varint": b"\x20" + b"\xff" * 11 + b"\x01",
           "length_past_end": b"\x0a\xff\xff\xff\xff\xff\xff\xff\xff\xff\x01",
           "scalar_for_message": b"\x08\x01"}[damage]
    with pytest.raises(tc.TcError) as e:
        from_serialized(bad)
    assert "protowire" in str(e.value)


def test_protobuf_reads_a_cache_file_and_the_library_reads_protobufs(messages):
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "cache.bin")
        listing = scaffold_query("options_cache_write_sample", path)
        m = messages["HipOptionsCacheProto"]()
        m.ParseFromString(open(path, "rb").read())
        assert m.IsInitialized() and len(m.keys) == len(m.values) == 4
        by_id = {}
        for k, v in zip(m.keys, m.values):
            by_id.setdefault(k.id, []).append((k, v))
        assert sorted(by_id) == ["tcA", "tcB"] and len(by_id["tcA"]) == 3
        k, _ = by_id["tcA"][0]
        assert k.backend_str == "dev" and [list(t.shape) for t in k.inputs] == [[10, 16], [16, 20]]
        assert [list(t.strides) for t in k.inputs] == [[16, 1], [20, 1]] and [list(t.shape) for t in k.outputs] == [[10, 20]]
        assert (k.inputs[0].dtype.code, k.inputs[0].dtype.bits, k.inputs[0].dtype.lanes, k.inputs[0].alignment) == (2, 32, 1, 0)
        runtimes = sorted(sorted(v.recorded_runtimes) for _, v in by_id["tcA"])
        assert runtimes == [[10000, 20000, 30000], [15000], [50000]]          # nanoseconds
        tiled = [v for _, v in by_id["tcA"] if list(v.recorded_runtimes) == [15000]][0]
        assert list(tiled.kernel_options.generic_mapping_options.tiling.sizes) == [4, 4]
        assert tiled.kernel_options.generic_mapping_options.unroll == 8
        # written by protobuf, read by the library: same entries; then edited by protobuf
        again = os.path.join(d, "again.bin")
        open(again, "wb").write(m.SerializeToString())
        assert tc.host_query("options_cache_dump", again) == listing
        m.keys[0].id = "renamed"
        m.values[0].recorded_runtimes.append(1)
        m.values[0].kernel_options.block.x = 128
        open(again, "wb").write(m.SerializeToString())
        dumped = tc.host_query("options_cache_dump", again)
        renamed = [line for line in dumped.splitlines() if line.startswith("renamed |")]
        assert len(renamed) == 1 and "mapToThreads=128" in renamed[0]


def test_cache_semantics_of_the_reference():
    """test/cuda/test_compilation_cache.cc:133-510 on a cache with two TCs: multimap counts, ranking by the
    median of all runs of an option, misses on any differing key part, pruning, wire and file round trips."""
    with tempfile.TemporaryDirectory() as d:
        lines = dict(line.split("=", 1) for line in scaffold_query("options_cache_selftest", os.path.join(d, "c.bin")).splitlines())
    assert lines["size"] == "4" and lines["count_tcA"] == "3" and lines["keys"] == "2"
    assert lines["top2_tcA"] == "o2@15000,o1@20000"             # o1 ran 10, 30 and 20 us: median 20
    assert [lines[k] for k in ("miss_other_tc", "miss_other_sizes", "miss_other_device", "miss_other_alignment")] == ["0"] * 4
    assert lines["retrievals"] == "5,1"
    assert lines["wire_copy_size"] == "4" and lines["wire_copy_top3_tcA"] == "o2@15000,o1@20000,o3@50000"
    assert lines["pruned_size"] == "2" and lines["pruned_top_tcA"] == "o2@15000"
    assert lines["file_loaded_size"] == "4" and lines["file_appended_size"] == "5"
