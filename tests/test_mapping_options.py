"""Mapping options: preset literal values (tc/core/mapping_options-inl.h:223-262,
tc/core/cuda/cuda_mapping_options.cc:327-384 with wave64 block shapes), serialisation round trip,
C++ printer, validation."""
import pytest

import tensorcomprehensions_amd as tc
from tensorcomprehensions_amd import MappingOptions


def fields(o):
    return dict(kv.split("=") for kv in o.normalized().split(";"))


def test_preset_values():
    n = fields(MappingOptions.naive())
    assert n["tile"] == "32,32,32" and n["unroll"] == "1" and n["mapToBlocks"] == "256,256"
    assert n["mapToThreads"] == "64,4"                       # 256 threads, x a whole wavefront
    assert n["outerScheduleFusionStrategy"] == "Preserve3Coincident"
    assert n["useSharedMemory"] == "0" and n["matchLibraryCalls"] == "0"
    st = fields(MappingOptions.single_thread())
    assert (st["tile"], st["mapToThreads"], st["mapToBlocks"]) == ("1", "1", "1")
    pw = fields(MappingOptions.pointwise())
    assert pw["unroll"] == "128" and pw["mapToBlocks"] == "100,100,100" and pw["mapToThreads"] == "64,2,2"
    mlp = fields(MappingOptions.mlp())
    assert mlp["outerScheduleFusionStrategy"] == "Max" and mlp["tile"] == "1" and mlp["mapToThreads"] == "128"
    assert fields(MappingOptions.conv())["tile"] == "4,8,8,8"
    assert fields(MappingOptions.group_conv())["tile"] == "1,1"


def test_serialisation_round_trip():
    o = (MappingOptions.naive().tile(1, 2, 2, 0).mapToThreads(256).mapToBlocks(32, 256).unroll(64).vectorWidth(4)
         .useSharedMemory(True).maxSharedMemory(40000).scheduleFusionStrategy("Max").sharedDepth(3).privateDepth(2)
         .matchLibraryCalls(True).collapseContiguous(False).reductionBlocks(16))
    data = o.serialize()
    back = MappingOptions.deserialize(data)
    assert back == o
    assert back.normalized() == o.normalized()
    assert MappingOptions.deserialize(MappingOptions.naive().serialize()) != o
    # generic options message is field 1, block field 2, grid field 3 (tc/proto/mapping_options.proto:74-96)
    assert data[0] == 0x0A


def test_cpp_printer_is_a_chain_starting_from_naive():
    cpp = MappingOptions.naive().tile(4, 8).unroll(16).to_cpp()
    lines = cpp.split("\n")
    assert lines[0] == "tc::HipMappingOptions::makeNaiveMappingOptions()"
    assert "    .outerScheduleFusionStrategy(tc::FusionStrategy::Preserve3Coincident)" in lines
    assert "    .tile(4, 8)" in lines and "    .unroll(16)" in lines
    assert "    .mapToThreads(64, 4)" in lines and "    .useSharedMemory(false)" in lines


@pytest.mark.parametrize("bad", ["naive;vectorWidth=3", "naive;noSuchOption=1", "nosuchpreset", "naive;mapToThreads=1,2,3,4",
                                 "naive;outerScheduleFusionStrategy=Sideways"])
def test_invalid_options_are_rejected(bad):
    with pytest.raises(tc.TcError):
        MappingOptions(bad).normalized()
