"""The reference's own callers of the operator boundary against this library.

oracle/Makefile (target ref_boundary) compiles the reference's StaticMemoryArena, OpTable /
StaticOpSlot / PlanAclnnOp, AclDeviceOps and handle guards from its sources where they lie, with
include/compat standing in for the CANN headers, and links oracle/ref_boundary_probe.cpp (ours)
to libmoe_kv_hip.so with no undefined symbol allowed. The CPU test builds it (only where the
reference tree is mounted) and checks that, without a device, the reference's backend reports
that explicitly. The GPU test runs the prebuilt binary: the reference's code reserves the arena,
builds the descriptors, plans the two operators, swaps the cache slices per layer and launches
through its StaticOpSlot, and the outputs are compared with the CPU oracle."""
import json
import math
import os
import subprocess

import numpy as np
import pytest

import oracle_ffi as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROBE = os.path.join(ROOT, "oracle", "_ref", "ref_boundary_probe")
REFERENCE = "/root/reference"
HEADS, LATENT, ROPE = 64, 512, 64
ROW = LATENT + ROPE


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE, "src")), reason="the reference tree is not mounted here")
def test_reference_callers_compile_and_link_against_the_library(tmp_path):
    proc = subprocess.run(["make", "-B", "-C", os.path.join(ROOT, "oracle"), "ref_boundary"], capture_output=True, text=True)
    assert proc.returncode == 0, proc.stdout[-3000:] + proc.stderr[-3000:]
    assert "--no-undefined" in proc.stdout          # the link line refuses any symbol the library does not export
    assert os.path.isfile(PROBE)
    # the reference headers saw this library's declarations, not its own stand-ins
    assert "include/compat" in proc.stdout and "mock/include" not in proc.stdout
    needed = subprocess.run(["readelf", "-d", PROBE], capture_output=True, text=True).stdout
    assert "libmoe_kv_hip.so" in needed
    if not os.path.exists("/dev/kfd"):
        # no device here: the reference's backend makes that an explicit outcome (device_ops.hpp:55-58)
        blob = tmp_path / "in.bin"
        blob.write_bytes(np.zeros((ROW + HEADS * ROW) * 1, dtype=np.uint16).tobytes())
        run = subprocess.run([PROBE, str(blob), str(tmp_path / "out.bin"), "1", "1", "64", "256", "1", "1"],
                             capture_output=True, text=True)
        assert run.returncode == 1 and "ref_boundary_probe:" in run.stderr


def _bf16_bits(rng, shape):
    return (rng.standard_normal(shape).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)


@pytest.mark.gpu
@pytest.mark.parametrize("live,identity", [(1, 1), (0, 0)])
def test_reference_callers_drive_the_kernels(live, identity, tmp_path):
    """live=1, identity=1: the table is written and the live context attended to. live=0,
    identity=0: exactly what the reference's code asks for -- the reserved context as kv length
    and the zero block table it never writes, so every logical block reads physical block 0."""
    if not os.path.isfile(PROBE):
        pytest.skip("oracle/_ref/ref_boundary_probe was not built (it needs the reference tree at build time)")
    layers, steps, bs, max_ctx = 2, 5, 64, 256
    blocks = max_ctx // bs
    rng = np.random.default_rng(17)
    items = _bf16_bits(rng, (steps, layers, ROW + HEADS * ROW))
    (tmp_path / "in.bin").write_bytes(items.tobytes())
    run = subprocess.run([PROBE, str(tmp_path / "in.bin"), str(tmp_path / "out.bin"), str(layers), str(steps), str(bs), str(max_ctx),
                          str(live), str(identity)], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, run.stdout + run.stderr
    report = json.loads(run.stdout.strip().splitlines()[-1])
    assert report["backend"] == "acl" and report["scatter_found"] == 1 and report["attention_found"] == 1
    assert report["rms_norm_found"] == 0                        # the engine's other operators are not this library's
    assert report["allocations_after_commit"] == 1              # one allocation at Commit (static_arena.cpp:108-118)
    assert report["allocations_after_build"] == report["allocations_after_steps"] == 2   # + the workspace; none in a step
    got = np.frombuffer((tmp_path / "out.bin").read_bytes(), dtype=np.uint16).reshape(steps, layers, HEADS, LATENT)
    got = orc.bf16_to_f32(got.reshape(-1)).reshape(got.shape)
    scale = 1.0 / math.sqrt(192.0)
    table = (np.arange(blocks, dtype=np.int32) if identity else np.zeros(blocks, dtype=np.int32)).reshape(1, blocks)
    for layer in range(layers):
        latent_plane = np.zeros(blocks * bs * LATENT, dtype=np.uint16)
        rope_plane = np.zeros(blocks * bs * ROPE, dtype=np.uint16)
        for position in range(steps):
            item = items[position, layer]
            latent_plane[position * LATENT:(position + 1) * LATENT] = item[:LATENT]          # slot = position (pipeline.cpp:517)
            rope_plane[position * ROPE:(position + 1) * ROPE] = item[LATENT:ROW]
            q_b = item[ROW:]
            # the reference's descriptors are contiguous views into q_b (static_arena_manager.cpp:481-485)
            q_latent = np.ascontiguousarray(q_b[:HEADS * LATENT].reshape(1, HEADS, LATENT))
            q_rope = np.ascontiguousarray(q_b[LATENT:LATENT + HEADS * ROPE].reshape(1, HEADS, ROPE))
            length = position + 1 if live else max_ctx
            expected, _ = orc.mla_decode(q_latent, q_rope, latent_plane, rope_plane, bs, table, [length], scale)
            peak = np.abs(expected).max()
            assert np.abs(got[position, layer] - expected[0]).max() <= 2e-2 * peak, (position, layer)
