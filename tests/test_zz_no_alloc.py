"""The entry point that allocates nothing (mk_rotated_packed_matvec_static, rotated
activations in the library's own fixed device array) against mk_rotated_packed_matvec with a
buffer of the caller's: bit-identical outputs through the C ABI, on two calls in a row of
which the second is smaller, and a clear refusal beyond the array's size."""

import numpy as np
import pytest
import torch

from oracle import matvec as oracle_matvec, scaling, transforms as oracle_transforms

import helpers

pytestmark = pytest.mark.gpu


def rotated_layer_call(samples, rows, width, dtype, seed):
    """Device tensors and the two argument lists (workspace entry point, static entry point)."""
    from mlkit_amd import native
    from mlkit_amd.quantization.transforms import OnlineRotation, random_signs

    weight = helpers.normal_weight(rows, width, seed=seed)
    layer = helpers.quantised_layer(weight, scaling.int_values(4), bits=4, group=128, integer=True)
    tensors = helpers.to_device(layer, torch.float16 if dtype == torch.float16 else torch.bfloat16)
    x = helpers.activations(samples, width, seed=seed + 1, dtype=dtype).cuda()
    order, power, basis, signs, scale, keep = OnlineRotation(seed).launch_arguments(width, x.device)
    matvec = (tensors["packed"].data_ptr(), tensors["scales"].data_ptr(), native.dtype_code(tensors["scales"]),
              tensors["values"].data_ptr(), 16, None, None, 0)
    shape = (samples, rows, width, 128, 4, 1, -8.0, 1.0, None)
    code = native.DTYPE_CODES[dtype]
    outputs = [torch.full((samples, rows), float("nan"), dtype=dtype, device="cuda") for _ in range(2)]
    workspace = torch.empty((samples, width), dtype=dtype, device="cuda")
    with_buffer = (x.data_ptr(), code, workspace.data_ptr(), order, power, basis, signs, scale, *matvec,
                   outputs[0].data_ptr(), *shape)
    without = (x.data_ptr(), code, order, power, basis, signs, scale, *matvec, outputs[1].data_ptr(), *shape)
    host_signs = random_signs(width, seed, "cuda").cpu().numpy()
    return with_buffer, without, outputs, (x, layer, host_signs, tensors, keep, workspace)


def test_static_buffer_entry_point_equals_the_workspace_entry_point():
    from mlkit_amd import native
    from mlkit_amd.kernels import hadamard

    lib = native.library()
    # a large call first, then a smaller one: the second must not see what the first left behind
    # (one fp16 sample of a power-of-two width is rotated inside the matvec kernel by both entry points)
    for samples, rows, width, dtype, seed in ((8, 512, 14336, torch.float16, 11), (2, 256, 4096, torch.float16, 12),
                                              (3, 128, 896, torch.bfloat16, 13), (1, 256, 4096, torch.float16, 14)):
        print(f"case samples={samples} rows={rows} width={width} {dtype}", flush=True)
        with_buffer, without, outputs, keep = rotated_layer_call(samples, rows, width, dtype, seed)
        native.check(lib.mk_rotated_packed_matvec(*with_buffer))
        native.check(lib.mk_rotated_packed_matvec_static(*without))
        torch.cuda.synchronize()
        assert not torch.isnan(outputs[0]).any()
        assert torch.equal(outputs[0], outputs[1])
        # and both are the rotated layer: oracle rotation of x, rounded to the input dtype, times the dense weight
        # (the matvec at its own tolerance on the activations the device rotated, and those within one unit in
        # the last place of the oracle's)
        x, layer, signs, _, _, workspace = keep
        inside = samples == 1 and width & (width - 1) == 0
        device_rotated = hadamard.transform(x.float(), signs_before=torch.from_numpy(signs).cuda()).to(dtype) if inside else workspace
        helpers.check_rotated_layer(outputs[1].float().cpu().numpy(), layer, device_rotated,
                                    oracle_transforms.randomized(x.float().cpu().numpy(), signs), dtype)


def test_static_buffer_entry_point_refuses_what_does_not_fit():
    from mlkit_amd import native

    lib = native.library()
    x = torch.zeros((8, 32768), device="cuda")                     # 8 x 32768 fp32 = 1 MiB > 512 KiB
    y = torch.zeros((8, 16), device="cuda")
    status = lib.mk_rotated_packed_matvec_static(
        x.data_ptr(), native.MK_F32, 1, 32768, None, None, 1.0, x.data_ptr(), x.data_ptr(), native.MK_F32, x.data_ptr(),
        16, None, None, 0, y.data_ptr(), 8, 16, 32768, 128, 4, 1, -8.0, 1.0, None)
    assert status == native.MK_ERR_INVALID
    assert "buffer holds 524288" in native.last_error() and "mk_rotated_packed_matvec" in native.last_error()
    torch.cuda.synchronize()
