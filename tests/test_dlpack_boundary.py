"""Argument validation of the DLPack-level entry points (include/tvmkv_dlpack.h).  Every check runs
before the first device call, so it can be exercised without a GPU: the tensors below describe host
memory and only claim to be ROCm tensors."""
import pytest
import torch

import tvm_amd
from tvm_amd import dlpack as dl

B, HQ, HKV, D, NP, PS = 3, 8, 2, 128, 10, 16


def decode_args(**override):
    """A consistent argument list of the decode slot; `override` swaps single entries."""
    f16, i32, f32 = torch.float16, torch.int32, torch.float32
    a = dict(
        q=dl.tensor(torch.zeros(B, HQ, D, dtype=f16)),
        pages=dl.tensor(torch.zeros(NP, 2, HKV, PS, D, dtype=f16)),
        page_indptr=dl.tensor(torch.zeros(B + 1, dtype=i32)),
        page_indices=dl.tensor(torch.zeros(7, dtype=i32)),
        length_info=dl.tensor(torch.zeros(B, dtype=i32)),
        k_rope_pos_offset=dl.tensor(torch.zeros(B, dtype=i32)),
        q_rope_position=dl.tensor(torch.zeros(B, dtype=i32)),
        out=dl.tensor(torch.zeros(B, HQ, D, dtype=f16)),
        lse=dl.tensor(torch.zeros(B, HQ, dtype=f32)),
    )
    a.update(override)
    return list(a.values()) + [0, 1.0, 1e4, D ** -0.5]


def fails(args, text, name="batch_decode_paged_kv"):
    with pytest.raises(tvm_amd.KVError) as e:
        dl.call(name, *args, stream=0)
    assert e.value.code == -1 and text in str(e.value), str(e.value)


def test_null_tensor_is_named():
    fails(decode_args(q=None), "q is NULL")
    fails(decode_args(lse=None), "lse is NULL")


def test_host_tensors_are_refused():
    cpu = dl.view(torch.zeros(B, HQ, D, dtype=torch.float16), 0, (B, HQ, D), device_type=1)
    fails(decode_args(q=cpu), "q must be a ROCm device tensor")


def test_dtype_is_checked():
    fails(decode_args(page_indptr=dl.tensor(torch.zeros(B + 1, dtype=torch.int64))), "page_indptr must be int32")
    fails(decode_args(lse=dl.tensor(torch.zeros(B, HQ, dtype=torch.float16))), "lse must be float32")
    fails(decode_args(q=dl.tensor(torch.zeros(B, HQ, D, dtype=torch.bfloat16))), "q must be float16")


def test_rank_and_shapes_are_checked():
    fails(decode_args(q=dl.tensor(torch.zeros(B, HQ * D, dtype=torch.float16))), "q has 2 dimensions, expected 3")
    fails(decode_args(lse=dl.tensor(torch.zeros(B + 1, HQ, dtype=torch.float32))), "lse has shape (4, 8), expected (rows of q, h_q)")
    fails(decode_args(k_rope_pos_offset=dl.tensor(torch.zeros(B + 2, dtype=torch.int32))), "k_rope_pos_offset has shape (5)")
    fails(decode_args(length_info=dl.tensor(torch.zeros(2, B, dtype=torch.int32))), "length_info has shape (2, 3), expected (3, batch)")
    fails(decode_args(pages=dl.tensor(torch.zeros(NP, 2, HKV, PS, 64, dtype=torch.float16))), "pages has shape")
    fails(decode_args(q=dl.tensor(torch.zeros(B + 1, HQ, D, dtype=torch.float16)),
                      out=dl.tensor(torch.zeros(B + 1, HQ, D, dtype=torch.float16)),
                      lse=dl.tensor(torch.zeros(B + 1, HQ, dtype=torch.float32)),
                      q_rope_position=dl.tensor(torch.zeros(B + 1, dtype=torch.int32))),
          "one query per page-table entry")


def test_byte_offset_alignment_and_layout():
    base = torch.zeros(B * HQ * D + 64, dtype=torch.float16)
    fails(decode_args(q=dl.view(base, 2, (B, HQ, D))), "q (data + byte_offset) must be aligned to 16 bytes")
    ints = torch.zeros(64, dtype=torch.int32)
    fails(decode_args(page_indptr=dl.view(ints, 6, (B + 1,))), "page_indptr (data + byte_offset) must be aligned to 4 bytes")
    strided = dl.view(torch.zeros(B, HQ, 2 * D, dtype=torch.float16), 0, (B, HQ, D), strides=(HQ * 2 * D, 2 * D, 1))
    fails(decode_args(q=strided), "q must be compact row-major")


def test_all_tensors_on_one_device():
    other = dl.tensor(torch.zeros(B, HQ, dtype=torch.float32))
    other.dl.device.device_id = 3
    fails(decode_args(lse=other), "lse is on device 3 but q is on device 0")


def test_other_slots_name_their_arguments():
    f16, i32 = torch.float16, torch.int32
    pages = dl.tensor(torch.zeros(NP, 2, HKV, PS, D, dtype=f16))
    k = dl.tensor(torch.zeros(5, HKV, D, dtype=f16))
    fails([pages, k, dl.tensor(torch.zeros(5, HKV, 64, dtype=f16)), dl.tensor(torch.zeros(5, dtype=i32))],
          "v_data has shape (5, 2, 64), expected the shape of k_data", name="transpose_append")
    fails([pages, dl.tensor(torch.zeros(4, dtype=i32)), dl.tensor(torch.zeros(2, 6, dtype=i32)), 7],
          "copy_length_indptr has 4 entries, fewer than batch_size + 1 = 8", name="compact_kv_copy")
    qkv = dl.tensor(torch.zeros(5, HQ + 2 * HKV + 1, D, dtype=f16))
    q = dl.tensor(torch.zeros(5, HQ, D, dtype=f16))
    fails([qkv, dl.tensor(torch.zeros(5, dtype=i32)), q, k, k, 1, None, None, 1.0, 1e4],
          "qkv has shape (5, 13, 128), expected (rows, h_q + 2 * h_kv, head_dim)", name="fused_rope")
    factors = dl.tensor(torch.zeros(D // 2, dtype=torch.float32))
    qkv = dl.tensor(torch.zeros(5, HQ + 2 * HKV, D, dtype=f16))
    fails([qkv, dl.tensor(torch.zeros(5, dtype=i32)), q, k, k, 1, factors, None, 1.0, 1e4],
          "rope_ext_factors has shape (64), expected (head_dim,)", name="fused_rope")
