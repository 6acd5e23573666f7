"""Host-side logic that needs no GPU: how the model call's keyword arguments are built for a sub-batch of a multimodal
batch (trl/trainer/grpo_trainer.py:1463-1510), and when the fused head keeps its stash."""
import torch


def _trainer():
    import trl_amd

    class Trainer(trl_amd.GRPOLossMixin):
        model_kwarg_keys = {"logits_to_keep"}

    return Trainer()


def test_patch_rows_follow_the_image_grid():
    """Qwen-style inputs: `pixel_values` holds the patch rows of all images back to back, `image_grid_thw` one row per
    image, `num_images` the images per sample.  Samples 0:2 own images 0..2 (4 + 6 + 4 patch rows), samples 2:4 own
    image 3 (sample 2 has no image)."""
    tr = _trainer()
    ids = torch.arange(4 * 5).view(4, 5)
    attn = torch.ones(4, 5, dtype=torch.long)
    grid = torch.tensor([[1, 2, 2], [1, 2, 3], [1, 1, 4], [1, 3, 2]])
    pixels = torch.arange(20 * 3).view(20, 3)
    kw = dict(pixel_values=pixels, image_grid_thw=grid, num_images=[1, 2, 0, 1], token_type_ids=ids + 100,
              mm_token_type_ids=ids + 200)
    first = tr._model_inputs(ids, attn, 0, 2, 3, False, **kw)
    assert torch.equal(first["pixel_values"], pixels[0:14]) and torch.equal(first["image_grid_thw"], grid[0:3])
    assert torch.equal(first["input_ids"], ids[0:2]) and torch.equal(first["token_type_ids"], ids[0:2] + 100)
    assert torch.equal(first["mm_token_type_ids"], ids[0:2] + 200)
    assert first["logits_to_keep"] == 4 and first["use_cache"] is False and "output_router_logits" not in first
    second = tr._model_inputs(ids, attn, 2, 4, 3, True, **kw)
    assert torch.equal(second["pixel_values"], pixels[14:20]) and torch.equal(second["image_grid_thw"], grid[3:4])
    assert second["output_router_logits"] is True
    only_third = tr._model_inputs(ids, attn, 2, 3, 3, False, **kw)  # a sample without images
    assert only_third["pixel_values"].shape[0] == 0 and only_third["image_grid_thw"].shape[0] == 0
    for out in (first, second):  # the lists that steer the slicing are no model arguments
        assert "num_images" not in out and "num_tiles" not in out and "image_position_ids" not in out
    whole = tr._model_inputs(ids, attn, 0, 4, 3, False, **kw)
    assert torch.equal(whole["pixel_values"], pixels) and torch.equal(whole["image_grid_thw"], grid)


def test_image_and_tile_indexed_inputs():
    tr = _trainer()
    ids = torch.zeros(3, 4, dtype=torch.long)
    attn = torch.ones(3, 4, dtype=torch.long)
    # image-indexed tensors with position ids
    pixels = torch.arange(5 * 2).view(5, 2)
    pos = torch.arange(5 * 3).view(5, 3)
    out = tr._model_inputs(ids, attn, 1, 3, 2, False, pixel_values=pixels, image_position_ids=pos, num_images=[2, 1, 2])
    assert torch.equal(out["pixel_values"], pixels[2:5]) and torch.equal(out["image_position_ids"], pos[2:5])
    # tile-indexed tensors: pixel_values, pixel_attention_mask and spatial_shapes move together
    tiles = torch.arange(6 * 2).view(6, 2)
    pam = torch.arange(6 * 4).view(6, 4)
    shapes = torch.arange(6 * 2).view(6, 2) + 50
    out = tr._model_inputs(ids, attn, 0, 2, 2, False, pixel_values=tiles, pixel_attention_mask=pam, spatial_shapes=shapes,
                           num_tiles=[1, 3, 2])
    assert torch.equal(out["pixel_values"], tiles[0:4]) and torch.equal(out["pixel_attention_mask"], pam[0:4])
    assert torch.equal(out["spatial_shapes"], shapes[0:4]) and "num_tiles" not in out
    # sample-indexed tensors
    px = torch.arange(3 * 2).view(3, 2)
    sizes = torch.arange(3 * 2).view(3, 2) + 9
    mask = torch.arange(3 * 2).view(3, 2) + 20
    out = tr._model_inputs(ids, attn, 1, 2, 2, False, pixel_values=px, pixel_attention_mask=mask, image_sizes=sizes)
    assert torch.equal(out["pixel_values"], px[1:2]) and torch.equal(out["pixel_attention_mask"], mask[1:2])
    assert torch.equal(out["image_sizes"], sizes[1:2])
    # text only: nothing but the text arguments
    out = tr._model_inputs(ids, attn, 0, 3, 2, False)
    assert set(out) == {"input_ids", "attention_mask", "logits_to_keep", "use_cache"}


def test_head_stash_budget_and_shape(monkeypatch):
    """The stash of the fused head: its size comes from the library (2 bytes per logit + one reference exponent per 64
    logits + the targets' logits, both dimensions padded to 256) and the host keeps it only within its budget."""
    from trl_amd import ops

    n, v = 300, 1000
    rows, ld, four = ops._head_stash_shape(n, v)
    vpad = 1024
    assert (rows, ld, four) == (vpad // 4 + vpad // 128 + 1, 512, 4)
    nbytes = rows * ld * four * 2
    monkeypatch.setenv("TRL_AMD_HEAD_STASH_GIB", str((nbytes + 1) / 2**30))
    assert ops.head_stash_fits(n, v)
    monkeypatch.setenv("TRL_AMD_HEAD_STASH_GIB", str((nbytes - 1) / 2**30))
    assert not ops.head_stash_fits(n, v)
    monkeypatch.setenv("TRL_AMD_HEAD_STASH_GIB", "0")
    assert not ops.head_stash_fits(n, v) and not ops.head_stash_fits(1, 1)
    monkeypatch.delenv("TRL_AMD_HEAD_STASH_GIB")
    assert ops.head_stash_fits(32768, 151936) and not ops.head_stash_fits(0, v)  # 10.3 GB of the default 24 GiB
    assert not ops.head_stash_fits(131072, 151936)  # 41 GB
