"""What a tuning start-up measured for the package's own kernels is kept in a file and read again."""

import json

from clockwork_amd import ops


def test_choices_written_and_read_back(tmp_path):
    path = str(tmp_path / "choices.json")
    first = ops.ProductPolicy()
    first.k_split_choices[(1536, 8960)] = 6
    first.wide_partial_choices[(1536, 8960)] = 4
    first.swiglu_choices[(17920, 1536)] = False
    first.product_choices[(3584, 1024, True)] = True
    first.write_choices(path)

    later = ops.ProductPolicy()
    later.k_split_choices[(1536, 8960)] = 3          # what this process measured itself stays
    assert later.read_choices(path) == 4
    # remembered, not in use: another model's shapes never show among this engine's choices
    assert later.k_split_choices == {(1536, 8960): 3} and not later.wide_partial_choices and not later.swiglu_choices
    assert later.recall("k_split_choices", (1536, 8960)) is None          # its own choice stands
    assert later.recall("wide_partial_choices", (1536, 8960)) == 4
    assert later.recall("wide_partial_choices", (1536, 8960)) is None     # in use now: nothing left to recall
    assert later.recall("swiglu_choices", (17920, 1536)) is False
    assert later.recall("swiglu_choices", (9, 9)) is None
    assert later.wide_partial_choices == {(1536, 8960): 4} and later.swiglu_choices == {(17920, 1536): False}
    assert not later.product_choices and not ops.DEFAULT_POLICY.k_split_choices
    # what it leaves behind: everything remembered, its own choices on top
    again = str(tmp_path / "again.json")
    later.write_choices(again)
    third = ops.ProductPolicy()
    assert third.read_choices(again) == 4
    assert third.recall("k_split_choices", (1536, 8960)) == 3
    assert third.recall("product_choices", (3584, 1024, True)) is True


def test_choices_of_another_build_or_a_broken_file_are_passed_over(tmp_path):
    path = tmp_path / "choices.json"
    policy = ops.ProductPolicy()
    assert policy.read_choices(str(path)) == 0                      # no file
    path.write_text("{ not json")
    assert policy.read_choices(str(path)) == 0
    record = {"made_for": ["another card", 1, 2, "0.0", "gemm-0.so", "gemm_tile-0.so", "core-0.so"],
              "k_split_choices": [[[1536, 8960], 6]]}
    path.write_text(json.dumps(record))
    assert policy.read_choices(str(path)) == 0 and policy.recall("k_split_choices", (1536, 8960)) is None
    record["made_for"] = ops._choices_made_for()
    path.write_text(json.dumps(record))
    assert policy.read_choices(str(path)) == 1 and policy.recall("k_split_choices", (1536, 8960)) == 6
    assert policy.k_split_choices == {(1536, 8960): 6}
    # a folder that cannot be written: nothing is kept, nothing is raised
    policy.write_choices(str(tmp_path / "missing" / "choices.json"))


def test_choices_file_follows_the_environment(monkeypatch, tmp_path):
    monkeypatch.setenv("CLOCKWORK_AMD_CHOICES_FILE", str(tmp_path / "c.json"))
    assert ops.choices_file() == str(tmp_path / "c.json")
    monkeypatch.delenv("CLOCKWORK_AMD_CHOICES_FILE")
    assert "clockwork_amd_choices_" in ops.choices_file()


def test_the_card_is_known_by_more_than_its_name(monkeypatch):
    """Under a profiler the card's marketing name comes back empty: what identifies it to the
    choices file is its architecture, its compute units and its memory, and another card has
    another file."""
    import types

    import torch

    def card(arch, units):
        return types.SimpleNamespace(name="", gcnArchName=arch, multi_processor_count=units, total_memory=1 << 38)

    monkeypatch.setattr(torch.cuda, "is_available", lambda: True)
    monkeypatch.setattr(torch.cuda, "current_device", lambda: 0)
    monkeypatch.setattr(torch.cuda, "get_device_properties", lambda d: card("gfx950:sramecc+:xnack-", 256))
    made_for, path = ops._choices_made_for(), ops.choices_file()
    assert made_for[:3] == ["gfx950:sramecc+:xnack-", 256, 1 << 38]
    monkeypatch.setattr(torch.cuda, "get_device_properties", lambda d: card("gfx950:sramecc+:xnack-", 128))
    assert ops._choices_made_for() != made_for and ops.choices_file() != path
