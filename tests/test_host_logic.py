"""The modules' order knobs on the host (no GPU): the rules for pieces and partitions, and the engine's tuned values
where crit's kernel build has written them beside a module (the generated _crit_tuning accessor, kernels/crit_kernels/
build.py:255-313, stood in for by a class with the same knobs() call)."""


def test_latent_partitions_follow_the_rule_or_the_engines_tuning():
    import torch
    import crit_amd.latent_attention as la
    device = torch.device("cuda", 0)
    held = dict(la._CUS)
    la._CUS[0] = 256                                   # an MI355X's compute units (no device is asked)
    try:
        # (128 heads of a (512, 64) cache, 16-bit or E4M3: the many-heads kernel, a workgroup a compute unit; pages of no
        # multiple of 16, another shape or the small tiles asked for: the rule of the small tiles)
        assert [la.partitions(device, h, 512, 64, 64) for h in (1, 16, 32, 64, 128)] == [64, 64, 64, 32, 8]
        assert la.partitions(device, 128, 512, 64, 64, 1) == 8 and la.partitions(device, 128, 512, 64, 24) == 16
        assert la.partitions(device, 128, 512, 64, 64, 0, 16) == 16 and la.partitions(device, 128, 256, 64, 64) == 16
        assert la.tile_rows(128, 512, 64, 64) == 128 and la.tile_rows(256, 512, 64, 16) == 128
        assert la.tile_rows(64, 512, 64, 64) == 16 and la.tile_rows(128, 512, 64, 64, asked=16) == 16

        class Tuning:
            @staticmethod
            def knobs(structure, key, rows):
                return {"PARTS": 12 if key["H"] == 128 else 0, "PIECE": 0, "TILE_ROWS": 16 if key["PAGE"] == 32 else 0}

        la._crit_tuning = Tuning
        assert la.partitions(device, 128, 512, 64, 64) == 12 and la.partitions(device, 16, 512, 64, 64) == 64
        assert la.tile_rows(128, 512, 64, 32) == 16 and la.tile_rows(128, 512, 64, 64) == 128
    finally:
        la._crit_tuning = None
        la._CUS.clear(), la._CUS.update(held)


def test_the_split_launchs_order_knobs_follow_the_rule_or_the_engines_tuning():
    import crit_amd.paged_kv_attention as pk
    assert pk.piece_size(128, 128, "bf16", 8) == 512 and pk.piece_size(128, 128, "fp8", 8) == 1536

    class Tuning:
        @staticmethod
        def knobs(structure, key, rows):
            assert structure == "split" and set(key) == {"D", "DV", "HKV", "KIND"}
            return {"PIECE": 768 if key["KIND"] == 1 else 0, "PARTS": 16 if key["HKV"] == 4 else 0}

    pk._crit_tuning = Tuning
    try:
        assert pk.piece_size(128, 128, "fp8", 8) == 768 and pk.piece_size(128, 128, "bf16", 8) == 512
        assert pk.piece_size(128, 128, "fp8") == 1536                      # no geometry, no tuning
        assert pk.partitions("cpu", 4, "bf16", 128, 128) == 16
    finally:
        pk._crit_tuning = None
