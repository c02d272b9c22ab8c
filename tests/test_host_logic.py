

def test_latent_partitions_follow_the_rule_or_the_engines_tuning():
    import torch
    import crit_amd.latent_attention as la
    device = torch.device("cuda", 0)
    held = dict(la._CUS)
    la._CUS[0] = 256                                   # an MI355X's compute units (no device is asked)
    try:
        assert [la.partitions(device, h, 512, 64, 64) for h in (1, 16, 32, 64, 128)] == [64, 64, 64, 32, 16]

        class Tuning:
            @staticmethod
            def knobs(structure, key, rows):
                return {"PARTS": 8 if key["H"] == 128 else 0, "PIECE": 0}

        la._crit_tuning = Tuning
        assert la.partitions(device, 128, 512, 64, 64) == 8 and la.partitions(device, 16, 512, 64, 64) == 64
    finally:
        la._crit_tuning = None
        la._CUS.clear(), la._CUS.update(held)
