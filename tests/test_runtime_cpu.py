"""The copies of matrices that decode steps read (`Runtime.tile_for_decode`): asked for while a model is built, made
when it is whole, the ones every step reads first, within half of the memory that is free then."""
import torch

from fllm_amd.parts.runtime import Runtime


class Matrix:
    """Stands for a matrix on the device: the runtime asks only where it is and how large."""
    is_cuda = True

    def __init__(self, name, mib):
        self.name, self.mib = name, mib

    def numel(self):
        return self.mib << 19

    def element_size(self):
        return 2


class Library:
    def __init__(self):
        self.made = []

    def tile_for_decode(self, w, gate_up=False):
        self.made.append((w.name, gate_up))
        return True


def build(rt):
    rt.collect_tile_requests()
    for layer in range(3):
        rt.tile_for_decode(Matrix(f"o{layer}", 32))
        rt.tile_for_decode(Matrix(f"qkv{layer}", 48), priority=1)
        rt.tile_for_decode(Matrix(f"down{layer}", 112))
        rt.tile_for_decode(Matrix(f"gate_up{layer}", 224), gate_up=True, priority=1)
    return rt.tiles_for_model()


def test_copies_are_made_by_priority_within_half_of_the_free_memory(monkeypatch):
    every = [(f"{kind}{layer}", False) for layer in range(3) for kind in ("o", "down")] + \
            [(f"{kind}{layer}", kind == "gate_up") for layer in range(3) for kind in ("qkv", "gate_up")]
    for free_mib, want in ((1 << 20, every),                       # plenty: all twelve, the first kind first
                           (2 * (3 * 144 + 48 + 224 + 48 + 10), every[:6] + [("qkv0", False), ("gate_up0", True), ("qkv1", False)]),
                           (2 * 300, [("o0", False), ("down0", False), ("o1", False), ("down1", False)]),
                           (2 * 40, [("o0", False)])):
        monkeypatch.setattr(torch.cuda, "mem_get_info", lambda device=None: (free_mib << 20, 1 << 40))
        lib = Library()
        made = build(Runtime(torch.device("cpu"), torch.bfloat16, lib, 128, decode_weight_tiles="auto"))
        assert lib.made == want, (free_mib, lib.made)
        assert made == sum(m << 20 for m in (dict(o=32, qkv=48, down=112, gate_up=224)[n.rstrip("012")] for n, _ in want))
    # switched on: no budget; switched off, or another precision: nothing
    lib = Library()
    build(Runtime(torch.device("cpu"), torch.bfloat16, lib, 128, decode_weight_tiles=True))
    assert lib.made == every
    for rt in (Runtime(torch.device("cpu"), torch.bfloat16, Library(), 128, decode_weight_tiles=False),
               Runtime(torch.device("cpu"), torch.float32, Library(), 128)):
        assert build(rt) == 0 and rt.ops.made == []


def test_outside_a_model_a_copy_is_made_at_once(monkeypatch):
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda device=None: (100 << 20, 1 << 40))
    lib = Library()
    rt = Runtime(torch.device("cpu"), torch.bfloat16, lib, 128)
    rt.tile_for_decode(Matrix("small", 4))
    rt.tile_for_decode(Matrix("large", 16))             # more than a twentieth of what is free
    rt.tile_for_decode(Matrix("pair", 2), gate_up=True)
    assert lib.made == [("small", False), ("pair", True)]
