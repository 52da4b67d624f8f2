"""Scene dumps in the format the reference's timing harness reads
(tests/rasterizer_test.cpp:145-212): a TorchScript module whose attributes are the rasterizer's
inputs — tensors ``means_3d, means_2d, shs, opacities, scales, rotations, viewmatrix, projmatrix,
campos`` (matrices in the API's transposed convention) and scalars ``image_height, image_width,
tanfovx, tanfovy, scale_modifier, sh_degree``.

``save_scene`` writes such a dump from a dict (for example a ``ds_splat_amd.synthetic`` scene),
``load_scene`` reads one back into a dict.  ``torch.jit.load`` runs the archive's code: only
load dumps you made or trust.
"""
import torch

TENSORS = ("means_3d", "means_2d", "shs", "opacities", "scales", "rotations", "viewmatrix", "projmatrix", "campos")
INTS = ("image_height", "image_width", "sh_degree")
FLOATS = ("tanfovx", "tanfovy", "scale_modifier")


class SceneDump(torch.nn.Module):
    image_height: int
    image_width: int
    sh_degree: int
    tanfovx: float
    tanfovy: float
    scale_modifier: float

    def __init__(self, scene):
        super().__init__()
        for name in TENSORS:
            self.register_buffer(name, scene[name].detach().cpu().contiguous())
        self.image_height = int(scene["image_height"])
        self.image_width = int(scene["image_width"])
        self.sh_degree = int(scene["sh_degree"])
        self.tanfovx = float(scene["tanfovx"])
        self.tanfovy = float(scene["tanfovy"])
        self.scale_modifier = float(scene["scale_modifier"])

    def forward(self):
        return self.means_3d


def scene_from_synthetic(sc):
    """A dump dict from a ``ds_splat_amd.synthetic.make_scene`` scene."""
    d = {k: sc[k] for k in ("means_3d", "shs", "opacities", "scales", "rotations", "viewmatrix", "projmatrix",
                            "campos", "tanfovx", "tanfovy", "sh_degree")}
    d["means_2d"] = torch.zeros_like(sc["means_3d"])
    d["image_height"], d["image_width"] = sc["height"], sc["width"]
    d["scale_modifier"] = sc.get("scale_modifier", 1.0)
    return d


def save_scene(path, scene):
    torch.jit.script(SceneDump(scene)).save(path)


def load_scene(path, device="cpu"):
    m = torch.jit.load(path, map_location="cpu")
    d = {name: getattr(m, name).to(device) for name in TENSORS}
    for name in INTS:
        d[name] = int(getattr(m, name))
    for name in FLOATS:
        d[name] = float(getattr(m, name))
    return d
