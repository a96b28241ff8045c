"""Stack of Clebsch-Gordan layers with the l=0 skip-connection embedding: the reference's
``SphericalCNN`` (CGNet/CGNet.py:14-69) on top of the HIP-backed ``CGBN_cuda`` layers."""
import torch
from torch import nn

from . import CG_layers as cglayers


class SphericalCNN(nn.Module):
    def __init__(self, lmax, taus, cuda=True, norm=True, skipconn=True, sparse_flag=False, device=None):
        """
        :param lmax: degrees l = 0..lmax
        :param taus: list of lists; taus[i] are the channels per degree entering layer i,
            taus[i+1] the channels leaving it
        :param cuda: must be True (the layers only run on the GPU)
        :param norm: fragment normalisation on/off
        :param skipconn: concatenate the l=0 fragments of the input and of every layer output;
            otherwise only the last layer's l=0 fragment is returned
        :param sparse_flag: True selects the minimum-spanning-tree subset of (l1, l2) pairs
        :param device: overrides the device implied by ``cuda`` (e.g. 'cpu' to inspect parameters)
        """
        assert cuda, "Do not support these parameters yet"
        super().__init__()
        self.lmax = lmax
        self.taus = taus
        self.n_layers = len(taus) - 1
        dev = 'cuda' if device is None else device
        self.cgs = nn.ModuleList([cglayers.CGBN_cuda(lmax, taus[i], taus[i + 1], batchnorm=norm,
                                                     sparse_flag=sparse_flag, device=dev)
                                  for i in range(self.n_layers)])
        self.skipconn = skipconn
        if self.skipconn:
            self.output_length = 2 * sum(int(t[0]) for t in taus)
        else:
            self.output_length = 2 * int(taus[-1][0])
        self.to(dev)

    def forward(self, f_input):
        if isinstance(f_input, (list, tuple)):
            B = f_input[0].shape[0]
            first = f_input[0].reshape(B, -1)
        else:
            B = f_input.shape[0]
            first = f_input[:, 0:int(self.taus[0][0]), :].reshape(B, -1)
        embedding = [first] if self.skipconn else []
        fs = f_input
        for layer in self.cgs:
            fs = layer(fs, straight_output=False)
            if self.skipconn:
                embedding.append(fs[0].reshape(B, -1))
        if self.skipconn:
            return torch.cat(embedding, 1)
        return fs[0].reshape(B, -1)


def normalisation_counts(module):
    """{module path: bn_cnt} of every fragment-normalisation layer under ``module``.  The count is a plain
    python attribute in the reference (``CG_layers.py:92,130``) and therefore missing from ``state_dict``;
    store this dict next to a checkpoint and hand it to ``load_normalisation_counts`` when resuming."""
    return {name: float(m.bn_cnt) for name, m in module.named_modules() if hasattr(m, "bn_cnt")}


def load_normalisation_counts(module, counts):
    named = dict(module.named_modules())
    for name, cnt in counts.items():
        if name not in named or not hasattr(named[name], "bn_cnt"):
            raise KeyError("no fragment-normalisation layer named %r" % name)
        named[name].bn_cnt = float(cnt)


class SphericalCNN_fast(SphericalCNN):
    """The stack under the constructor the reference's Shrec17 script calls
    (Shrec17/Shrec17_main_fast.py:78-79): ``SphericalCNN(lmax, taus, nlayers, skip_type=, num_channels_input=)``
    with ``taus`` ONE list of channels per degree shared by all layers.  The class itself is not part of the
    reference (the script imports it from a module the repository does not hold), so the meaning of the
    arguments is taken from that call site and from ``SphericalCNN``:

    * the input carries ``num_channels_input`` channels in every degree (6 spherical signals per SHREC17 mesh);
    * ``nlayers`` layers follow, each producing ``taus``;
    * ``skip_type`` 0 returns the last layer's l=0 fragment only, 1 the concatenation of the l=0 fragments of the
      input and of every layer (``skipconn``); the script routes other values to residual classes that are not
      in the reference either, and they are refused here.
    """

    def __init__(self, lmax, taus, nlayers, skip_type=1, num_channels_input=1, norm=True, sparse_flag=False,
                 device=None):
        if skip_type not in (0, 1):
            raise NotImplementedError("skip_type=%r: only 0 (last l=0 fragment) and 1 (skip connections) exist" % (skip_type,))
        if len(taus) != lmax + 1:
            raise AssertionError("taus must have lmax+1 entries")
        if int(nlayers) < 1 or int(num_channels_input) < 1:
            raise AssertionError("nlayers and num_channels_input must be positive")
        per_layer = [[int(num_channels_input)] * (lmax + 1)] + [[int(t) for t in taus] for _ in range(int(nlayers))]
        super().__init__(lmax, per_layer, cuda=True, norm=norm, skipconn=bool(skip_type), sparse_flag=sparse_flag,
                         device=device)
        self.skip_type = skip_type
        self.num_channels_input = int(num_channels_input)
