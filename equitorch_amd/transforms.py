"""Graph data transforms (``equitorch/transforms/__init__.py``): radius graph with edge vectors, vector norms,
spherical harmonics of the edge vectors and length embeddings, written onto a PyTorch Geometric style data object.

With PyTorch Geometric installed the classes are ``BaseTransform`` subclasses registered under the reference's
functional names, and ``RadiusGraph`` calls ``torch_geometric.nn.radius_graph``.  Without it they are plain
callables on any object with attribute access (``data.pos``, ``data.batch`` ...), applied to a shallow copy as
``BaseTransform.__call__`` does, and the radius graph is found by blocked brute force on the device of ``pos``.
"""
import copy
from typing import Callable, Optional

import torch
from torch import Tensor

try:                                       # pragma: no cover - depends on the installation
    import torch_geometric
    from torch_geometric.data.datapipes import functional_transform
    from torch_geometric.transforms import BaseTransform
except ImportError:
    torch_geometric = None

    class BaseTransform:                   # the two behaviours of PyG's base class the transforms rely on
        def __call__(self, data):
            return self.forward(copy.copy(data))

        def forward(self, data):
            raise NotImplementedError

        def __repr__(self) -> str:
            return f"{self.__class__.__name__}()"

    def functional_transform(name: str):
        return lambda cls: cls


def radius_graph(pos: Tensor, r: float, batch: Optional[Tensor] = None, loop: bool = False,
                 max_num_neighbors: int = 32, flow: str = "source_to_target", block: int = 4096) -> Tensor:
    """``edge_index (2, E)`` of all pairs closer than ``r`` inside one example of the batch: for every centre node,
    in index order, its first ``max_num_neighbors`` neighbours in index order.  ``source_to_target`` puts the
    neighbour in row 0 and the centre in row 1 (messages flow into the centre), as
    ``torch_geometric.nn.radius_graph`` does."""
    assert flow in ("source_to_target", "target_to_source")
    n = pos.shape[0]
    centres, neighbours = [], []
    index = torch.arange(n, device=pos.device)
    for start in range(0, n, block):
        rows = index[start:start + block]
        close = torch.cdist(pos[rows], pos) < r
        if batch is not None:
            close &= batch[rows, None] == batch[None, :]
        if not loop:
            close[torch.arange(rows.numel(), device=pos.device), rows] = False
        close &= close.cumsum(dim=1) <= max_num_neighbors
        c, nb = close.nonzero(as_tuple=True)
        centres.append(rows[c])
        neighbours.append(nb)
    centre, neighbour = torch.cat(centres), torch.cat(neighbours)
    return torch.stack([neighbour, centre] if flow == "source_to_target" else [centre, neighbour])


@functional_transform('radius_graph_eqt')
class RadiusGraph(BaseTransform):
    r"""Adds ``edge_index`` (all pairs within ``r``) and ``edge_vec = pos[edge_index[1]] - pos[edge_index[0]]``
    (reference ``:17-107``; attribute names configurable)."""

    def __init__(self, r: float, loop: bool = False, max_num_neighbors: int = 32, flow: str = 'source_to_target',
                 pos_attr: str = 'pos', edge_index_attr: str = 'edge_index', edge_vector_attr: str = 'edge_vec',
                 num_workers: int = 1) -> None:
        self.r = r
        self.loop = loop
        self.max_num_neighbors = max_num_neighbors
        self.flow = flow
        self.num_workers = num_workers
        self.pos_attr = pos_attr
        self.edge_index_attr = edge_index_attr
        self.edge_vector_attr = edge_vector_attr

    def forward(self, data):
        pos = getattr(data, self.pos_attr)
        batch = getattr(data, 'batch', None)
        if torch_geometric is not None:    # pragma: no cover
            edge_index = torch_geometric.nn.radius_graph(pos, self.r, batch, self.loop,
                                                         max_num_neighbors=self.max_num_neighbors, flow=self.flow,
                                                         num_workers=self.num_workers)
        else:
            edge_index = radius_graph(pos, self.r, batch, self.loop, self.max_num_neighbors, self.flow)
        setattr(data, self.edge_index_attr, edge_index)
        # the reference reads ``data.pos`` here whatever ``pos_attr`` says (``:100-102``); the configured one is meant
        setattr(data, self.edge_vector_attr, pos[edge_index[1]] - pos[edge_index[0]])
        return data

    def __repr__(self) -> str:
        return f'{self.__class__.__name__}(r={self.r})'


@functional_transform('add_vector_norm')
class AddVectorNorm(BaseTransform):
    r"""``data.<norm_attr> = |data.<vector_attr>|`` along the last axis (reference ``:109-151``)."""

    def __init__(self, vector_attr: str = 'edge_vec', norm_attr: str = 'edge_norm') -> None:
        self.vector_attr = vector_attr
        self.norm_attr = norm_attr

    def forward(self, data):
        setattr(data, self.norm_attr, getattr(data, self.vector_attr).norm(dim=-1))
        return data


@functional_transform('add_spherical_harmonics')
class AddSphericalHarmonics(BaseTransform):
    r"""``data.<sh_attr> = Y_0..l_max(data.<vector_attr>)``, ``(E, (l_max + 1)^2)``, on the spherical-harmonics kernel
    (reference ``:153-201``).  As there, the vectors are taken as they are: for a vector of length ``r`` the degree-``l``
    block is ``r^l`` times the harmonic of its direction."""

    def __init__(self, l_max: int, vector_attr: str = 'edge_vec', sh_attr: str = 'edge_sh',
                 integral_normalize: bool = False) -> None:
        self.l_max = l_max
        self.vector_attr = vector_attr
        self.sh_attr = sh_attr
        self.integral_normalize = integral_normalize

    def forward(self, data):
        from .nn.functional.sphericals import spherical_harmonics
        vec = getattr(data, self.vector_attr)
        setattr(data, self.sh_attr, spherical_harmonics(vec, self.l_max, integral_normalize=self.integral_normalize))
        return data


@functional_transform('add_vector_length_embedding')
class AddVectorLengthEmbedding(BaseTransform):
    r"""``data.<embedding_attr> = emb(|data.<vector_attr>|)`` for a callable ``emb`` such as ``BesselBasis``
    (reference ``:203-253``)."""

    def __init__(self, emb: Callable[[Tensor], Tensor], vector_attr: str = 'edge_vec',
                 embedding_attr: str = 'edge_emb') -> None:
        self.emb = emb
        self.vector_attr = vector_attr
        self.embedding_attr = embedding_attr

    def forward(self, data):
        setattr(data, self.embedding_attr, self.emb(getattr(data, self.vector_attr).norm(dim=-1)))
        return data


__all__ = ['RadiusGraph', 'AddSphericalHarmonics', 'AddVectorNorm', 'AddVectorLengthEmbedding']
