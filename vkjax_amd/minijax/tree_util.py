'''Pytree flatten / unflatten for tuples, lists, dicts and None (what the
reference uses from jax: tree_flatten, tree_leaves, tree_structure, tree_unflatten,
tree_map / tree_multimap; reference: vkjax/function.py:26-43,
vkjax/kompute_jaxpr_interpreter.py:69).'''
import typing as tp

import numpy as np


class TreeDef:
    '''Hashable description of a container nest; leaves are `*`.'''
    __slots__ = ('kind', 'meta', 'children', 'num_leaves', '_hash')

    def __init__(self, kind, meta, children):
        self.kind       = kind       #'leaf' | 'none' | 'tuple' | 'list' | 'dict'
        self.meta       = meta       #dict keys (sorted) for 'dict'
        self.children   = tuple(children)
        self.num_leaves = 1 if kind == 'leaf' else sum(c.num_leaves for c in self.children)
        self._hash      = hash((kind, meta, tuple(c._hash for c in self.children)))   #children are hashed once

    def _key(self):
        return (self.kind, self.meta, self.children)

    def __eq__(self, other):
        if self is other:
            return True
        return isinstance(other, TreeDef) and self._hash == other._hash and self._key() == other._key()

    def __hash__(self):
        return self._hash

    def __repr__(self):
        if self.kind == 'leaf':
            return '*'
        if self.kind == 'none':
            return 'None'
        if self.kind == 'dict':
            return '{' + ', '.join(f'{k!r}: {c!r}' for k, c in zip(self.meta, self.children)) + '}'
        inner = ', '.join(map(repr, self.children))
        return f'({inner})' if self.kind == 'tuple' else f'[{inner}]'


_LEAF = TreeDef('leaf', None, ())


_NONE = TreeDef('none', None, ())
_ARRAY = np.ndarray


def tree_flatten(tree) -> tp.Tuple[list, TreeDef]:
    leaves = []

    def rec(x):
        if type(x) is _ARRAY:                       #by far the most frequent node: no further tests
            leaves.append(x)
            return _LEAF
        if x is None:
            return _NONE
        if isinstance(x, tuple) and not hasattr(x, '_fields'):
            return TreeDef('tuple', None, [rec(c) for c in x])
        if isinstance(x, list):
            return TreeDef('list', None, [rec(c) for c in x])
        if isinstance(x, dict):
            keys = tuple(sorted(x.keys()))
            return TreeDef('dict', keys, [rec(x[k]) for k in keys])
        leaves.append(x)
        return _LEAF

    treedef = rec(tree)
    return leaves, treedef


def tree_leaves(tree) -> list:
    '''The leaves alone, in tree_flatten's order, without building the structure.'''
    leaves = []

    def rec(x):
        if type(x) is _ARRAY:
            leaves.append(x)
        elif x is None:
            pass
        elif (isinstance(x, tuple) and not hasattr(x, '_fields')) or isinstance(x, list):
            for c in x:
                rec(c)
        elif isinstance(x, dict):
            for k in sorted(x.keys()):
                rec(x[k])
        else:
            leaves.append(x)

    rec(tree)
    return leaves


def tree_structure(tree) -> TreeDef:
    return tree_flatten(tree)[1]


def tree_unflatten(treedef: TreeDef, leaves):
    it = iter(leaves)

    def rec(td):
        if td.kind == 'leaf':
            return next(it)
        if td.kind == 'none':
            return None
        children = [rec(c) for c in td.children]
        if td.kind == 'tuple':
            return tuple(children)
        if td.kind == 'list':
            return children
        return dict(zip(td.meta, children))

    out = rec(treedef)
    rest = list(it)
    if rest:
        raise ValueError(f'too many leaves for {treedef}: {len(rest)} left over')
    return out


def tree_map(f, tree, *rest):
    leaves, treedef = tree_flatten(tree)
    others = []
    for r in rest:
        l, td = tree_flatten(r)
        if td != treedef:
            raise ValueError(f'tree structures differ: {treedef} vs {td}')
        others.append(l)
    return tree_unflatten(treedef, [f(*xs) for xs in zip(leaves, *others)])


tree_multimap = tree_map
