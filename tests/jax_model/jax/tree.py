"""jax.tree.map for the pytrees the binding uses: dicts, lists, tuples and leaves."""


def map(f, tree, *rest, is_leaf=None):  # noqa: A001
    if is_leaf is not None and is_leaf(tree):
        return f(tree, *rest)
    if isinstance(tree, dict):
        return {k: map(f, tree[k], *[r[k] for r in rest], is_leaf=is_leaf) for k in tree}
    if isinstance(tree, (list, tuple)):
        return type(tree)(map(f, t, *[r[i] for r in rest], is_leaf=is_leaf) for i, t in enumerate(tree))
    return f(tree, *rest)
