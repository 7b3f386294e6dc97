"""jax.tree_util of the model (dict pytrees only)."""


class DictKey:
    def __init__(self, key):
        self.key = key

    def __str__(self):
        return str(self.key)


def tree_flatten_with_path(tree, prefix=()):
    out = []
    if isinstance(tree, dict):
        for k in tree:
            out += tree_flatten_with_path(tree[k], prefix + (DictKey(k),))[0]
    else:
        out.append((prefix, tree))
    return out, None
