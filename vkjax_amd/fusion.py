'''Peephole fusion over the op list of one program (placeholder pass-through until the
per-primitive path is verified on the device).'''


def fuse_ops(all_ops, bufferpool, outvars):
    return all_ops
