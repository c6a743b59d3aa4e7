"""Python faces of the bfloat16 attention kernels (csrc/attention_bf16.hip)."""


def attention(q, k_pages, v_pages, batch, table, scale, window):
    """The fast kernel's result, or None if no fast kernel takes this shape."""
    return None
