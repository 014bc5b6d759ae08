"""Small helpers shared by the host-side classes."""


def dict_to_str(d, indent=0):
    """Vertically formatted string of a dictionary, one "key: value" line per entry (the layout the reference prints
    its actions / performance tables in, src/utils.py:23-30)."""
    pad = indent * " "
    lines = [pad + "{"]
    keys = list(d)
    for i, key in enumerate(keys):
        lines.append(pad + "  " + str(key) + ": " + str(d[key]) + ("," if i < len(keys) - 1 else ""))
    lines.append(pad + "}")
    return "\n".join(lines)
