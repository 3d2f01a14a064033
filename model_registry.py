"""Lists the models this engine knows by name, family by family, and the architectures
it can build (output in the manner of the reference's model_registry.py:8-22)."""

from __future__ import annotations

from tokensprint_amd.config import architecture_names, models_by_family


def listing() -> str:
    families = models_by_family()
    if not families:
        return "No models are currently registered."
    lines = ["Registered models:"]
    for family, models in sorted(families.items()):
        lines += ["", f"{family}:"] + [f"  - {m.short} ({m.repo_id})" for m in models]
    lines += ["", "Architectures: " + ", ".join(architecture_names())]
    return "\n".join(lines)


if __name__ == "__main__":
    print(listing())
