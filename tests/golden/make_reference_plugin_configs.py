"""Writes tests/golden/reference_plugin_configs.json from the three plugin-description files the reference
keeps beside the plugins on this path:

    plugin/skipLayerNormPlugin/CustomSkipLayerNormPluginDynamic_PluginConfig.yaml
    plugin/embLayerNormPlugin/CustomEmbLayerNormPluginDynamic_PluginConfig.yaml
    plugin/bertQKVToContextPlugin/CustomQKVToContextPluginDynamic_PluginConfig.yaml

They are data for the reference's plugin test harness: per plugin version the input and output names, the
accepted input types, the PluginField attributes with their types and which are required, the output shape
expressions, the comparison tolerances and a few named test configurations.  (The "golden_reference_script"
files they name are not part of the reference checkout, so there are no expected output values to take.)
Only the keys the tests use are kept; the YAML is read as data with yaml.safe_load.

    python tests/golden/make_reference_plugin_configs.py [/root/reference]
"""
import json
import os
import sys

import yaml

FILES = [
    "plugin/skipLayerNormPlugin/CustomSkipLayerNormPluginDynamic_PluginConfig.yaml",
    "plugin/embLayerNormPlugin/CustomEmbLayerNormPluginDynamic_PluginConfig.yaml",
    "plugin/bertQKVToContextPlugin/CustomQKVToContextPluginDynamic_PluginConfig.yaml",
]
KEYS = ["inputs", "outputs", "input_dims", "input_dim_constraints", "supported_input_types", "output_dims",
        "attributes", "attribute_types", "attribute_dims", "attribute_options", "attributes_required", "abs_tol",
        "rel_tol", "fp16_atol", "fp16_rtol", "configs"]


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    out = {}
    for rel in FILES:
        with open(os.path.join(root, rel)) as fh:
            doc = yaml.safe_load(fh)
        versions = {}
        for version, body in doc["versions"].items():
            versions[str(version)] = {k: body[k] for k in KEYS if k in body}
        out[doc["name"]] = {"source": rel, "interface": doc.get("interface"), "versions": versions}
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_plugin_configs.json")
    with open(dst, "w") as fh:
        json.dump(out, fh, indent=1, sort_keys=True)
        fh.write("\n")
    print(f"wrote {dst}")


if __name__ == "__main__":
    main()
