"""Import-path alias: ``from jvp_flash_attention.jvp_attention import JVPAttn, attention`` (the
reference's import line, README.md:41) resolves to the MI355X implementation."""
