"""elf_amd: MI355X-native execution path of one ELF pipeline stage (see include/elf_stage.h)."""
