# Top-level build.  `make` builds the two product libraries; the per-block executables keep the
# reference's target names and land in this directory, because the llama-*.py drivers run
# `make <target>` and then `./<target> ...` from their working directory.
PKG     := zkllm-ccs2024_amd
TARGETS := main ppgen commit-param self-attn ffn rmsnorm skip-connection

all: libs

libs:
	$(MAKE) -C $(PKG)/csrc
	$(MAKE) -C $(PKG)/host

$(TARGETS): libs
	$(MAKE) -C $(PKG)/host $@
	cp $(PKG)/host/$@ ./$@

oracle:
	$(MAKE) -C oracle

clean:
	$(MAKE) -C $(PKG)/csrc clean
	$(MAKE) -C $(PKG)/host clean
	rm -f $(TARGETS)

.PHONY: all libs oracle clean
