"""Parts a layer is put together from.  See `parts.base` for the interfaces and the
registries, `parts.plan` for the data that selects and sizes them."""
