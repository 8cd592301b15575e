"""Step function, scheduler, engine facade and trace replay."""
