"""Stream logger with the level and no-propagate behaviour of dlblas/utils/logger.py:32-39."""
import logging

_FORMAT = '%(asctime)s - %(levelname)s - %(message)s (%(filename)s:%(lineno)d)'
_COLOURS = {
    logging.DEBUG: '\x1b[1;34m',
    logging.INFO: '\x1b[1;32m',
    logging.WARNING: '\x1b[33;20m',
    logging.ERROR: '\x1b[31;20m',
    logging.CRITICAL: '\x1b[31;1m',
}


class _Colour(logging.Formatter):

    def format(self, record):
        colour = _COLOURS.get(record.levelno, '')
        return logging.Formatter(f'{colour}{_FORMAT}\x1b[0m').format(record)


def get_logger(name: str) -> logging.Logger:
    logger = logging.getLogger(name)
    if not getattr(logger, '_dlblas_configured', False):
        logger.setLevel(logging.INFO)
        handler = logging.StreamHandler()
        handler.setFormatter(_Colour())
        logger.addHandler(handler)
        logger.propagate = False
        logger._dlblas_configured = True
    return logger
